"""Gated linear attention: a matrix state per head whose rows decay each by a factor that the token sets.

    q = Wq x / sqrt(dim),  k = Wk x   heads x dim;     v = Wv x   heads x vdim
    alpha = sigmoid(Wa2 (Wa1 x) + b)^(1/tau)           heads x dim, one decay per key channel, through a low rank
    S_t = diag(alpha_t) S_(t-1) + k_t v_t^T            a [dim, vdim] matrix per (sequence, head), zero at the start
    o_t = S_t^T q_t
    out = Wo ( rms(o_t over each head's vdim) * w_norm * silu(Wg x) )      w_norm [vdim], the same for all heads

(The recurrence is that of S. Yang, B. Wang, Y. Shen, R. Panda, Y. Kim, "Gated Linear Attention Transformers with
Hardware-Efficient Training".)  q, k, v and g are one stacked product; the decays' pre-activations are a second, float32
product of the low-rank rows.  The state is a fixed-size float32 region of the cache (kind "state"): a step continues from
what the sequence's slot holds, whatever the step's cut, and a slot starts at zero.  The decays (through the logarithm of
the sigmoid), the state and both products of the recurrence are float32; the projections have the engine's activation
type.  One kernel walks a sequence's rows of the step in order (`gla_scan`, prompts and decode steps alike; long
sequences in chunks side by side, after which the chunks' states are joined in order and every chunk's rows get what they owe
the state their chunk started from), one norms and gates (`gated_group_rmsnorm` with the gate behind the norm).  Every size and constant is a constructor parameter.
"""

from __future__ import annotations

import torch

from ..weights.binder import TensorSpec
from .base import MIXERS, CacheNeed
from .linear import Linear


class GatedLinearAttention:
    graph_safe = True      # forward reads only the step's device tensors
    graph_safe_rows = None
    writes_fresh = True    # forward(..., fresh=True) writes its result instead of adding it

    def __init__(self, hidden: int, n_heads: int, dim: int, vdim: int, decay_rank: int, tau: float, norm_eps: float, prefix: str):
        if not tau > 0.0:
            raise ValueError(f"tau must be positive, got {tau}")
        self.hidden, self.n_heads, self.dim, self.vdim = int(hidden), int(n_heads), int(dim), int(vdim)
        self.decay_rank, self.tau, self.norm_eps, self.prefix = int(decay_rank), float(tau), float(norm_eps), prefix
        key_width, value_width = self.n_heads * self.dim, self.n_heads * self.vdim
        self.q_off, self.k_off, self.v_off, self.g_off = 0, key_width, 2 * key_width, 2 * key_width + value_width
        self.proj = Linear(hidden, [key_width, key_width, value_width, value_width],
                           [prefix + "q", prefix + "k", prefix + "v", prefix + "g"])
        self.decay_down = Linear(hidden, self.decay_rank, prefix + "a1")
        self.decay_up = Linear(self.decay_rank, key_width, prefix + "a2")
        self.out = Linear(value_width, hidden, prefix + "o")
        self.norm_weight = self.decay_bias = None

    def tensor_specs(self):
        return (self.proj.tensor_specs() + self.decay_down.tensor_specs() + self.decay_up.tensor_specs() + self.out.tensor_specs() + [
            TensorSpec(self.prefix + "a2.b", (self.n_heads * self.dim,), "norm"), TensorSpec(self.prefix + "norm", (self.vdim,), "norm")])

    def load(self, get):
        for linear in (self.proj, self.decay_down, self.decay_up, self.out):
            linear.load(get)
        # one weight for all heads, laid out once per head for the kernel that norms the heads of a row side by side
        self.norm_weight = get(self.prefix + "norm").to(torch.float32).repeat(self.n_heads).contiguous()
        self.decay_bias = get(self.prefix + "a2.b").to(torch.float32).contiguous()

    def prepare(self, kernels):
        for linear in (self.proj, self.decay_down, self.decay_up, self.out):
            linear.prepare(kernels)

    def cache_need(self):
        return CacheNeed(kind="state", state_shape=(self.n_heads, self.dim, self.vdim), state_dtype=torch.float32)

    def working_bytes(self, step) -> int:
        width = self.n_heads * self.vdim
        chunks = 0
        if step.sizes is not None and hasattr(step.sizes, "gla_chunk_bytes"):
            chunks = step.sizes.gla_chunk_bytes(step.seqs, step.rows, step.max_rows_per_seq, self.n_heads, self.dim, self.vdim)
        return (chunks + self.proj.working_bytes(step, step.rows) + self.decay_down.working_bytes(step, step.rows)
                + self.decay_up.working_bytes(step, step.rows, out_size=4) + step.matrix(step.rows, width, 4)
                + step.matrix(step.rows, width, reader=self.out.reader_for_plan(step.act_size))
                + self.out.working_bytes(step, step.rows, accumulate=True))

    def forward(self, ctx, x, hidden, cache, then_norm=None, fresh=False):
        k = ctx.kernels
        width = self.n_heads * self.vdim
        proj = self.proj.forward(ctx, x)
        decays = self.decay_up.forward(ctx, self.decay_down.forward(ctx, x), out_dtype=torch.float32)
        mixed = ctx.new_f32(ctx.n_rows, width)
        k.gla_scan(proj, self.q_off, self.k_off, self.v_off, decays, self.decay_bias, self.tau, self.dim ** -0.5, cache.state,
                   ctx.seq_start, ctx.seq_slot, mixed, self.n_heads, self.dim, self.vdim, max_rows_per_seq=ctx.max_rows_per_seq)
        gated = ctx.new_activations(ctx.n_rows, width, reader=self.out.reader())
        k.gated_group_rmsnorm(mixed, proj, self.g_off, self.norm_weight, self.norm_eps, gated, self.n_heads, gate_after=True)
        self.out.forward(ctx, gated, out=hidden, accumulate=not fresh)
        return None


@MIXERS.register("gated_linear_attention")
def _build_gated_linear_attention(config, layer_index, prefix, shared):
    sizes = config.layers[layer_index].mixer
    return GatedLinearAttention(config.hidden, sizes.heads, sizes.dim, sizes.vdim, sizes.decay_rank, sizes.tau, config.rms_eps,
                                prefix + "mix.")
