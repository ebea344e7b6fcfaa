"""A matrix memory with exponential gates (the mLSTM of the xLSTM family), kept as a recurrent state.

    q = Wq x / sqrt(dim),  k = Wk x   heads x dim;     v = Wv x   heads x vdim
    i_t = cap tanh((Wi x + bi) / cap)                   log input gate, one number a head
    f_t = logsigmoid(cap tanh((Wf x + bf) / cap))       log forget gate
    m_t = max(f_t + m_(t-1), i_t)                       running maximum of the exponents, 0 when a sequence starts
    S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T       [dim, vdim], zero at the start
    n_t = the same with k_t alone                                           [dim]
    o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
    out = Wo ( o_t / rms(o_t over each head's vdim) * w_norm * sigmoid(Wg x) )

q, k, v and the gate g are one stacked product in the activation type; the two gates' pre-activations are a second,
small product with float32 results.  n is S's column for a value that is always one, so per sequence and head the layer
keeps vdim + 1 columns of dim floats and m in one float32 region of the cache.  Gates, their exponentials, the maximum,
the state and both products of the recurrence are float32 in both engines.  Three kernels: `mlstm_gates` walks the
m of a sequence's rows in order and leaves exp(f + m' - m), exp(i - m) and m for every row; `mlstm_scan` walks the
columns with those factors from the slot's state (prompts, portions and decode steps are one code path, so a
position's result does not depend on the cut) and leaves S^T q and n . q; `mlstm_finish` divides, norms head by head
and gates.  A step of one row a sequence (a decode step) does all three in one launch where the kernel set has it
(`mlstm_step`).  Every size and constant is a constructor parameter.
"""

from __future__ import annotations

import torch

from ..weights.binder import TensorSpec
from .base import MIXERS, CacheNeed
from .linear import Linear


class MatrixMemory:
    graph_safe = True
    graph_safe_rows = None
    writes_fresh = True    # forward(..., fresh=True) writes its result instead of adding it

    def __init__(self, hidden: int, n_heads: int, dim: int, vdim: int, gate_cap: float, norm_eps: float, prefix: str):
        if not gate_cap > 0.0:
            raise ValueError(f"the gates' cap must be positive, got {gate_cap}")
        self.hidden, self.n_heads, self.dim, self.vdim = int(hidden), int(n_heads), int(dim), int(vdim)
        self.gate_cap, self.norm_eps, self.prefix = float(gate_cap), float(norm_eps), prefix
        key_width, value_width = self.n_heads * self.dim, self.n_heads * self.vdim
        self.q_off, self.k_off, self.v_off, self.g_off = 0, key_width, 2 * key_width, 2 * key_width + value_width
        self.proj = Linear(hidden, [key_width, key_width, value_width, value_width],
                           [prefix + "q", prefix + "k", prefix + "v", prefix + "g"])
        self.gates = Linear(hidden, [self.n_heads, self.n_heads], [prefix + "i", prefix + "f"])
        self.out = Linear(value_width, hidden, prefix + "o")
        self.state_floats = self.n_heads * ((self.vdim + 1) * self.dim + 1)      # kernels: mlstm_state_floats
        self.norm_weight = self.gate_bias = None

    def tensor_specs(self):
        return self.proj.tensor_specs() + self.gates.tensor_specs() + self.out.tensor_specs() + [
            TensorSpec(self.prefix + "i.b", (self.n_heads,), "linear"), TensorSpec(self.prefix + "f.b", (self.n_heads,), "linear"),
            TensorSpec(self.prefix + "norm", (self.n_heads * self.vdim,), "norm")]

    def load(self, get):
        self.proj.load(get)
        self.gates.load(get)
        self.out.load(get)
        self.norm_weight = get(self.prefix + "norm").to(torch.float32).contiguous()
        self.gate_bias = torch.cat([get(self.prefix + "i.b").to(torch.float32), get(self.prefix + "f.b").to(torch.float32)]).contiguous()

    def prepare(self, kernels):
        self.proj.prepare(kernels)
        self.gates.prepare(kernels)
        self.out.prepare(kernels)

    def cache_need(self):
        return CacheNeed(kind="state", state_shape=(self.state_floats,), state_dtype=torch.float32)

    def working_bytes(self, step) -> int:
        width = self.n_heads * self.vdim
        return (self.proj.working_bytes(step, step.rows) + self.gates.working_bytes(step, step.rows, out_size=4)
                + step.matrix(step.rows, width, 4) + step.matrix(step.rows, 4 * self.n_heads, 4)
                + step.matrix(step.rows, width, reader=self.out.reader_for_plan(step.act_size))
                + self.out.working_bytes(step, step.rows, accumulate=True))

    def forward(self, ctx, x, hidden, cache, then_norm=None, fresh=False):
        k = ctx.kernels
        n, width = ctx.n_rows, self.n_heads * self.vdim
        proj = self.proj.forward(ctx, x)
        pre = self.gates.forward(ctx, x, out_dtype=torch.float32)
        gated = ctx.new_activations(n, width, reader=self.out.reader())
        one_launch = getattr(k, "mlstm_step", None)
        if one_launch is not None and ctx.max_rows_per_seq == 1:      # a decode step: gates, recurrence and read-out in one launch
            one_launch(proj, self.q_off, self.k_off, self.v_off, self.g_off, pre, self.gate_bias, self.gate_cap, cache.state, ctx.seq_slot,
                       self.norm_weight, self.norm_eps, gated, self.n_heads, self.dim, self.vdim)
        else:
            read = ctx.new_f32(n, width)                  # S^T q of every row and head
            beside = ctx.new_f32(n, 4 * self.n_heads)     # the gates' two factors, m and n . q of every row and head
            k.mlstm_gates(pre, self.gate_bias, self.gate_cap, cache.state, ctx.seq_start, ctx.seq_slot, beside, self.n_heads, self.dim,
                          self.vdim)
            k.mlstm_scan(proj, self.q_off, self.k_off, self.v_off, beside, cache.state, ctx.seq_start, ctx.seq_slot, read, self.n_heads,
                         self.dim, self.vdim)
            k.mlstm_finish(read, beside, proj, self.g_off, self.norm_weight, self.norm_eps, gated, self.n_heads, self.vdim)
        self.out.forward(ctx, gated, out=hidden, accumulate=not fresh)
        return None


@MIXERS.register("mlstm")
def _build_mlstm(config, layer_index, prefix, shared):
    sizes = config.layers[layer_index].mixer
    return MatrixMemory(config.hidden, sizes.heads, sizes.dim, sizes.vdim, sizes.gate_cap, config.rms_eps, prefix + "mix.")
