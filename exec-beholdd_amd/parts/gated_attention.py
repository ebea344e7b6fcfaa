"""Grouped softmax attention with biased projections, per-head query and key norms, a rotation over part of a head,
keys seen within a chunk or a window, and a gate on the heads' outputs.

    q, k, v = Wq x + bq, Wk x + bk, Wv x + bv          heads x dim, kv_heads x dim, kv_heads x vdim
    q <- rms(q over each head's dim) * wq;  k likewise   one weight [dim] for all heads, before the rotation
    dimensions i and i + turned/2 (i < turned/2) of every head of q and k turned by position * base^(-2i/turned)
    query at position p sees key at j <= p where   chunk c: floor(p / c) = floor(j / c);   window w: p - j < w;   else all
    softmax of q.k * scale; query head h reads key/value head h // (heads / kv_heads)
    out = Wo (heads * sigmoid(Wg x))

The four projections are one stacked product [q | k | v | g]; the biases are added, the heads normed and turned, and
keys and values written into the pages by one kernel (`head_norm_rope_write`).  Keys have `dim` dimensions a head and
values `vdim`; both are cached as heads of one padded size (zeros beyond), which the paged attention kernels take as it
is.  Chunks are counted from a sequence's position 0, so what a row sees does not depend on how a prompt was cut; the
cache keeps a chunk's (or a window's) span of positions and gives older pages back.  Norm statistics, angles and the
softmax are float32.  Every size and constant is a constructor parameter; each mechanism can be switched off: without
`gate` there is no Wg and the heads go to Wo as they are; `rotation` (a `RotaryFrequencies`) replaces `turned` and `base`
where the frequencies are not the plain powers of the base; `neighbours` pairs dimensions 2i and 2i + 1.
"""

from __future__ import annotations

import torch

from ..weights.binder import TensorSpec
from .base import MIXERS, CacheNeed
from .conv_attention import padded_head
from .linear import Linear
from .rope import RotaryFrequencies


class GatedAttention:
    graph_safe = True
    graph_safe_rows = None
    writes_fresh = True    # forward(..., fresh=True) writes its result instead of adding it

    def __init__(self, hidden: int, n_heads: int, n_kv_heads: int, dim: int, vdim: int, scale: float, prefix: str, *,
                 bias: bool = True, head_norm_eps: float | None = None, turned: int = 0, base: float = 10000.0,
                 chunk: int = 0, window: int = 0, gate: bool = True, rotation: RotaryFrequencies | None = None,
                 neighbours: bool = False):
        """`head_norm_eps` None: no query and key norms; `turned` 0: no rotation; `chunk` and `window` 0: every earlier key."""
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} query heads do not group evenly into {n_kv_heads} kv heads")
        if chunk and window:
            raise ValueError("keys are seen by chunk or by window, not both")
        if rotation is not None:
            turned = rotation.dims
        if turned % 2 or turned > dim:
            raise ValueError(f"the rotation turns pairs of a head's {dim} dimensions, got {turned}")
        self.hidden, self.n_heads, self.n_kv_heads, self.dim, self.vdim = int(hidden), int(n_heads), int(n_kv_heads), int(dim), int(vdim)
        self.scale, self.prefix, self.bias, self.head_norm_eps = float(scale), prefix, bool(bias), head_norm_eps
        self.turned, self.chunk, self.window = int(turned), int(chunk), int(window)
        self.q_width, self.k_width, self.v_width = self.n_heads * self.dim, self.n_kv_heads * self.dim, self.n_kv_heads * self.vdim
        self.qkv_width = self.q_width + self.k_width + self.v_width
        self.gate_width = self.n_heads * self.vdim
        self.pad = padded_head(dim, vdim)
        self.gate, self.neighbours = bool(gate), bool(neighbours)
        self.rotation = rotation if rotation is not None else (RotaryFrequencies(self.turned, base) if self.turned else None)
        self.proj = Linear(hidden, [self.q_width, self.k_width, self.v_width] + ([self.gate_width] if self.gate else []),
                           [prefix + "q", prefix + "k", prefix + "v"] + ([prefix + "g"] if self.gate else []))
        self.out = Linear(self.gate_width, hidden, prefix + "o")
        self.q_norm = self.k_norm = self.qkv_bias = None

    @property
    def input_reader(self):
        return self.proj.reader()

    def tensor_specs(self):
        specs = self.proj.tensor_specs() + self.out.tensor_specs()
        if self.bias:
            specs += [TensorSpec(self.prefix + "q.b", (self.q_width,), "linear"), TensorSpec(self.prefix + "k.b", (self.k_width,), "linear"),
                      TensorSpec(self.prefix + "v.b", (self.v_width,), "linear")]
        if self.head_norm_eps is not None:
            specs += [TensorSpec(self.prefix + "q.norm", (self.dim,), "norm"), TensorSpec(self.prefix + "k.norm", (self.dim,), "norm")]
        return specs

    def load(self, get):
        self.proj.load(get)
        self.out.load(get)
        if self.bias:
            self.qkv_bias = torch.cat([get(self.prefix + name).to(torch.float32) for name in ("q.b", "k.b", "v.b")]).contiguous()
        if self.head_norm_eps is not None:
            self.q_norm = get(self.prefix + "q.norm").to(torch.float32).contiguous()
            self.k_norm = get(self.prefix + "k.norm").to(torch.float32).contiguous()

    def prepare(self, kernels):
        self.proj.prepare(kernels)
        self.out.prepare(kernels)

    def cache_need(self):
        # a chunk is at most `chunk` positions long: nothing older than that is ever seen again
        return CacheNeed(kind="kv", kv_heads=self.n_kv_heads, head_dim=self.pad, window=self.chunk or self.window)

    def working_bytes(self, step) -> int:
        total = self.proj.working_bytes(step, step.rows) + 2 * step.matrix(step.rows, self.n_heads * self.pad)
        total += step.matrix(step.rows, self.gate_width, reader=self.out.reader_for_plan(step.act_size))
        if step.sizes is not None:
            total += step.sizes.attention_working_bytes(step.rows, step.seqs, step.max_rows_per_seq, self.n_heads, self.n_kv_heads,
                                                        self.pad, step.max_position, step.act_size)
        return total + self.out.working_bytes(step, step.rows, accumulate=True)

    def forward(self, ctx, x, hidden, cache, then_norm=None, fresh=False):
        k = ctx.kernels
        n = ctx.n_rows
        proj = self.proj.forward(ctx, x)
        q = ctx.new_activations(n, self.n_heads * self.pad)
        freq = self.rotation.frequencies(ctx.device) if self.rotation is not None else None
        turning = dict(neighbours=self.neighbours, magnitude=self.rotation.magnitude) if self.rotation is not None and (
            self.neighbours or self.rotation.magnitude != 1.0) else {}
        k.head_norm_rope_write(proj, 0, self.qkv_bias, self.q_norm, self.k_norm, self.head_norm_eps or 0.0, freq, self.turned,
                               ctx.positions, ctx.row_seq, q, cache.k_pages, cache.v_pages, cache.page_table, self.n_heads,
                               self.n_kv_heads, self.dim, self.vdim, self.pad, cache.writes, **turning)
        plain = not self.gate and self.pad == self.vdim      # the attended heads are the output projection's input as they are
        attended = ctx.new_activations(n, self.n_heads * self.pad, reader=self.out.reader() if plain else None)
        k.attention(q, attended, cache.k_pages, cache.v_pages, cache.page_table, ctx.row_seq, ctx.positions, self.n_heads,
                    self.n_kv_heads, self.pad, self.scale, self.window, layout=ctx, chunk=self.chunk)
        if plain:
            gated = attended
        else:
            gated = ctx.new_activations(n, self.gate_width, reader=self.out.reader())
            k.gate_heads(attended, self.pad, proj if self.gate else None, self.qkv_width, gated, self.n_heads, self.vdim)
        self.out.forward(ctx, gated, out=hidden, accumulate=not fresh)
        return None


@MIXERS.register("gated_attention")
def _build_gated_attention(config, layer_index, prefix, shared):
    sizes = config.layers[layer_index].mixer
    return GatedAttention(config.hidden, sizes.heads, sizes.kv_heads, sizes.dim, sizes.vdim, sizes.scale, prefix + "mix.",
                          bias=getattr(sizes, "bias", True), head_norm_eps=config.rms_eps, turned=sizes.rot_dims,
                          base=sizes.rot_base, chunk=getattr(sizes, "chunk", 0), window=getattr(sizes, "window", 0))
