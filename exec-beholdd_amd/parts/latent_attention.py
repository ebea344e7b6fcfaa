"""Attention over a cached latent (low-rank keys and values with one rotated key part for all heads).

    q = Wq x                 per head [q_c (dim, not rotated) | q_r (rot_dim, rotated)]
    Wdkv x = [c_raw | k_r]   c = rms(c_raw) * w_c  (kv_rank),  k_r (rot_dim) rotated, one for all heads
    k_c = Wuk c,  v = Wuv c  per head (dim and vdim)
    score_ij = (q_c,i . k_c,j + R_i q_r,i . R_j k_r,j) * scale,  causal softmax,  out = Wo concat_h sum_j p_ij v_j

Only c and k_r are cached.  The up-projections never run over cached positions: since q_c . (Wuk c) = (Wuk^T q_c) . c
and sum_j p_j (Wuv c_j) = Wuv (sum_j p_j c_j), a head's query is carried into the latent's space and its attended
latent into the head's values, by one small matrix per head each (`heads_linear`).  What is left in between is the
paged attention kernels' own case of one key/value head of size kv_rank + rot_dim shared by all query heads, with
key [c | k_r] and value [c | 0]; prompts and decode steps take the same path, so a position's result does not
depend on the cut.  The rotation turns the first `rotation.dims` dimensions of the rot_dim part, dimension i with
i + dims/2, by position * base^(-2i/dims) (angles in float32, no table, no longest position).  A model without a
rotated part has rot_dim 0 and no rotation; with a `window` a query sees the last `window` positions only (its own
among them) and the cache gives older pages back; with `gate` the heads' values are multiplied by sigmoid(Wg x) ahead
of the output projection, the gate being one more slice of the stacked projection (`gate="head"`: one gate a head,
Wg x has `heads` numbers).  With `query_rank` the queries go through a latent of their own,
q = Wuq (rms(Wdq x) * w_q), Wdq being one more slice of the stacked projection.  With `sinks` every head's softmax sum
has one more term exp(sink_h), a learned number without key or value.  `neighbours`: the rotation pairs dimensions
2i and 2i + 1; its frequencies and the factor on its cosines and sines are the `rotation` object's.
Every size and constant is a constructor parameter.
"""

from __future__ import annotations

import torch

from ..weights.binder import TensorSpec
from .base import MIXERS, CacheNeed
from .linear import Linear
from .rope import RotaryFrequencies


class LatentAttention:
    graph_safe = True      # forward reads only the step's device tensors
    graph_safe_rows = None
    writes_fresh = True    # forward(..., fresh=True) writes its result instead of adding it

    def __init__(self, hidden: int, n_heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int, scale: float,
                 rotation: RotaryFrequencies | None, norm_eps: float, prefix: str, window: int = 0, gate=False,
                 query_rank: int = 0, sinks: bool = False, neighbours: bool = False):
        if (rotation.dims if rotation is not None else 0) > rot_dim:
            raise ValueError(f"the rotation turns {rotation.dims} dimensions, the rotated part has {rot_dim}")
        if window < 0:
            raise ValueError(f"a window is a count of positions (0: all), got {window}")
        self.hidden, self.n_heads, self.dim, self.rot_dim = int(hidden), int(n_heads), int(dim), int(rot_dim)
        self.vdim, self.kv_rank, self.scale = int(vdim), int(kv_rank), float(scale)
        self.rotation, self.norm_eps, self.prefix = rotation, float(norm_eps), prefix
        if gate not in (False, True, "head"):
            raise ValueError(f"a gate is absent, one a value (True) or one a head ('head'), got {gate!r}")
        self.window, self.gate, self.gate_per_head = int(window), bool(gate), gate == "head"
        self.query_rank, self.has_sinks, self.neighbours = int(query_rank), bool(sinks), bool(neighbours)
        self.q_head = self.dim + self.rot_dim                 # a head of the projected query
        self.kv_head = self.kv_rank + self.rot_dim            # the one cached key/value head
        # the stacked projection's first slice: the queries themselves, or the latent they are made from
        first_width, first_name = (self.query_rank, "dq") if self.query_rank else (self.n_heads * self.q_head, "q")
        self.down_off = first_width                           # where [c_raw | k_r] begins in a projected row
        self.gate_off = self.down_off + self.kv_head         # where the gate begins, if there is one
        gate_width = [self.n_heads if self.gate_per_head else self.n_heads * self.vdim] if self.gate else []
        self.proj = Linear(hidden, [first_width, self.kv_head] + gate_width,
                           [prefix + first_name, prefix + "dkv"] + ([prefix + "g"] if self.gate else []))
        self.query_up = Linear(self.query_rank, self.n_heads * self.q_head, prefix + "uq") if self.query_rank else None
        self.out = Linear(self.n_heads * self.vdim, hidden, prefix + "o")
        self.latent_weight = self.key_up = self.value_up = self.frequencies = self.query_weight = self.sinks = None

    @property
    def input_reader(self):
        return self.proj.reader()

    def tensor_specs(self):
        specs = self.proj.tensor_specs() + self.out.tensor_specs() + [
            TensorSpec(self.prefix + "dkv.norm", (self.kv_rank,), "norm"),
            TensorSpec(self.prefix + "uk", (self.n_heads * self.dim, self.kv_rank), "linear"),
            TensorSpec(self.prefix + "uv", (self.n_heads * self.vdim, self.kv_rank), "linear")]
        if self.query_up is not None:
            specs += self.query_up.tensor_specs() + [TensorSpec(self.prefix + "dq.norm", (self.query_rank,), "norm")]
        if self.has_sinks:
            specs.append(TensorSpec(self.prefix + "sink", (self.n_heads,), "norm"))
        return specs

    def load(self, get):
        self.proj.load(get)
        self.out.load(get)
        self.latent_weight = get(self.prefix + "dkv.norm").to(torch.float32).contiguous()
        # one matrix per head, [inputs, outputs]: queries go dim -> kv_rank through Wuk as stored, attended latents
        # kv_rank -> vdim through Wuv transposed
        self.key_up = get(self.prefix + "uk").view(self.n_heads, self.dim, self.kv_rank).contiguous()
        self.value_up = get(self.prefix + "uv").view(self.n_heads, self.vdim, self.kv_rank).transpose(1, 2).contiguous()
        self.frequencies = self.rotation.frequencies(self.latent_weight.device) if self.rotation is not None else None
        if self.query_up is not None:
            self.query_up.load(get)
            self.query_weight = get(self.prefix + "dq.norm").to(torch.float32).contiguous()
        if self.has_sinks:
            self.sinks = get(self.prefix + "sink").to(torch.float32).contiguous()

    def prepare(self, kernels):
        self.proj.prepare(kernels)
        self.out.prepare(kernels)
        if self.query_up is not None:
            self.query_up.prepare(kernels)

    def cache_need(self):
        return CacheNeed(kind="kv", kv_heads=1, head_dim=self.kv_head, window=self.window)

    def working_bytes(self, step) -> int:
        total = self.proj.working_bytes(step, step.rows) + 2 * step.matrix(step.rows, self.n_heads * self.kv_head)
        total += (2 if self.gate else 1) * step.matrix(step.rows, self.n_heads * self.vdim)
        if self.query_up is not None:
            total += step.matrix(step.rows, self.query_rank) + self.query_up.working_bytes(step, step.rows)
        if step.sizes is not None:
            total += step.sizes.attention_working_bytes(step.rows, step.seqs, step.max_rows_per_seq, self.n_heads, 1,
                                                        self.kv_head, step.max_position, step.act_size)
        return total + self.out.working_bytes(step, step.rows, accumulate=True)

    def forward(self, ctx, x, hidden, cache, then_norm=None, fresh=False):
        k = ctx.kernels
        heads, rank, turned = self.n_heads, self.kv_rank, self.rotation.dims if self.rotation is not None else 0
        proj = self.proj.forward(ctx, x)
        if self.query_up is not None:      # the queries from their own normed latent
            query_latent = ctx.new_activations(ctx.n_rows, self.query_rank, reader=self.query_up.reader())
            k.slice_rmsnorm(proj, 0, self.query_weight, self.norm_eps, query_latent)
            heads_rows = self.query_up.forward(ctx, query_latent)
        else:
            heads_rows = proj
        turning = dict(neighbours=self.neighbours, magnitude=self.rotation.magnitude) if self.rotation is not None and (
            self.neighbours or self.rotation.magnitude != 1.0) else {}
        if heads_rows is not proj:
            turning["query_source"] = heads_rows
        sinking = dict(sinks=self.sinks) if self.has_sinks else {}
        query = ctx.new_activations(ctx.n_rows, heads * self.kv_head)
        # one launch: c and k_r into the cache, and the heads' rotated query parts into their places
        if self.rot_dim:
            k.latent_write(proj, self.down_off, self.latent_weight, self.norm_eps, self.frequencies, turned, ctx.positions,
                           ctx.row_seq, cache.k_pages, cache.v_pages, cache.page_table, rank, self.rot_dim, write=cache.writes,
                           query=query, query_head=self.kv_head, query_first=rank, source_head=self.q_head, source_first=self.dim,
                           n_heads=heads, **turning)
        elif cache.writes:
            k.latent_write(proj, self.down_off, self.latent_weight, self.norm_eps, None, 0, ctx.positions, ctx.row_seq,
                           cache.k_pages, cache.v_pages, cache.page_table, rank, 0)
        k.heads_linear(heads_rows, self.q_head, 0, self.key_up, query, self.kv_head, 0, heads)
        attended = ctx.new_activations(ctx.n_rows, heads * self.kv_head)
        k.attention(query, attended, cache.k_pages, cache.v_pages, cache.page_table, ctx.row_seq, ctx.positions,
                    heads, 1, self.kv_head, self.scale, self.window, layout=ctx, **sinking)
        if self.gate:
            values = ctx.new_activations(ctx.n_rows, heads * self.vdim)
            k.heads_linear(attended, self.kv_head, 0, self.value_up, values, self.vdim, 0, heads)
            gated = ctx.new_activations(ctx.n_rows, heads * self.vdim, reader=self.out.reader())
            k.gate_heads(values, self.vdim, proj, self.gate_off, gated, heads, self.vdim, **(dict(per_head=True) if self.gate_per_head else {}))
            values = gated
        else:
            values = ctx.new_activations(ctx.n_rows, heads * self.vdim, reader=self.out.reader())
            k.heads_linear(attended, self.kv_head, 0, self.value_up, values, self.vdim, 0, heads)
        self.out.forward(ctx, values, out=hidden, accumulate=not fresh)
        return None


@MIXERS.register("latent_attention")
def _build_latent_attention(config, layer_index, prefix, shared):
    sizes = config.layers[layer_index].mixer
    rotation = RotaryFrequencies(sizes.rot_dims, sizes.rot_base, getattr(sizes, "rot_stretch", None)) if sizes.rot_dims else None
    return LatentAttention(config.hidden, sizes.heads, sizes.dim, sizes.rot_dim, sizes.vdim, sizes.kv_rank, sizes.scale,
                           rotation, config.rms_eps, prefix + "mix.", window=getattr(sizes, "window", 0),
                           gate=getattr(sizes, "gate", False), query_rank=getattr(sizes, "q_rank", 0),
                           sinks=getattr(sizes, "sinks", False), neighbours=getattr(sizes, "neighbours", False))
