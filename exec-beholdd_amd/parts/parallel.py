"""Several mixers side by side: all read the same input, and their results are added with fixed weights,

    out = sum_i scale_i * M_i(x).

Each mixer keeps what it keeps: the cache need of the whole is the mixers' needs joined, paged keys and values of one of
them with the fixed-size state of another beside the pages (`CacheNeed` of kind "kv" with a `state_shape`), and every mixer
is handed the same `LayerCache`, of which it touches its own part.  At most one of the mixers may need pages and at most one
a state.  The results are float32 matrices of their own and the weighted sum is float32 (`weighted_sum`).
"""

from __future__ import annotations

from .base import MIXERS, CacheNeed, graph_rows_allowed
from .gated_attention import GatedAttention
from .gla import GatedLinearAttention
from .rope import RotaryFrequencies


class ParallelMixers:
    writes_fresh = True    # forward(..., fresh=True) writes its result instead of adding it

    def __init__(self, mixers, scales):
        self.mixers, self.scales = list(mixers), [float(scale) for scale in scales]
        if len(self.mixers) < 2 or len(self.mixers) != len(self.scales):
            raise ValueError("two or more mixers side by side, and a scale for each")
        needs = [need for need in (mixer.cache_need() for mixer in self.mixers) if need is not None]
        paged = [need for need in needs if need.kind == "kv"]
        fixed = [need for need in needs if need.kind == "state"]
        if len(paged) > 1 or len(fixed) > 1 or any(need.state_shape for need in paged):
            raise ValueError("mixers side by side: at most one of them keeps pages and at most one a state")
        if paged and fixed:
            self._need = CacheNeed(kind="kv", kv_heads=paged[0].kv_heads, head_dim=paged[0].head_dim, window=paged[0].window,
                                   state_shape=fixed[0].state_shape, state_dtype=fixed[0].state_dtype)
        else:
            self._need = (paged or fixed or [None])[0]

    @property
    def graph_safe(self):
        return all(getattr(mixer, "graph_safe", False) for mixer in self.mixers)

    @property
    def graph_safe_rows(self):
        return graph_rows_allowed(self.mixers)

    def tensor_specs(self):
        return [spec for mixer in self.mixers for spec in mixer.tensor_specs()]

    def load(self, get):
        for mixer in self.mixers:
            mixer.load(get)

    def prepare(self, kernels):
        for mixer in self.mixers:
            if hasattr(mixer, "prepare"):
                mixer.prepare(kernels)

    def cache_need(self):
        return self._need

    def working_bytes(self, step) -> int:
        total = len(self.mixers) * step.matrix(step.rows, self.mixers[0].hidden, 4)
        return total + sum(mixer.working_bytes(step) for mixer in self.mixers if hasattr(mixer, "working_bytes"))

    def _run(self, ctx, x, mixer, cache, rows, width):
        result = ctx.new_f32(rows, width)
        if getattr(mixer, "writes_fresh", False):
            mixer.forward(ctx, x, result, cache, fresh=True)
        else:
            result.zero_()
            mixer.forward(ctx, x, result, cache)
        return result

    def forward(self, ctx, x, hidden, cache, then_norm=None, fresh=False):
        k = ctx.kernels
        rows, width = hidden.shape
        total = self._run(ctx, x, self.mixers[0], cache, rows, width)
        scale = self.scales[0]
        for mixer, weight in zip(self.mixers[1:-1], self.scales[1:-1]):
            k.weighted_sum(total, total, scale, self._run(ctx, x, mixer, cache, rows, width), weight)
            scale = 1.0
        last = self._run(ctx, x, self.mixers[-1], cache, rows, width)
        if fresh:
            k.weighted_sum(hidden, total, scale, last, self.scales[-1])
        else:
            k.weighted_sum(total, total, scale, last, self.scales[-1])
            k.weighted_sum(hidden, hidden, 1.0, total, 1.0)
        return None


@MIXERS.register("parallel_attention_gla")
def _build_parallel_attention_gla(config, layer_index, prefix, shared):
    """Windowed softmax attention (`mixer.left`, tensors under mix.left.) beside gated linear attention (`mixer.right`, tensors
    under mix.right.)."""
    sizes = config.layers[layer_index].mixer
    left, right = sizes.left, sizes.right
    rotation = RotaryFrequencies(left.rot_dims, left.rot_base, left.rot_stretch) if left.rot_dims else None
    attention = GatedAttention(config.hidden, left.heads, left.kv_heads, left.dim, left.vdim, left.scale, prefix + "mix.left.",
                               bias=False, head_norm_eps=config.rms_eps, window=left.window, gate=False, rotation=rotation,
                               neighbours=True)
    linear = GatedLinearAttention(config.hidden, right.heads, right.dim, right.vdim, right.decay_rank, right.tau, config.rms_eps,
                                  prefix + "mix.right.")
    return ParallelMixers([attention, linear], [sizes.left_scale, sizes.right_scale])
