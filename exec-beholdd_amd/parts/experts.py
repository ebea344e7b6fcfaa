"""Routed experts: a mixture of small gated feed-forward layers of which every token uses a few, and a shared one.

    z = Wr h + br                       router logits, float32 (h in the activation type); the bias is optional
    chosen = the `top` largest of z;  their weights = softmax over the chosen logits alone (which is also what the
                                        chosen ones' shares of a softmax over all experts are once divided by their sum)
    expert(h) = Wd (g' * sigmoid(alpha g') * (u' + 1)),  g' = min(Wg h, limit),  u' = clamp(Wu h, -limit, limit)
    out = sum over chosen of weight * expert(h)  +  shared(h)        (the shared expert has the same form and runs for all)

Variants, each a constructor parameter: `scoring="sigmoid"` weighs a chosen expert by the sigmoid of its own logit (no
norming over the chosen); `weigh_input=True` puts the weight on the expert's input, out = sum expert(weight * h), which for
these experts is a factor on the gate and up sums ahead of the activation (W (w h) = w (W h)); `limit`, `alpha` and `shift`
shape the activation g' * sigmoid(alpha g') * (u' + shift), an infinite limit with alpha 1 and shift 0 being silu(g) * u; the
shared expert is any feed-forward part.

The experts' matrices are kept stacked: gate and up rows of an expert in one [2 ff, width] block, [experts, ...] in
all.  The (row, choice) pairs are grouped by expert on the device (`experts_group`).  A step of few rows then runs a
workgroup per expert and block of outputs that reads the expert's rows from memory once for all of its pairs
(`experts_rows`), with nothing that depends on the routing on the host, so that decode steps can be captured.  A step
of many rows (a prompt) reads the experts' counts on the host (the step waits for the device there), lays the pairs'
inputs side by side, expert after expert, and runs all experts' products in one launch on the matrix cores
(`experts_products`, over a table of row tiles made from the counts; the activation rides in the first product), or,
for sizes and element types that kernel does not take, the framework's matrix products on each expert's stretch.  Sizes
that the grouped kernels do not take go pair by pair (`experts_gate_up`, `experts_down`).  In every form a row's
experts' shares are added in the order of its own choice, so its result depends on its batch-mates by rounding at most.  The routing is left in
`ctx.extras["routing"]` ((chosen, weights) of the last layer that ran).  Every size and constant is a constructor
parameter.
"""

from __future__ import annotations

import torch

from ..weights.binder import TensorSpec
from .base import FEED_FORWARDS
from .linear import Linear

GATE_SLOPE = 1.702      # alpha of the gate's sigmoid


class ClampedGLU:
    """One gated feed-forward of the form above, for every row: out = Wd act(Wg h, Wu h), added to the residual."""
    graph_safe = True
    graph_safe_rows = None

    def __init__(self, hidden: int, ff: int, limit: float, prefix: str, alpha: float = GATE_SLOPE):
        self.hidden, self.ff, self.limit, self.alpha = int(hidden), int(ff), float(limit), float(alpha)
        self.gate_up = Linear(hidden, [ff, ff], [prefix + "gate", prefix + "up"])
        self.down = Linear(ff, hidden, prefix + "down")

    @property
    def input_reader(self):
        return self.gate_up.reader()

    def tensor_specs(self):
        return self.gate_up.tensor_specs() + self.down.tensor_specs()

    def load(self, get):
        self.gate_up.load(get)
        self.down.load(get)

    def prepare(self, kernels):
        self.gate_up.prepare(kernels)
        self.down.prepare(kernels)

    def working_bytes(self, step) -> int:
        return (self.gate_up.working_bytes(step, step.rows) + step.matrix(step.rows, self.ff, reader=self.down.reader_for_plan(step.act_size))
                + self.down.working_bytes(step, step.rows, accumulate=True))

    def forward(self, ctx, x, hidden, then_norm=None):
        both = self.gate_up.forward(ctx, x)
        inner = ctx.new_activations(both.shape[0], self.ff, reader=self.down.reader())
        ctx.kernels.clamped_glu(both, inner, self.limit, self.alpha)
        self.down.forward(ctx, inner, out=hidden, accumulate=True)
        return None


class RoutedExperts:
    graph_safe = True
    graph_safe_rows = 1       # steps of several rows a sequence may read the experts' counts on the host
    PRODUCT_PAIRS = 16        # from that many pairs an expert on average, a step of many rows runs matrix products
    PACK_FOR_PROMPTS = True   # keep a second copy of every expert's matrices in the form the products of many rows read fastest
    ONE_LAUNCH_WORK = 1.5e11  # up to that many operations a layer, a prompt's experts run as one launch over all of them: the
                              # one kernel reaches about 120 TFLOP/s whatever the size (tiles of 128 x 64 outputs re-read their
                              # operands through the L2), the products per expert cost about 25 us each and then run faster

    def __init__(self, hidden: int, n_experts: int, top: int, ff: int, limit: float, prefix: str, shared=None,
                 alpha: float = GATE_SLOPE, router_bias: bool = True, scoring: str = "softmax", weigh_input: bool = False,
                 shift: float = 1.0):
        if not 1 <= top <= n_experts:
            raise ValueError(f"a row uses 1 to {n_experts} experts, got {top}")
        if scoring not in ("softmax", "sigmoid"):
            raise ValueError(f"experts are weighed by 'softmax' over the chosen or by each one's 'sigmoid', got {scoring!r}")
        self.scoring, self.weigh_input, self.shift = scoring, bool(weigh_input), float(shift)
        self.hidden, self.n_experts, self.top, self.ff = int(hidden), int(n_experts), int(top), int(ff)
        self.limit, self.alpha, self.prefix, self.shared = float(limit), float(alpha), prefix, shared
        self.router = Linear(hidden, n_experts, prefix + "router")
        self.has_router_bias = bool(router_bias)
        self.router_bias = self.w_gate_up = self.w_down = None
        self.for_products = None      # per expert (gate and up, down) as the matrix products take them
        self.in_one_launch = False    # a prompt's products run as one launch over all experts (kernels.experts_products)

    def tensor_specs(self):
        specs = self.router.tensor_specs()
        if self.has_router_bias:
            specs.append(TensorSpec(self.prefix + "router.b", (self.n_experts,), "linear"))
        for e in range(self.n_experts):
            specs += [TensorSpec(f"{self.prefix}e{e}.gate", (self.ff, self.hidden), "linear"),
                      TensorSpec(f"{self.prefix}e{e}.up", (self.ff, self.hidden), "linear"),
                      TensorSpec(f"{self.prefix}e{e}.down", (self.hidden, self.ff), "linear")]
        return specs + (self.shared.tensor_specs() if self.shared is not None else [])

    def load(self, get):
        self.router.load(get)
        self.router_bias = get(self.prefix + "router.b").to(torch.float32).contiguous() if self.has_router_bias else None
        first = get(f"{self.prefix}e0.gate")
        self.w_gate_up = torch.empty((self.n_experts, 2 * self.ff, self.hidden), dtype=first.dtype, device=first.device)
        self.w_down = torch.empty((self.n_experts, self.hidden, self.ff), dtype=first.dtype, device=first.device)
        for e in range(self.n_experts):
            self.w_gate_up[e, :self.ff].copy_(first if e == 0 else get(f"{self.prefix}e{e}.gate"))
            self.w_gate_up[e, self.ff:].copy_(get(f"{self.prefix}e{e}.up"))
            self.w_down[e].copy_(get(f"{self.prefix}e{e}.down"))
        if self.shared is not None:
            self.shared.load(get)

    def prepare(self, kernels):
        """The stacked matrices stay row after row (the kernels for steps of few rows read them so).  For prompts every expert's
        matrices are kept a second time in the kernel library's own form, where it has one for them: its products of many rows
        read that form several times as fast, and a GPU with hundreds of GB holds both."""
        self.router.prepare(kernels)
        if self.shared is not None:
            self.shared.prepare(kernels)
        takes = getattr(kernels, "experts_products_take", None)
        self.in_one_launch = bool(takes is not None and takes(self.w_gate_up.dtype, self.hidden, self.ff) and takes(self.w_down.dtype, self.ff, self.hidden))
        if self.PACK_FOR_PROMPTS and hasattr(kernels, "pack_weight"):
            self.for_products = [(kernels.pack_weight(self.w_gate_up[e]), kernels.pack_weight(self.w_down[e])) for e in range(self.n_experts)]

    def working_bytes(self, step) -> int:
        total = self.router.working_bytes(step, step.rows, out_size=4) + 2 * step.matrix(step.rows, self.top, 4)
        pairs = step.rows * self.top
        total += step.matrix(self.n_experts, step.rows, 4) + step.matrix(pairs, self.ff) + step.matrix(pairs, self.hidden, 4)
        if step.rows > step.seqs and pairs >= self.PRODUCT_PAIRS * self.n_experts:      # a step of many rows: the pairs' inputs, gate and up
            total += step.matrix(pairs, self.hidden) + step.matrix(pairs, 2 * self.ff) + step.matrix(pairs, 1, 4)
        return total + (self.shared.working_bytes(step) if self.shared is not None else 0)

    def forward(self, ctx, x, hidden, then_norm=None):
        k = ctx.kernels
        n = x.shape[0]
        logits = self.router.forward(ctx, x, out_dtype=torch.float32)
        chosen = torch.empty((n, self.top), dtype=torch.int32, device=ctx.device)
        weights = ctx.new_f32(n, self.top)
        k.route_top_k(logits, self.router_bias, chosen, weights, **({"scoring": self.scoring} if self.scoring != "softmax" else {}))
        ctx.extras["routing"] = (chosen, weights)
        # where the weight goes: on the expert's input (the kernels that make gate and up take it) or on its output
        act = {} if self.shift == 1.0 else {"shift": self.shift}
        ahead = dict(act, in_weights=weights) if self.weigh_input else act
        behind = None if self.weigh_input else weights
        pairs = n * self.top
        takes = getattr(k, "experts_rows_take", None)
        if takes is None or not (takes(self.hidden) and takes(self.ff)):
            inner = ctx.new_activations(pairs, self.ff)
            k.experts_gate_up(x, chosen, self.w_gate_up, inner, self.limit, self.alpha, **ahead)
            k.experts_down(inner, chosen, behind, self.w_down, hidden)
        else:
            lists = torch.empty((self.n_experts, n), dtype=torch.int32, device=ctx.device)
            counts = torch.empty((self.n_experts,), dtype=torch.int32, device=ctx.device)
            k.experts_group(chosen, lists, counts)
            if ctx.is_decode or pairs < self.PRODUCT_PAIRS * self.n_experts:
                inner = ctx.new_activations(pairs, self.ff)
                k.experts_rows(x, self.top, lists, counts, self.w_gate_up, inner, gated=True, limit=self.limit, alpha=self.alpha, **ahead)
                y = ctx.new_f32(pairs, self.hidden)
                k.experts_rows(inner, 1, lists, counts, self.w_down, y)
                self._combine(k, y, None, behind, hidden)
            else:
                self._as_products(ctx, x, lists, counts, weights, hidden)
        if self.shared is not None:
            self.shared.forward(ctx, x, hidden)
        return None


    def _combine(self, k, y, place, weights, hidden):
        if weights is not None:
            k.experts_combine(y, place, weights, hidden)
        else:
            k.experts_combine(y, place, None, hidden, top=self.top)

    def _as_products(self, ctx, x, lists, counts, weights, hidden):
        """Every expert's pairs as one stretch of rows through the framework's matrix products."""
        k = ctx.kernels
        act = {} if self.shift == 1.0 else {"shift": self.shift}
        behind = None if self.weigh_input else weights
        n, pairs = x.shape[0], x.shape[0] * self.top
        matrices = self.for_products or [(self.w_gate_up[e], self.w_down[e]) for e in range(self.n_experts)]
        held = counts.cpu().tolist()              # the host waits for the routing here
        starts, at = [], 0
        for count in held:
            starts.append(at)
            at += count
        offsets = torch.tensor(starts, dtype=torch.int32, device=ctx.device)
        gathered = ctx.new_activations(pairs, self.hidden)
        place = torch.empty((pairs,), dtype=torch.int32, device=ctx.device)
        k.experts_gather(x, self.top, lists, counts, offsets, gathered, place, **({"in_weights": weights} if self.weigh_input else {}))
        if self.in_one_launch and 6.0 * pairs * self.ff * self.hidden <= self.ONE_LAUNCH_WORK:
            tiles = torch.tensor([(e, first + at, min(128, count - at)) for e, (first, count) in enumerate(zip(starts, held))
                                  for at in range(0, count, 128)], dtype=torch.int32, device=ctx.device)
            inner = ctx.new_activations(pairs, self.ff)
            k.experts_products(gathered, self.w_gate_up, tiles, inner, gated=True, limit=self.limit, alpha=self.alpha, **act)
            y = ctx.new_f32(pairs, self.hidden)
            k.experts_products(inner, self.w_down, tiles, y)
            self._combine(k, y, place, behind, hidden)
            return
        both = ctx.new_activations(pairs, 2 * self.ff)
        for e, (first, count) in enumerate(zip(starts, held)):
            if count:
                k.gemm(gathered[first:first + count], matrices[e][0], both[first:first + count])
        inner = ctx.new_activations(pairs, self.ff)
        k.clamped_glu(both, inner, self.limit, self.alpha, **act)
        y = ctx.new_f32(pairs, self.hidden)
        for e, (first, count) in enumerate(zip(starts, held)):
            if count:
                k.gemm(inner[first:first + count], matrices[e][1], y[first:first + count])
        self._combine(k, y, place, behind, hidden)


@FEED_FORWARDS.register("routed_experts")
def _build_routed_experts(config, layer_index, prefix, shared):
    sizes = config.layers[layer_index].mlp
    common = ClampedGLU(config.hidden, sizes.shared.ff, sizes.shared.limit, prefix + "mlp.shared.") if sizes.shared is not None else None
    return RoutedExperts(config.hidden, sizes.experts, sizes.top, sizes.expert.ff, sizes.expert.limit, prefix + "mlp.", shared=common,
                         router_bias=getattr(sizes, "router_bias", True))


@FEED_FORWARDS.register("routed_silu_experts")
def _build_routed_silu_experts(config, layer_index, prefix, shared):
    """Experts of the form Wd (silu(Wg h) * (Wu h)), each weighed by the sigmoid of its own router logit, the weight on the
    expert's input; a shared expert of the same form."""
    from .mlp import SwiGLU

    sizes = config.layers[layer_index].mlp
    names = ("gate", "up", "down")
    common = SwiGLU(config.hidden, sizes.shared_ff, prefix + "mlp.shared.", names=names) if sizes.shared_ff else None
    return RoutedExperts(config.hidden, sizes.experts, sizes.top, sizes.expert_ff, float("inf"), prefix + "mlp.", shared=common,
                         alpha=1.0, router_bias=False, scoring="sigmoid", weigh_input=True, shift=0.0)
