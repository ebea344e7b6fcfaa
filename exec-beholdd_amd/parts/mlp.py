"""Dense SwiGLU feed-forward: out = Wd (silu(Wg x) * (Wu x)), added to the residual.

crates/beholdd-model/src/qwen3moe/forward.rs:1270-1298 with silu(x) = x / (1 + exp(-x)) and no
clamp (crates/beholdd-kernel/src/vecops.rs:91-110, limit 0 at forward.rs:1288).  The gate and
up matrices are stacked so that one product computes both.
"""

from __future__ import annotations

from .base import FEED_FORWARDS
from .linear import Linear


class SwiGLU:
    graph_safe = True      # forward reads only the step's device tensors
    graph_safe_rows = None # ... whatever the number of tokens a sequence brings
    prepares_next_norm = True      # the down projection can carry the norm that follows
    takes_prepared_input = True    # x goes to the gate/up product untouched
    def __init__(self, hidden: int, intermediate: int, prefix: str, names=("gate_proj.weight", "up_proj.weight", "down_proj.weight")):
        """`names`: what the gate, up and down matrices are called behind `prefix`."""
        self.hidden, self.intermediate = hidden, intermediate
        self.gate_up = Linear(hidden, [intermediate, intermediate], [prefix + names[0], prefix + names[1]])
        self.down = Linear(intermediate, hidden, prefix + names[2])

    @property
    def input_reader(self):
        return self.gate_up.reader(swiglu=True)    # x goes to that product and nowhere else

    def tensor_specs(self):
        return self.gate_up.tensor_specs() + self.down.tensor_specs()

    def load(self, get):
        self.gate_up.load(get)
        self.down.load(get)

    def prepare(self, kernels):
        self.gate_up.prepare(kernels)
        self.down.prepare(kernels)

    def working_bytes(self, step) -> int:
        activated = step.matrix(step.rows, self.intermediate, reader=self.down.reader_for_plan(step.act_size))
        return (activated + self.gate_up.working_bytes(step, step.rows, accumulate=True, swiglu=True)
                + self.down.working_bytes(step, step.rows, accumulate=True, then_norm=True))

    def forward(self, ctx, x, hidden, then_norm=None):
        activated = ctx.new_activations(x.shape[0], self.intermediate, reader=self.down.reader())
        ctx.kernels.gemm_swiglu(x, self.gate_up.weight, activated)     # both products and the gate in one pass
        return self.down.add_into(ctx, activated, hidden, then_norm)


@FEED_FORWARDS.register("swiglu")
def _build_swiglu(config, layer_index, prefix, shared):
    return SwiGLU(config.hidden, config.intermediate, prefix + "mlp.")


class SquaredReLU:
    """Dense feed-forward with one inner matrix: out = Wd relu(Wu x)^2.  Its result is added to `hidden`, or written
    there when the caller says that `hidden` holds nothing yet (`fresh`)."""
    graph_safe = True
    graph_safe_rows = None
    writes_fresh = True

    def __init__(self, hidden: int, inner: int, prefix: str):
        self.hidden, self.inner = hidden, inner
        self.up = Linear(hidden, inner, prefix + "up")
        self.down = Linear(inner, hidden, prefix + "down")

    @property
    def input_reader(self):
        return self.up.reader()

    def tensor_specs(self):
        return self.up.tensor_specs() + self.down.tensor_specs()

    def load(self, get):
        self.up.load(get)
        self.down.load(get)

    def prepare(self, kernels):
        self.up.prepare(kernels)
        self.down.prepare(kernels)

    def working_bytes(self, step) -> int:
        return (2 * step.matrix(step.rows, self.inner) + self.up.working_bytes(step, step.rows, accumulate=True)
                + self.down.working_bytes(step, step.rows, accumulate=True))

    def forward(self, ctx, x, hidden, fresh=False):
        inner = self.up.forward(ctx, x)
        activated = ctx.new_activations(inner.shape[0], self.inner, reader=self.down.reader())      # as the down product reads it
        ctx.kernels.relu_squared(inner, activated)
        self.down.forward(ctx, activated, out=hidden, accumulate=not fresh)


class GeluTanh(SquaredReLU):
    """The same with the tanh form of GELU between the two matrices: out = Wd gelu(Wu x),
    gelu(z) = z/2 (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))."""

    def forward(self, ctx, x, hidden, fresh=False):
        inner = self.up.forward(ctx, x)
        activated = ctx.new_activations(inner.shape[0], self.inner, reader=self.down.reader())
        ctx.kernels.gelu_tanh(inner, activated)
        self.down.forward(ctx, activated, out=hidden, accumulate=not fresh)


@FEED_FORWARDS.register("gelu_tanh")
def _build_gelu_tanh(config, layer_index, prefix, shared):
    return GeluTanh(config.hidden, config.layers[layer_index].mlp.ff, prefix + "mlp.")


@FEED_FORWARDS.register("squared_relu")
def _build_squared_relu(config, layer_index, prefix, shared):
    return SquaredReLU(config.hidden, config.layers[layer_index].ff, prefix + "mlp.")


@FEED_FORWARDS.register("none")
def _build_no_feed_forward(config, layer_index, prefix, shared):
    return None


@FEED_FORWARDS.register("clamped_glu")
def _build_clamped_glu(config, layer_index, prefix, shared):
    from .experts import ClampedGLU

    sizes = config.layers[layer_index].mlp
    return ClampedGLU(config.hidden, sizes.ff, sizes.limit, prefix + "mlp.")
