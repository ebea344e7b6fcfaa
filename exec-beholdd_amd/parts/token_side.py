"""A per-layer input from the token itself, and the matrix through which a looped stretch of layers is entered.

Token side input (after a layer's feed-forward), with a table that holds `dim` numbers per (token, layer):

    e = table[token][layer * dim : (layer + 1) * dim]
    g = gelu_tanh(Wgate x) * e;   y = Wproj g;   x <- x + y / sqrt(mean(y^2) + eps) * w

x is the float32 residual; the two products read it and g in the activation type, the norm and the sum are float32.
The table is one tensor for all layers (`TokenSideTable`, shared); a layer that runs several times reads the same part.

Loop input (before the first layer of every pass of a looped stretch):  x <- Win [x ; x0], x0 being the embedding's
output, which `LoopInput.keep` copies before the first layer changes the residual.
"""

from __future__ import annotations

import torch

from ..weights.binder import TensorSpec
from .linear import Linear


class TokenSideTable:
    """The table [vocab, layers * dim], owned by the model and read by every layer's `TokenSideInput`."""
    graph_safe = True
    graph_safe_rows = None

    def __init__(self, vocab: int, n_layers: int, dim: int, name: str):
        self.vocab, self.n_layers, self.dim, self.name = int(vocab), int(n_layers), int(dim), name
        self.weight = None

    def tensor_specs(self):
        return [TensorSpec(self.name, (self.vocab, self.n_layers * self.dim), "linear")]

    def load(self, get):
        self.weight = get(self.name)


class TokenSideInput:
    graph_safe = True
    graph_safe_rows = None

    def __init__(self, hidden: int, dim: int, layer: int, table: TokenSideTable, eps: float, prefix: str):
        self.hidden, self.dim, self.layer, self.table, self.eps, self.prefix = int(hidden), int(dim), int(layer), table, float(eps), prefix
        self.gate = Linear(hidden, dim, prefix + "gate")
        self.proj = Linear(dim, hidden, prefix + "proj")
        self.norm_weight = None

    def tensor_specs(self):
        return self.gate.tensor_specs() + self.proj.tensor_specs() + [TensorSpec(self.prefix + "norm", (self.hidden,), "norm")]

    def load(self, get):
        self.gate.load(get)
        self.proj.load(get)
        self.norm_weight = get(self.prefix + "norm").to(torch.float32).contiguous()

    def prepare(self, kernels):
        self.gate.prepare(kernels)
        self.proj.prepare(kernels)

    def working_bytes(self, step) -> int:
        return (step.matrix(step.rows, self.hidden) + 2 * step.matrix(step.rows, self.dim) + step.matrix(step.rows, self.hidden, 4)
                + self.gate.working_bytes(step, step.rows, accumulate=True) + self.proj.working_bytes(step, step.rows, accumulate=True))

    def forward(self, ctx, hidden):
        k = ctx.kernels
        n = hidden.shape[0]
        x = ctx.new_activations(n, self.hidden, reader=self.gate.reader())
        k.cast_concat(hidden, None, x)
        gate = self.gate.forward(ctx, x)
        gated = ctx.new_activations(n, self.dim, reader=self.proj.reader())
        if ctx.token_src is not None:
            k.gelu_gate_table(gate, ctx.tokens, self.table.weight, self.layer * self.dim, gated, token_src=ctx.token_src, fed_tokens=ctx.fed_tokens)
        else:
            k.gelu_gate_table(gate, ctx.tokens, self.table.weight, self.layer * self.dim, gated)
        y = self.proj.forward(ctx, gated, out_dtype=torch.float32)
        k.rms_scale_add(hidden, y, self.norm_weight, self.eps)


class LoopInput:
    graph_safe = True
    graph_safe_rows = None

    def __init__(self, hidden: int, name: str):
        self.hidden = int(hidden)
        self.linear = Linear(2 * self.hidden, self.hidden, name)

    def tensor_specs(self):
        return self.linear.tensor_specs()

    def load(self, get):
        self.linear.load(get)

    def prepare(self, kernels):
        self.linear.prepare(kernels)

    def working_bytes(self, step) -> int:
        return (step.matrix(step.rows, self.hidden, 4) + step.matrix(step.rows, 2 * self.hidden)
                + self.linear.working_bytes(step, step.rows, accumulate=True))

    def keep(self, ctx, hidden):
        """A copy of the embedding's output, for the passes to read."""
        return hidden.clone()

    def forward(self, ctx, hidden, first):
        """hidden <- Win [hidden ; first], in place."""
        both = ctx.new_activations(hidden.shape[0], 2 * self.hidden, reader=self.linear.reader())
        ctx.kernels.cast_concat(hidden, first, both)
        self.linear.forward(ctx, both, out=hidden)


class EmbeddingAgain:
    """The entry of a later pass of a looped stretch that adds the embedding's output to the residual: x <- x + x0, in
    float32, x0 being what `keep` copied before the first layer changed the residual."""
    graph_safe = True
    graph_safe_rows = None

    def __init__(self, hidden: int):
        self.hidden = int(hidden)

    def tensor_specs(self):
        return []

    def load(self, get):
        pass

    def working_bytes(self, step) -> int:
        return step.matrix(step.rows, self.hidden, 4)      # the copy of the embedding's output

    def keep(self, ctx, hidden):
        return hidden.clone()

    def forward(self, ctx, hidden, first):
        ctx.kernels.weighted_sum(hidden, hidden, 1.0, first, 1.0)
