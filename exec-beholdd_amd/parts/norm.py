"""RMSNorm: y = (x * inv) * w with inv = 1/sqrt(mean(x^2) + eps).

crates/beholdd-kernel/src/vecops.rs:54-64: the weight is a plain multiplier (no 1 + w) and the
order of the two multiplications is (x * inv) * w.  The statistic is computed in float32 on
the float32 residual; only the result is rounded to the activation type.
"""

from __future__ import annotations

import torch

from ..weights.binder import TensorSpec
from .base import NORMS, NormRequest


class RMSNorm:
    graph_safe = True      # forward reads only the step's device tensors
    graph_safe_rows = None # ... whatever the number of tokens a sequence brings
    def __init__(self, width: int, eps: float, name: str):
        if not (eps > 0.0):
            raise ValueError(f"RMSNorm epsilon must be positive, got {eps}")
        self.width, self.eps, self.name = int(width), float(eps), name
        self.weight: torch.Tensor | None = None

    def tensor_specs(self):
        return [TensorSpec(self.name, (self.width,), "norm")]

    def load(self, get):
        self.weight = get(self.name)

    serves_reader = True   # forward and request take the product that reads the output

    def forward(self, ctx, hidden, rows=None, reader=None):
        n = hidden.shape[0] if rows is None else rows.shape[0]
        out = ctx.new_activations(n, self.width, reader=reader)
        ctx.kernels.rmsnorm(hidden, self.weight, self.eps, out, rows=rows)
        return out

    def working_bytes(self, step, rows: int | None = None, reader=None) -> int:
        return step.matrix(step.rows if rows is None else rows, self.width, reader=reader)

    def request(self, reader=None):
        """This norm as the product that completes its input may prepare it."""
        return NormRequest(self.weight, self.eps, reader)


class ZeroCentredRMSNorm(RMSNorm):
    """RMSNorm whose stored weight lies around zero: y = x / sqrt(mean(x^2) + eps) * (1 + w).  The sum 1 + w is made
    once, in float32, when the weight is loaded, and kept in float32 (a bfloat16 could not hold it).  The input is
    the float32 residual, or several residual streams [n, streams, width] of which the norm reads a weighted sum
    (`take` [streams] float32; None: every stream once): sum and statistic in float32 in one kernel."""

    reads_streams = True

    def tensor_specs(self):
        return [TensorSpec(self.name, (self.width,), "linear")]      # a random one lies around zero, like a stored one

    def load(self, get):
        self.weight = (get(self.name).to(torch.float32) + 1.0).contiguous()

    def forward(self, ctx, hidden, rows=None, reader=None, take=None):
        if hidden.dim() == 2:
            return super().forward(ctx, hidden, rows=rows, reader=reader)
        n = hidden.shape[0] if rows is None else rows.shape[0]
        out = ctx.new_activations(n, self.width, reader=reader)
        ctx.kernels.streams_rmsnorm(hidden, take, self.weight, self.eps, out, rows=rows)
        return out

    def update_then_forward(self, ctx, hidden, result, mix, give, scale, reader=None, take=None):
        """The streams' update by a sublayer's `result` (`kernels.streams_update`) and this norm of what they have become,
        in one kernel; None where the kernel set has none (then update, and call `forward`)."""
        fused = getattr(ctx.kernels, "streams_update_rmsnorm", None)
        if fused is None or hidden.dim() != 3:
            return None
        out = ctx.new_activations(hidden.shape[0], self.width, reader=reader)
        fused(hidden, result, mix, give, scale, take, self.weight, self.eps, out)
        return out

    def request(self, reader=None):
        raise NotImplementedError("this norm does not ride on the products around it")


class LayerNorm:
    """y = (x - mean) / sqrt(var + eps) * w + b, the variance being the mean of the squared deviations; mean, variance
    and the result are float32 on the float32 residual, only the output is rounded to the activation type.  The bias
    is the tensor `name + bias_suffix` (None: no bias).  Weight and bias are kept in float32."""
    graph_safe = True
    graph_safe_rows = None
    serves_reader = True

    def __init__(self, width: int, eps: float, name: str, bias_suffix: str | None = ".b"):
        if not (eps > 0.0):
            raise ValueError(f"LayerNorm epsilon must be positive, got {eps}")
        self.width, self.eps, self.name = int(width), float(eps), name
        self.bias_name = name + bias_suffix if bias_suffix is not None else None
        self.weight = self.bias = None

    def tensor_specs(self):
        specs = [TensorSpec(self.name, (self.width,), "norm")]
        if self.bias_name is not None:
            specs.append(TensorSpec(self.bias_name, (self.width,), "linear"))
        return specs

    def load(self, get):
        self.weight = get(self.name).to(torch.float32).contiguous()
        self.bias = get(self.bias_name).to(torch.float32).contiguous() if self.bias_name is not None else None

    def forward(self, ctx, hidden, rows=None, reader=None):
        n = hidden.shape[0] if rows is None else rows.shape[0]
        out = ctx.new_activations(n, self.width, reader=reader)
        ctx.kernels.layernorm(hidden, self.weight, self.bias, self.eps, out, rows=rows)
        return out

    def working_bytes(self, step, rows: int | None = None, reader=None) -> int:
        return step.matrix(step.rows if rows is None else rows, self.width, reader=reader)

    def sum_forward(self, ctx, hidden, result, alpha: float, reader=None, rounded: bool = True):
        """hidden <- norm(alpha * hidden + result), row by row and in place: the weighted sum, the statistics and the result
        are float32.  Returns what a sublayer that reads the new residual takes as its input: the residual itself where
        the activations are float32, else a copy rounded to the activation type, written by the same kernel (in the form
        `reader` reads fastest); None when `rounded` says that nobody reads one."""
        if ctx.act_dtype == torch.float32:
            ctx.kernels.sum_layernorm(hidden, result, alpha, self.weight, self.bias, self.eps, None)
            return hidden if rounded else None
        out = ctx.new_activations(hidden.shape[0], self.width, reader=reader) if rounded else None
        ctx.kernels.sum_layernorm(hidden, result, alpha, self.weight, self.bias, self.eps, out)
        return out


@NORMS.register("layernorm")
def _build_layernorm(config, width, name, shared):
    return LayerNorm(width, config.rms_eps, name)


@NORMS.register("rmsnorm")
def _build_rmsnorm(config, width, name, shared):
    return RMSNorm(width, config.rms_eps, name)


@NORMS.register("rmsnorm_zero_centred")
def _build_rmsnorm_zero_centred(config, width, name, shared):
    return ZeroCentredRMSNorm(width, config.rms_eps, name)
