"""Norm operator modules.  RMSNorm: arithmetic in csrc/elementwise.hip (nvh_rmsnorm / nvh_add_rmsnorm).
StreamNorm: a layer norm or RMS norm of the fp32 residual stream, applied together with the residual add in front of it by
nvh_residual_norm (csrc/stream_f32.hip).
DynamicTanh: a norm without statistics, tanh(alpha x) * weight + bias, applied together with the residual add around
it by nvh_residual_dyt (csrc/stream_f32.hip) over an fp32 residual stream.
PostSumRMSNorm: an RMS norm taken AFTER the residual sum (the stream itself is the normed value), with the old stream's
weight in the sum, a per-column scale of the sublayer's result and a weight stored around zero (nvh_residual_postnorm).

SublayerOutputNorm: an RMS norm of a sublayer's RESULT, which then joins the stream with a multiplier (nvh_residual_subnorm).

Interface of the reference's nanovllm/layers/layernorm.py:48-165: ``RMSNorm(hidden_size,
eps)``, ``.weight``, ``forward(x)`` -> y, ``forward(x, residual)`` -> (y, new_residual).
"""
import torch
from torch import nn

from .. import ops


class RMSNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float = 1e-6) -> None:
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(hidden_size), requires_grad=False)

    def forward(self, x, residual: torch.Tensor | None = None):
        """x: tensor, or a SplitKOutput (unreduced projection; only with a residual)."""
        slabs = getattr(x, "slabs", None)
        if residual is None:
            if slabs is not None:
                x = x.reduce()
            return ops.rmsnorm(x, self.weight.data, self.eps)
        # the residual stream is updated in place: new_residual aliases `residual`
        if slabs is not None:
            return ops.add_rmsnorm(None, residual, self.weight.data, self.eps, partials=slabs)
        return ops.add_rmsnorm(x, residual, self.weight.data, self.eps)


class DynamicTanh(nn.Module):
    """tanh(alpha * x) * weight + bias with a learned scalar alpha; no mean, no variance, no epsilon.

    The module holds the parameters; the arithmetic runs fused with a residual add (ops.residual_dyt), which takes the
    `triple()` of the norm after the sublayer and of the norm that opens the next one."""

    def __init__(self, hidden_size: int, alpha: float = 0.5) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size), requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(hidden_size), requires_grad=False)
        self.alpha = nn.Parameter(torch.full((1,), alpha), requires_grad=False)
        self.alpha.weight_loader = lambda param, t: param.data.copy_(t.reshape(1))

    def triple(self):
        return self.alpha.data, self.weight.data, self.bias.data

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """x fp32 [rows, dim] -> normalised rows in the parameters' type (x is left as it is)."""
        return ops.residual_dyt(x, nxt=self.triple())


class StreamNorm(nn.Module):
    """Norm of an fp32 residual stream with statistics: kind "layer" = (x - mean) / sqrt(var + eps) * weight + bias (var: the mean
    squared deviation), kind "rms" = x * rsqrt(mean of squares + eps) * weight.  The module holds the parameters; the arithmetic
    runs fused with the residual add that precedes it (ops.residual_norm takes `spec()`)."""

    def __init__(self, hidden_size: int, eps: float, kind: str = "layer", bias: bool = True) -> None:
        super().__init__()
        assert kind in ("layer", "rms")
        self.kind, self.eps = kind, eps
        self.weight = nn.Parameter(torch.ones(hidden_size), requires_grad=False)
        if bias and kind == "layer":
            self.bias = nn.Parameter(torch.zeros(hidden_size), requires_grad=False)
        else:
            self.register_parameter("bias", None)

    def spec(self) -> dict:
        return dict(norm=self.kind, weight=self.weight.data, bias=None if self.bias is None else self.bias.data, eps=self.eps)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """x fp32 [rows, dim] -> normalised rows in the parameters' type (x is left as it is)."""
        return ops.residual_norm(x, **self.spec())


class PostSumRMSNorm(nn.Module):
    """The close of a sublayer in a stack that norms after the sum:

        x <- rms_norm(alpha x + scale * sublayer(x)) * (offset + weight)

    alpha weighs the old stream in the sum, `scale` (one factor per column, optional) the sublayer's result, and `offset` = 1
    serves a weight that is stored around zero.  The stream x is fp32 and is replaced in place; `close` returns it once
    more in the activation type, the input of the next sublayer."""

    def __init__(self, hidden_size: int, eps: float, alpha: float = 1.0, weight_offset: float = 0.0, layer_scale: bool = False) -> None:
        super().__init__()
        self.eps, self.alpha, self.weight_offset = eps, float(alpha), float(weight_offset)
        self.weight = nn.Parameter(torch.zeros(hidden_size) if weight_offset else torch.ones(hidden_size), requires_grad=False)
        if layer_scale:
            self.scale = nn.Parameter(torch.ones(hidden_size), requires_grad=False)
        else:
            self.register_parameter("scale", None)

    def close(self, x: torch.Tensor, y: torch.Tensor | None = None, y32: torch.Tensor | None = None, want_h: bool = True):
        """y: the sublayer's result in the activation type, y32: in fp32 (either, both or none)."""
        return ops.residual_postnorm(x, self.weight.data, self.eps, y, y32, None if self.scale is None else self.scale.data, self.alpha,
                                     self.weight_offset, want_h)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """The norm alone (no sum, the stream taken once): x fp32 [rows, dim] -> normed rows in the activation type (x is left as it is)."""
        return ops.residual_postnorm(x, self.weight.data, self.eps, None, None, None, 1.0, self.weight_offset, True, in_place=False)


class SublayerOutputNorm(nn.Module):
    """The close of a sublayer whose result, not its input, is normed:

        x <- x + mult * weight * y / sqrt(mean(y^2) + eps),      y = the sublayer's result (a sum of up to three terms)

    `weight` is ONE number for all columns (hidden_size None) or one per column.  The stream x is fp32 and is updated in place; `close`
    returns it once more in the activation type, the input of a sublayer that reads the stream as it is."""

    def __init__(self, eps: float, mult: float = 1.0, hidden_size: int | None = None) -> None:
        super().__init__()
        self.eps, self.mult = eps, float(mult)
        self.weight = nn.Parameter(torch.ones(hidden_size or 1), requires_grad=False)
        self.weight.weight_loader = lambda param, t: param.data.copy_(t.reshape(param.shape))

    def close(self, x: torch.Tensor, a=None, a_scale: float = 1.0, b=None, b_scale: float = 1.0, c32=None, want_h: bool = True):
        """a, b: terms of the result in the activation type (with their factors), c32: a term in fp32."""
        return ops.residual_subnorm(x, self.weight.data, self.eps, self.mult, a, a_scale, b, b_scale, c32, want_h)
