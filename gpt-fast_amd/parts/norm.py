"""RMS norm (reference model.py:230-241)."""
import torch

from ..config.spec import NormSpec
from ..ops import kernels as K
from .base import Param, Part, Runtime, check_bound, register_norm


class RMSNorm(Part):
    """``x * rsqrt(mean(x^2) + eps) * (weight + weight_offset)`` over the last dimension;
    statistics and scaling in float32 from the float32 residual stream, one rounding to the
    compute type at the store.  ``eps``, the width and the offset (1 for weights stored
    around zero) are the spec's; the offset is added once, when the weight is bound."""

    replayable = True

    def __init__(self, spec: NormSpec, runtime: Runtime):
        self.spec = spec
        self.rt = runtime
        self.weight = None

    def parameters(self):
        init = "around_zero" if getattr(self.spec, "weight_offset", 0.0) else "norm"
        return {"weight": Param((self.spec.dim,), role="vector", init=init)}

    def bind(self, tensors):
        check_bound("RMSNorm", self.parameters(), tensors)
        self.weight = tensors["weight"].to(torch.float32).contiguous()
        offset = float(getattr(self.spec, "weight_offset", 0.0))
        if offset:
            self.weight = self.weight + offset

    def forward(self, residual: torch.Tensor, rows=None) -> torch.Tensor:
        return K.rmsnorm(residual, self.weight, self.spec.eps, self.rt.dtype, rows=rows)

    def row_and_column_form(self):
        """This norm is a factor per row, rsqrt(mean(x^2) + eps), times a weight per column:
        (column weights, eps).  A kernel that completes the residual stream can apply it in
        the same pass."""
        return self.weight, self.spec.eps


class ScalarRMSNorm(RMSNorm):
    """``x * rsqrt(mean(x^2) + eps) * g`` with ONE stored number g for all elements.  The number
    is spread over a vector when it is bound, so every kernel that takes a norm's weights per
    column takes this norm as well."""

    def parameters(self):
        return {"weight": Param((), role="vector", init="norm")}

    def bind(self, tensors):
        check_bound("ScalarRMSNorm", self.parameters(), tensors)
        g = tensors["weight"].to(torch.float32).reshape(1)
        self.weight = (g + float(getattr(self.spec, "weight_offset", 0.0))).expand(self.spec.dim).contiguous()


class NoNorm(Part):
    """No norm: the rows of the stream in the compute type, for a sublayer that reads the stream
    itself.  ``plain_rows`` tells a kernel that completes the stream to hand the new rows on as
    they are."""

    replayable = True
    plain_rows = True

    def __init__(self, spec: NormSpec, runtime: Runtime):
        self.spec = spec
        self.rt = runtime

    def forward(self, residual: torch.Tensor, rows=None) -> torch.Tensor:
        return K.cast_rows(residual, self.rt.dtype, rows=rows)


class LayerNorm(Part):
    """``(x - mean) * rsqrt(mean((x - mean)^2) + eps) * weight`` over the last dimension, no
    bias; statistics in float32 from the float32 stream, one rounding to the compute type at
    the store.  ``layer_form()`` tells a kernel that completes the stream how to apply it on
    its way."""

    replayable = True

    def __init__(self, spec: NormSpec, runtime: Runtime):
        self.spec = spec
        self.rt = runtime
        self.weight = None

    def parameters(self):
        return {"weight": Param((self.spec.dim,), role="vector", init="norm")}

    def bind(self, tensors):
        check_bound("LayerNorm", self.parameters(), tensors)
        self.weight = tensors["weight"].to(torch.float32).contiguous()

    def forward(self, residual: torch.Tensor, rows=None) -> torch.Tensor:
        return K.layer_norm(residual, self.weight, self.spec.eps, self.rt.dtype, rows=rows)

    def layer_form(self):
        return self.weight, self.spec.eps


register_norm("rms", RMSNorm)
register_norm("layer", LayerNorm)
register_norm("rms_scalar", ScalarRMSNorm)
register_norm("none", NoNorm)
