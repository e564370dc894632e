"""RMSNorm fused with the residual addition that precedes it.

y = x * rsqrt(mean(x^2) + eps) * w, all in float32, rounded once to the storage
type (the reference's float32 path, operators/src/cuda/rms_norm_cuda.cu:99-100;
its bfloat16 path rounds twice, :91-98, which this implementation does not copy).
The weight is kept in float32 whatever it was stored in.
"""
from __future__ import annotations

import torch

from ..csrc import lib
from ..weights.loader import ParamSpec


class RMSNorm:
    capture_safe = True      # only capturable kernels, no allocation per step

    @classmethod
    def kernel_libraries(cls, spec, dtype):
        return ("rowwise",)

    @classmethod
    def parameters(cls, spec, width):
        return {"weight": ParamSpec((width,), init="norm")}

    def __init__(self, spec, width, params, dtype, device):
        self.eps = float(spec.eps)
        self.width = width
        self.weight = params["weight"].to(device=device, dtype=torch.float32).contiguous()

    def add_norm(self, ctx, residual, delta, out_name, rows=None, write_residual=True):
        """residual += delta (all splits); returns rmsnorm(residual)[rows] * weight in
        the step's storage type."""
        n = residual.shape[0] if rows is None else rows.numel()
        out = ctx.buffer(out_name, (n, self.width))
        lib.add_rmsnorm(residual, delta, self.weight, self.eps, out, rows=rows,
                        write_residual=write_residual)
        return out

    def norm_add(self, ctx, residual, delta, cast_name=None, bias=None):
        """residual += rmsnorm(delta (+ bias)) * weight (the norm on a sublayer's output; `bias`
        is what the sublayer's last product left to this kernel).  With `cast_name`, also
        returns the new residual rows in the step's storage type, in the buffer of that name
        (what the next sublayer's product reads)."""
        cast = None
        if cast_name is not None:
            cast = ctx.buffer(cast_name, tuple(residual.shape))
        lib.norm_add(residual, delta, self.weight, self.eps, cast_out=cast, bias=bias)
        return cast


class LayerNorm:
    """y = (x - mean) / sqrt(mean((x - mean)^2) + eps) * w + b: a norm with a mean, a weight
    and a bias, in float32, rounded once to the storage type.  It sits where an `RMSNorm` sits:
    before a sublayer (`add_norm`) or on its output (`norm_add`).  Weight and bias are kept in
    float32 whatever they were stored in."""

    capture_safe = True      # only capturable kernels, no allocation per step
    centred = True

    @classmethod
    def kernel_libraries(cls, spec, dtype):
        return ("norms",)

    @classmethod
    def parameters(cls, spec, width):
        return {"weight": ParamSpec((width,), init="norm"), "bias": ParamSpec((width,), scale=0.1)}

    def __init__(self, spec, width, params, dtype, device):
        self.eps = float(spec.eps)
        self.width = width
        self.weight = params["weight"].to(device=device, dtype=torch.float32).contiguous()
        self.bias = params["bias"].to(device=device, dtype=torch.float32).contiguous()

    def scale_by(self, vector) -> None:
        """Fold a multiplier [width] (or a number) on the norm's result into weight and bias."""
        self.weight = (self.weight * vector).contiguous()
        self.bias = (self.bias * vector).contiguous()

    conv_widths = 4      # `conv` of the two methods below is taken for widths that are multiples

    def add_norm(self, ctx, residual, delta, out_name, rows=None, write_residual=True, conv=None):
        """residual += delta (all splits); returns layernorm(residual)[rows] in the step's
        storage type.  `conv` (a decode step only; see `lib.stream_norm`): the rows returned
        are h + conv(h) for the normed rows h."""
        n = residual.shape[0] if rows is None else rows.numel()
        out = ctx.buffer(out_name, (n, self.width))
        lib.stream_norm(residual, delta, out, w_next=self.weight, b_next=self.bias, eps=self.eps,
                        centred=True, rows=rows, write_residual=write_residual, conv=conv)
        return out

    def norm_add(self, ctx, residual, delta, cast_name=None, bias=None):
        """residual += layernorm(delta (+ bias)) (the norm on a sublayer's output; `bias` is
        what the sublayer's last product left to this kernel)."""
        if cast_name is not None:
            raise ValueError("layernorm: the stream's rounded copy is not implemented here")
        lib.stream_norm(residual, delta, None, w_after=self.weight, b_after=self.bias,
                        eps=self.eps, centred=True, delta_bias=bias)
        return None

    def norm_add_then(self, ctx, residual, delta, following, out_name, bias=None, conv=None):
        """residual += layernorm(delta (+ bias)), and then the rows of `following`, a norm of
        this kind before the next sublayer, in one pass: returns following(residual) (with
        `conv`, a decode step only: those rows with their convolution added)."""
        out = ctx.buffer(out_name, tuple(residual.shape))
        lib.stream_norm(residual, delta, out, w_after=self.weight, b_after=self.bias,
                        w_next=following.weight, b_next=following.bias, eps=self.eps,
                        centred=True, delta_bias=bias, conv=conv)
        return out
