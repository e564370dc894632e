"""Feed-forward parts.  `GatedMLP`: down(act(gate(x)) * up(x)) with act silu or the tanh form
of gelu, or the clamped swish: with g = min(gate(x), limit) and u = clamp(up(x), -limit, limit),
down(g sigmoid(alpha g) (u + 1)); `DenseMLP`:
down(act(up(x))) with act one of relu squared, relu, silu, tanh-gelu.

The gated one:

runtime/include/execution/decoder.hpp:161-166 of the reference; gate and up are
two checkpoint matrices that become one [2I, H] matrix when the part is built: in strips
of 16 rows, the gate rows of 16 outputs followed by their up rows (when I is a multiple of
16; else all gate rows, then all up rows).  A wave of the few-rows kernel owns 16 rows, so
neighbouring waves hold a strip's gate and up sums and the kernel can write
silu(gate) * up itself; otherwise the activation kernel reads the same layout.
Optional biases (runtime/include/models/qwen3_model.hpp:396-403) follow their rows.
"""
from __future__ import annotations

import torch

from ..csrc import lib
from ..weights.loader import ParamSpec
from .linear import Linear


class GatedMLP:
    @property
    def capture_safe(self):
        """Only capturable kernels and no allocation per step, as long as its products do."""
        return self.gate_up.capture_safe and self.down.capture_safe

    @property
    def capture_rows(self):
        return min(self.gate_up.capture_rows, self.down.capture_rows)

    @classmethod
    def kernel_libraries(cls, spec, dtype):
        return ("rowwise", *Linear.kernel_libraries(dtype))

    @classmethod
    def parameters(cls, spec, hidden):
        params = {
            "gate_proj.weight": ParamSpec((spec.intermediate_size, hidden)),
            "up_proj.weight": ParamSpec((spec.intermediate_size, hidden)),
            "down_proj.weight": ParamSpec((hidden, spec.intermediate_size)),
        }
        wanted = getattr(spec, "bias", None)
        if wanted is not False:
            optional = wanted is not True
            params["gate_proj.bias"] = ParamSpec((spec.intermediate_size,), optional=optional)
            params["up_proj.bias"] = ParamSpec((spec.intermediate_size,), optional=optional)
            params["down_proj.bias"] = ParamSpec((hidden,), optional=optional)
        return params

    def __init__(self, spec, hidden, params, dtype, device):
        if spec.activation not in lib.GATE_ACTIVATIONS:
            raise ValueError(f"gated_mlp: activation '{spec.activation}' is not implemented; "
                             f"known: {sorted(lib.GATE_ACTIVATIONS)}")
        self.spec = spec
        gate, up = params["gate_proj.weight"], params["up_proj.weight"]
        inter = spec.intermediate_size
        self.strip = lib.GATE_STRIP if inter % lib.GATE_STRIP == 0 else 0
        if self.strip:
            both = torch.stack([gate.reshape(inter // self.strip, self.strip, hidden),
                                up.reshape(inter // self.strip, self.strip, hidden)], dim=1)
            both = both.reshape(2 * inter, hidden)
        else:
            both = torch.cat([gate, up], dim=0)
        both_bias = None
        if "gate_proj.bias" in params or "up_proj.bias" in params:   # an absent one is zero
            zero = gate.new_zeros(inter)
            gate_bias = params.get("gate_proj.bias", zero)
            up_bias = params.get("up_proj.bias", zero)
            if self.strip:    # the same interleaving as the rows
                both_bias = torch.stack([gate_bias.reshape(-1, self.strip),
                                         up_bias.reshape(-1, self.strip)], dim=1).reshape(-1)
            else:
                both_bias = torch.cat([gate_bias, up_bias])
        self.gate_up = Linear(both, dtype, device, bias=both_bias)
        self.down = Linear(params["down_proj.weight"], dtype, device,
                           bias=params.get("down_proj.bias"))

    bias_later = True      # forward(..., bias_later=True) hands the last product's bias on

    def forward(self, ctx, x, bias_later=False):
        """The feed-forward's rows; with `bias_later`, (rows, float32 bias of the down
        projection that is still to be added, or None): a caller whose next kernel reads the
        rows anyway adds it there and saves a launch."""
        n = x.shape[0]
        # (the few-rows product that applies the gate itself knows silu only)
        act = (self.gate_up.forward_gated(ctx, x, "mlp.act")
               if self.strip and self.spec.activation == "silu" else None)
        if act is None:
            # (the activation kernel adds the bias itself where the product left it to it)
            gate_up, bias = self.gate_up.forward(ctx, x, "mlp.gate_up", bias_later=True)
            act = ctx.buffer("mlp.act", (n, self.spec.intermediate_size))
            lib.swiglu(gate_up, act, self.strip, self.spec.activation, bias=bias,
                       limit=getattr(self.spec, "limit", 0.0), alpha=getattr(self.spec, "alpha", 1.0))
            ctx.release(gate_up)
        out = self.down.forward(ctx, act, "mlp.down", bias_later=bias_later)
        ctx.release(act)
        return out


class DenseMLP:
    """down(act(up(x))): two matrices and an elementwise activation between them
    (`spec.activation`: "relu2" = relu(z)^2, "relu", "silu", "gelu_tanh").  The activation
    kernel sums the float32 slices of a few-rows product while it reads them."""

    @property
    def capture_safe(self):
        return self.up.capture_safe and self.down.capture_safe

    @property
    def capture_rows(self):
        return min(self.up.capture_rows, self.down.capture_rows)

    @classmethod
    def kernel_libraries(cls, spec, dtype):
        return ("rowwise", *Linear.kernel_libraries(dtype))

    @classmethod
    def parameters(cls, spec, hidden):
        return {
            "up_proj.weight": ParamSpec((spec.intermediate_size, hidden)),
            "down_proj.weight": ParamSpec((hidden, spec.intermediate_size)),
            "up_proj.bias": ParamSpec((spec.intermediate_size,), optional=True),
            "down_proj.bias": ParamSpec((hidden,), optional=True),
        }

    def __init__(self, spec, hidden, params, dtype, device):
        if spec.activation not in lib.ACTIVATIONS:
            raise ValueError(f"dense_mlp: activation '{spec.activation}' is not implemented; "
                             f"known: {sorted(lib.ACTIVATIONS)}")
        self.spec = spec
        self.up = Linear(params["up_proj.weight"], dtype, device, bias=params.get("up_proj.bias"))
        self.down = Linear(params["down_proj.weight"], dtype, device,
                           bias=params.get("down_proj.bias"))

    def forward(self, ctx, x):
        n = x.shape[0]
        up = self.up.forward(ctx, x, "mlp.up")
        act = ctx.buffer("mlp.act", (n, self.spec.intermediate_size))
        lib.activation(up, act, self.spec.activation)
        ctx.release(up)
        out = self.down.forward(ctx, act, "mlp.down")
        ctx.release(act)
        return out
