"""Routed feed-forward: a mixture of experts.

For every row x: router logits z = W_router x in float32 (the router matrix is kept in
float32; x is read as the step stores it), the `top` experts with the largest logits, their
weights p = softmax over the chosen logits alone, and

    y = sum over the chosen e of p_e W_down,e (silu(W_gate,e x) * (W_up,e x)).

With `scoring = "softmax_all"` the scores are the softmax over all router outputs, the choice
goes by score plus a learned `correction` per output (where the spec has one), and the weights
are the chosen scores themselves; with `identity = I` the router has I outputs beyond the
experts, and one of them chosen adds p x itself.

The experts' matrices are stacked when the part is built (gate and up [E, F, H], down
[E, H, F]); routing stays on the device, so a step with this part is captured like any
other.  In bfloat16 with widths that are multiples of 64 the experts run as grouped matrix
products on the matrix cores (the pairs of (row, choice) laid out by expert on the device);
otherwise, and in float32, a kernel takes one pair at a time.  Kernels: `csrc/moe.hip`.
"""
from __future__ import annotations

import torch

from ..csrc import lib
from ..weights.loader import ParamSpec


class RoutedMLP:
    capture_safe = True      # only this library's kernels, nothing read back, no allocation

    @classmethod
    def kernel_libraries(cls, spec, dtype):
        return ("moe", "rowwise")

    @classmethod
    def parameters(cls, spec, hidden):
        outputs = spec.n_experts + getattr(spec, "identity", 0)
        params = {"router.weight": ParamSpec((outputs, hidden), scale=0.2)}
        if getattr(spec, "correction", False):
            params["router.correction"] = ParamSpec((outputs,), scale=0.05)
        for expert in range(spec.n_experts):
            prefix = f"experts.{expert}."
            params[prefix + "gate_proj.weight"] = ParamSpec((spec.intermediate_size, hidden))
            params[prefix + "up_proj.weight"] = ParamSpec((spec.intermediate_size, hidden))
            params[prefix + "down_proj.weight"] = ParamSpec((hidden, spec.intermediate_size))
        return params

    @classmethod
    def check(cls, spec):
        if not 1 <= spec.n_experts <= 512:
            raise ValueError(f"routed_mlp: 1 to 512 experts, got {spec.n_experts}")
        identity = getattr(spec, "identity", 0)
        if identity < 0 or spec.n_experts + identity > 512:
            raise ValueError("routed_mlp: a router has at most 512 outputs")
        if not 1 <= spec.top <= min(spec.n_experts + identity, 64):
            raise ValueError(f"routed_mlp: top must lie in 1..min(router outputs, 64), got {spec.top}")
        if getattr(spec, "scoring", "softmax_chosen") not in lib.ROUTER_SCORINGS:
            raise ValueError(f"routed_mlp: unknown scoring '{spec.scoring}'")
        if getattr(spec, "correction", False) and spec.scoring != "softmax_all":
            raise ValueError("routed_mlp: a correction belongs to the scoring 'softmax_all'")
        if spec.intermediate_size < 1:
            raise ValueError("routed_mlp: an expert's width must be positive")

    def __init__(self, spec, hidden, params, dtype, device):
        self.check(spec)
        self.spec = spec
        self.hidden = hidden

        def stacked(name):
            return torch.stack([params[f"experts.{expert}.{name}.weight"]
                                for expert in range(spec.n_experts)]).to(
                                    device=device, dtype=dtype).contiguous()
        self.w_gate, self.w_up, self.w_down = stacked("gate_proj"), stacked("up_proj"), stacked("down_proj")
        self.router = params["router.weight"].to(device=device, dtype=torch.float32).contiguous()
        self.scoring = getattr(spec, "scoring", "softmax_chosen")
        self.correction = None
        if getattr(spec, "correction", False):
            self.correction = params["router.correction"].to(device=device, dtype=torch.float32).contiguous()
        self.grouped = lib.moe_grouped_supported(dtype, hidden, spec.intermediate_size,
                                                 spec.n_experts)

    def forward(self, ctx, x):
        spec = self.spec
        n = x.shape[0]
        expert = ctx.buffer("moe.expert", (n, spec.top), torch.int32)
        weight = ctx.buffer("moe.weight", (n, spec.top), torch.float32)
        lib.moe_route(x, self.router, ctx.meta.row_seq, expert, weight, scoring=self.scoring,
                      correction=self.correction)
        act = ctx.buffer("moe.act", (n * spec.top, spec.intermediate_size))
        out = ctx.buffer("moe.out", (n, self.hidden), torch.float32)
        if self.grouped:
            pairs = n * spec.top
            order = ctx.buffer("moe.order", (2 * pairs + spec.n_experts + 1,), torch.int32)
            sums = ctx.buffer("moe.sums", (pairs, self.hidden), torch.float32)
            lib.moe_experts_grouped(x, self.w_gate, self.w_up, self.w_down, expert, weight,
                                    order[:pairs], order[pairs:2 * pairs], order[2 * pairs:], act,
                                    sums, out)
            ctx.release(order, sums)
        else:
            lib.moe_experts(x, self.w_gate, self.w_up, self.w_down, expert, weight, act, out)
        ctx.release(expert, weight, act)
        return out
