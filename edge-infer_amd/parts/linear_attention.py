"""Linear attention with a fixed decay per head.

For token t and head h, with x the mixer's input (the recurrence, the norm and the gate in
float32):

    q = silu(W_q x), k = silu(W_k x)        heads x key_dim
    v = silu(W_v x)                         heads x value_dim
    S_t = decay_h S_(t-1) + k_t v_t^T       S is [key_dim, value_dim], zero before the sequence
    o_t = S_t^T q_t
    out = W_o (rmsnorm(o over all heads) * out_norm * sigmoid(W_g x))

The four projections are one product.  Per sequence the cache holds one float32 row
(`StateRequest`): S of every head.  The row has two versions: a step reads one and writes the
whole other one, and the session makes that one current when the step is committed, so a
prompt may arrive whole, in portions of any size or token by token.  Kernels:
`csrc/linear_attention.hip`.
"""
from __future__ import annotations

import torch

from ..csrc import lib
from ..weights.loader import ParamSpec
from .base import StateRequest
from .linear import Linear


class LinearAttention:
    ACTIVATE_ROWS = 64       # from so many rows of a prompt step on, q, k and v are activated aside

    @property
    def capture_safe(self):
        """Only this library's kernels, nothing allocated per step, what varies read from the
        step's metadata on the device: as long as its products say the same."""
        return self.proj.capture_safe and self.o.capture_safe

    @property
    def capture_rows(self):
        return min(self.proj.capture_rows, self.o.capture_rows)

    @classmethod
    def parameters(cls, spec, hidden):
        return {
            "q_proj.weight": ParamSpec((spec.qk_width, hidden)),
            "k_proj.weight": ParamSpec((spec.qk_width, hidden)),
            "v_proj.weight": ParamSpec((spec.v_width, hidden)),
            "gate_proj.weight": ParamSpec((spec.v_width, hidden)),
            "out_norm.weight": ParamSpec((spec.v_width,), init="norm"),
            "o_proj.weight": ParamSpec((hidden, spec.v_width)),
        }

    @classmethod
    def cache_request(cls, spec):
        return StateRequest(shape=(lib.la_state_floats(spec.n_heads, spec.key_dim,
                                                       spec.value_dim),), two_versions=True)

    @classmethod
    def kernel_libraries(cls, spec, dtype):
        return ("linear_attention", *Linear.kernel_libraries(dtype))

    @classmethod
    def check(cls, spec):
        if spec.n_heads < 1 or spec.value_dim < 1:
            raise ValueError("linear_attention: heads and value_dim must be positive")
        if not 1 <= spec.key_dim <= 256:
            raise ValueError(f"linear_attention: key_dim must lie in 1..256, got {spec.key_dim}")
        if len(spec.decay) != spec.n_heads:
            raise ValueError("linear_attention: one decay a head")

    def __init__(self, spec, hidden, params, dtype, device, positions=None):
        self.check(spec)
        self.spec = spec
        self.proj = Linear(torch.cat([params["q_proj.weight"], params["k_proj.weight"],
                                      params["v_proj.weight"], params["gate_proj.weight"]], dim=0),
                           dtype, device)
        self.o = Linear(params["o_proj.weight"], dtype, device)
        self.decay = torch.tensor(list(spec.decay), dtype=torch.float64).to(
            device=device, dtype=torch.float32).contiguous()
        self.out_norm = params["out_norm.weight"].to(device=device, dtype=torch.float32).contiguous()
        self.gate_column = 2 * spec.qk_width + spec.v_width

    def forward(self, ctx, x, entry):
        if not entry.writes_cache:
            raise ValueError("linear_attention: a run that only reads another run's state is not "
                             "implemented")
        spec, meta = self.spec, ctx.meta
        n = x.shape[0]
        state = ctx.cache.state(entry.cache)                 # [2 (slots + 1), state floats]
        proj = self.proj.forward(ctx, x, "la.proj")
        o_raw = ctx.buffer("la.o_raw", (n, spec.v_width), torch.float32)
        rows, activated = proj, False
        if not ctx.decode and n >= self.ACTIVATE_ROWS:
            # many tokens a sequence: silu of q, k and v once, not once a block of the scan
            rows = ctx.buffer("la.act", (n, self.gate_column), torch.float32)
            lib.la_activate(proj, rows)
            activated = True
        lib.la_scan(rows, self.decay, state, meta.seq_state_in, meta.seq_state_out, meta.seq_count,
                    meta.seq_row0, o_raw, spec.n_heads, spec.key_dim, spec.value_dim,
                    activated=activated)
        if activated:
            ctx.release(rows)
        gated = ctx.buffer("la.gated", (n, spec.v_width))
        lib.la_out(o_raw, proj, self.gate_column, self.out_norm, spec.norm_eps, meta.row_seq, gated)
        ctx.release(o_raw, proj)
        delta = self.o.forward(ctx, gated, "la.o")
        ctx.release(gated)
        return delta
