"""Selective state-space mixer with one decay per head (Mamba-2).

For token t and head h (its B and C come from group h // (heads / groups)), with x the mixer's
input, inner = heads * head_dim and N = state (all of the recurrence in float32):

    [z | xBC | dt] = W_in x                   z: inner, xBC: inner + 2 groups N, dt: heads
    xBC            = silu(conv(xBC) + b)      short causal convolution over time, one filter a
                                              channel, zeros before the sequence
    dt             = softplus(dt + dt_bias)   (no clamp)
    S_t            = exp(-exp(a_log_h) dt_t) S_{t-1} + dt_t B_t x_t^T        S is [N, head_dim]
    y_t            = S_t^T C_t + skip_h x_t
    out            = W_o (rmsnorm_parts(y * silu(z)) * out_norm)

The gate comes before the norm, which divides each of `norm_parts` equal parts of the row by
its own root mean square.  Per sequence the cache holds one float32 row (`StateRequest`): S of
every head, then the last taps - 1 inputs of every convolved channel, so a prompt may arrive
whole, in portions of any size or token by token.  The row has two versions: a step reads one
and writes the whole other one, and the session makes that one current when the step is
committed.  Kernels: `csrc/ssm.hip`.
"""
from __future__ import annotations

import torch

from ..csrc import lib
from ..weights.loader import ParamSpec
from .base import StateRequest
from .linear import Linear


class StateSpace:
    @property
    def capture_safe(self):
        """Only this library's kernels, nothing allocated per step, what varies read from the
        step's metadata on the device: as long as its products say the same."""
        return self.proj.capture_safe and self.o.capture_safe

    @property
    def capture_rows(self):
        return min(self.proj.capture_rows, self.o.capture_rows)

    @classmethod
    def shape_of(cls, spec) -> lib.SsmShape:
        return lib.SsmShape(spec.n_heads, spec.groups, spec.head_dim, spec.state, spec.conv_taps)

    @classmethod
    def parameters(cls, spec, hidden):
        channels = spec.inner + 2 * spec.groups * spec.state
        return {
            "in_proj.weight": ParamSpec((spec.inner + channels + spec.n_heads, hidden)),
            "conv.weight": ParamSpec((channels, spec.conv_taps), scale=0.5),
            "conv.bias": ParamSpec((channels,), scale=0.1),
            "dt_bias": ParamSpec((spec.n_heads,), init="uniform", low=-4.0, high=0.0),
            "a_log": ParamSpec((spec.n_heads,), init="uniform", low=-3.0, high=0.5),
            "skip": ParamSpec((spec.n_heads,), init="norm"),
            "out_norm.weight": ParamSpec((spec.inner,), init="norm"),
            "o_proj.weight": ParamSpec((hidden, spec.inner)),
        }

    @classmethod
    def cache_request(cls, spec):
        return StateRequest(shape=(cls.shape_of(spec).state_floats,), two_versions=True)

    @classmethod
    def kernel_libraries(cls, spec, dtype):
        return ("ssm", *Linear.kernel_libraries(dtype))

    @classmethod
    def check(cls, spec):
        if spec.n_heads < 1 or spec.groups < 1 or spec.n_heads % spec.groups:
            raise ValueError("mamba2: n_heads must be a multiple of groups")
        if not 1 <= spec.state <= 1024:
            raise ValueError(f"mamba2: state must lie in 1..1024, got {spec.state}")
        if spec.head_dim < 1:
            raise ValueError("mamba2: head_dim must be positive")
        if not 1 <= spec.conv_taps <= 64:
            raise ValueError(f"mamba2: conv_taps must lie in 1..64, got {spec.conv_taps}")
        if spec.norm_parts < 1 or spec.inner % spec.norm_parts:
            raise ValueError("mamba2: norm_parts must divide heads * head_dim")

    def __init__(self, spec, hidden, params, dtype, device, positions=None):
        self.check(spec)
        self.spec = spec
        self.shape = self.shape_of(spec)
        self.proj = Linear(params["in_proj.weight"], dtype, device)
        self.o = Linear(params["o_proj.weight"], dtype, device)

        def f32(tensor):
            return tensor.to(device=device, dtype=torch.float32).contiguous()
        self.conv_w = f32(params["conv.weight"])
        self.conv_b = f32(params["conv.bias"])
        self.dt_bias = f32(params["dt_bias"])
        self.a_log = f32(params["a_log"])
        self.skip = f32(params["skip"])
        self.out_norm = f32(params["out_norm.weight"])

    def forward(self, ctx, x, entry):
        if not entry.writes_cache:
            raise ValueError("mamba2: a run that only reads another run's state is not "
                             "implemented")
        shape, meta = self.shape, ctx.meta
        n = x.shape[0]
        state = ctx.cache.state(entry.cache)                 # [2 (slots + 1), state_floats]
        rows_in, rows_out = meta.seq_state_in, meta.seq_state_out
        proj = self.proj.forward(ctx, x, "ssm.proj")
        conv = ctx.buffer("ssm.conv", (n, shape.channels), torch.float32)
        lib.ssm_conv(proj, self.conv_w, self.conv_b, state, shape, meta.row_pos, meta.row_seq,
                     rows_in, rows_out, meta.seq_start, meta.seq_count, meta.seq_row0, conv)
        y_raw = ctx.buffer("ssm.y_raw", (n, shape.inner), torch.float32)
        lib.ssm_scan(conv, proj, self.a_log, self.dt_bias, self.skip, state, shape, rows_in,
                     rows_out, meta.seq_count, meta.seq_row0, y_raw)
        ctx.release(conv)
        gated = ctx.buffer("ssm.gated", (n, shape.inner))
        lib.ssm_out(y_raw, proj, self.out_norm, self.spec.norm_eps, shape, self.spec.norm_parts,
                    meta.row_seq, gated)
        ctx.release(y_raw, proj)
        delta = self.o.forward(ctx, gated, "ssm.o")
        ctx.release(gated)
        return delta
