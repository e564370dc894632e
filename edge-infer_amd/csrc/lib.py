"""ctypes bindings of the HIP kernel libraries.

Each function takes torch tensors that live on the GPU, checks what the kernel
assumes about them (device, dtype, contiguity, sizes) and launches on torch's
current stream.  A library is loaded (and compiled, when it is not yet) the first
time one of its functions is called.  There is no other implementation behind
these functions: if a library cannot be built or loaded the call raises.
"""
from __future__ import annotations

import ctypes
import functools
import os
from ctypes import c_float, c_int, c_longlong, c_ulonglong, c_void_p
from typing import Dict, Optional

import torch

from . import build

F32, BF16 = 0, 1
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}
PAGE_TOKENS = 64

_SIGNATURES = {
    "rowwise": {
        "ei_embed_gather": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_float,
                            c_void_p],
        "ei_add_rmsnorm": [c_void_p, c_void_p, c_int, c_int, c_longlong, c_void_p, c_void_p,
                           c_float, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
        "ei_swiglu": [c_void_p, c_int, c_int, c_longlong, c_void_p, c_int, c_int, c_int, c_int,
                      c_int, c_void_p, c_float, c_float, c_void_p],
        "ei_norm_rows": [c_void_p, c_void_p, c_float, c_longlong, c_int, c_void_p],
        "ei_gate_rows": [c_void_p, c_int, c_int, c_longlong, c_longlong, c_int, c_void_p, c_int,
                         c_longlong, c_int, c_void_p],
        "ei_scale_cap": [c_void_p, c_float, c_float, c_longlong, c_void_p],
        "ei_norm_add_norm": [c_void_p, c_void_p, c_int, c_int, c_longlong, c_void_p, c_void_p,
                             c_float, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p],
        "ei_concat_cast": [c_void_p, c_void_p, c_void_p, c_int, c_longlong, c_int, c_void_p],
        "ei_set_rows": [c_void_p, c_int, c_int, c_longlong, c_void_p, c_void_p, c_longlong, c_int,
                        c_void_p],
        "ei_sum_slices": [c_void_p, c_int, c_longlong, c_void_p, c_longlong, c_void_p],
        "ei_bias_rows": [c_void_p, c_void_p, c_longlong, c_int, c_int, c_void_p],
        "ei_norm_add": [c_void_p, c_void_p, c_int, c_int, c_longlong, c_void_p, c_float, c_void_p,
                        c_int, c_int, c_int, c_void_p, c_void_p],
        "ei_cast_rows": [c_void_p, c_void_p, c_int, c_longlong, c_void_p],
        "ei_activation": [c_void_p, c_int, c_int, c_longlong, c_void_p, c_int, c_longlong, c_int,
                          c_void_p],
    },
    "rope_store": {
        "ei_qk_norm_rope_store": [c_void_p, c_int, c_int, c_longlong, c_void_p, c_void_p, c_float,
                                  c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                  c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                  c_void_p],
        "ei_head_store": [c_void_p, c_int, c_int, c_longlong, c_longlong, c_void_p, c_void_p,
                          c_float, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                          c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int,
                          c_int, c_int, c_int, c_int, c_float, c_int, c_void_p, c_longlong,
                          c_void_p],
        "ei_projection_norm_store": [c_void_p, c_int, c_int, c_longlong, c_void_p, c_void_p, c_void_p,
                                     c_float, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                     c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                     c_int, c_void_p],
    },
    "ssm": {
        "ei_ssm_state_floats": [c_int, c_int, c_int, c_int, c_int],
        "ei_ssm_conv": [c_void_p, c_int, c_int, c_longlong, c_longlong, c_void_p, c_void_p,
                        c_void_p, c_longlong, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                        c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                        c_int, c_void_p],
        "ei_ssm_scan": [c_void_p, c_void_p, c_int, c_int, c_longlong, c_longlong, c_void_p,
                        c_void_p, c_void_p, c_void_p, c_longlong, c_void_p, c_void_p, c_void_p,
                        c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
        "ei_ssm_out": [c_void_p, c_void_p, c_int, c_int, c_longlong, c_longlong, c_void_p,
                       c_float, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
    },
    "norms": {
        "ei_stream_norm": [c_void_p, c_void_p, c_int, c_int, c_longlong, c_void_p, c_void_p,
                           c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_int, c_void_p, c_int,
                           c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                           c_int, c_int, c_void_p],
        "ei_norm_mean": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_float,
                         c_void_p, c_int, c_int, c_void_p],
    },
    "input_conv": {
        "ei_input_conv": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p,
                          c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                          c_int, c_int, c_int, c_void_p],
    },
    "linear_attention": {
        "ei_la_scan": [c_void_p, c_int, c_int, c_longlong, c_longlong, c_void_p, c_void_p,
                       c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                       c_int, c_int, c_void_p],
        "ei_la_activate": [c_void_p, c_int, c_int, c_longlong, c_longlong, c_void_p, c_int, c_int,
                           c_void_p],
        "ei_la_out": [c_void_p, c_void_p, c_int, c_int, c_longlong, c_longlong, c_longlong,
                      c_void_p, c_float, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    },
    "moe": {
        "ei_moe_route": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                         c_int, c_int, c_int, c_void_p, c_void_p],
        "ei_moe_experts": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                           c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
        "ei_moe_grouped_supported": [c_int, c_int, c_int, c_int],
        "ei_moe_experts_grouped": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                   c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                   c_int, c_int, c_int, c_int, c_int, c_void_p],
    },
    "delta_rule": {
        "ei_delta_conv": [c_void_p, c_int, c_int, c_longlong, c_int, c_void_p, c_int, c_void_p,
                          c_longlong, c_longlong, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                          c_void_p, c_int, c_int, c_int, c_void_p],
        "ei_delta_tail": [c_void_p, c_int, c_int, c_longlong, c_int, c_int, c_void_p, c_longlong,
                          c_longlong, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                          c_void_p],
        "ei_delta_rule": [c_void_p, c_void_p, c_int, c_int, c_longlong, c_int, c_int, c_int,
                          c_void_p, c_void_p, c_void_p, c_longlong, c_void_p, c_void_p, c_void_p,
                          c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_float,
                          c_void_p],
        "ei_delta_out": [c_void_p, c_void_p, c_int, c_int, c_longlong, c_int, c_int, c_void_p,
                         c_float, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
    },
    "attention_generic": {
        "ei_attn_heads_per_block": [c_int],
        "ei_attn_positions_per_item": [c_int],
        "ei_attention": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int,
                         c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int,
                         c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_float,
                         c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p],
        "ei_pool_store": [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                          c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int,
                          c_void_p],
    },
    "attention_wide": {
        "ei_attn_wide_supported": [c_int, c_int, c_int],
        "ei_attn_wide_positions": [c_int],
        "ei_attention_wide": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                              c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                              c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_float, c_int,
                              c_int, c_int, c_void_p, c_void_p],
    },
    "head_ops": {
        "ei_latent_down_store": [c_void_p, c_int, c_int, c_longlong, c_void_p, c_void_p, c_float,
                                 c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                 c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                 c_void_p],
        "ei_head_matmul": [c_void_p, c_int, c_int, c_longlong, c_longlong, c_int, c_int, c_void_p,
                           c_int, c_void_p, c_int, c_longlong, c_int, c_int, c_int, c_int, c_int,
                           c_int, c_void_p],
        "ei_rotate_pairs": [c_void_p, c_int, c_int, c_longlong, c_longlong, c_int, c_int, c_void_p,
                            c_void_p, c_void_p, c_int, c_longlong, c_int, c_int, c_int, c_int,
                            c_int, c_void_p],
        "ei_mix_heads": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                         c_void_p],
    },
    "mlstm": {
        "ei_mlstm_state_floats": [c_int, c_int, c_int],
        "ei_mlstm_proj_width": [c_int, c_int, c_int],
        "ei_mlstm_walk": [c_void_p, c_int, c_int, c_longlong, c_void_p, c_void_p, c_void_p,
                          c_longlong, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                          c_int, c_int, c_int, c_float, c_float, c_float, c_int, c_void_p],
        "ei_mlstm_out": [c_void_p, c_void_p, c_int, c_int, c_longlong, c_void_p, c_float,
                         c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    },
    "attention_mfma": {
        "ei_attn_decode_mfma_supported": [c_int, c_int],
        "ei_attn_prefill_mfma_positions": [c_int],
        "ei_attention_prefill_mfma": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int,
                                      c_int, c_int, c_float, c_int, c_int, c_void_p],
        "ei_attention_decode_mfma": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                     c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                     c_int, c_int, c_float, c_int, c_int, c_int, c_void_p,
                                     c_void_p],
        "ei_attention_prefill_mfma_ext": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                          c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p,
                                          c_int, c_int, c_int, c_int, c_float, c_int, c_int,
                                          c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
        "ei_attention_decode_mfma_ext": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                         c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int,
                                         c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int,
                                         c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
        "ei_attention_decode_mfma_fused": [c_void_p, c_int, c_longlong, c_void_p, c_void_p, c_float,
                                           c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                           c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int,
                                           c_int, c_int, c_int, c_int, c_float, c_int, c_int,
                                           c_int, c_void_p, c_void_p],
    },
    "gemm_f32": {
        "ei_gemm_f32": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_longlong, c_longlong,
                        c_longlong, c_void_p],
    },
    "gemm_bf16": {
        "ei_skinny_gemm_splits": [c_int, c_int, c_int, c_int],
        "ei_gemm_bf16_skinny": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                c_void_p],
        "ei_gemm_bf16_skinny_packed": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                       c_void_p],
        "ei_gemm_bf16_skinny_gated": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                      c_void_p],
    },
    "sampling": {
        "ei_argmax": [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_longlong, c_void_p],
        "ei_argmax_partial_size": [c_int, c_int],
        "ei_argmax_static": [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p],
        "ei_argmax_static_prepare": [],
        "ei_sample": [c_void_p, c_int, c_int, c_float, c_float, c_int, c_ulonglong, c_void_p,
                      c_void_p, c_void_p, c_void_p, c_void_p, c_longlong, c_void_p],
        "ei_sample_scratch_size": [c_int, c_int],
    },
    "peaks": {
        "ei_stream_read": [c_void_p, c_longlong, c_int, c_void_p, c_void_p],
        "ei_mfma_loop": [c_int, c_int, c_int, c_void_p, c_void_p],
        "ei_empty_launches": [c_int, c_int, c_void_p],
    },
}

_loaded: Dict[str, ctypes.CDLL] = {}


class KernelError(RuntimeError):
    pass


def library(name: str) -> ctypes.CDLL:
    lib = _loaded.get(name)
    if lib is not None:
        return lib
    path = build.build_library(name)
    try:
        lib = ctypes.CDLL(str(path))
    except OSError as error:
        raise KernelError(f"cannot load kernel library {path}: {error}") from error
    for symbol, argtypes in _SIGNATURES.get(name, {}).items():
        function = getattr(lib, symbol)
        function.argtypes = argtypes
        function.restype = c_int
    lib.ei_last_error.restype = ctypes.c_char_p
    _loaded[name] = lib
    return lib


def loaded_libraries():
    return sorted(_loaded)


def prepare(names) -> None:
    """Compile the kernel libraries `names` that are not built yet, at the same time.  A
    model says which ones it will need when it is made; each is still loaded at its first use."""
    build.build_libraries([name for name in names if name not in _loaded])


launches = 0        # calls of kernel entry points so far (most launch one kernel, a few two)


def _check(lib, status: int, what: str) -> None:
    global launches
    launches += 1
    if status != 0:
        message = lib.ei_last_error().decode(errors="replace")
        raise KernelError(f"{what}: {message} (status {status})")


# torch's own shortcut to the current stream's handle (no Stream object is made); a step of
# few rows launches some 300 kernels and is bound by what each launch costs the host
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


@functools.lru_cache(maxsize=None)
def _compute_units(index: int) -> int:
    return int(torch.cuda.get_device_properties(index).multi_processor_count)


def compute_units(device=None) -> int:
    """Compute units of a device (the current one by default): 256 on an MI355X.  The one
    place on the Python side where launch plans take the chip's size from."""
    if device is None:
        index = torch.cuda.current_device()
    else:
        device = torch.device(device)
        index = torch.cuda.current_device() if device.index is None else device.index
    return _compute_units(index)


def _stream() -> int:
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _gpu(tensor: torch.Tensor, name: str, dtype=None) -> int:
    if not tensor.is_cuda:
        raise KernelError(f"{name} must live on the GPU")
    if not tensor.is_contiguous():
        raise KernelError(f"{name} must be contiguous")
    if dtype is not None and tensor.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, got {tensor.dtype}")
    return tensor.data_ptr()


def _code(tensor: torch.Tensor, name: str) -> int:
    try:
        return _DTYPE_CODE[tensor.dtype]
    except KeyError:
        raise KernelError(f"{name} has unsupported dtype {tensor.dtype}") from None


def _splits(tensor: torch.Tensor, rows: int, width: int, name: str):
    """(nsplit, stride) of a [rows, width] or [nsplit, rows, width] tensor."""
    if tensor.dim() == 2 and tuple(tensor.shape) == (rows, width):
        return 1, 0
    if tensor.dim() == 3 and tuple(tensor.shape[1:]) == (rows, width):
        return tensor.shape[0], rows * width
    raise KernelError(f"{name} must be [{rows}, {width}] or [splits, {rows}, {width}], "
                      f"got {list(tensor.shape)}")


# ---------------------------------------------------------------------------
def embed_gather(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor,
                 scale: float = 1.0) -> None:
    """out[r] = table[ids[r]] * scale as float32."""
    lib = library("rowwise")
    n = ids.numel()
    vocab, hidden = table.shape
    if tuple(out.shape) != (n, hidden):
        raise KernelError(f"embed_gather: out must be [{n}, {hidden}], got {list(out.shape)}")
    status = lib.ei_embed_gather(_gpu(ids, "ids", torch.int32), _gpu(table, "table"),
                                 _code(table, "table"), _gpu(out, "out", torch.float32), n,
                                 hidden, vocab, float(scale), _stream())
    _check(lib, status, "embed_gather")


def add_rmsnorm(residual: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor,
                eps: float, out: torch.Tensor, rows: Optional[torch.Tensor] = None,
                write_residual: bool = True) -> None:
    """residual [R, H] float32 (+= sum of delta splits, stored back unless told not
    to); out[i] = rmsnorm(residual[rows[i] if rows else i]) * weight."""
    lib = library("rowwise")
    total_rows, hidden = residual.shape
    n = out.shape[0]
    if out.dim() != 2 or out.shape[1] != hidden:
        raise KernelError(f"add_rmsnorm: out must be [*, {hidden}], got {list(out.shape)}")
    if weight.numel() != hidden:
        raise KernelError(f"add_rmsnorm: weight must have {hidden} elements")
    if rows is None and n != total_rows:
        raise KernelError("add_rmsnorm: out and residual row counts differ")
    if rows is not None and rows.numel() != n:
        raise KernelError("add_rmsnorm: rows and out row counts differ")
    nsplit, stride, delta_ptr, delta_code = 0, 0, None, F32
    if delta is not None:
        nsplit, stride = _splits(delta, total_rows, hidden, "delta")
        delta_ptr, delta_code = _gpu(delta, "delta"), _code(delta, "delta")
    status = lib.ei_add_rmsnorm(
        _gpu(residual, "residual", torch.float32), delta_ptr, delta_code, nsplit, stride,
        None if rows is None else _gpu(rows, "rows", torch.int32),
        _gpu(weight, "weight", torch.float32), float(eps), _gpu(out, "out"), _code(out, "out"), n,
        hidden, int(write_residual), _stream())
    _check(lib, status, "add_rmsnorm")


GATE_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1, "clamped_swish": 2}


def swiglu(gate_up: torch.Tensor, out: torch.Tensor, strip: int = 0,
           activation: str = "silu", bias: Optional[torch.Tensor] = None,
           limit: float = 0.0, alpha: float = 1.0) -> None:
    """out = act(gate) * up of [n, 2*inter] rows (or float32 slices of them), act "silu" or
    "gelu_tanh"; or "clamped_swish": with g = min(gate, limit) and u = clamp(up, -limit, limit),
    out = g sigmoid(alpha g) (u + 1).  strip = 0: the gate columns come first, then the up
    columns; strip > 0: `strip` gate columns, their `strip` up columns, and so on.  bias:
    float32 [2*inter] in the rows' own column order, added before the activation."""
    lib = library("rowwise")
    if activation not in GATE_ACTIVATIONS:
        raise KernelError(f"swiglu: unknown gate activation '{activation}'; "
                          f"known: {sorted(GATE_ACTIVATIONS)}")
    n, inter = out.shape
    nsplit, stride = _splits(gate_up, n, 2 * inter, "gate_up")
    if bias is not None and bias.numel() != 2 * inter:
        raise KernelError("swiglu: the bias must be as wide as a row of gate_up")
    status = lib.ei_swiglu(_gpu(gate_up, "gate_up"), _code(gate_up, "gate_up"), nsplit, stride,
                           _gpu(out, "out"), _code(out, "out"), n, inter, int(strip),
                           GATE_ACTIVATIONS[activation],
                           None if bias is None else _gpu(bias, "bias", torch.float32),
                           float(limit), float(alpha), _stream())
    _check(lib, status, "swiglu")


def norm_rows(x: torch.Tensor, weight: torch.Tensor, eps: float) -> None:
    """x [rows, H] float32 <- x / sqrt(mean(x^2) + eps) * weight, in place."""
    lib = library("rowwise")
    rows, hidden = x.shape
    if weight.numel() != hidden:
        raise KernelError("norm_rows: the weight must be as wide as a row")
    status = lib.ei_norm_rows(_gpu(x, "x", torch.float32), _gpu(weight, "weight", torch.float32),
                              float(eps), rows, hidden, _stream())
    _check(lib, status, "norm_rows")


def gate_rows(gate: torch.Tensor, first_column: int, out: torch.Tensor) -> None:
    """out [n, w] *= sigmoid(gate[:, first_column : first_column + w]) for gate [n, g] in out's
    type or float32, or float32 slices [s, n, g] (summed first)."""
    lib = library("rowwise")
    n, width = out.shape
    stride = gate.shape[-1]
    nsplit, split_stride = _splits(gate, n, stride, "gate")
    if not 0 <= first_column <= stride - width:
        raise KernelError("gate_rows: the gate's columns lie outside its rows")
    status = lib.ei_gate_rows(_gpu(gate, "gate"), _code(gate, "gate"), nsplit, split_stride,
                              stride, int(first_column), _gpu(out, "out"), _code(out, "out"), n,
                              width, _stream())
    _check(lib, status, "gate_rows")


def scale_cap(x: torch.Tensor, scale: float, cap: Optional[float]) -> None:
    """x (float32) <- cap tanh(scale x / cap), or scale x without a cap, in place."""
    lib = library("rowwise")
    status = lib.ei_scale_cap(_gpu(x, "x", torch.float32), float(scale), float(cap or 0.0),
                              x.numel(), _stream())
    _check(lib, status, "scale_cap")


def sum_slices(slices: torch.Tensor, out: torch.Tensor) -> None:
    """out = slices.sum(0) for float32 [s, ...] in slice order."""
    lib = library("rowwise")
    n = out.numel()
    if slices.dim() < 2 or slices[0].numel() != n:
        raise KernelError("sum_slices: out must have the shape of one slice")
    status = lib.ei_sum_slices(_gpu(slices, "slices", torch.float32), slices.shape[0], n,
                               _gpu(out, "out", torch.float32), n, _stream())
    _check(lib, status, "sum_slices")


def bias_rows(bias: torch.Tensor, out: torch.Tensor, accumulate: bool) -> None:
    """out[r, :] = bias (accumulate False) or out[r, :] + bias, float32 [rows, width]."""
    lib = library("rowwise")
    if out.dim() != 2 or bias.numel() != out.shape[1]:
        raise KernelError(f"bias_rows: bias of {bias.numel()} for rows {list(out.shape)}")
    status = lib.ei_bias_rows(_gpu(bias, "bias", torch.float32), _gpu(out, "out", torch.float32),
                              out.shape[0], out.shape[1], int(accumulate), _stream())
    _check(lib, status, "bias_rows")


def _row_bias(bias, hidden, what):
    if bias is None:
        return None
    if bias.numel() != hidden:
        raise KernelError(f"{what}: the bias must have {hidden} elements")
    return _gpu(bias, "bias", torch.float32)


def norm_add(residual: torch.Tensor, delta: torch.Tensor, weight: torch.Tensor, eps: float,
             cast_out: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None) -> None:
    """residual [R, H] float32 += rmsnorm(sum of delta's slices (+ bias [H])) * weight;
    `cast_out` [R, H] (optional) receives the new residual rows in its own type."""
    lib = library("rowwise")
    rows, hidden = residual.shape
    nsplit, stride = _splits(delta, rows, hidden, "delta")
    if weight.numel() != hidden:
        raise KernelError(f"norm_add: weight must have {hidden} elements")
    if cast_out is not None and tuple(cast_out.shape) != (rows, hidden):
        raise KernelError("norm_add: cast_out must have the residual's shape")
    status = lib.ei_norm_add(_gpu(residual, "residual", torch.float32), _gpu(delta, "delta"),
                             _code(delta, "delta"), nsplit, stride,
                             _gpu(weight, "weight", torch.float32), float(eps),
                             None if cast_out is None else _gpu(cast_out, "cast_out"),
                             F32 if cast_out is None else _code(cast_out, "cast_out"), rows, hidden,
                             _row_bias(bias, hidden, "norm_add"), _stream())
    _check(lib, status, "norm_add")


def norm_add_norm(residual: torch.Tensor, delta: torch.Tensor, w_after: torch.Tensor,
                  w_next: torch.Tensor, eps: float, out: torch.Tensor,
                  bias: Optional[torch.Tensor] = None) -> None:
    """residual [R, H] float32 += rmsnorm(sum of delta's slices (+ bias [H])) * w_after, then
    out [R, H] = rmsnorm(residual) * w_next in out's type: one pass over the rows."""
    lib = library("rowwise")
    rows, hidden = residual.shape
    nsplit, stride = _splits(delta, rows, hidden, "delta")
    if w_after.numel() != hidden or w_next.numel() != hidden:
        raise KernelError(f"norm_add_norm: weights must have {hidden} elements")
    if tuple(out.shape) != (rows, hidden):
        raise KernelError("norm_add_norm: out must have the residual's shape")
    status = lib.ei_norm_add_norm(_gpu(residual, "residual", torch.float32), _gpu(delta, "delta"),
                                  _code(delta, "delta"), nsplit, stride,
                                  _gpu(w_after, "w_after", torch.float32),
                                  _gpu(w_next, "w_next", torch.float32), float(eps),
                                  _gpu(out, "out"), _code(out, "out"), rows, hidden,
                                  _row_bias(bias, hidden, "norm_add_norm"), _stream())
    _check(lib, status, "norm_add_norm")


def concat_cast(a: torch.Tensor, b: torch.Tensor, out: torch.Tensor) -> None:
    """out [R, 2H] = [a | b] for float32 a, b [R, H], in out's type."""
    lib = library("rowwise")
    rows, hidden = a.shape
    if tuple(b.shape) != (rows, hidden) or tuple(out.shape) != (rows, 2 * hidden):
        raise KernelError("concat_cast: a and b must be [rows, H] and out [rows, 2 H]")
    status = lib.ei_concat_cast(_gpu(a, "a", torch.float32), _gpu(b, "b", torch.float32),
                                _gpu(out, "out"), _code(out, "out"), rows, hidden, _stream())
    _check(lib, status, "concat_cast")


def set_rows(x: torch.Tensor, out: torch.Tensor, vector: Optional[torch.Tensor] = None) -> None:
    """out [R, H] float32 = sum of x's slices (+ vector [H]): a product's result becomes the
    float32 stream."""
    lib = library("rowwise")
    rows, hidden = out.shape
    nsplit, stride = _splits(x, rows, hidden, "x")
    if vector is not None and vector.numel() != hidden:
        raise KernelError(f"set_rows: the vector must have {hidden} elements")
    status = lib.ei_set_rows(_gpu(x, "x"), _code(x, "x"), nsplit, stride,
                             None if vector is None else _gpu(vector, "vector", torch.float32),
                             _gpu(out, "out", torch.float32), rows, hidden, _stream())
    _check(lib, status, "set_rows")


def cast_rows(source: torch.Tensor, out: torch.Tensor) -> None:
    """out = source (float32) in out's type, elementwise."""
    lib = library("rowwise")
    if source.numel() != out.numel():
        raise KernelError("cast_rows: sizes differ")
    status = lib.ei_cast_rows(_gpu(source, "source", torch.float32), _gpu(out, "out"),
                              _code(out, "out"), source.numel(), _stream())
    _check(lib, status, "cast_rows")


ACTIVATIONS = {"relu2": 0, "relu": 1, "silu": 2, "gelu_tanh": 3}


def activation(x: torch.Tensor, out: torch.Tensor, kind: str) -> None:
    """out [n, w] = act(x) for x [n, w] or float32 slices [s, n, w] (summed first); kind:
    "relu2" (relu squared), "relu", "silu", "gelu_tanh"."""
    lib = library("rowwise")
    n, width = out.shape
    nsplit, stride = _splits(x, n, width, "x")
    if kind not in ACTIVATIONS:
        raise KernelError(f"activation: unknown kind '{kind}'; known: {sorted(ACTIVATIONS)}")
    status = lib.ei_activation(_gpu(x, "x"), _code(x, "x"), nsplit, stride, _gpu(out, "out"),
                               _code(out, "out"), out.numel(), ACTIVATIONS[kind], _stream())
    _check(lib, status, "activation")


def _rotated_width(rope_table, head_dim: int, what: str) -> int:
    """The width of a rotation table [positions, R]: R/2 cosines, then R/2 sines, for the
    pairs (i, i + R/2) of a head's first R <= head_dim elements; the rest pass unrotated."""
    if rope_table is None:
        return head_dim
    if rope_table.dim() != 2 or rope_table.shape[1] % 2 or not 2 <= rope_table.shape[1] <= head_dim:
        raise KernelError(f"{what}: the rotation table must be [positions, R] with R even and at "
                          f"most head_dim = {head_dim}, got {list(rope_table.shape)}")
    return rope_table.shape[1]


def qk_norm_rope_store(qkv, q_norm_w, k_norm_w, eps, rope_table, row_pos, row_seq, page_table,
                       q_out, k_pages, v_pages, n_heads, n_kv_heads, head_dim,
                       write_cache=True) -> None:
    """Per-head RMSNorm of queries and keys (weights or None), rotation by `rope_table`
    (float32 [positions, R], R <= head_dim; or None), queries to `q_out`, keys and values to
    their cache pages."""
    lib = library("rope_store")
    n = q_out.shape[0]
    width = (n_heads + 2 * n_kv_heads) * head_dim
    nsplit, stride = _splits(qkv, n, width, "qkv")
    if tuple(q_out.shape) != (n, n_heads * head_dim):
        raise KernelError("qk_norm_rope_store: q_out has the wrong shape")
    if row_pos.numel() < n or row_seq.numel() < n:
        raise KernelError("qk_norm_rope_store: row metadata shorter than the rows")
    rot_dim = _rotated_width(rope_table, head_dim, "qk_norm_rope_store")
    if write_cache:
        expect = (n_kv_heads, PAGE_TOKENS, head_dim)
        if tuple(k_pages.shape[1:]) != expect or tuple(v_pages.shape) != tuple(k_pages.shape):
            raise KernelError(f"qk_norm_rope_store: pages must be [*, {expect}]")
        if k_pages.dtype != q_out.dtype or v_pages.dtype != q_out.dtype:
            raise KernelError("qk_norm_rope_store: cache and q_out dtypes differ")
    status = lib.ei_qk_norm_rope_store(
        _gpu(qkv, "qkv"), _code(qkv, "qkv"), nsplit, stride,
        None if q_norm_w is None else _gpu(q_norm_w, "q_norm", torch.float32),
        None if k_norm_w is None else _gpu(k_norm_w, "k_norm", torch.float32), float(eps),
        None if rope_table is None else _gpu(rope_table, "rope_table", torch.float32), rot_dim,
        _gpu(row_pos, "row_pos", torch.int32), _gpu(row_seq, "row_seq", torch.int32),
        _gpu(page_table, "page_table", torch.int32), page_table.shape[-1],
        _gpu(q_out, "q_out"), _gpu(k_pages, "k_pages") if write_cache else None,
        _gpu(v_pages, "v_pages") if write_cache else None, _code(q_out, "q_out"), n, n_heads,
        n_kv_heads, head_dim, int(write_cache), _stream())
    _check(lib, status, "qk_norm_rope_store")


def attention_heads_per_block(group: int) -> int:
    return library("attention_generic").ei_attn_heads_per_block(group)


def attention_positions_per_item(group: int) -> int:
    return library("attention_generic").ei_attn_positions_per_item(group)


def attention(q, k_pages, v_pages, item_seq, item_row0, item_npos, n_items, row_pos, row_seq,
              page_table, out, n_heads, n_kv_heads, head_dim, window=None, scale=None,
              n_splits=1, part_o=None, part_ml=None, value_dim=None, chunk=None, slopes=None,
              sinks=None, key_heads=1, values_in_keys=False, gate=None, pool=None,
              pool_k=None, pool_v=None, pool_table=None, pool_only=False) -> None:
    """Generic causal attention over the paged cache (see attention_generic.hip).
    value_dim: head size of the values and of `out` (None: head_dim); chunk: a query sees only
    the keys of its own block of that many positions; slopes, sinks: float32 [n_heads], the
    distance term's slope and the softmax's sink of every query head (None: none).
    key_heads: 1, or n_kv_heads: a query row is then n_kv_heads * head_dim wide and meets the
    keys of all kv heads of a position laid end to end (scores mixed over heads: see
    `mix_heads`).  values_in_keys: the values are the first value_dim elements of the key
    rows and `v_pages` is not read.  gate: float32 [rows, heads]; the output of a row and
    head is multiplied by sigmoid(gate).  pool: P (needs a window): a query also sees the
    entries of the pooled cache (`pool_k`, `pool_v`: pages shaped like the tokens' pages, found
    through `pool_table`) whose blocks of P positions lie wholly before its window.
    pool_only: the tokens are left out; `out` is not written, and part_o [rows, heads,
    value_dim] and part_ml [rows, heads, 2] receive every row's unnormalised sums over the
    pooled entries, the largest score and the sum of weights (n_splits 1)."""
    lib = library("attention_generic")
    n = q.shape[0]
    value_dim = head_dim if value_dim is None else int(value_dim)
    key_heads = int(key_heads)
    if key_heads not in (1, n_kv_heads):
        raise KernelError("attention: key_heads must be 1 or the number of kv heads")
    if tuple(q.shape) != (n, n_heads * key_heads * head_dim) or \
            tuple(out.shape) != (n, n_heads * value_dim):
        raise KernelError("attention: q must be [rows, heads * key_heads * head_dim] and out "
                          "[rows, heads * value_dim]")
    expect = (n_kv_heads, PAGE_TOKENS, head_dim)
    expect_v = (k_pages.shape[0], n_kv_heads, PAGE_TOKENS, value_dim)
    if tuple(k_pages.shape[1:]) != expect:
        raise KernelError(f"attention: key pages must be [*, {expect}]")
    if values_in_keys:
        if value_dim > head_dim:
            raise KernelError("attention: values inside the keys cannot be wider than the keys")
        v_pages = k_pages
    elif tuple(v_pages.shape) != expect_v:
        raise KernelError(f"attention: value pages must be {list(expect_v)}")
    if not (q.dtype == k_pages.dtype == v_pages.dtype == out.dtype):
        raise KernelError("attention: q, cache and out dtypes differ")
    if gate is not None and (gate.dtype != torch.float32 or gate.numel() != n * n_heads):
        raise KernelError("attention: the gate must be float32 [rows, heads]")
    if item_seq.numel() < n_items or item_row0.numel() < n_items or item_npos.numel() < n_items:
        raise KernelError("attention: work item arrays shorter than n_items")
    for name, per_head in (("slopes", slopes), ("sinks", sinks)):
        if per_head is not None and per_head.numel() != n_heads:
            raise KernelError(f"attention: {name} must have one value per query head")
    if pool_only and (not pool or n_splits != 1 or gate is not None):
        raise KernelError("attention: the pooled entries alone are taken in one slice")
    if n_splits > 1 or pool_only:
        need_o = n * n_heads * n_splits * value_dim
        if part_o is None or part_ml is None or part_o.numel() < need_o \
                or part_ml.numel() < n * n_heads * n_splits * 2:
            raise KernelError("attention: split scratch missing or too small")
    if pool:
        if not window or pool_k is None or pool_v is None or pool_table is None:
            raise KernelError("attention: pooled blocks need a window and their cache")
        if tuple(pool_k.shape[1:]) != expect or tuple(pool_v.shape[1:]) != expect_v[1:] \
                or pool_k.dtype != q.dtype or pool_v.dtype != q.dtype \
                or pool_table.shape[-1] != page_table.shape[-1]:
            raise KernelError("attention: the pooled cache must be shaped like the tokens'")
    if scale is None:
        scale = head_dim ** -0.5
    status = lib.ei_attention(
        _gpu(q, "q"), _gpu(k_pages, "k_pages"), _gpu(v_pages, "v_pages"), _code(q, "q"),
        _gpu(item_seq, "item_seq", torch.int32), _gpu(item_row0, "item_row0", torch.int32),
        _gpu(item_npos, "item_npos", torch.int32), n_items, _gpu(row_pos, "row_pos", torch.int32),
        _gpu(row_seq, "row_seq", torch.int32), _gpu(page_table, "page_table", torch.int32),
        page_table.shape[-1], _gpu(out, "out"),
        None if part_o is None else _gpu(part_o, "part_o", torch.float32),
        None if part_ml is None else _gpu(part_ml, "part_ml", torch.float32), n, n_heads,
        n_kv_heads, head_dim, value_dim, int(window or 0), int(chunk or 0),
        None if slopes is None else _gpu(slopes, "slopes", torch.float32),
        None if sinks is None else _gpu(sinks, "sinks", torch.float32), float(scale), n_splits,
        key_heads, int(bool(values_in_keys)),
        None if gate is None else _gpu(gate, "gate", torch.float32), int(pool or 0),
        _gpu(pool_k, "pool_k") if pool else None, _gpu(pool_v, "pool_v") if pool else None,
        _gpu(pool_table, "pool_table", torch.int32) if pool else None, int(bool(pool_only)),
        _stream())
    _check(lib, status, "attention")


def pool_store(k_pages, v_pages, row_pos, row_seq, page_table, pool_table, pool_k, pool_v, n_rows,
               pool, row_list=None) -> None:
    """For every row whose position ends a block of `pool` positions: the means of the block's
    cached keys and values (all kv heads) into entry position // pool of the pooled cache.
    row_list (int32, optional): the rows to look at instead of all `n_rows` (-1: skipped)."""
    lib = library("attention_generic")
    n_kv_heads, head_dim, value_dim = k_pages.shape[1], k_pages.shape[3], v_pages.shape[3]
    if tuple(pool_k.shape[1:]) != tuple(k_pages.shape[1:]) or \
            tuple(pool_v.shape[1:]) != tuple(v_pages.shape[1:]) or \
            not (k_pages.dtype == v_pages.dtype == pool_k.dtype == pool_v.dtype) or \
            pool_table.shape[-1] != page_table.shape[-1]:
        raise KernelError("pool_store: the pooled cache must be shaped like the tokens'")
    if row_pos.numel() < n_rows or row_seq.numel() < n_rows or pool < 1:
        raise KernelError("pool_store: row metadata shorter than the rows")
    status = lib.ei_pool_store(
        _gpu(k_pages, "k_pages"), _gpu(v_pages, "v_pages"), _code(k_pages, "k_pages"),
        _gpu(row_pos, "row_pos", torch.int32), _gpu(row_seq, "row_seq", torch.int32),
        _gpu(page_table, "page_table", torch.int32), _gpu(pool_table, "pool_table", torch.int32),
        page_table.shape[-1], _gpu(pool_k, "pool_k"), _gpu(pool_v, "pool_v"), n_rows, n_kv_heads,
        head_dim, value_dim, int(pool),
        None if row_list is None else _gpu(row_list, "row_list", torch.int32),
        0 if row_list is None else row_list.numel(), _stream())
    _check(lib, status, "pool_store")


def attention_wide_supported(dtype, query_width: int, head_dim: int, value_dim: int) -> bool:
    """Whether the matrix-core kernel for wide keys takes these sizes (asked without loading
    its library): bfloat16, query rows (key_heads * head_dim) a multiple of 32 up to 1024, the
    stored key head size a multiple of 8, values a multiple of 16 up to 512."""
    return (dtype == torch.bfloat16 and 32 <= query_width <= 1024 and query_width % 32 == 0
            and head_dim % 8 == 0 and 16 <= value_dim <= 512 and value_dim % 16 == 0)


def attention_wide_positions(group: int) -> int:
    """Positions of one sequence that a work item of `attention_wide` may hold: a block has
    64 query rows, positions x heads of a kv group."""
    return 64 // min(group, 64)


def attention_wide(q, k_pages, v_pages, item_seq, item_row0, item_npos, n_items, row_pos, row_seq,
                   page_table, out, n_heads, n_kv_heads, head_dim, window=None, scale=None,
                   n_splits=1, part_o=None, part_ml=None, value_dim=None, sinks=None, key_heads=1,
                   values_in_keys=False, gate=None) -> None:
    """bfloat16 attention on the matrix cores for wide keys (see attention_wide.hip); arguments
    as `attention`'s."""
    lib = library("attention_wide")
    n = q.shape[0]
    value_dim = head_dim if value_dim is None else int(value_dim)
    key_heads = int(key_heads)
    if key_heads not in (1, n_kv_heads):
        raise KernelError("attention_wide: key_heads must be 1 or the number of kv heads")
    if not attention_wide_supported(q.dtype, key_heads * head_dim, head_dim, value_dim):
        raise KernelError("attention_wide: these head sizes or this type are not supported")
    if tuple(q.shape) != (n, n_heads * key_heads * head_dim) or \
            tuple(out.shape) != (n, n_heads * value_dim):
        raise KernelError("attention_wide: q must be [rows, heads * key_heads * head_dim] and out "
                          "[rows, heads * value_dim]")
    if tuple(k_pages.shape[1:]) != (n_kv_heads, PAGE_TOKENS, head_dim):
        raise KernelError("attention_wide: key pages have the wrong shape")
    if values_in_keys:
        if value_dim > head_dim:
            raise KernelError("attention_wide: values inside the keys cannot be wider than them")
        v_pages = k_pages
    elif tuple(v_pages.shape) != (k_pages.shape[0], n_kv_heads, PAGE_TOKENS, value_dim):
        raise KernelError("attention_wide: value pages have the wrong shape")
    if not (k_pages.dtype == v_pages.dtype == out.dtype == torch.bfloat16):
        raise KernelError("attention_wide: q, cache and out must be bfloat16")
    if item_seq.numel() < n_items or item_row0.numel() < n_items or item_npos.numel() < n_items:
        raise KernelError("attention_wide: work item arrays shorter than n_items")
    if sinks is not None and sinks.numel() != n_heads:
        raise KernelError("attention_wide: sinks must have one value per query head")
    if gate is not None and (gate.dtype != torch.float32 or gate.numel() != n * n_heads):
        raise KernelError("attention_wide: the gate must be float32 [rows, heads]")
    if n_splits > 1:
        if part_o is None or part_ml is None or part_o.numel() < n * n_heads * n_splits * value_dim \
                or part_ml.numel() < n * n_heads * n_splits * 2:
            raise KernelError("attention_wide: split scratch missing or too small")
    if scale is None:
        scale = head_dim ** -0.5
    status = lib.ei_attention_wide(
        _gpu(q, "q"), _gpu(k_pages, "k_pages"), _gpu(v_pages, "v_pages"),
        _gpu(item_seq, "item_seq", torch.int32), _gpu(item_row0, "item_row0", torch.int32),
        _gpu(item_npos, "item_npos", torch.int32), n_items, _gpu(row_pos, "row_pos", torch.int32),
        _gpu(row_seq, "row_seq", torch.int32), _gpu(page_table, "page_table", torch.int32),
        page_table.shape[-1], _gpu(out, "out"),
        None if part_o is None else _gpu(part_o, "part_o", torch.float32),
        None if part_ml is None else _gpu(part_ml, "part_ml", torch.float32), n, n_heads,
        n_kv_heads, head_dim, value_dim, int(window or 0),
        None if sinks is None else _gpu(sinks, "sinks", torch.float32), float(scale), n_splits,
        key_heads, int(bool(values_in_keys)),
        None if gate is None else _gpu(gate, "gate", torch.float32), _stream())
    _check(lib, status, "attention_wide")


# ---------------------------------------------------------------------------
# per-head operations (head_ops.hip)
def _rows_of(x, name):
    """(rows, row width, nsplit, split stride) of [rows, width] or float32 slices of it."""
    if x.dim() == 2:
        return x.shape[0], x.shape[1], 1, 0
    if x.dim() == 3 and x.dtype == torch.float32:
        return x.shape[1], x.shape[2], x.shape[0], x.shape[1] * x.shape[2]
    raise KernelError(f"{name} must be [rows, width] or float32 [slices, rows, width]")


def latent_down_store(proj, q_norm_w, c_norm_w, eps, frequencies, row_pos, row_seq, page_table,
                      q_latent, k_pages, gate_out, q_rank, kv_rank, rot_dim, n_gate,
                      write_cache=True) -> None:
    """One row of a fused down-projection [q_rank | kv_rank | rot_dim | n_gate]: the first two
    parts are RMS-normed with their weights; the queries' latent goes to `q_latent` [rows,
    q_rank], the keys' latent and the rotated last part (neighbouring pairs, angle position *
    frequencies[i]) to the row's cache page `k_pages` [pages, 1, 64, kv_rank + rot_dim], the gate
    logits to `gate_out` float32 [rows, n_gate]."""
    lib = library("head_ops")
    n, width, nsplit, stride = _rows_of(proj, "proj")
    if width != q_rank + kv_rank + rot_dim + n_gate:
        raise KernelError("latent_down_store: the projection's width does not fit its parts")
    if tuple(q_latent.shape) != (n, q_rank):
        raise KernelError("latent_down_store: q_latent must be [rows, q_rank]")
    if q_norm_w.numel() != q_rank or c_norm_w.numel() != kv_rank:
        raise KernelError("latent_down_store: norm weights must be as wide as the latents")
    if rot_dim and (frequencies is None or frequencies.numel() != rot_dim // 2):
        raise KernelError("latent_down_store: one frequency for every rotated pair")
    if n_gate and (gate_out is None or gate_out.numel() < n * n_gate):
        raise KernelError("latent_down_store: gate_out must be float32 [rows, n_gate]")
    if row_pos.numel() < n or row_seq.numel() < n:
        raise KernelError("latent_down_store: row metadata shorter than the rows")
    if write_cache:
        if tuple(k_pages.shape[1:]) != (1, PAGE_TOKENS, kv_rank + rot_dim):
            raise KernelError("latent_down_store: pages must be [*, 1, 64, kv_rank + rot_dim]")
        if k_pages.dtype != q_latent.dtype:
            raise KernelError("latent_down_store: cache and q_latent dtypes differ")
    status = lib.ei_latent_down_store(
        _gpu(proj, "proj"), _code(proj, "proj"), nsplit, stride,
        _gpu(q_norm_w, "q_norm_w", torch.float32), _gpu(c_norm_w, "c_norm_w", torch.float32),
        float(eps), None if frequencies is None else _gpu(frequencies, "frequencies", torch.float32),
        _gpu(row_pos, "row_pos", torch.int32), _gpu(row_seq, "row_seq", torch.int32),
        _gpu(page_table, "page_table", torch.int32), page_table.shape[-1],
        _gpu(q_latent, "q_latent"), _gpu(k_pages, "k_pages") if write_cache else None,
        None if gate_out is None else _gpu(gate_out, "gate_out", torch.float32),
        _code(q_latent, "q_latent"), n, q_rank, kv_rank, rot_dim, n_gate, int(write_cache),
        _stream())
    _check(lib, status, "latent_down_store")


def head_matmul(x, matrices, y, heads, x_head, x_first, y_head, y_first) -> None:
    """y[n, h * y_head + y_first + j] = sum_i x[n, h * x_head + x_first + i] * matrices[h, i, j]
    for matrices [heads, K, J] of the storage type; x [rows, width] or float32 slices of it."""
    lib = library("head_ops")
    n, x_row, nsplit, stride = _rows_of(x, "x")
    if matrices.dim() != 3 or matrices.shape[0] != heads:
        raise KernelError("head_matmul: matrices must be [heads, K, J]")
    if y.dim() != 2 or y.shape[0] != n:
        raise KernelError("head_matmul: y must be [rows, width]")
    _, k, j = matrices.shape
    status = lib.ei_head_matmul(_gpu(x, "x"), _code(x, "x"), nsplit, stride, x_row, int(x_head),
                                int(x_first), _gpu(matrices, "matrices"),
                                _code(matrices, "matrices"), _gpu(y, "y"), _code(y, "y"),
                                y.shape[1], int(y_head), int(y_first), n, heads, k, j, _stream())
    _check(lib, status, "head_matmul")


def rotate_pairs(x, frequencies, row_pos, y, heads, rot_dim, x_head, x_first, y_head,
                 y_first) -> None:
    """Elements (2i, 2i + 1) of x[n, h * x_head + x_first + 0..rot_dim] turn by the angle
    row_pos[n] * frequencies[i] and go to y[n, h * y_head + y_first + ...]."""
    lib = library("head_ops")
    n, x_row, nsplit, stride = _rows_of(x, "x")
    if y.dim() != 2 or y.shape[0] != n:
        raise KernelError("rotate_pairs: y must be [rows, width]")
    if frequencies.numel() != rot_dim // 2 or row_pos.numel() < n:
        raise KernelError("rotate_pairs: one frequency a pair and one position a row")
    status = lib.ei_rotate_pairs(_gpu(x, "x"), _code(x, "x"), nsplit, stride, x_row, int(x_head),
                                 int(x_first), _gpu(frequencies, "frequencies", torch.float32),
                                 _gpu(row_pos, "row_pos", torch.int32), _gpu(y, "y"),
                                 _code(y, "y"), y.shape[1], int(y_head), int(y_first), n, heads,
                                 int(rot_dim), _stream())
    _check(lib, status, "rotate_pairs")


def mix_heads(q, talk, out, heads, kv_heads, head_dim) -> None:
    """out[n, h, c, :] = sum over the heads g of kv head c of talk[h, g] q[n, g, :]: with
    `attention(..., key_heads=kv_heads)` the scores of these rows are the scores of q mixed
    over heads by `talk` [heads, heads] (float32)."""
    lib = library("head_ops")
    n = q.shape[0]
    if tuple(q.shape) != (n, heads * head_dim) or \
            tuple(out.shape) != (n, heads * kv_heads * head_dim) or q.dtype != out.dtype:
        raise KernelError("mix_heads: q must be [rows, heads * head_dim] and out "
                          "[rows, heads * kv_heads * head_dim] of one type")
    if talk.numel() != heads * heads:
        raise KernelError("mix_heads: the mixing matrix must be [heads, heads]")
    status = lib.ei_mix_heads(_gpu(q, "q"), _code(q, "q"), _gpu(talk, "talk", torch.float32),
                              _gpu(out, "out"), n, heads, kv_heads, head_dim, _stream())
    _check(lib, status, "mix_heads")


# ---------------------------------------------------------------------------
# matrix memory (mlstm.hip)
def mlstm_state_floats(heads: int, key_dim: int, value_dim: int) -> int:
    """Floats of one sequence's state: per head S^T [value_dim, key_dim], n [key_dim], m, padded
    to a multiple of 4 (16-byte accesses)."""
    return heads * ((value_dim * key_dim + key_dim + 1 + 3) // 4 * 4)


def mlstm_proj_width(heads: int, key_dim: int, value_dim: int) -> int:
    """Width of the fused projection [q | k | v | i | f | g]."""
    return 2 * heads * key_dim + 2 * heads * value_dim + 2 * heads


def mlstm_walk(proj, i_bias, f_bias, state, seq_in, seq_out, seq_count, seq_row0, o_raw, heads,
               key_dim, value_dim, cap, q_scale, bottom_eps) -> None:
    """The matrix memory's walk over the rows of a step (see mlstm.hip): proj [rows, width] or
    float32 slices; state float32 [table rows, state floats]; o_raw float32 [rows, heads *
    value_dim]."""
    lib = library("mlstm")
    n, width, nsplit, stride = _rows_of(proj, "proj")
    if width != mlstm_proj_width(heads, key_dim, value_dim):
        raise KernelError("mlstm_walk: the projection's width does not fit the shape")
    if state.dim() != 2 or state.shape[1] < mlstm_state_floats(heads, key_dim, value_dim):
        raise KernelError("mlstm_walk: state rows too short")
    n_seqs = seq_count.numel()
    if seq_in.numel() < n_seqs or seq_out.numel() < n_seqs or seq_row0.numel() < n_seqs:
        raise KernelError("mlstm_walk: sequence metadata shorter than the sequences")
    if tuple(o_raw.shape) != (n, heads * value_dim):
        raise KernelError("mlstm_walk: o_raw must be [rows, heads * value_dim]")
    if i_bias.numel() != heads or f_bias.numel() != heads:
        raise KernelError("mlstm_walk: one gate bias a head")
    status = lib.ei_mlstm_walk(
        _gpu(proj, "proj"), _code(proj, "proj"), nsplit, stride,
        _gpu(i_bias, "i_bias", torch.float32), _gpu(f_bias, "f_bias", torch.float32),
        _gpu(state, "state", torch.float32), state.shape[1],
        _gpu(seq_in, "seq_in", torch.int32), _gpu(seq_out, "seq_out", torch.int32),
        _gpu(seq_count, "seq_count", torch.int32), _gpu(seq_row0, "seq_row0", torch.int32),
        _gpu(o_raw, "o_raw", torch.float32), n_seqs, heads, key_dim, value_dim, float(cap),
        float(q_scale), float(bottom_eps), n, _stream())
    _check(lib, status, "mlstm_walk")


def mlstm_out(o_raw, proj, norm_w, eps, row_seq, out, heads, key_dim, value_dim) -> None:
    """out = rmsnorm per head (o_raw) * norm_w [heads * value_dim] * sigmoid(gate columns of
    proj), in out's type."""
    lib = library("mlstm")
    n, width, nsplit, stride = _rows_of(proj, "proj")
    if width != mlstm_proj_width(heads, key_dim, value_dim):
        raise KernelError("mlstm_out: the projection's width does not fit the shape")
    if tuple(o_raw.shape) != (n, heads * value_dim) or tuple(out.shape) != tuple(o_raw.shape):
        raise KernelError("mlstm_out: o_raw and out must be [rows, heads * value_dim]")
    if norm_w.numel() != heads * value_dim or row_seq.numel() < n:
        raise KernelError("mlstm_out: the weight spans all heads; one sequence index a row")
    status = lib.ei_mlstm_out(_gpu(o_raw, "o_raw", torch.float32), _gpu(proj, "proj"),
                              _code(proj, "proj"), nsplit, stride,
                              _gpu(norm_w, "norm_w", torch.float32), float(eps),
                              _gpu(row_seq, "row_seq", torch.int32), _gpu(out, "out"),
                              _code(out, "out"), n, heads, key_dim, value_dim, _stream())
    _check(lib, status, "mlstm_out")


def projection_norm_store(qkv, q_norm_w, k_norm_w, eps, row_pos, row_seq, page_table, q_out,
                          k_pages, v_pages, n_heads, n_kv_heads, head_dim, value_dim,
                          write_cache=True, bias=None) -> None:
    """One RMS norm over the whole query projection and one over the whole key projection
    (weights [heads * head_dim] and [kv heads * head_dim], or None for no norm), no rotation;
    queries to `q_out`, keys [*, kv heads, 64, head_dim] and values [*, kv heads, 64, value_dim]
    to their cache pages.  bias: float32 [q | k | v width], added to the projection first."""
    lib = library("rope_store")
    n = q_out.shape[0]
    width = n_heads * head_dim + n_kv_heads * (head_dim + value_dim)
    if bias is not None and bias.numel() != width:
        raise KernelError("projection_norm_store: the bias must be as wide as the projection")
    nsplit, stride = _splits(qkv, n, width, "qkv")
    if tuple(q_out.shape) != (n, n_heads * head_dim):
        raise KernelError("projection_norm_store: q_out has the wrong shape")
    if row_pos.numel() < n or row_seq.numel() < n:
        raise KernelError("projection_norm_store: row metadata shorter than the rows")
    if (q_norm_w is None) != (k_norm_w is None):
        raise KernelError("projection_norm_store: both norm weights or neither")
    if q_norm_w is not None and (q_norm_w.numel() != n_heads * head_dim
                                 or k_norm_w.numel() != n_kv_heads * head_dim):
        raise KernelError("projection_norm_store: norm weights must be as wide as the projections")
    if write_cache:
        if tuple(k_pages.shape[1:]) != (n_kv_heads, PAGE_TOKENS, head_dim) or \
                tuple(v_pages.shape) != (k_pages.shape[0], n_kv_heads, PAGE_TOKENS, value_dim):
            raise KernelError("projection_norm_store: pages have the wrong shape")
        if k_pages.dtype != q_out.dtype or v_pages.dtype != q_out.dtype:
            raise KernelError("projection_norm_store: cache and q_out dtypes differ")
    status = lib.ei_projection_norm_store(
        _gpu(qkv, "qkv"), _code(qkv, "qkv"), nsplit, stride,
        None if bias is None else _gpu(bias, "bias", torch.float32),
        None if q_norm_w is None else _gpu(q_norm_w, "q_norm", torch.float32),
        None if k_norm_w is None else _gpu(k_norm_w, "k_norm", torch.float32), float(eps),
        _gpu(row_pos, "row_pos", torch.int32), _gpu(row_seq, "row_seq", torch.int32),
        _gpu(page_table, "page_table", torch.int32), page_table.shape[-1], _gpu(q_out, "q_out"),
        _gpu(k_pages, "k_pages") if write_cache else None,
        _gpu(v_pages, "v_pages") if write_cache else None, _code(q_out, "q_out"), n, n_heads,
        n_kv_heads, head_dim, value_dim, int(write_cache), _stream())
    _check(lib, status, "projection_norm_store")


def head_store(proj, q_norm_w, k_norm_w, eps, frequencies, row_pos, row_seq, page_table, q_out,
               k_pages, v_pages, n_heads, n_kv_heads, head_dim, value_dim, write_cache=True,
               v_first=None, v_mode=0, v_lambda=None, query_temperature=None, gate_out=None,
               gate_column=0) -> None:
    """(query_temperature (coef, every): a query at position p is multiplied by
    1 + coef ln(floor((p + 1) / every) + 1); gate_out float32 [n, heads]: receives the rows'
    columns gate_column .. gate_column + heads - 1, summed over slices; n_kv_heads 0: the rows
    hold queries only and the cache is not written.)
    Rows that begin with [q | k | v] (and may go on with other columns), as [n, g] or float32
    slices [s, n, g]: per-head RMS norm of queries and keys (weights [head_dim], or None), the
    rotation of every head's first R elements in pairs (i, i + R/2) by position *
    frequencies[i] (float64 [R/2], or None for no rotation), queries to `q_out`, keys
    [*, kv heads, 64, head_dim] and values [*, kv heads, 64, value_dim] to their pages.
    v_mode 1: the values are also written to `v_first` (float32 [n, kv heads * value_dim]);
    v_mode 2: what is stored is (1 - lambda) v + lambda v_first, `v_lambda` one float32 on the
    device."""
    lib = library("rope_store")
    n = q_out.shape[0]
    stride = proj.shape[-1]
    nsplit, split_stride = _splits(proj, n, stride, "proj")
    if stride < n_heads * head_dim + n_kv_heads * (head_dim + value_dim):
        raise KernelError("head_store: the rows are narrower than the projections")
    if tuple(q_out.shape) != (n, n_heads * head_dim):
        raise KernelError("head_store: q_out has the wrong shape")
    if row_pos.numel() < n or row_seq.numel() < n:
        raise KernelError("head_store: row metadata shorter than the rows")
    for weight in (q_norm_w, k_norm_w):
        if weight is not None and weight.numel() != head_dim:
            raise KernelError("head_store: a norm weight must be as wide as a head")
    rot_dim = 0
    if frequencies is not None:
        rot_dim = 2 * frequencies.numel()
        if frequencies.dim() != 1 or not 2 <= rot_dim <= head_dim:
            raise KernelError("head_store: the frequencies must be [R/2] with R at most head_dim")
    if write_cache:
        if tuple(k_pages.shape[1:]) != (n_kv_heads, PAGE_TOKENS, head_dim) or \
                tuple(v_pages.shape) != (k_pages.shape[0], n_kv_heads, PAGE_TOKENS, value_dim):
            raise KernelError("head_store: pages have the wrong shape")
        if k_pages.dtype != q_out.dtype or v_pages.dtype != q_out.dtype:
            raise KernelError("head_store: cache and q_out dtypes differ")
    if v_mode not in (0, 1, 2):
        raise KernelError("head_store: v_mode must be 0, 1 or 2")
    if v_mode and (v_first is None or tuple(v_first.shape) != (n, n_kv_heads * value_dim)):
        raise KernelError("head_store: v_first must be float32 [rows, kv heads * value_dim]")
    if v_mode == 2 and (v_lambda is None or v_lambda.numel() != 1):
        raise KernelError("head_store: mixing values needs its one weight")
    temp = (0.0, 0) if query_temperature is None else query_temperature
    if temp[1] < 0:
        raise KernelError("head_store: the temperature's step must be positive")
    if gate_out is not None and (tuple(gate_out.shape) != (n, n_heads)
                                 or stride < gate_column + n_heads):
        raise KernelError("head_store: gate_out must be [rows, heads] and the rows hold its columns")
    if n_kv_heads == 0 and write_cache:
        raise KernelError("head_store: rows without keys cannot write the cache")
    status = lib.ei_head_store(
        _gpu(proj, "proj"), _code(proj, "proj"), nsplit, split_stride, stride,
        None if q_norm_w is None else _gpu(q_norm_w, "q_norm", torch.float32),
        None if k_norm_w is None else _gpu(k_norm_w, "k_norm", torch.float32), float(eps),
        None if frequencies is None else _gpu(frequencies, "frequencies", torch.float64), rot_dim,
        _gpu(row_pos, "row_pos", torch.int32), _gpu(row_seq, "row_seq", torch.int32),
        _gpu(page_table, "page_table", torch.int32), page_table.shape[-1], _gpu(q_out, "q_out"),
        _gpu(k_pages, "k_pages") if write_cache else None,
        _gpu(v_pages, "v_pages") if write_cache else None, _code(q_out, "q_out"),
        None if not v_mode else _gpu(v_first, "v_first", torch.float32), int(v_mode),
        None if v_mode != 2 else _gpu(v_lambda, "v_lambda", torch.float32), n, n_heads,
        n_kv_heads, head_dim, value_dim, int(write_cache), float(temp[0]), int(temp[1]),
        None if gate_out is None else _gpu(gate_out, "gate_out", torch.float32), int(gate_column),
        _stream())
    _check(lib, status, "head_store")


MFMA_HEAD_DIMS = (64, 128)


def attention_decode_mfma_supported(head_dim: int, group: int) -> bool:
    """Whether the matrix-core attention kernels take this head size (asked without
    loading their library, so that models which do not need it never compile it)."""
    return head_dim in MFMA_HEAD_DIMS and group >= 1


def attention_prefill_mfma_heads(group: int) -> int:
    """Query heads of a kv group that one block of the matrix-core prefill kernel takes: the
    largest of 4, 2, 1 that divides the group."""
    return 4 if group % 4 == 0 else (2 if group % 2 == 0 else 1)


def attention_prefill_mfma_positions(group: int, key_ways: int = 1) -> int:
    """Positions of a sequence per work item of the matrix-core prefill kernel: a block of 8
    waves holds 4, 2 or 1 heads of a kv group, each wave 32 positions of one head; with
    `key_ways` = 2 two waves share the keys of every page for the same positions, so an item
    is half as long (0: the group has no such form)."""
    heads = attention_prefill_mfma_heads(group)
    if key_ways not in (1, 2) or heads * key_ways > 8:
        return 0
    return 32 * (8 // (heads * key_ways))


def attention_prefill_mfma(q, k_pages, v_pages, item_seq, item_row0, item_npos, n_items, row_pos,
                           page_table, out, n_heads, n_kv_heads, head_dim, window=None,
                           scale=None, key_ways=1, pair_items=True, largest_item=None,
                           chunk=None, slopes=None, sinks=None, pool_o=None, pool_ml=None,
                           gate=None) -> None:
    """bfloat16 prefill attention on the matrix cores; an item holds up to
    `attention_prefill_mfma_positions(group, key_ways)` positions of one sequence.
    pair_items: with enough items a block may take item i and then item n_items - 1 - i
    (equal work a block where the items are those of one prompt, longest first).
    largest_item: the most positions any item holds, from the host's copy of the list (the
    kernel gives a block's waves fixed rows of an item and would leave the rows of a larger
    one out); None: looked up from `item_npos` on the device, which waits for the device.
    chunk, slopes, sinks: as for `attention` (any of them takes the kernel's extended form)."""
    lib = library("attention_mfma")
    n = q.shape[0]
    capacity = attention_prefill_mfma_positions(n_heads // max(1, n_kv_heads), key_ways)
    if capacity == 0:
        raise KernelError(f"attention_prefill: no form with key_ways = {key_ways} for groups of "
                          f"{n_heads // max(1, n_kv_heads)} heads")
    if largest_item is None:
        largest_item = int(item_npos[:n_items].max().item())
    if not 0 <= int(largest_item) <= capacity:
        raise KernelError(f"attention_prefill: an item of {largest_item} positions; a block "
                          f"takes at most {capacity} with key_ways = {key_ways}")
    if tuple(q.shape) != (n, n_heads * head_dim) or tuple(out.shape) != tuple(q.shape):
        raise KernelError("attention_prefill: q and out must be [rows, heads * head_dim]")
    expect = (n_kv_heads, PAGE_TOKENS, head_dim)
    if tuple(k_pages.shape[1:]) != expect or tuple(v_pages.shape) != tuple(k_pages.shape):
        raise KernelError(f"attention_prefill: pages must be [*, {expect}]")
    if item_seq.numel() < n_items or item_row0.numel() < n_items or item_npos.numel() < n_items:
        raise KernelError("attention_prefill: work item arrays shorter than n_items")
    if scale is None:
        scale = head_dim ** -0.5
    common = (
        _gpu(q, "q", torch.bfloat16), _gpu(k_pages, "k_pages", torch.bfloat16),
        _gpu(v_pages, "v_pages", torch.bfloat16), _gpu(item_seq, "item_seq", torch.int32),
        _gpu(item_row0, "item_row0", torch.int32), _gpu(item_npos, "item_npos", torch.int32),
        n_items, _gpu(row_pos, "row_pos", torch.int32),
        _gpu(page_table, "page_table", torch.int32), page_table.shape[-1],
        _gpu(out, "out", torch.bfloat16), n_heads, n_kv_heads, head_dim, int(window or 0),
        float(scale), int(key_ways), int(bool(pair_items)))
    if chunk or slopes is not None or sinks is not None or pool_o is not None or gate is not None:
        status = lib.ei_attention_prefill_mfma_ext(*common, *_attention_extras(
            chunk, slopes, sinks, n_heads, n, head_dim, pool_o, pool_ml, gate), _stream())
    else:
        status = lib.ei_attention_prefill_mfma(*common, _stream())
    _check(lib, status, "attention_prefill")


def _attention_extras(chunk, slopes, sinks, n_heads, rows=0, head_dim=0, pool_o=None,
                      pool_ml=None, gate=None):
    """(chunk, slopes, sinks, pool_o, pool_ml, gate pointers) for the extended forms of the
    matrix-core kernels.  pool_o float32 [rows * heads * head_dim] and pool_ml [rows * heads *
    2]: what `attention(..., pool_only=True)` left for every row and head, taken in as one more
    slice of the softmax; gate float32 [rows, heads]: the output is multiplied by its sigmoid."""
    for name, per_head in (("slopes", slopes), ("sinks", sinks)):
        if per_head is not None and per_head.numel() != n_heads:
            raise KernelError(f"attention: {name} must have one value per query head")
    if (pool_o is None) != (pool_ml is None):
        raise KernelError("attention: the pooled sums and their weights come together")
    if pool_o is not None and (pool_o.numel() < rows * n_heads * head_dim
                               or pool_ml.numel() < rows * n_heads * 2):
        raise KernelError("attention: the pooled sums are too small for these rows")
    if gate is not None and gate.numel() < rows * n_heads:
        raise KernelError("attention: the gate must be float32 [rows, heads]")

    def f32(tensor, name):
        return None if tensor is None else _gpu(tensor, name, torch.float32)
    return (int(chunk or 0), f32(slopes, "slopes"), f32(sinks, "sinks"), f32(pool_o, "pool_o"),
            f32(pool_ml, "pool_ml"), f32(gate, "gate"))


class DecodeProjection:
    """What `attention_decode_mfma` needs to make queries, key and value itself: the fused
    projection as float32 partial sums [slices, rows, (heads + 2 kv heads) * head_dim], the
    per-head RMSNorm weights (float32 [head_dim], or None), their eps, the rotation table
    (float32 [positions, R] with R <= head_dim, or None), and whether the position's key and value are
    stored in the pages."""

    def __init__(self, qkv, q_norm_w, k_norm_w, eps, rope_table, write_cache):
        self.qkv, self.q_norm_w, self.k_norm_w = qkv, q_norm_w, k_norm_w
        self.eps, self.rope_table, self.write_cache = eps, rope_table, write_cache


def attention_decode_mfma(q, k_pages, v_pages, row_pos, row_seq, page_table, out, n_heads,
                          n_kv_heads, head_dim, window=None, scale=None, n_splits=1, part_o=None,
                          part_ml=None, waves=4, longest=None, heads=0, chunk=None, slopes=None,
                          sinks=None, pool_o=None, pool_ml=None, gate=None) -> None:
    """bfloat16 decode attention on the matrix cores: one query row per sequence.  `waves`
    (4, 8 or 16) of a block share its key range tile by tile; more suit fewer sequences (few
    blocks), whose ranges then need fewer slices or none.  `heads` (a power of two, or 0 for
    as many as the block size allows): query heads of a kv group that one block takes; fewer
    give more, lighter blocks.  `longest` (int32 [1] on the
    device): the most tokens a sequence of the step holds; every sequence's range is then
    cut into slices of the longest one's share, so that unequal lengths give equal blocks.
    `q` is the queries [rows, heads * head_dim], or a `DecodeProjection`: the kernel then does
    the work of `qk_norm_rope_store` for its rows as well.  chunk, slopes, sinks: as for
    `attention` (any of them takes the kernel's extended form, which the fused one lacks)."""
    lib = library("attention_mfma")
    n = out.shape[0]
    fused = isinstance(q, DecodeProjection)
    extended = (bool(chunk) or slopes is not None or sinks is not None or pool_o is not None
                or gate is not None)
    if (pool_o is not None or gate is not None) and n_splits < 2:
        raise KernelError("attention_decode: pooled sums and the gate are taken in by the merge "
                          "of at least two slices")
    if fused and extended:
        raise KernelError("attention_decode: the fused projection has no extended form")
    if tuple(out.shape) != (n, n_heads * head_dim) or (not fused and tuple(q.shape) != tuple(out.shape)):
        raise KernelError("attention_decode: q and out must be [rows, heads * head_dim]")
    if fused:
        width = (n_heads + 2 * n_kv_heads) * head_dim
        if q.qkv.dim() != 3 or tuple(q.qkv.shape[1:]) != (n, width):
            raise KernelError(f"attention_decode: the projection must be [slices, {n}, {width}], "
                              f"got {list(q.qkv.shape)}")
        for name in ("q_norm_w", "k_norm_w"):
            weight = getattr(q, name)
            if weight is not None and weight.numel() != head_dim:
                raise KernelError(f"attention_decode: {name} must have {head_dim} elements")
        rot_dim = _rotated_width(q.rope_table, head_dim, "attention_decode")
    expect = (n_kv_heads, PAGE_TOKENS, head_dim)
    if tuple(k_pages.shape[1:]) != expect or tuple(v_pages.shape) != tuple(k_pages.shape):
        raise KernelError(f"attention_decode: pages must be [*, {expect}]")
    if row_pos.numel() < n or row_seq.numel() < n or page_table.shape[0] < n:
        raise KernelError("attention_decode: row metadata shorter than the rows")
    if n_splits > 1:
        if part_o is None or part_ml is None or part_o.numel() < n * n_heads * n_splits * head_dim \
                or part_ml.numel() < n * n_heads * n_splits * 2:
            raise KernelError("attention_decode: split scratch missing or too small")
    if scale is None:
        scale = head_dim ** -0.5
    if fused:
        def opt(tensor, name):
            return None if tensor is None else _gpu(tensor, name, torch.float32)
        status = lib.ei_attention_decode_mfma_fused(
            _gpu(q.qkv, "qkv", torch.float32), q.qkv.shape[0], n * width,
            opt(q.q_norm_w, "q_norm"), opt(q.k_norm_w, "k_norm"), float(q.eps),
            opt(q.rope_table, "rope_table"), rot_dim, int(bool(q.write_cache)),
            _gpu(k_pages, "k_pages", torch.bfloat16), _gpu(v_pages, "v_pages", torch.bfloat16),
            _gpu(row_pos, "row_pos", torch.int32), _gpu(row_seq, "row_seq", torch.int32),
            _gpu(page_table, "page_table", torch.int32), page_table.shape[-1],
            _gpu(out, "out", torch.bfloat16),
            None if part_o is None else _gpu(part_o, "part_o", torch.float32),
            None if part_ml is None else _gpu(part_ml, "part_ml", torch.float32), n, n_heads,
            n_kv_heads, head_dim, int(window or 0), float(scale), n_splits, int(waves),
            int(heads), None if longest is None else _gpu(longest, "longest", torch.int32),
            _stream())
        _check(lib, status, "attention_decode")
        return
    common = (
        _gpu(q, "q", torch.bfloat16), _gpu(k_pages, "k_pages", torch.bfloat16),
        _gpu(v_pages, "v_pages", torch.bfloat16), _gpu(row_pos, "row_pos", torch.int32),
        _gpu(row_seq, "row_seq", torch.int32), _gpu(page_table, "page_table", torch.int32),
        page_table.shape[-1], _gpu(out, "out", torch.bfloat16),
        None if part_o is None else _gpu(part_o, "part_o", torch.float32),
        None if part_ml is None else _gpu(part_ml, "part_ml", torch.float32), n, n_heads,
        n_kv_heads, head_dim, int(window or 0), float(scale), n_splits, int(waves), int(heads),
        None if longest is None else _gpu(longest, "longest", torch.int32))
    if extended:
        status = lib.ei_attention_decode_mfma_ext(*common, *_attention_extras(
            chunk, slopes, sinks, n_heads, q.shape[0], head_dim, pool_o, pool_ml, gate), _stream())
    else:
        status = lib.ei_attention_decode_mfma(*common, _stream())
    _check(lib, status, "attention_decode")


# -- gated delta rule -----------------------------------------------------------------------
def delta_state_floats(n_heads: int, n_kv_heads: int, key_dim: int, value_dim: int,
                       taps: int) -> int:
    """float32 elements of one sequence's state: S^T of every head [heads, value_dim, key_dim],
    then the last taps - 1 inputs of every convolved channel [taps - 1, channels], rounded up
    to a multiple of 4.  (No kernel library is needed to know it.)"""
    channels = 2 * n_kv_heads * key_dim + n_heads * value_dim
    return (n_heads * value_dim * key_dim + (taps - 1) * channels + 3) // 4 * 4


class DeltaShape:
    """Sizes of a gated-delta mixer and where its parts lie in a row of its fused projection
    [q | k | v | beta | decay | gate]."""

    def __init__(self, n_heads, n_kv_heads, key_dim, value_dim, taps):
        self.n_heads, self.n_kv_heads = int(n_heads), int(n_kv_heads)
        self.key_dim, self.value_dim, self.taps = int(key_dim), int(value_dim), int(taps)
        self.qk_width = self.n_kv_heads * self.key_dim
        self.v_width = self.n_heads * self.value_dim
        self.channels = 2 * self.qk_width + self.v_width          # what the convolution covers
        self.beta_col = self.channels
        self.decay_col = self.beta_col + self.n_heads
        self.gate_col = self.decay_col + self.n_heads
        self.width = self.gate_col + self.v_width
        self.tail_offset = self.n_heads * self.value_dim * self.key_dim
        self.state_floats = delta_state_floats(n_heads, n_kv_heads, key_dim, value_dim, taps)


def _delta_proj(proj, rows, shape):
    nsplit, stride = _splits(proj, rows, shape.width, "proj")
    return _gpu(proj, "proj"), _code(proj, "proj"), nsplit, stride


def _delta_state(state, shape):
    if state.dim() != 2 or state.shape[1] != shape.state_floats:
        raise KernelError(f"delta: the state must be [rows, {shape.state_floats}], "
                          f"got {list(state.shape)}")
    return _gpu(state, "state", torch.float32)


def _delta_rows(seq_in, seq_out, n_seqs):
    """A sequence's state is read from row seq_in[s] of the state table and written to row
    seq_out[s] (the same row, or the other of two versions)."""
    if seq_in.numel() < n_seqs or seq_out.numel() < n_seqs:
        raise KernelError("delta: state row lists shorter than the sequences")
    return _gpu(seq_in, "seq_in", torch.int32), _gpu(seq_out, "seq_out", torch.int32)


DELTA_FEW_TAPS = 8      # up to so many taps `delta_conv` can renew the tails itself


def delta_conv(proj, conv_w, state, shape: DeltaShape, row_pos, row_seq, seq_in, seq_out,
               seq_start, out, renew_tail=False) -> None:
    """out [rows, channels] float32 = silu(causal convolution) of the q, k, v columns of
    `proj` ([rows, width] or float32 slices of it); conv_w float32 [channels, taps]; inputs
    from before this step come from the sequences' tails in `state` [rows, state_floats], row
    seq_in[s] for sequence s.  renew_tail: every sequence brings exactly one row (the caller vouches for it) and the
    tails become the last taps - 1 inputs here, written to row seq_out[s], so `delta_tail` is
    not needed (at most `DELTA_FEW_TAPS` taps)."""
    lib = library("delta_rule")
    rows = out.shape[0]
    if tuple(out.shape) != (rows, shape.channels) or tuple(conv_w.shape) != (shape.channels, shape.taps):
        raise KernelError("delta_conv: out must be [rows, channels] and conv_w [channels, taps]")
    if row_pos.numel() < rows or row_seq.numel() < rows:
        raise KernelError("delta_conv: row metadata shorter than the rows")
    pointer, code, nsplit, stride = _delta_proj(proj, rows, shape)
    status = lib.ei_delta_conv(pointer, code, nsplit, stride, shape.width,
                               _gpu(conv_w, "conv_w", torch.float32), shape.taps,
                               _delta_state(state, shape), shape.state_floats, shape.tail_offset,
                               _gpu(row_pos, "row_pos", torch.int32),
                               _gpu(row_seq, "row_seq", torch.int32),
                               *_delta_rows(seq_in, seq_out, seq_start.numel()),
                               _gpu(seq_start, "seq_start", torch.int32),
                               _gpu(out, "out", torch.float32), rows, shape.channels,
                               int(bool(renew_tail)), _stream())
    _check(lib, status, "delta_conv")


def delta_tail(proj, state, shape: DeltaShape, rows, seq_in, seq_out, seq_count, seq_row0) -> None:
    """The sequences' tails become the last taps - 1 inputs after this step (of `rows` packed
    rows; sequence s brings seq_count[s] of them from row seq_row0[s] on): read from row
    seq_in[s] of `state` where the step brought fewer, written to row seq_out[s]."""
    if shape.taps < 2:
        return
    lib = library("delta_rule")
    n_seqs = seq_count.numel()
    if seq_row0.numel() < n_seqs:
        raise KernelError("delta_tail: sequence metadata shorter than the sequences")
    pointer, code, nsplit, stride = _delta_proj(proj, rows, shape)
    status = lib.ei_delta_tail(pointer, code, nsplit, stride, shape.width, shape.taps,
                               _delta_state(state, shape), shape.state_floats, shape.tail_offset,
                               *_delta_rows(seq_in, seq_out, n_seqs),
                               _gpu(seq_count, "seq_count", torch.int32),
                               _gpu(seq_row0, "seq_row0", torch.int32), n_seqs, shape.channels,
                               _stream())
    _check(lib, status, "delta_tail")


def delta_rule(conv, proj, a_log, dt_bias, state, shape: DeltaShape, seq_in, seq_out, seq_count,
               seq_row0, o_raw, q_scale: float, unit_eps: float) -> None:
    """The recurrence over every sequence's rows of this step, in order; reads S from row
    seq_in[s] of `state` and writes it to row seq_out[s]; o_raw [rows, heads * value_dim]
    float32 receives S^T q of every row."""
    lib = library("delta_rule")
    rows = conv.shape[0]
    n_seqs = seq_count.numel()
    if tuple(conv.shape) != (rows, shape.channels) or tuple(o_raw.shape) != (rows, shape.v_width):
        raise KernelError("delta_rule: conv must be [rows, channels] and o_raw [rows, heads * value_dim]")
    if a_log.numel() != shape.n_heads or dt_bias.numel() != shape.n_heads:
        raise KernelError("delta_rule: one decay rate and bias per head")
    if seq_row0.numel() < n_seqs:
        raise KernelError("delta_rule: sequence metadata shorter than the sequences")
    pointer, code, nsplit, stride = _delta_proj(proj, rows, shape)
    status = lib.ei_delta_rule(_gpu(conv, "conv", torch.float32), pointer, code, nsplit, stride,
                               shape.width, shape.beta_col, shape.decay_col,
                               _gpu(a_log, "a_log", torch.float32),
                               _gpu(dt_bias, "dt_bias", torch.float32), _delta_state(state, shape),
                               shape.state_floats, *_delta_rows(seq_in, seq_out, n_seqs),
                               _gpu(seq_count, "seq_count", torch.int32),
                               _gpu(seq_row0, "seq_row0", torch.int32),
                               _gpu(o_raw, "o_raw", torch.float32), n_seqs, shape.n_heads,
                               shape.n_kv_heads, shape.key_dim, shape.value_dim, float(q_scale),
                               float(unit_eps), _stream())
    _check(lib, status, "delta_rule")


def delta_out(o_raw, proj, norm_w, eps, shape: DeltaShape, row_seq, out) -> None:
    """out [rows, heads * value_dim] = o / sqrt(mean(o^2) + eps) * norm_w * silu(gate) per head."""
    lib = library("delta_rule")
    rows = o_raw.shape[0]
    if tuple(o_raw.shape) != (rows, shape.v_width) or tuple(out.shape) != tuple(o_raw.shape):
        raise KernelError("delta_out: o_raw and out must be [rows, heads * value_dim]")
    if norm_w.numel() != shape.value_dim:
        raise KernelError("delta_out: the norm weight must have value_dim elements")
    pointer, code, nsplit, stride = _delta_proj(proj, rows, shape)
    status = lib.ei_delta_out(_gpu(o_raw, "o_raw", torch.float32), pointer, code, nsplit, stride,
                              shape.width, shape.gate_col, _gpu(norm_w, "norm_w", torch.float32),
                              float(eps), _gpu(row_seq, "row_seq", torch.int32), _gpu(out, "out"),
                              _code(out, "out"), rows, shape.n_heads, shape.value_dim, _stream())
    _check(lib, status, "delta_out")


# ---------------------------------------------------------------------------
class SsmShape:
    """Sizes of a state-space mixer: heads of `head_dim` columns each, `groups` pairs of B and C
    vectors of `state` elements, `taps` of the convolution.  A projection row is
    [z: inner | x: inner | B: groups * state | C: groups * state | dt: heads]."""

    def __init__(self, heads, groups, head_dim, state, taps):
        self.heads, self.groups, self.head_dim = int(heads), int(groups), int(head_dim)
        self.state, self.taps = int(state), int(taps)
        self.inner = self.heads * self.head_dim
        self.channels = self.inner + 2 * self.groups * self.state      # what is convolved
        self.proj_width = self.inner + self.channels + self.heads
        # S of every head [head][column][row], then the convolution's last taps - 1 inputs
        self.state_floats = self.inner * self.state + (self.taps - 1) * self.channels

    @property
    def sizes(self):
        return (self.heads, self.groups, self.head_dim, self.state, self.taps)


def _ssm_proj(proj, rows, shape):
    if proj.shape[-1] != shape.proj_width:
        raise KernelError(f"ssm: the projection must be {shape.proj_width} wide")
    return _splits(proj, rows, shape.proj_width, "proj")


def _ssm_state(state, shape):
    if state.dim() != 2 or state.shape[1] != shape.state_floats:
        raise KernelError(f"ssm: the state table must be [rows, {shape.state_floats}]")
    return _gpu(state, "state", torch.float32)


def ssm_conv(proj, conv_w, conv_b, state, shape: SsmShape, row_pos, row_seq, seq_in, seq_out,
             seq_start, seq_count, seq_row0, conv) -> None:
    """conv [n, channels] float32 = silu(causal convolution of the x, B and C columns of `proj`
    + bias), earlier inputs taken from the step's rows or the sequence's tail in row
    `seq_in[s]` of `state`; the new tails are written to row `seq_out[s]`."""
    lib = library("ssm")
    n = conv.shape[0]
    nsplit, stride = _ssm_proj(proj, n, shape)
    n_seqs = seq_in.numel()
    if tuple(conv.shape) != (n, shape.channels) or tuple(conv_w.shape) != (shape.channels, shape.taps):
        raise KernelError("ssm_conv: conv or its filters have the wrong shape")
    if conv_b is not None and conv_b.numel() != shape.channels:
        raise KernelError("ssm_conv: the bias must have one value a channel")
    if row_pos.numel() < n or row_seq.numel() < n or min(
            seq_out.numel(), seq_start.numel(), seq_count.numel(), seq_row0.numel()) < n_seqs:
        raise KernelError("ssm_conv: metadata shorter than the step")
    status = lib.ei_ssm_conv(
        _gpu(proj, "proj"), _code(proj, "proj"), nsplit, stride, shape.proj_width,
        _gpu(conv_w, "conv_w", torch.float32),
        None if conv_b is None else _gpu(conv_b, "conv_b", torch.float32),
        _ssm_state(state, shape), state.shape[1], _gpu(row_pos, "row_pos", torch.int32),
        _gpu(row_seq, "row_seq", torch.int32), _gpu(seq_in, "seq_in", torch.int32),
        _gpu(seq_out, "seq_out", torch.int32), _gpu(seq_start, "seq_start", torch.int32),
        _gpu(seq_count, "seq_count", torch.int32), _gpu(seq_row0, "seq_row0", torch.int32),
        _gpu(conv, "conv", torch.float32), n, n_seqs, *shape.sizes, _stream())
    _check(lib, status, "ssm_conv")


def ssm_scan(conv, proj, a_log, dt_bias, d_skip, state, shape: SsmShape, seq_in, seq_out,
             seq_count, seq_row0, y_raw) -> None:
    """The recurrence over every sequence's rows: S <- exp(-exp(a_log) dt) S + dt B x^T from row
    `seq_in[s]` of `state`, y = S^T C + d_skip x to `y_raw` [n, inner] float32, the last S to row
    `seq_out[s]`; dt = softplus(proj's dt column + dt_bias)."""
    lib = library("ssm")
    n = y_raw.shape[0]
    nsplit, stride = _ssm_proj(proj, n, shape)
    n_seqs = seq_in.numel()
    if tuple(conv.shape) != (n, shape.channels) or tuple(y_raw.shape) != (n, shape.inner):
        raise KernelError("ssm_scan: conv or y_raw has the wrong shape")
    for name, per_head in (("a_log", a_log), ("dt_bias", dt_bias), ("d_skip", d_skip)):
        if per_head.numel() != shape.heads:
            raise KernelError(f"ssm_scan: {name} must have one value a head")
    if min(seq_out.numel(), seq_count.numel(), seq_row0.numel()) < n_seqs:
        raise KernelError("ssm_scan: metadata shorter than the step")
    status = lib.ei_ssm_scan(
        _gpu(conv, "conv", torch.float32), _gpu(proj, "proj"), _code(proj, "proj"), nsplit, stride,
        shape.proj_width, _gpu(a_log, "a_log", torch.float32),
        _gpu(dt_bias, "dt_bias", torch.float32), _gpu(d_skip, "d_skip", torch.float32),
        _ssm_state(state, shape), state.shape[1], _gpu(seq_in, "seq_in", torch.int32),
        _gpu(seq_out, "seq_out", torch.int32), _gpu(seq_count, "seq_count", torch.int32),
        _gpu(seq_row0, "seq_row0", torch.int32), _gpu(y_raw, "y_raw", torch.float32), n_seqs,
        *shape.sizes, _stream())
    _check(lib, status, "ssm_scan")


def ssm_out(y_raw, proj, norm_w, eps, shape: SsmShape, parts, row_seq, out) -> None:
    """out [n, inner] = rmsnorm over each of `parts` equal parts of (y_raw * silu(z)) * norm_w,
    z the first `inner` columns of `proj`."""
    lib = library("ssm")
    n = out.shape[0]
    nsplit, stride = _ssm_proj(proj, n, shape)
    if tuple(y_raw.shape) != (n, shape.inner) or tuple(out.shape) != (n, shape.inner):
        raise KernelError("ssm_out: y_raw and out must be [rows, inner]")
    if norm_w.numel() != shape.inner or parts < 1 or shape.inner % parts:
        raise KernelError("ssm_out: the weight must be [inner] and the parts divide it")
    status = lib.ei_ssm_out(_gpu(y_raw, "y_raw", torch.float32), _gpu(proj, "proj"),
                            _code(proj, "proj"), nsplit, stride, shape.proj_width,
                            _gpu(norm_w, "norm_w", torch.float32), float(eps),
                            _gpu(row_seq, "row_seq", torch.int32), _gpu(out, "out"),
                            _code(out, "out"), n, shape.inner, int(parts), _stream())
    _check(lib, status, "ssm_out")


# ---------------------------------------------------------------------------
def stream_norm(residual, delta, out, *, w_after=None, b_after=None, w_next=None, b_next=None,
                eps: float, centred: bool, rows=None, write_residual: bool = True,
                delta_bias=None, conv=None) -> None:
    """One pass over the rows of the float32 stream `residual` [R, H].  With d the sum of
    delta's slices (+ delta_bias [H]): if `w_after` is given, d <- norm(d) * w_after + b_after
    (the norm on a sublayer's output); residual += d (stored back unless told not to); if
    `out` is given, out[i] = norm(residual[rows[i] if rows else i]) * w_next + b_next in out's
    type.  centred: norms with a mean (layer norms; the biases may be None), else RMS norms.
    delta None: nothing is added.  conv = (weight [taps, H] float32, state, part, parts,
    seq_in, seq_out) (a decode step only: row r is sequence r, widths that are multiples of
    4): `out` receives h + conv(h) for the normed rows h, as `input_conv` gives it, and the
    sequences' state moves on by the row."""
    lib = library("norms")
    total_rows, hidden = residual.shape
    n = total_rows if rows is None else rows.numel()
    if out is not None and tuple(out.shape) != (n, hidden):
        raise KernelError(f"stream_norm: out must be [{n}, {hidden}], got {list(out.shape)}")
    if (out is None) != (w_next is None):
        raise KernelError("stream_norm: an output and its norm's weight come together")
    if delta is None and (w_after is not None or delta_bias is not None):
        raise KernelError("stream_norm: a norm on a sublayer's output needs that output")
    for name, vector in (("w_after", w_after), ("b_after", b_after), ("w_next", w_next),
                         ("b_next", b_next), ("delta_bias", delta_bias)):
        if vector is not None and vector.numel() != hidden:
            raise KernelError(f"stream_norm: {name} must have {hidden} elements")
    nsplit, stride, delta_ptr, delta_code = 0, 0, None, F32
    if delta is not None:
        nsplit, stride = _splits(delta, total_rows, hidden, "delta")
        delta_ptr, delta_code = _gpu(delta, "delta"), _code(delta, "delta")

    def f32(vector, name):
        return None if vector is None else _gpu(vector, name, torch.float32)
    conv_args = (None, None, None, None, 0, 0, 0)
    if conv is not None:
        weight, state, part, parts, seq_in, seq_out = conv
        taps = weight.shape[0]
        if out is None or rows is not None or tuple(weight.shape) != (taps, hidden) or hidden % 4:
            raise KernelError("stream_norm: the convolution needs normed rows that are the "
                              "step's sequences and a width that is a multiple of 4")
        if taps > 1 and (state is None or state.shape[1] != parts * (taps - 1) * hidden
                         or seq_in.numel() < n or seq_out.numel() < n):
            raise KernelError("stream_norm: the convolution's state does not fit")
        conv_args = (_gpu(weight, "conv weight", torch.float32),
                     None if taps == 1 else _gpu(state, "state", torch.float32),
                     None if taps == 1 else _gpu(seq_in, "seq_in", torch.int32),
                     None if taps == 1 else _gpu(seq_out, "seq_out", torch.int32), taps,
                     int(part), int(parts))
    status = lib.ei_stream_norm(
        _gpu(residual, "residual", torch.float32), delta_ptr, delta_code, nsplit, stride,
        f32(delta_bias, "delta_bias"), None if rows is None else _gpu(rows, "rows", torch.int32),
        f32(w_after, "w_after"), f32(b_after, "b_after"), f32(w_next, "w_next"),
        f32(b_next, "b_next"), float(eps), int(bool(centred)),
        None if out is None else _gpu(out, "out"), F32 if out is None else _code(out, "out"), n,
        hidden, int(write_residual), *conv_args, _stream())
    _check(lib, status, "stream_norm")


def norm_mean(branches, weights, eps: float, out: torch.Tensor) -> None:
    """out [n, h] float32 = the mean over the branches b of rmsnorm(x_b) * w_b; every x_b is
    [n, h] or float32 slices [s, n, h], of its own type."""
    lib = library("norms")
    rows, hidden = out.shape
    count = len(branches)
    if not 1 <= count <= 4 or len(weights) != count:
        raise KernelError("norm_mean: 1 to 4 branches, each with its weight")
    pointers = (c_void_p * count)()
    weight_pointers = (c_void_p * count)()
    nsplits = (c_int * count)()
    strides = (c_longlong * count)()
    codes = (c_int * count)()
    for index, (x, w) in enumerate(zip(branches, weights)):
        nsplits[index], strides[index] = _splits(x, rows, hidden, "a branch")
        pointers[index] = _gpu(x, "a branch")
        codes[index] = _code(x, "a branch")
        if w.numel() != hidden:
            raise KernelError(f"norm_mean: a weight must have {hidden} elements")
        weight_pointers[index] = _gpu(w, "weight", torch.float32)
    status = lib.ei_norm_mean(pointers, nsplits, strides, codes, weight_pointers, count,
                              float(eps), _gpu(out, "out", torch.float32), rows, hidden, _stream())
    _check(lib, status, "norm_mean")


def input_conv(h, weight, state, part: int, parts: int, row_pos, row_seq, seq_in, seq_out,
               seq_start, seq_count, seq_row0, out) -> None:
    """out [n, w] = h + conv(h): a causal convolution over the rows of every sequence with
    the filter weight [taps, w] (float32, tap by tap), the inputs before the step's rows taken from part
    `part` of the sequence's state row (float32 rows of parts * (taps - 1) * w, two versions:
    `seq_in` names the row read, `seq_out` the row whose part is written anew).  state None
    with one tap."""
    lib = library("input_conv")
    n, width = h.shape
    taps = weight.shape[0]
    n_seqs = seq_count.numel()
    if tuple(weight.shape) != (taps, width) or tuple(out.shape) != (n, width) or out.dtype != h.dtype:
        raise KernelError("input_conv: shapes do not fit")
    if out.data_ptr() == h.data_ptr():
        raise KernelError("input_conv: the result needs a buffer of its own")
    if taps > 1:
        if state is None or state.dim() != 2 or state.shape[1] != parts * (taps - 1) * width:
            raise KernelError("input_conv: state rows must hold parts * (taps - 1) * width floats")
        if seq_in.numel() < n_seqs or seq_out.numel() < n_seqs:
            raise KernelError("input_conv: state rows missing")
    if row_pos.numel() < n or row_seq.numel() < n or seq_start.numel() < n_seqs \
            or seq_row0.numel() < n_seqs:
        raise KernelError("input_conv: row metadata shorter than the rows")
    status = lib.ei_input_conv(
        _gpu(h, "h"), _code(h, "h"), _gpu(weight, "weight", torch.float32),
        None if taps == 1 else _gpu(state, "state", torch.float32), int(part), int(parts), taps,
        _gpu(row_pos, "row_pos", torch.int32), _gpu(row_seq, "row_seq", torch.int32),
        None if taps == 1 else _gpu(seq_in, "seq_in", torch.int32),
        None if taps == 1 else _gpu(seq_out, "seq_out", torch.int32),
        _gpu(seq_start, "seq_start", torch.int32), _gpu(seq_count, "seq_count", torch.int32),
        _gpu(seq_row0, "seq_row0", torch.int32), _gpu(out, "out"), n, width, n_seqs, _stream())
    _check(lib, status, "input_conv")


def la_state_floats(heads: int, key_dim: int, value_dim: int) -> int:
    """float32 elements of one sequence's linear-attention state: S [heads, key_dim, value_dim]."""
    return heads * key_dim * value_dim


def la_activate(proj, act) -> None:
    """act [n, w] float32 = silu of the first w columns of proj's rows ([n, g] or float32 slices
    [s, n, g]): q, k and v of linear attention, activated once for every block of the scan."""
    lib = library("linear_attention")
    n, width = act.shape
    stride = proj.shape[-1]
    nsplit, split_stride = _splits(proj, n, stride, "proj")
    if stride < width:
        raise KernelError("la_activate: the rows are narrower than what is asked of them")
    status = lib.ei_la_activate(_gpu(proj, "proj"), _code(proj, "proj"), nsplit, split_stride,
                                stride, _gpu(act, "act", torch.float32), n, width, _stream())
    _check(lib, status, "la_activate")


def la_scan(proj, decay, state, seq_in, seq_out, seq_count, seq_row0, o_raw, heads, key_dim,
            value_dim, activated: bool = False) -> None:
    """The recurrence of linear attention with a decay per head over the rows of every
    sequence: proj rows [q | k | v | ...] ([n, g] or float32 slices [s, n, g]), silu on all
    three, S_t = decay_h S_(t-1) + k_t v_t^T, o_raw [n, heads * value_dim] float32 = S_t^T q_t.
    state: float32 rows of heads * key_dim * value_dim, two versions (`seq_in`, `seq_out`).
    activated: the rows hold q, k and v as `la_activate` left them, and silu is not taken again."""
    lib = library("linear_attention")
    if activated and proj.dtype != torch.float32:
        raise KernelError("la_scan: activated rows are float32")
    n = o_raw.shape[0]
    stride = proj.shape[-1]
    nsplit, split_stride = _splits(proj, n, stride, "proj")
    n_seqs = seq_count.numel()
    if tuple(o_raw.shape) != (n, heads * value_dim) or decay.numel() != heads:
        raise KernelError("la_scan: shapes do not fit")
    if state.dim() != 2 or state.shape[1] != la_state_floats(heads, key_dim, value_dim):
        raise KernelError("la_scan: state rows must hold heads * key_dim * value_dim floats")
    if stride < heads * (2 * key_dim + value_dim):
        raise KernelError("la_scan: the rows are narrower than q, k and v")
    if seq_in.numel() < n_seqs or seq_out.numel() < n_seqs or seq_row0.numel() < n_seqs:
        raise KernelError("la_scan: sequence metadata shorter than the sequences")
    status = lib.ei_la_scan(
        _gpu(proj, "proj"), _code(proj, "proj"), nsplit, split_stride, stride,
        _gpu(decay, "decay", torch.float32), _gpu(state, "state", torch.float32),
        _gpu(seq_in, "seq_in", torch.int32), _gpu(seq_out, "seq_out", torch.int32),
        _gpu(seq_count, "seq_count", torch.int32), _gpu(seq_row0, "seq_row0", torch.int32),
        _gpu(o_raw, "o_raw", torch.float32), n_seqs, heads, key_dim, value_dim,
        int(bool(activated)), _stream())
    _check(lib, status, "la_scan")


def la_out(o_raw, proj, gate_column: int, norm_w, eps: float, row_seq, out) -> None:
    """out [n, v] = rmsnorm(o_raw) * norm_w * sigmoid(g), g the columns gate_column ..
    gate_column + v - 1 of proj's rows (summed over slices)."""
    lib = library("linear_attention")
    n, width = o_raw.shape
    stride = proj.shape[-1]
    nsplit, split_stride = _splits(proj, n, stride, "proj")
    if tuple(out.shape) != (n, width) or norm_w.numel() != width or stride < gate_column + width:
        raise KernelError("la_out: shapes do not fit")
    status = lib.ei_la_out(
        _gpu(o_raw, "o_raw", torch.float32), _gpu(proj, "proj"), _code(proj, "proj"), nsplit,
        split_stride, stride, int(gate_column), _gpu(norm_w, "norm_w", torch.float32), float(eps),
        None if row_seq is None else _gpu(row_seq, "row_seq", torch.int32), _gpu(out, "out"),
        _code(out, "out"), n, width, _stream())
    _check(lib, status, "la_out")


ROUTER_SCORINGS = {"softmax_chosen": 0, "softmax_all": 1}


def moe_route(x, router_w, row_seq, expert, weight, scoring: str = "softmax_chosen",
              correction=None) -> None:
    """For every row of x [n, w]: the `top` experts of largest float32 logit router_w [E, w] . x
    into `expert` (int32 [n, top], largest first), the softmax over their logits into `weight`
    (float32 [n, top]).  Rows with row_seq < 0 get weights of 0.  scoring "softmax_all": the
    scores are the softmax over all E logits, the choice is by score + correction [E] (None:
    by the score), and the weights are the chosen scores themselves."""
    lib = library("moe")
    if scoring not in ROUTER_SCORINGS:
        raise KernelError(f"moe_route: unknown scoring '{scoring}'")
    if correction is not None and (scoring != "softmax_all" or correction.numel() != router_w.shape[0]):
        raise KernelError("moe_route: a correction belongs to the scoring 'softmax_all' and has "
                          "one number a router output")
    n, width = x.shape
    n_experts = router_w.shape[0]
    top = expert.shape[1]
    if tuple(router_w.shape) != (n_experts, width) or tuple(expert.shape) != (n, top) \
            or tuple(weight.shape) != (n, top):
        raise KernelError("moe_route: shapes do not fit")
    if row_seq is not None and row_seq.numel() < n:
        raise KernelError("moe_route: row metadata shorter than the rows")
    status = lib.ei_moe_route(_gpu(x, "x"), _code(x, "x"), _gpu(router_w, "router_w", torch.float32),
                              None if row_seq is None else _gpu(row_seq, "row_seq", torch.int32),
                              _gpu(expert, "expert", torch.int32),
                              _gpu(weight, "weight", torch.float32), n, width, n_experts, top,
                              ROUTER_SCORINGS[scoring],
                              None if correction is None else _gpu(correction, "correction", torch.float32),
                              _stream())
    _check(lib, status, "moe_route")


def moe_experts(x, w_gate, w_up, w_down, expert, weight, act, out) -> None:
    """out [n, w] float32 = sum over a row's choices k of weight[r, k] *
    w_down[e] (silu(w_gate[e] x_r) * (w_up[e] x_r)), e = expert[r, k]; w_gate and w_up
    [E, f, w], w_down [E, w, f], all of x's type; `act` [n * top, f] of that type is scratch.
    A choice e >= E is an identity expert: it adds weight[r, k] * x_r."""
    lib = library("moe")
    n, width = x.shape
    n_experts, inter = w_gate.shape[0], w_gate.shape[1]
    top = expert.shape[1]
    if tuple(w_gate.shape) != (n_experts, inter, width) or tuple(w_up.shape) != tuple(w_gate.shape) \
            or tuple(w_down.shape) != (n_experts, width, inter):
        raise KernelError("moe_experts: the stacked matrices have the wrong shapes")
    if tuple(expert.shape) != (n, top) or tuple(weight.shape) != (n, top) \
            or tuple(act.shape) != (n * top, inter) or tuple(out.shape) != (n, width):
        raise KernelError("moe_experts: shapes do not fit")
    if not (x.dtype == w_gate.dtype == w_up.dtype == w_down.dtype == act.dtype):
        raise KernelError("moe_experts: x, the matrices and act must have one type")
    status = lib.ei_moe_experts(_gpu(x, "x"), _gpu(w_gate, "w_gate"), _gpu(w_up, "w_up"),
                                _gpu(w_down, "w_down"), _code(x, "x"),
                                _gpu(expert, "expert", torch.int32),
                                _gpu(weight, "weight", torch.float32), _gpu(act, "act"),
                                _gpu(out, "out", torch.float32), n, width, inter, n_experts, top,
                                _stream())
    _check(lib, status, "moe_experts")


def moe_grouped_supported(dtype, width: int, inter: int, n_experts: int) -> bool:
    """Whether `moe_experts_grouped` takes these sizes (bfloat16, widths that are multiples of
    the matrix cores' K-tile)."""
    if dtype != torch.bfloat16:
        return False
    return bool(library("moe").ei_moe_grouped_supported(BF16, width, inter, n_experts))


def moe_experts_grouped(x, w_gate, w_up, w_down, expert, weight, sorted_pairs, place, starts, act,
                        sums, out) -> None:
    """`moe_experts` as grouped matrix products on the matrix cores: the (row, choice) pairs are
    laid out by expert on the device, every expert's pairs meet its matrices in tiles, and the
    rows' weighted sums are taken last.  Scratch: sorted_pairs, place [n * top] and starts
    [E + 1] int32, act [n * top, f] bfloat16, sums [n * top, w] float32."""
    lib = library("moe")
    n, width = x.shape
    n_experts, inter = w_gate.shape[0], w_gate.shape[1]
    top = expert.shape[1]
    pairs = n * top
    if tuple(w_gate.shape) != (n_experts, inter, width) or tuple(w_up.shape) != tuple(w_gate.shape) \
            or tuple(w_down.shape) != (n_experts, width, inter):
        raise KernelError("moe_experts_grouped: the stacked matrices have the wrong shapes")
    if tuple(expert.shape) != (n, top) or tuple(weight.shape) != (n, top) \
            or tuple(act.shape) != (pairs, inter) or tuple(sums.shape) != (pairs, width) \
            or tuple(out.shape) != (n, width) or sorted_pairs.numel() < pairs \
            or place.numel() < pairs or starts.numel() < n_experts + 1:
        raise KernelError("moe_experts_grouped: shapes do not fit")
    if not moe_grouped_supported(x.dtype, width, inter, n_experts):
        raise KernelError("moe_experts_grouped: bfloat16 and widths that are multiples of 64 only")
    status = lib.ei_moe_experts_grouped(
        _gpu(x, "x", torch.bfloat16), _gpu(w_gate, "w_gate", torch.bfloat16),
        _gpu(w_up, "w_up", torch.bfloat16), _gpu(w_down, "w_down", torch.bfloat16),
        _gpu(expert, "expert", torch.int32), _gpu(weight, "weight", torch.float32),
        _gpu(sorted_pairs, "sorted_pairs", torch.int32), _gpu(place, "place", torch.int32),
        _gpu(starts, "starts", torch.int32), _gpu(act, "act", torch.bfloat16),
        _gpu(sums, "sums", torch.float32), _gpu(out, "out", torch.float32), n, width, inter,
        n_experts, top, _stream())
    _check(lib, status, "moe_experts_grouped")


# ---------------------------------------------------------------------------
def gemm_f32(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> None:
    """out[M, N] = a[M, K] . w[N, K]^T in float32."""
    lib = library("gemm_f32")
    m, k = a.shape
    n = w.shape[0]
    if w.shape[1] != k or tuple(out.shape) != (m, n):
        raise KernelError(f"gemm_f32: shapes {list(a.shape)} x {list(w.shape)}^T -> "
                          f"{list(out.shape)} do not agree")
    status = lib.ei_gemm_f32(_gpu(a, "a", torch.float32), _gpu(w, "w", torch.float32),
                             _gpu(out, "out", torch.float32), m, n, k, k, k, n, _stream())
    _check(lib, status, "gemm_f32")


def argmax_partial_size(rows: int, vocab: int) -> int:
    """float32 elements of scratch with which `argmax` searches a wide vocabulary with many
    blocks a row (0: one block a row is used anyway)."""
    return 2 * library("sampling").ei_argmax_partial_size(rows, vocab)


def argmax(logits: torch.Tensor, tokens: torch.Tensor, probabilities=None, partial=None) -> None:
    lib = library("sampling")
    rows, vocab = logits.shape
    if tokens.numel() < rows:
        raise KernelError("argmax: tokens shorter than the rows")
    status = lib.ei_argmax(_gpu(logits, "logits", torch.float32), rows, vocab,
                           _gpu(tokens, "tokens", torch.int32),
                           None if probabilities is None
                           else _gpu(probabilities, "probabilities", torch.float32),
                           None if partial is None else _gpu(partial, "partial", torch.float32),
                           0 if partial is None else partial.numel() // 2, _stream())
    _check(lib, status, "argmax")


ARGMAX_STATIC_MAX_PARTIALS = 65536


def argmax_static(logits: torch.Tensor, tokens: torch.Tensor, probabilities=None) -> None:
    """`argmax` without a buffer from the caller and without any allocation: the partial results
    of a wide vocabulary live in a device array of the library (at most 65536 pairs of row and
    chunk of 4096 logits; larger requests are refused).  Calls that overlap on one GPU race."""
    lib = library("sampling")
    rows, vocab = logits.shape
    if tokens.numel() < rows:
        raise KernelError("argmax_static: tokens shorter than the rows")
    status = lib.ei_argmax_static(_gpu(logits, "logits", torch.float32), rows, vocab,
                                  _gpu(tokens, "tokens", torch.int32),
                                  None if probabilities is None
                                  else _gpu(probabilities, "probabilities", torch.float32),
                                  _stream())
    _check(lib, status, "argmax_static")


def sample_scratch_size(rows: int, vocab: int) -> int:
    """int32 elements of zeroed scratch that `sample` takes for many blocks a row (0: none)."""
    return library("sampling").ei_sample_scratch_size(rows, vocab)


def sample(logits, temperature, top_p, top_k, seed, streams, counters, tokens,
           probabilities=None, scratch=None) -> None:
    """`scratch` (int32, zero before its first use, see `sample_scratch_size`) lets a wide
    vocabulary be searched by many blocks a row; the tokens are the same without it."""
    lib = library("sampling")
    rows, vocab = logits.shape
    if tokens.numel() < rows or streams.numel() < rows or counters.numel() < rows:
        raise KernelError("sample: per-row arrays shorter than the rows")
    status = lib.ei_sample(_gpu(logits, "logits", torch.float32), rows, vocab, float(temperature),
                           float(top_p), int(top_k), int(seed) & (2**64 - 1),
                           _gpu(streams, "streams", torch.int32),
                           _gpu(counters, "counters", torch.int32),
                           _gpu(tokens, "tokens", torch.int32),
                           None if probabilities is None
                           else _gpu(probabilities, "probabilities", torch.float32),
                           None if scratch is None else _gpu(scratch, "scratch", torch.int32),
                           0 if scratch is None else scratch.numel(), _stream())
    _check(lib, status, "sample")


# ---------------------------------------------------------------------------
def has_skinny_gemm() -> bool:
    return "gemm_bf16" in build.available_libraries()


_SKINNY_MAX_SPLITS = int(os.environ.get("EDGE_INFER_SKINNY_MAX_SPLITS", "0"))   # 0: no cap


def skinny_gemm_splits(rows: int, n: int, k: int) -> int:
    """K slices the weight-streaming product uses for [rows, k] x [n, k]^T."""
    return library("gemm_bf16").ei_skinny_gemm_splits(rows, n, k, _SKINNY_MAX_SPLITS)


# most rows for which the weight-streaming product is taken instead of the library's
SKINNY_ROWS = int(os.environ.get("EDGE_INFER_SKINNY_ROWS", "256"))
if not 1 <= SKINNY_ROWS <= 256:
    raise KernelError("EDGE_INFER_SKINNY_ROWS must lie in 1..256")


def skinny_gemm_ok(rows: int, k: int) -> bool:
    return rows <= SKINNY_ROWS and k % 8 == 0


def gemm_bf16_skinny(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> None:
    """out[s, m, n] = sum over the s-th slice of K of x[m, :] . w[n, :] (float32), for at
    most 256 rows; out.shape[0] says into how many slices K is cut."""
    lib = library("gemm_bf16")
    m, k = x.shape
    n = w.shape[0]
    if out.dim() != 3 or w.shape[1] != k or tuple(out.shape[1:]) != (m, n):
        raise KernelError(f"gemm_bf16_skinny: shapes {list(x.shape)} x {list(w.shape)}^T -> "
                          f"{list(out.shape)} do not agree")
    status = lib.ei_gemm_bf16_skinny(_gpu(x, "x", torch.bfloat16), _gpu(w, "w", torch.bfloat16),
                                     _gpu(out, "out", torch.float32), m, n, k, out.shape[0],
                                     _stream())
    _check(lib, status, "gemm_bf16_skinny")


def pack_weight(w: torch.Tensor) -> torch.Tensor:
    """The streaming copy of a bfloat16 matrix [n, k] for `gemm_bf16_skinny_packed`:
    [8*ceil(k/256), ceil(n/16), 4, 16, 8] where element (kt, strip, c, r, e) is
    w[strip*16 + r, kt*32 + c*8 + e], zero outside the matrix (k is padded to whole
    K-tiles of the kernel, 256 wide).  Made once when the weights
    are loaded; a data movement, no arithmetic."""
    if w.dtype != torch.bfloat16 or w.dim() != 2:
        raise KernelError("pack_weight: a bfloat16 matrix is expected")
    n, k = w.shape
    strips, tiles = (n + 15) // 16, 8 * ((k + 255) // 256)
    if (strips * 16, tiles * 32) != (n, k):
        padded = torch.zeros((strips * 16, tiles * 32), dtype=w.dtype, device=w.device)
        padded[:n, :k] = w
        w = padded
    return w.view(strips, 16, tiles, 4, 8).permute(2, 0, 3, 1, 4).contiguous()


def gemm_bf16_skinny_packed(x: torch.Tensor, packed: torch.Tensor, n: int,
                            out: torch.Tensor) -> None:
    """`gemm_bf16_skinny` with the weight given as `pack_weight(w)` of a matrix [n, k]."""
    lib = library("gemm_bf16")
    m, k = x.shape
    if (out.dim() != 3 or tuple(out.shape[1:]) != (m, n) or packed.dim() != 5
            or tuple(packed.shape) != (8 * ((k + 255) // 256), (n + 15) // 16, 4, 16, 8)):
        raise KernelError(f"gemm_bf16_skinny_packed: shapes {list(x.shape)} x packed "
                          f"{list(packed.shape)} (n = {n}) -> {list(out.shape)} do not agree")
    status = lib.ei_gemm_bf16_skinny_packed(_gpu(x, "x", torch.bfloat16),
                                            _gpu(packed, "packed", torch.bfloat16),
                                            _gpu(out, "out", torch.float32), m, n, k,
                                            out.shape[0], _stream())
    _check(lib, status, "gemm_bf16_skinny_packed")


GATE_STRIP = 16     # gate rows and up rows alternate in strips of this many (one MFMA tile)


def gemm_bf16_skinny_gated(x: torch.Tensor, w: torch.Tensor, n: int, act: torch.Tensor,
                           packed: bool) -> None:
    """act[m, i] = silu(x[m] . gate_i) * (x[m] . up_i) for a weight [n, k] whose rows are, in
    strips of 16, the gate rows of 16 outputs followed by their up rows; `w` is that matrix or
    (packed) its `pack_weight` copy.  For at most 256 rows; K is not sliced, so it pays where
    `skinny_gemm_splits` is 1."""
    lib = library("gemm_bf16")
    m, k = x.shape
    if tuple(act.shape) != (m, n // 2) or n % (2 * GATE_STRIP):
        raise KernelError(f"gemm_bf16_skinny_gated: {list(x.shape)} x [{n}, {k}] -> "
                          f"{list(act.shape)} do not agree")
    expect = (8 * ((k + 255) // 256), (n + 15) // 16, 4, 16, 8) if packed else (n, k)
    if tuple(w.shape) != expect:
        raise KernelError(f"gemm_bf16_skinny_gated: weight {list(w.shape)}, expected {list(expect)}")
    status = lib.ei_gemm_bf16_skinny_gated(_gpu(x, "x", torch.bfloat16), _gpu(w, "w", torch.bfloat16),
                                           _gpu(act, "act", torch.bfloat16), m, n, k, int(packed),
                                           _stream())
    _check(lib, status, "gemm_bf16_skinny_gated")


# ---------------------------------------------------------------------------
def stream_read(data: torch.Tensor, sink: torch.Tensor, blocks: int = 4096) -> None:
    """Read every byte of `data` once with a plain kernel (a yardstick for memory-bound steps)."""
    lib = library("peaks")
    nbytes = data.numel() * data.element_size()
    status = lib.ei_stream_read(_gpu(data, "data"), nbytes - nbytes % 16, int(blocks),
                                _gpu(sink, "sink", torch.int32), _stream())
    _check(lib, status, "stream_read")


MFMA_LOOP_FLOPS = 8 * 16 * 16 * 32 * 2      # per wave and iteration of `mfma_loop`


def mfma_loop(iters: int, blocks: int, sink: torch.Tensor, wide: bool = False) -> None:
    """`blocks` x 4 waves multiply bfloat16 tiles on registers: `iters` rounds of 8 products of
    16x16x32, or (wide) of 4 products of 32x32x16; `MFMA_LOOP_FLOPS` a wave and round."""
    lib = library("peaks")
    status = lib.ei_mfma_loop(int(iters), int(blocks), int(wide),
                              _gpu(sink, "sink", torch.float32), _stream())
    _check(lib, status, "mfma_loop")


def empty_launches(count: int, blocks: int = 256) -> None:
    """`count` launches of a kernel that does nothing (`blocks` blocks of one wave), one after
    the other on the current stream: the floor under a chain of that many dependent kernels."""
    lib = library("peaks")
    _check(lib, lib.ei_empty_launches(int(count), int(blocks), _stream()), "empty_launches")
