"""ctypes binding of libllmq_gfx950.so (the C ABI declared in include/llmq.h).

Nothing here computes: tensors are validated by the callers, this module passes raw device
pointers, sizes and the current HIP stream to C and turns a negative status into RuntimeError.
There is no fallback: if the library is missing the import of any op fails loudly.
"""
from __future__ import annotations

import ctypes
import pathlib

import torch

_LIB_PATH = pathlib.Path(__file__).resolve().parent / "lib" / "libllmq_gfx950.so"

BF16, F16, F32 = 0, 1, 2
E4M3, E5M2 = 0, 1

_DTYPE_CODE = {torch.bfloat16: BF16, torch.float16: F16, torch.float32: F32}

_vp, _i64, _int, _f32, _sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float, ctypes.c_size_t

# name -> (restype, argtypes); must list every symbol of include/llmq.h
SIGNATURES = {
    "llmq_abi_version": (_int, []),
    "llmq_status_string": (ctypes.c_char_p, [_int]),
    "llmq_quant_i8_per_token": (_int, [_vp, _int, _i64, _i64, _i64, _vp, _vp, _int, _vp]),
    "llmq_quant_i8_weight_per_channel": (_int, [_vp, _int, _i64, _i64, _i64, _vp, _vp, _vp]),
    "llmq_quant_i8_per_tensor": (_int, [_vp, _int, _i64, _i64, _i64, _vp, _vp, _int, _vp, _sz, _vp]),
    "llmq_quant_i8_per_token_floor": (_int, [_vp, _int, _i64, _i64, _i64, _vp, _vp, _int, _f32, _vp]),
    "llmq_quant_i8_per_tensor_floor": (_int, [_vp, _int, _i64, _i64, _i64, _vp, _vp, _int, _f32, _vp, _sz, _vp]),
    "llmq_quant_fp8_per_token": (_int, [_vp, _int, _i64, _i64, _i64, _vp, _vp, _vp]),
    "llmq_quant_fp8_per_tensor": (_int, [_vp, _int, _i64, _i64, _i64, _vp, _vp, _vp, _sz, _vp]),
    "llmq_quant_fp8_static": (_int, [_vp, _int, _i64, _i64, _i64, _vp, _vp, _int, _vp]),
    "llmq_rmsnorm": (_int, [_vp, _int, _i64, _i64, _i64, _vp, _f32, _vp, _vp, _vp]),
    "llmq_rmsnorm_quant_i8_per_token": (_int, [_vp, _int, _i64, _i64, _i64, _vp, _f32, _vp, _vp, _vp, _int, _vp, _vp]),
    "llmq_rmsnorm_quant_fp8_per_token": (_int, [_vp, _int, _i64, _i64, _i64, _vp, _f32, _vp, _vp, _vp, _vp, _vp]),
    "llmq_quant_workspace_bytes": (_sz, []),
    "llmq_gemm_w8a8": (_int, [_vp, _i64, _vp, _i64, _vp, _vp, _f32, _vp, _vp, _int, _f32, _vp, _int, _i64,
                              _i64, _i64, _i64, _vp, _vp, _sz, _vp]),
    "llmq_gemm_fp8": (_int, [_vp, _int, _i64, _vp, _i64, _vp, _vp, _f32, _vp, _vp, _int, _f32, _vp, _int, _i64,
                             _i64, _i64, _i64, _vp, _vp, _sz, _vp]),
    "llmq_gemm_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "llmq_gemm_w8a8_static": (_int, [_vp, _i64, _vp, _i64, _vp, _vp, _f32, _vp, _vp, _int, _f32, _vp, _int, _i64,
                                     _i64, _i64, _i64, _vp]),
    "llmq_gemm_static_scratch_bytes": (_sz, []),
    "llmq_gemm_f16": (_int, [_vp, _i64, _vp, _i64, _f32, _vp, _int, _f32, _vp, _int, _i64, _i64, _i64, _i64, _vp, _vp, _sz, _vp]),
    "llmq_gemm_f16_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "llmq_linear_i8_dynamic": (_int, [_vp, _int, _i64, _vp, _i64, _vp, _vp, _int, _vp, _int, _i64, _i64, _i64, _i64, _vp, _vp, _vp, _vp]),
    "llmq_linear_fp8_dynamic": (_int, [_vp, _int, _i64, _vp, _i64, _vp, _vp, _int, _vp, _int, _i64, _i64, _i64, _i64, _vp, _vp, _vp, _vp]),
    "llmq_linear_dynamic_max_tokens": (_int, [_i64]),
    "llmq_linear_dynamic_force_variant": (_int, [_int]),
    "llmq_gemm_fp8_quantized_output": (_int, [_vp, _int, _i64, _vp, _i64, _vp, _vp, _f32, _vp, _vp, _int, _f32, _vp, _vp, _int,
                                              _i64, _i64, _i64, _i64, _vp, _sz, _vp]),
    "llmq_gemm_fp8_quantized_output_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "llmq_gemm_force_plan": (_int, [_int, _int]),
    "llmq_gemm_num_configs": (_int, []),
    "llmq_awq_gemm": (_int, [_vp, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _sz, _vp]),
    "llmq_awq_gemm_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "llmq_awq_force_plan": (_int, [_int, _int, _int]),
    "llmq_awq_workspace_ticket_bytes": (_sz, []),
    "llmq_awq_workspace_init": (_int, [_vp, _sz, _vp]),
    "llmq_awq_dequant": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "llmq_awq_dequant_t": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
}

_lib = None


def lib_path() -> pathlib.Path:
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    """Load the shared library once.  Raises (never falls back) when it has not been built."""
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            raise RuntimeError(
                f"{_LIB_PATH} is missing: build it with `python -m llmqrt_amd.csrc.build` "
                "(there is no CPU or PyTorch fallback for these ops)")
        handle = ctypes.CDLL(str(_LIB_PATH))
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


def check(status: int, what: str) -> None:
    if status != 0:
        msg = lib().llmq_status_string(status).decode()
        raise RuntimeError(f"{what}: {msg} (llmq status {status})")


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dt]
    except KeyError:
        raise RuntimeError(f"unsupported dtype {dt}") from None


def ptr(t) -> int | None:
    return None if t is None else t.data_ptr()


def stream_of(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


class _Workspaces:
    """One grow-only scratch tensor per (device, stream): the C library never allocates.
    zeroed: every new buffer starts as zeros (the AWQ workspace begins with arrival counters that must be zero before
    the first call and that every call leaves zero)."""

    def __init__(self, zeroed: bool = False):
        self._buf = {}
        self._zeroed = zeroed

    def get(self, device: torch.device, nbytes: int) -> torch.Tensor | None:
        if nbytes == 0:
            return None
        key = (device.index, torch.cuda.current_stream(device).cuda_stream)
        buf = self._buf.get(key)
        if buf is None or buf.numel() < nbytes:
            alloc = torch.zeros if self._zeroed else torch.empty
            buf = alloc(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
            self._buf[key] = buf
        return buf


workspaces = _Workspaces()
awq_workspaces = _Workspaces(zeroed=True)  # never shared with another op: their partial sums would overwrite the counters
