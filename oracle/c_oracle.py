"""ctypes view of oracle/liboracle.so (scalar C oracle).  Test infrastructure only."""
import ctypes
import pathlib

import numpy as np
import torch

_HERE = pathlib.Path(__file__).resolve().parent
_lib = None

BF16, F16 = 0, 1


def lib():
    global _lib
    if _lib is None:
        path = _HERE / "liboracle.so"
        if not path.exists():
            from . import build_oracle
            build_oracle.build()
        _lib = ctypes.CDLL(str(path))
        _lib.orc_e4m3_decode.restype = ctypes.c_float
        _lib.orc_e4m3_decode.argtypes = [ctypes.c_uint8]
        _lib.orc_e4m3_encode.restype = ctypes.c_uint8
        _lib.orc_e4m3_encode.argtypes = [ctypes.c_float]
        _lib.orc_f32_to_bf16.restype = ctypes.c_uint16
        _lib.orc_f32_to_bf16.argtypes = [ctypes.c_float]
        _lib.orc_f32_to_f16.restype = ctypes.c_uint16
        _lib.orc_f32_to_f16.argtypes = [ctypes.c_float]
        _lib.orc_f16_to_f32.restype = ctypes.c_float
        _lib.orc_f16_to_f32.argtypes = [ctypes.c_uint16]
    return _lib


def _p(a):
    return ctypes.c_void_p(a.ctypes.data)


def _dt(t):
    return {torch.bfloat16: BF16, torch.float16: F16}[t.dtype]


def _u16(t):
    return np.ascontiguousarray(t.contiguous().view(torch.int16).numpy().view(np.uint16))


def quant_i8_per_token(x: torch.Tensor):
    M, K = x.shape
    xb = _u16(x)
    q = np.empty((M, K), np.int8)
    s = np.empty((M,), np.uint16)
    lib().orc_quant_i8_per_token(_p(xb), _dt(x), ctypes.c_long(M), ctypes.c_long(K), _p(q), _p(s))
    return torch.from_numpy(q), torch.from_numpy(s.view(np.int16)).view(x.dtype).view(M, 1)


def quant_i8_per_tensor(x: torch.Tensor):
    xb = _u16(x)
    q = np.empty(xb.shape, np.int8)
    s = np.empty((1,), np.uint16)
    lib().orc_quant_i8_per_tensor(_p(xb), _dt(x), ctypes.c_long(xb.size), _p(q), _p(s))
    return torch.from_numpy(q), torch.from_numpy(s.view(np.int16)).view(x.dtype).view(())


def quant_fp8_per_token(x: torch.Tensor):
    M, K = x.shape
    xb = _u16(x)
    q = np.empty((M, K), np.uint8)
    s = np.empty((M,), np.float32)
    lib().orc_quant_fp8_per_token(_p(xb), _dt(x), ctypes.c_long(M), ctypes.c_long(K), _p(q), _p(s))
    return torch.from_numpy(q).view(torch.float8_e4m3fn), torch.from_numpy(s).view(M, 1)


def quant_fp8_per_tensor(x: torch.Tensor):
    xb = _u16(x)
    q = np.empty(xb.shape, np.uint8)
    s = np.empty((1,), np.float32)
    lib().orc_quant_fp8_per_tensor(_p(xb), _dt(x), ctypes.c_long(xb.size), _p(q), _p(s))
    return torch.from_numpy(q).view(torch.float8_e4m3fn), torch.from_numpy(s).view(())


def gemm_i8(a: torch.Tensor, b_nk: torch.Tensor):
    M, K = a.shape
    N = b_nk.shape[0]
    an, bn = np.ascontiguousarray(a.numpy()), np.ascontiguousarray(b_nk.numpy())
    acc = np.empty((M, N), np.int32)
    lib().orc_gemm_i8(_p(an), _p(bn), ctypes.c_long(M), ctypes.c_long(N), ctypes.c_long(K), _p(acc))
    return torch.from_numpy(acc)


def awq_dequant(qweight, qzeros, scales, group):
    K, Nw = qweight.shape
    N = Nw * 8
    qw, qz = np.ascontiguousarray(qweight.numpy()), np.ascontiguousarray(qzeros.numpy())
    sc = _u16(scales)
    out = np.empty((K, N), np.uint16)
    lib().orc_awq_dequant(_p(qw), _p(qz), _p(sc), ctypes.c_long(K), ctypes.c_long(N), ctypes.c_long(group), _p(out))
    return torch.from_numpy(out.view(np.int16)).view(torch.float16)


def awq_gemm(x, qweight, qzeros, scales, group):
    M, K = x.shape
    N = qweight.shape[1] * 8
    xb = _u16(x)
    qw, qz = np.ascontiguousarray(qweight.numpy()), np.ascontiguousarray(qzeros.numpy())
    sc = _u16(scales)
    out = np.empty((M, N), np.uint16)
    lib().orc_awq_gemm(_p(xb), _p(qw), _p(qz), _p(sc), ctypes.c_long(M), ctypes.c_long(N),
                       ctypes.c_long(K), ctypes.c_long(group), _p(out))
    return torch.from_numpy(out.view(np.int16)).view(torch.float16)


def e4m3_decode_table():
    return np.array([lib().orc_e4m3_decode(c) for c in range(256)], np.float32)


def e4m3_encode(values):
    return np.array([lib().orc_e4m3_encode(float(v)) for v in values], np.uint8)


def rmsnorm_given_inv(x: torch.Tensor, weight: torch.Tensor, inv: torch.Tensor) -> torch.Tensor:
    M, K = x.shape
    xb, wb = _u16(x), _u16(weight)
    iv = np.ascontiguousarray(inv.reshape(M).to(torch.float32).numpy())
    y = np.empty((M, K), np.uint16)
    lib().orc_rmsnorm_given_inv(_p(xb), _p(wb), _p(iv), _dt(x), ctypes.c_long(M), ctypes.c_long(K), _p(y))
    return torch.from_numpy(y.view(np.int16)).view(x.dtype)


def inv_rms_f64(x: torch.Tensor, eps: float) -> torch.Tensor:
    M, K = x.shape
    xb = _u16(x)
    out = np.empty((M,), np.float64)
    lib().orc_inv_rms_f64(_p(xb), _dt(x), ctypes.c_long(M), ctypes.c_long(K), ctypes.c_double(eps), _p(out))
    return torch.from_numpy(out)
