"""ctypes access to the compiled test oracles.  TEST INFRASTRUCTURE ONLY.

``liboracle.so``                  — oracle.c, the plain-C restatement.
``_ref/libtessera_x86_ref.so``    — the reference's own x86 kernels for this path,
                                    compiled from the reference checkout by
                                    ``oracle/Makefile`` (present only where that
                                    build ran; needs an AVX-512 host to call).
"""
from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path
from typing import Optional

import numpy as np

HERE = Path(__file__).resolve().parent
_c_vp, _c_int, _c_f, _c_i64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_int64


def build(force: bool = False) -> None:
    """Run ``make`` for the C oracle (and ``_ref`` when the reference is mounted)."""
    if force:
        subprocess.run(["make", "-C", str(HERE), "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", str(HERE)], check=True, capture_output=True)


_lib: Optional[ctypes.CDLL] = None
_ref: Optional[ctypes.CDLL] = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        path = HERE / "liboracle.so"
        if not path.is_file():
            build()
        _lib = ctypes.CDLL(str(path))
        _lib.orc_moe_route.restype = _c_int
    return _lib


def host_has_avx512() -> bool:
    try:
        flags = Path("/proc/cpuinfo").read_text()
    except OSError:
        return False
    return all(f in flags for f in ("avx512f", "avx512bw", "avx512vl", "avx512dq"))


def ref() -> Optional[ctypes.CDLL]:
    """The compiled reference kernels, or None when not built / not runnable here."""
    global _ref
    if _ref is None:
        path = HERE / "_ref" / "libtessera_x86_ref.so"
        if not path.is_file() or not host_has_avx512():
            return None
        _ref = ctypes.CDLL(str(path))
    return _ref


def _p(a: np.ndarray):
    return a.ctypes.data_as(_c_vp)


def gemm_bf16_f32(a_bits: np.ndarray, b_bits: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a_bits, np.uint16)
    b = np.ascontiguousarray(b_bits, np.uint16)
    M, K = a.shape
    N = b.shape[1]
    c = np.empty((M, N), np.float32)
    lib().orc_gemm_bf16_f32(_p(a), _p(b), _p(c), M, N, K)
    return c


def gemm_bf16_f64(a_bits: np.ndarray, b_bits: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a_bits, np.uint16)
    b = np.ascontiguousarray(b_bits, np.uint16)
    M, K = a.shape
    N = b.shape[1]
    c = np.empty((M, N), np.float64)
    lib().orc_gemm_bf16_f64(_p(a), _p(b), _p(c), M, N, K)
    return c


def gemm_s8s8_s32(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, np.int8)
    b = np.ascontiguousarray(b, np.int8)
    M, K = a.shape
    N = b.shape[1]
    c = np.empty((M, N), np.int32)
    lib().orc_gemm_s8s8_s32(_p(a), _p(b), _p(c), M, N, K)
    return c


def flash_attn_f32(q, k, v, scale: float, causal: bool):
    q = np.ascontiguousarray(q, np.float32)
    k = np.ascontiguousarray(k, np.float32)
    v = np.ascontiguousarray(v, np.float32)
    B, Hq, Sq, D = q.shape
    _, Hkv, Sk, _ = k.shape
    o = np.empty_like(q)
    lse = np.empty((B, Hq, Sq), np.float32)
    lib().orc_flash_attn_f32(_p(q), _p(k), _p(v), B, Hq, Hkv, Sq, Sk, D, _c_f(scale), 1 if causal else 0,
                             _p(o), _p(lse))
    return o, lse


def fpquant_f32(x, max_normal=448.0, mantissa_bits=3, min_exp=-6) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty_like(x)
    lib().orc_fpquant_f32(_p(x), _c_i64(x.size), _c_f(max_normal), mantissa_bits, min_exp, _p(out))
    return out


def moe_route(scores, k: int, normalize: bool = True, capacity: int = 0):
    s = np.ascontiguousarray(scores, np.float32)
    T, E = s.shape
    S = T * k
    tos = np.empty(S, np.int32)
    eos = np.empty(S, np.int32)
    cw = np.empty(S, np.float32)
    gs = np.empty(E, np.int32)
    go = np.empty(E + 1, np.int32)
    n = lib().orc_moe_route(_p(s), T, E, k, 1 if normalize else 0, capacity, _p(tos), _p(eos), _p(cw), _p(gs), _p(go))
    if n < 0:
        raise MemoryError("orc_moe_route")
    return tos[:n].copy(), eos[:n].copy(), cw[:n].copy(), gs, go


# ---- the reference's compiled kernels (only where ref() is available) ----------

def ref_gemm_bf16(a_bits, b_bits) -> np.ndarray:
    a = np.ascontiguousarray(a_bits, np.uint16)
    b = np.ascontiguousarray(b_bits, np.uint16)
    M, K = a.shape
    N = b.shape[1]
    c = np.zeros((M, N), np.float32)
    ref().tessera_x86_reference_gemm_bf16(_p(a), _p(b), _p(c), M, N, K, _c_f(0.0))
    return c


def ref_gemm_u8s8(a_u8, b_s8) -> np.ndarray:
    a = np.ascontiguousarray(a_u8, np.uint8)
    b = np.ascontiguousarray(b_s8, np.int8)
    M, K = a.shape
    N = b.shape[1]
    c = np.zeros((M, N), np.int32)
    ref().tessera_x86_reference_gemm_u8s8_s32(_p(a), _p(b), _p(c), M, N, K, 0)
    return c


def ref_flash_attn_lse(q, k, v, scale: float, causal: bool, window: int = 0, softcap: float = 0.0, bias=None):
    q = np.ascontiguousarray(q, np.float32)
    k = np.ascontiguousarray(k, np.float32)
    v = np.ascontiguousarray(v, np.float32)
    B, Hq, Sq, D = q.shape
    _, Hkv, Sk, _ = k.shape
    o = np.empty_like(q)
    lse = np.empty((B, Hq, Sq), np.float32)
    i64 = _c_i64
    if bias is not None:
        bias = np.ascontiguousarray(np.broadcast_to(bias, (B, Hq, Sq, Sk)), np.float32)
    ref().tessera_x86_flash_attn_ext_lse_f32(_p(q), _p(k), _p(v), _p(bias) if bias is not None else None, i64(B), i64(Hq), i64(Hkv), i64(Sq), i64(Sk),
                                             i64(D), i64(D), _c_f(scale), 1 if causal else 0, i64(window), _c_f(softcap),
                                             _p(o), _p(lse))
    return o, lse


def ref_fpquant(x, max_normal=448.0, mantissa_bits=3, min_exp=-6) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty_like(x)
    ref().tessera_x86_avx512_fpquant_f32(_p(x), _c_i64(x.size), _c_f(max_normal), mantissa_bits, min_exp, _p(out))
    return out
