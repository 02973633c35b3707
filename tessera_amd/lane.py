"""ctypes binding of ``libtessera_gfx950.so`` — the MI355X execution lane.

The host side is ctypes-only (the reference never imports PyTorch,
``README.md:10-14``) and follows the loader discipline of the reference's ROCm
lanes (``python/tessera/runtime.py:1939-2033``):

* library path = ``TESSERA_GFX950_LIB`` override, else the in-tree build;
* ``ctypes.CDLL(..., mode=RTLD_LOCAL)`` — ``RTLD_GLOBAL`` corrupted interpreter
  shutdown for the reference (``runtime.py:1972-1978``);
* a cached host probe (:func:`available`) that callers consult before claiming a
  native execution;
* return codes 0/1/2/3 mapped to ``ValueError`` (bad shape), :class:`LaneUnavailable`
  (no device) and ``RuntimeError`` (device failure), as the executors do
  (``runtime.py:2137-2142``).

There is no CPU fallback here: when the library or the device is missing the
calls raise.
"""
from __future__ import annotations

import ctypes
import os
import threading
from pathlib import Path
from typing import Optional

import numpy as np

_PKG = Path(__file__).resolve().parent
_DEFAULT_LIB = _PKG / "lib" / "libtessera_gfx950.so"

OK, BAD_SHAPE, NO_DEVICE, DEVICE_FAILED = 0, 1, 2, 3


class LaneUnavailable(RuntimeError):
    """The gfx950 lane cannot run here (library not built, or no MI355X).

    The counterpart of the reference's ``_RocmCompiledUnavailable``: callers may
    treat it as "lane absent"; it is never converted into a CPU execution here."""


_lib: Optional[ctypes.CDLL] = None
_lib_lock = threading.Lock()
_probe: Optional[bool] = None

_c_int = ctypes.c_int
_c_vp = ctypes.c_void_p
_c_f = ctypes.c_float
_c_i64 = ctypes.c_int64
_c_sz = ctypes.c_size_t
_P = ctypes.POINTER


def library_path() -> Path:
    env = os.environ.get("TESSERA_GFX950_LIB")
    return Path(env) if env else _DEFAULT_LIB


# symbol -> argtypes; every entry point returns int.
_GEMM = [_c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int]
_SIGNATURES = {
    "tessera_gfx950_gpu_launcher": [ctypes.c_char_p, ctypes.c_char_p, _c_vp, _c_vp],
    "tessera_gfx950_flash_attn_bf16_bench": [_c_int] * 8 + [_P(ctypes.c_double)],
    "tessera_gfx950_abi_version": [],
    "tessera_gfx950_probe": [],
    "tessera_gfx950_device_name": [ctypes.c_char_p, _c_int],
    "tessera_gfx950_device_cus": [_P(_c_int)],
    "tessera_gfx950_malloc": [_P(_c_vp), _c_sz],
    "tessera_gfx950_free": [_c_vp],
    "tessera_gfx950_memcpy_h2d": [_c_vp, _c_vp, _c_sz],
    "tessera_gfx950_memcpy_d2h": [_c_vp, _c_vp, _c_sz],
    "tessera_gfx950_memset": [_c_vp, _c_int, _c_sz],
    "tessera_gfx950_memcpy_d2d_dev": [_c_vp, _c_vp, _c_sz, _c_vp],
    "tessera_gfx950_synchronize": [],
    "tessera_gfx950_timer_create": [_P(_c_vp)],
    "tessera_gfx950_timer_start": [_c_vp, _c_vp],
    "tessera_gfx950_timer_stop": [_c_vp, _c_vp],
    "tessera_gfx950_timer_elapsed_ms": [_c_vp, _P(_c_f)],
    "tessera_gfx950_timer_destroy": [_c_vp],
    "tessera_gfx950_gemm_f16": _GEMM,
    "tessera_gfx950_gemm_bf16": _GEMM,
    "tessera_gfx950_gemm_f16_f16": _GEMM,
    "tessera_gfx950_gemm_bf16_bf16": _GEMM,
    "tessera_gfx950_batched_gemm_f16": [_c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_int],
    "tessera_gfx950_batched_gemm_bf16": [_c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_int],
    "tessera_gfx950_gemm_i8_i32": _GEMM,
    "tessera_gfx950_gemm_w8a8_f32": [_c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int],
    "tessera_gfx950_gemm_e4m3_bf16": [_c_vp, _c_vp, _c_f, _c_f, _c_vp, _c_int, _c_int, _c_int],
    "tessera_gfx950_gemm_e5m2_bf16": [_c_vp, _c_vp, _c_f, _c_f, _c_vp, _c_int, _c_int, _c_int],
    "tessera_gfx950_gemm_e4m3_f32": [_c_vp, _c_vp, _c_f, _c_f, _c_vp, _c_int, _c_int, _c_int],
    "tessera_gfx950_gemm_e5m2_f32": [_c_vp, _c_vp, _c_f, _c_f, _c_vp, _c_int, _c_int, _c_int],
    "tessera_gfx950_gemm_f16_dev": _GEMM + [_c_vp],
    "tessera_gfx950_gemm_bf16_dev": _GEMM + [_c_vp],
    "tessera_gfx950_gemm_f16_f16_dev": _GEMM + [_c_vp],
    "tessera_gfx950_gemm_bf16_bf16_dev": _GEMM + [_c_vp],
    "tessera_gfx950_batched_gemm_f16_dev": [_c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_int, _c_vp],
    "tessera_gfx950_batched_gemm_bf16_dev": [_c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_int, _c_vp],
    "tessera_gfx950_batched_gemm_strided_f16_dev": [_c_vp] * 3 + [_c_int] * 4 + [_c_i64] * 3 + [_c_int, _c_vp],
    "tessera_gfx950_batched_gemm_strided_bf16_dev": [_c_vp] * 3 + [_c_int] * 4 + [_c_i64] * 3 + [_c_int, _c_vp],
    "tessera_gfx950_fake_quantize_nvfp4_f32": [_c_vp, _c_int, _c_int, _c_vp, _c_vp, _c_vp],
    "tessera_gfx950_fake_quantize_nvfp4_f32_dev": [_c_vp, _c_int, _c_int, _c_vp, _c_vp, _c_vp, _c_vp],
    "tessera_gfx950_quantize_i8_tensor_f32": [_c_vp, _c_i64, _c_f, _c_vp, _c_vp],
    "tessera_gfx950_quantize_i8_tensor_f32_dev": [_c_vp, _c_i64, _c_f, _c_vp, _c_vp, _c_vp],
    "tessera_gfx950_quantize_i8_smoothed_f32": [_c_vp, _c_int, _c_int, _c_vp, _c_vp, _c_vp],
    "tessera_gfx950_quantize_i8_smoothed_f32_dev": [_c_vp, _c_int, _c_int, _c_vp, _c_vp, _c_vp, _c_vp],
    "tessera_gfx950_fpquant_f32": [_c_vp, _c_i64, _c_f, _c_int, _c_int, _c_vp],
    "tessera_gfx950_fpquant_f32_dev": [_c_vp, _c_i64, _c_f, _c_int, _c_int, _c_vp, _c_vp],
    "tessera_gfx950_fake_quantize_fp_f32": [_c_vp, _c_i64, _c_f, _c_int, _c_int, _c_f, _c_vp, _c_vp, _c_vp],
    "tessera_gfx950_fake_quantize_fp_f32_dev": [_c_vp, _c_i64, _c_f, _c_int, _c_int, _c_f, _c_vp, _c_vp, _c_vp, _c_vp],
    "tessera_gfx950_scale_groups_f32": [_c_vp, _c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_int],
    "tessera_gfx950_scale_groups_f32_dev": [_c_vp, _c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_int, _c_vp],
    "tessera_gfx950_silu_mul_bf16": [_c_vp, _c_vp, _c_vp, _c_i64],
    "tessera_gfx950_silu_mul_bf16_dev": [_c_vp, _c_vp, _c_vp, _c_i64, _c_vp],
    "tessera_gfx950_silu_mul_f16": [_c_vp, _c_vp, _c_vp, _c_i64],
    "tessera_gfx950_silu_mul_f16_dev": [_c_vp, _c_vp, _c_vp, _c_i64, _c_vp],
    "tessera_gfx950_gemm_schedule": [_c_int] * 5 + [_c_vp] * 4,
    "tessera_gfx950_gemm_rest_split": [_c_int] * 4 + [_c_vp] * 2,
    "tessera_gfx950_gemm_bias_act_f16": [_c_vp, _c_vp, _c_vp, _c_int, _c_vp, _c_int, _c_int, _c_int],
    "tessera_gfx950_gemm_bias_act_bf16": [_c_vp, _c_vp, _c_vp, _c_int, _c_vp, _c_int, _c_int, _c_int],
    "tessera_gfx950_gemm_bias_act_f16_dev": [_c_vp, _c_vp, _c_vp, _c_int, _c_vp, _c_int, _c_int, _c_int, _c_vp],
    "tessera_gfx950_gemm_bias_act_bf16_dev": [_c_vp, _c_vp, _c_vp, _c_int, _c_vp, _c_int, _c_int, _c_int, _c_vp],
    "tessera_gfx950_gated_gemm_f16": [_c_vp, _c_vp, _c_vp, _c_int, _c_vp, _c_int, _c_int, _c_int],
    "tessera_gfx950_gated_gemm_bf16": [_c_vp, _c_vp, _c_vp, _c_int, _c_vp, _c_int, _c_int, _c_int],
    "tessera_gfx950_gated_gemm_f16_dev": [_c_vp, _c_vp, _c_vp, _c_int, _c_vp, _c_int, _c_int, _c_int, _c_vp],
    "tessera_gfx950_gated_gemm_bf16_dev": [_c_vp, _c_vp, _c_vp, _c_int, _c_vp, _c_int, _c_int, _c_int, _c_vp],
    "tessera_gfx950_gemm_i8_i32_dev": _GEMM + [_c_vp],
    "tessera_gfx950_gemm_w8a8_f32_dev": [_c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_vp],
    "tessera_gfx950_gemm_e4m3_bf16_dev": [_c_vp, _c_vp, _c_f, _c_f, _c_vp, _c_int, _c_int, _c_int, _c_vp],
    "tessera_gfx950_gemm_e5m2_bf16_dev": [_c_vp, _c_vp, _c_f, _c_f, _c_vp, _c_int, _c_int, _c_int, _c_vp],
    "tessera_gfx950_gemm_e4m3_f32_dev": [_c_vp, _c_vp, _c_f, _c_f, _c_vp, _c_int, _c_int, _c_int, _c_vp],
    "tessera_gfx950_gemm_e5m2_f32_dev": [_c_vp, _c_vp, _c_f, _c_f, _c_vp, _c_int, _c_int, _c_int, _c_vp],
    "tessera_gfx950_stream_release": [_c_vp],
    "tessera_gfx950_gemm_bf16_bench": [_c_int, _c_int, _c_int, _c_int, _P(ctypes.c_double)],
    "tessera_gfx950_gemm_f16_bench": [_c_int] * 6 + [_P(ctypes.c_double)],
    "tessera_gfx950_gemm_bf16_bench_rotating": [_c_int, _c_int, _c_int, _c_int, _c_int, _P(ctypes.c_double)],
    "tessera_gfx950_bench_last_timer_source": [],
    "tessera_gfx950_mfma_probe_bf16_dev": [_c_vp, _c_int, _c_vp, _P(ctypes.c_double), _c_vp],
    "tessera_gfx950_mfma_probe_dev": [_c_int, _c_vp, _c_int, _c_vp, _P(ctypes.c_double), _c_vp],
    "tessera_gfx950_quantize_e4m3_f32": [_c_vp, _c_i64, _c_f, _c_vp, _P(_c_f)],
    "tessera_gfx950_quantize_e5m2_f32": [_c_vp, _c_i64, _c_f, _c_vp, _P(_c_f)],
    "tessera_gfx950_quantize_i8_f32": [_c_vp, _c_int, _c_int, _c_int, _c_vp, _c_vp],
    "tessera_gfx950_quantize_e4m3_f32_dev": [_c_vp, _c_i64, _c_f, _c_vp, _c_vp, _c_vp],
    "tessera_gfx950_quantize_e5m2_f32_dev": [_c_vp, _c_i64, _c_f, _c_vp, _c_vp, _c_vp],
    "tessera_gfx950_quantize_i8_f32_dev": [_c_vp, _c_int, _c_int, _c_int, _c_vp, _c_vp, _c_vp],
    "tessera_gfx950_flash_attn_f16": [_c_vp, _c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_int, _c_int, _c_f, _c_int],
    "tessera_gfx950_flash_attn_bf16": [_c_vp, _c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_int, _c_int, _c_f, _c_int],
    "tessera_gfx950_flash_attn_gqa_f16": [_c_vp] * 5 + [_c_int] * 6 + [_c_f, _c_int],
    "tessera_gfx950_flash_attn_gqa_bf16": [_c_vp] * 5 + [_c_int] * 6 + [_c_f, _c_int],
    "tessera_gfx950_flash_attn_gqa_f16_dev": [_c_vp] * 5 + [_c_int] * 6 + [_c_f, _c_int, _c_int, _c_vp],
    "tessera_gfx950_flash_attn_gqa_bf16_dev": [_c_vp] * 5 + [_c_int] * 6 + [_c_f, _c_int, _c_int, _c_vp],
    "tessera_gfx950_flash_attn_ext_f16": [_c_vp] * 5 + [_c_int] * 6 + [_c_f, _c_int, _c_int, _c_f],
    "tessera_gfx950_flash_attn_ext_bf16": [_c_vp] * 5 + [_c_int] * 6 + [_c_f, _c_int, _c_int, _c_f],
    "tessera_gfx950_flash_attn_ext_f16_dev": [_c_vp] * 5 + [_c_int] * 6 + [_c_f, _c_int, _c_int, _c_f, _c_int, _c_vp],
    "tessera_gfx950_flash_attn_ext_bf16_dev": [_c_vp] * 5 + [_c_int] * 6 + [_c_f, _c_int, _c_int, _c_f, _c_int, _c_vp],
    "tessera_gfx950_flash_attn_strided_f16_dev": [_c_vp] * 5 + [_c_int] * 6 + [_c_vp, _c_f, _c_int, _c_int, _c_f, _c_int, _c_vp],
    "tessera_gfx950_flash_attn_strided_bf16_dev": [_c_vp] * 5 + [_c_int] * 6 + [_c_vp, _c_f, _c_int, _c_int, _c_f, _c_int, _c_vp],
    "tessera_gfx950_flash_attn_bias_f16": [_c_vp] * 6 + [_c_int] * 6 + [_c_f, _c_int, _c_int, _c_f],
    "tessera_gfx950_flash_attn_bias_bf16": [_c_vp] * 6 + [_c_int] * 6 + [_c_f, _c_int, _c_int, _c_f],
    "tessera_gfx950_flash_attn_bias_f16_dev": [_c_vp] * 6 + [_c_int] * 6 + [_c_f, _c_int, _c_int, _c_f, _c_int, _c_vp],
    "tessera_gfx950_flash_attn_bias_bf16_dev": [_c_vp] * 6 + [_c_int] * 6 + [_c_f, _c_int, _c_int, _c_f, _c_int, _c_vp],
    "tessera_gfx950_flash_attn_bwd_f16": [_c_vp] * 7 + [_c_int] * 6 + [_c_f, _c_int],
    "tessera_gfx950_flash_attn_bwd_bf16": [_c_vp] * 7 + [_c_int] * 6 + [_c_f, _c_int],
    "tessera_gfx950_flash_attn_bwd_f16_dev": [_c_vp] * 9 + [_c_int] * 6 + [_c_f, _c_int, _c_vp],
    "tessera_gfx950_flash_attn_bwd_bf16_dev": [_c_vp] * 9 + [_c_int] * 6 + [_c_f, _c_int, _c_vp],
    "tessera_gfx950_moe_route_f32": [_c_vp] + [_c_int] * 5 + [_c_vp] * 6,
    "tessera_gfx950_moe_route_f32_dev": [_c_vp] + [_c_int] * 5 + [_c_vp] * 6 + [_c_vp],
    "tessera_gfx950_moe_route_f32_noalloc_dev": [_c_vp] + [_c_int] * 5 + [_c_vp] * 6 + [_c_vp],
    "tessera_gfx950_moe_plan_f32": [_c_vp] * 3 + [_c_int] * 5 + [_c_vp] * 11,
    "tessera_gfx950_moe_plan_f32_dev": [_c_vp] * 3 + [_c_int] * 5 + [_c_vp] * 11 + [_c_vp],
    "tessera_gfx950_moe_unpack_combine_bf16": [_c_vp] * 4 + [_c_int] * 4,
    "tessera_gfx950_moe_unpack_combine_f32": [_c_vp] * 4 + [_c_int] * 4,
    "tessera_gfx950_moe_unpack_combine_bf16_dev": [_c_vp] * 4 + [_c_int] * 4 + [_c_vp],
    "tessera_gfx950_moe_unpack_combine_f32_dev": [_c_vp] * 4 + [_c_int] * 4 + [_c_vp],
    "tessera_gfx950_moe_dispatch": [_c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_int],
    "tessera_gfx950_moe_dispatch_dev": [_c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_int, _c_vp],
    "tessera_gfx950_moe_combine_bf16": [_c_vp, _c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int],
    "tessera_gfx950_moe_combine_f32": [_c_vp, _c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int],
    "tessera_gfx950_moe_combine_bf16_dev": [_c_vp, _c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_vp],
    "tessera_gfx950_moe_combine_f32_dev": [_c_vp, _c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_vp],
    "tessera_gfx950_grouped_gemm_bf16": [_c_vp, _c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_int],
    "tessera_gfx950_grouped_gemm_bf16_f32": [_c_vp, _c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_int],
    "tessera_gfx950_grouped_gemm_bf16_dev": [_c_vp, _c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_int, _c_vp],
    "tessera_gfx950_grouped_gemm_bf16_f32_dev": [_c_vp, _c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_int, _c_vp],
    "tessera_gfx950_grouped_gemm_f16": [_c_vp, _c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_int],
    "tessera_gfx950_grouped_gemm_f16_f32": [_c_vp, _c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_int],
    "tessera_gfx950_grouped_gemm_f16_dev": [_c_vp, _c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_int, _c_vp],
    "tessera_gfx950_grouped_gemm_f16_f32_dev": [_c_vp, _c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_int, _c_vp],
    "tessera_gfx950_moe_swiglu_block_bf16": [_c_vp] * 6 + [_c_int] * 5,
    "tessera_gfx950_moe_swiglu_block_bf16_dev": [_c_vp] * 7 + [_c_int] * 5 + [_c_vp],
    "tessera_gfx950_moe_swiglu_block_gather_bf16_dev": [_c_vp] * 8 + [_c_int] * 6 + [_c_vp],
    "tessera_gfx950_moe_layer_bf16": [_c_vp] * 6 + [_c_int] * 8 + [_c_vp] * 5,
    "tessera_gfx950_moe_layer_router_bf16": [_c_vp] * 6 + [_c_int] * 8 + [_c_vp] * 6,
    "tessera_gfx950_moe_layer_workspace_bytes": [_c_int] * 6 + [_P(_c_sz)],
    "tessera_gfx950_moe_layer_bf16_dev": [_c_vp] * 8 + [_c_sz] + [_c_int] * 8 + [_c_vp] * 6 + [_c_vp],
}


def exported_symbols() -> tuple[str, ...]:
    """Names of every entry point the header declares."""
    return tuple(_SIGNATURES)


def load() -> ctypes.CDLL:
    """Load the library once and bind every signature.  Raises
    :class:`LaneUnavailable` when the library is not built or not loadable."""
    global _lib
    if _lib is not None:
        return _lib
    with _lib_lock:
        if _lib is not None:
            return _lib
        path = library_path()
        if not path.is_file():
            raise LaneUnavailable(
                f"{path} not found — build it with `python -m tessera_amd.build` "
                "(or point TESSERA_GFX950_LIB at it)")
        try:
            lib = ctypes.CDLL(str(path), mode=ctypes.RTLD_LOCAL)
        except OSError as exc:
            raise LaneUnavailable(f"cannot load {path}: {exc}") from exc
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(lib, name, None)
            if fn is None:
                raise LaneUnavailable(f"{path} lacks symbol {name} — rebuild the library")
            fn.argtypes = argtypes
            fn.restype = _c_int
        _lib = lib
        return lib


def available() -> bool:
    """Cached host probe: True iff the library loads and device 0 is a gfx950."""
    global _probe
    if _probe is None:
        try:
            _probe = load().tessera_gfx950_probe() == OK
        except LaneUnavailable:
            _probe = False
    return _probe


def check(rc: int, what: str) -> None:
    """Map a lane return code to the exception the reference's executors raise."""
    if rc == OK:
        return
    if rc == BAD_SHAPE:
        raise ValueError(f"{what}: the gfx950 lane rejected the shape/arguments")
    if rc == NO_DEVICE:
        raise LaneUnavailable(f"{what}: no usable gfx950 (MI355X) device")
    raise RuntimeError(f"{what}: device operation failed (rc={rc})")


def ptr(a: Optional[np.ndarray]) -> Optional[int]:
    return None if a is None else a.ctypes.data


def device_name() -> str:
    buf = ctypes.create_string_buffer(256)
    check(load().tessera_gfx950_device_name(buf, 256), "device_name")
    return buf.value.decode()


def device_cus() -> int:
    n = _c_int(0)
    check(load().tessera_gfx950_device_cus(ctypes.byref(n)), "device_cus")
    return n.value


def synchronize() -> None:
    check(load().tessera_gfx950_synchronize(), "synchronize")


class DeviceBuffer:
    """A raw device allocation owned by Python (freed on ``close`` / GC)."""

    def __init__(self, nbytes: int):
        self.nbytes = int(nbytes)
        p = _c_vp()
        check(load().tessera_gfx950_malloc(ctypes.byref(p), self.nbytes), "malloc")
        self.ptr = p.value

    @classmethod
    def from_host(cls, a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        buf = cls(a.nbytes)
        buf.upload(a)
        return buf

    def upload(self, a: np.ndarray) -> None:
        a = np.ascontiguousarray(a)
        if a.nbytes > self.nbytes:
            raise ValueError("upload larger than the device buffer")
        check(load().tessera_gfx950_memcpy_h2d(self.ptr, a.ctypes.data, a.nbytes), "memcpy_h2d")

    def download(self, shape, dtype) -> np.ndarray:
        out = np.empty(shape, dtype)
        if out.nbytes > self.nbytes:
            raise ValueError("download larger than the device buffer")
        check(load().tessera_gfx950_memcpy_d2h(out.ctypes.data, self.ptr, out.nbytes), "memcpy_d2h")
        return out

    def zero(self) -> None:
        check(load().tessera_gfx950_memset(self.ptr, 0, self.nbytes), "memset")

    def close(self) -> None:
        if getattr(self, "ptr", None):
            try:
                load().tessera_gfx950_free(self.ptr)
            finally:
                self.ptr = None

    def __del__(self):  # pragma: no cover - best effort
        try:
            self.close()
        except Exception:
            pass


class DeviceTimer:
    """HIP-event stopwatch on the default stream."""

    def __init__(self):
        p = _c_vp()
        check(load().tessera_gfx950_timer_create(ctypes.byref(p)), "timer_create")
        self._t = p.value

    def start(self, stream=None) -> None:
        check(load().tessera_gfx950_timer_start(self._t, stream), "timer_start")

    def stop(self, stream=None) -> None:
        check(load().tessera_gfx950_timer_stop(self._t, stream), "timer_stop")

    def elapsed_ms(self) -> float:
        ms = _c_f(0)
        check(load().tessera_gfx950_timer_elapsed_ms(self._t, ctypes.byref(ms)), "timer_elapsed")
        return float(ms.value)

    def close(self) -> None:
        if getattr(self, "_t", None):
            load().tessera_gfx950_timer_destroy(self._t)
            self._t = None

    def __del__(self):  # pragma: no cover
        try:
            self.close()
        except Exception:
            pass
