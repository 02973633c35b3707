"""The typed-descriptor seam: a ``submit`` hook for the host's native-launcher registry.

The reference's third way into a backend is ``runtime.register_native_launcher(target,
binary_formats=..., submit=fn)`` (``python/tessera/runtime.py:279-306``): an artifact that
carries a native image and a launch descriptor is validated by the host and handed to the
hook registered for the image's exact target as
``submit(image, descriptor, buffers, scalars, stream)`` (``:30900-30955``); whatever the
hook returns becomes the launch's ``output``, and anything it raises becomes a
``device_error`` result.  The gfx1151 hook (``:3564-3908``) loads a compiler-built HSACO and
launches ``descriptor.entry_symbol`` from it.

This lane's kernels are compiled ahead of time into one shared library, so its images are of
the ``shared_object`` format (the format the reference's Apple GPU hook registers, ``:4715``):
``descriptor.entry_symbol`` names one of the library's C entry points and
``descriptor.abi_id`` says how the buffers, scalars and provenance map onto its arguments.
The ABI identifiers are the reference's (``compiler/rocm_native.py:55-69``), plus a bf16
matmul that the gfx1151 lane does not have.

Nothing here is a registry: :func:`register` calls the host's own function.
"""
from __future__ import annotations

from typing import Any, Mapping

import numpy as np

from . import bf16 as _bf16
from . import lane as _lane
from . import ops as _ops

TARGET = "rocm_gfx950"
BINARY_FORMATS = ("shared_object",)

MATMUL_F16_F32_ABI = "tessera.rocm.matmul.a_b_o_m_n_k.f16_f32.v1"
MATMUL_BF16_F32_ABI = "tessera.rocm.matmul.a_b_o_m_n_k.bf16_f32.v1"
ATTN_F16_ABI = "tessera.rocm.attention.q_k_v_o_dims.f16_f32out.v1"
ATTN_BF16_ABI = "tessera.rocm.attention.q_k_v_o_dims.bf16_f32out.v1"
MOE_DISPATCH_F32_ABI = "tessera.rocm.moe_dispatch.x_token_o_t_s_h.f32_i32.v1"

# abi id -> (kind, storage, the entry points a descriptor of that ABI may name)
_ABIS = {
    MATMUL_F16_F32_ABI: ("matmul", "f16", ("tessera_gfx950_gemm_f16",)),
    MATMUL_BF16_F32_ABI: ("matmul", "bf16", ("tessera_gfx950_gemm_bf16",)),
    ATTN_F16_ABI: ("attention", "f16", ("tessera_gfx950_flash_attn_gqa_f16", "tessera_gfx950_flash_attn_ext_f16",
                                        "tessera_gfx950_flash_attn_bias_f16")),
    ATTN_BF16_ABI: ("attention", "bf16", ("tessera_gfx950_flash_attn_gqa_bf16", "tessera_gfx950_flash_attn_ext_bf16",
                                          "tessera_gfx950_flash_attn_bias_bf16")),
    MOE_DISPATCH_F32_ABI: ("moe_dispatch", "f32", ("tessera_gfx950_moe_dispatch",)),
}


def supported_abis() -> tuple:
    return tuple(_ABIS)


def _is_storage(array: Any, storage: str) -> bool:
    if storage == "f16":
        return getattr(array, "dtype", None) == np.float16
    return _bf16.is_bf16(array)


def _filled(output: Any, result: np.ndarray) -> Any:
    """The host binds an output buffer; the result goes into it and it is what comes back."""
    if not output.flags.c_contiguous:
        raise RuntimeError("gfx950 native output must be contiguous")
    np.copyto(output, result.reshape(output.shape))
    return output


def submit(image: Any, descriptor: Any, buffers: Mapping[str, Any], scalars: Mapping[str, object], stream: Any) -> Any:
    """Run one typed launch.  ``buffers`` maps the descriptor's buffer names to host arrays
    (inputs first, the output last, by ordinal); shapes and dtypes are checked against the
    descriptor's scalars / provenance before anything touches the device, and a mismatch
    raises ``RuntimeError`` as the reference's hooks do."""
    del image, stream     # one ahead-of-time library, default stream, synchronised on return
    spec = _ABIS.get(descriptor.abi_id)
    if spec is None:
        raise RuntimeError(f"unsupported gfx950 descriptor ABI {descriptor.abi_id!r}")
    kind, storage, entries = spec
    if descriptor.entry_symbol not in entries:
        raise RuntimeError(f"gfx950 descriptor ABI {descriptor.abi_id!r} cannot launch {descriptor.entry_symbol!r}")
    if descriptor.entry_symbol not in _lane.exported_symbols():
        raise RuntimeError(f"gfx950 native symbol {descriptor.entry_symbol!r} not found")
    ordered = sorted(descriptor.buffers, key=lambda item: item.ordinal)
    provenance = getattr(descriptor, "provenance", None) or {}

    if kind == "matmul":
        if len(ordered) != 3:
            raise RuntimeError("gfx950 matmul descriptor requires 3 buffers")
        a, b, output = (buffers[item.name] for item in ordered)
        m, n, k = (int(scalars[key]) for key in ("M", "N", "K"))
        if (tuple(a.shape) != (m, k) or tuple(b.shape) != (k, n) or tuple(output.shape) != (m, n)
                or not _is_storage(a, storage) or not _is_storage(b, storage) or output.dtype != np.float32):
            raise RuntimeError("gfx950 matmul arrays disagree with M/N/K or descriptor dtype")
        return _filled(output, _ops.gemm(a, b, out="f32"))

    if kind == "attention":
        with_bias = bool(provenance.get("bias"))
        if len(ordered) != (5 if with_bias else 4):
            raise RuntimeError(f"gfx950 attention descriptor requires {5 if with_bias else 4} buffers")
        q, key, value = (buffers[item.name] for item in ordered[:3])
        bias = buffers[ordered[3].name] if with_bias else None
        output = buffers[ordered[-1].name]
        b_, hq, hkv, sq, sk, d, dv = (int(x) for x in provenance["shape"])
        if (tuple(q.shape) != (b_, hq, sq, d) or tuple(key.shape) != (b_, hkv, sk, d)
                or tuple(value.shape) != (b_, hkv, sk, dv) or tuple(output.shape) != (b_, hq, sq, dv) or dv != d
                or not all(_is_storage(x, storage) for x in (q, key, value)) or output.dtype != np.float32):
            raise RuntimeError("gfx950 attention arrays disagree with descriptor shape/dtype")
        if with_bias and (tuple(bias.shape) != (b_, hq, sq, sk) or bias.dtype != np.float32):
            raise RuntimeError("gfx950 attention bias disagrees with descriptor")
        if float(provenance.get("dropout_p", 0.0)) > 0.0:
            raise RuntimeError("gfx950 attention has no dropout form")
        # the carrier stores an inclusive left offset (key >= q - left); the kernel takes
        # the band width, left + 1 (runtime.py:3857-3864)
        left = int(provenance.get("window_left", -1))
        result = _ops._attention(q, key, value, float(provenance["scale"]), bool(provenance["causal"]), False, "f32",
                                 True, window=left + 1 if left >= 0 else 0,
                                 logit_softcap=float(provenance.get("softcap", 0.0)), attn_bias=bias)
        return _filled(output, result)

    # moe_dispatch: x f32 (T,H), token i32 (S) -> out f32 (S,H), an exact gather
    if len(ordered) != 3:
        raise RuntimeError("gfx950 MoE dispatch descriptor requires 3 buffers")
    x, token, output = (buffers[item.name] for item in ordered)
    tokens, slots, hidden = (int(scalars[key]) for key in ("T", "S", "H"))
    if (tuple(x.shape) != (tokens, hidden) or tuple(token.shape) != (slots,) or tuple(output.shape) != (slots, hidden)
            or tokens <= 0 or slots <= 0 or hidden <= 0 or np.any(token < 0) or np.any(token >= tokens)):
        raise RuntimeError("gfx950 MoE dispatch arrays disagree with descriptor scalars")
    if x.dtype != np.float32 or token.dtype != np.int32 or output.dtype != np.float32:
        raise RuntimeError("gfx950 MoE dispatch requires f32 input/output and i32 indices")
    if not output.flags.c_contiguous:
        raise RuntimeError("gfx950 native output must be contiguous")
    xa, ta = np.ascontiguousarray(x), np.ascontiguousarray(token)
    _lane.check(_lane.load().tessera_gfx950_moe_dispatch(xa.ctypes.data, ta.ctypes.data, output.ctypes.data,
                                                         tokens, slots, hidden, 4), "moe_dispatch")
    return output


def register(runtime_module: Any, *, replace: bool = False) -> str:
    """Register :func:`submit` with the host (its ``runtime`` module, or any object with a
    ``register_native_launcher(target, *, binary_formats, submit, replace)``); returns the target."""
    runtime_module.register_native_launcher(TARGET, binary_formats=BINARY_FORMATS, submit=submit, replace=replace)
    return TARGET
