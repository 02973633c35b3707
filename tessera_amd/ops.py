"""The dense-op surface of ``tessera.ops`` / ``tessera.nn.functional`` on the
gfx950 lane.

Same names, argument meaning and error behaviour as the reference's numpy
definitions, but every function computes on the MI355X through the C ABI
(:mod:`tessera_amd.lane`).  There is no CPU path: without the library or the
device the calls raise :class:`~tessera_amd.lane.LaneUnavailable`.

Reference definitions mirrored here (paths under ``python/tessera``):

=====================  ==========================================================
``gemm`` / ``matmul``   ``__init__.py:239-254`` + storage rule ``:5783-5855``
``batched_gemm``
``flash_attn``          ``__init__.py:1304-1356``
``gqa_attention``       ``nn/functional.py:349-356``
``grouped_gemm``        ``__init__.py:291-351``
``moe_swiglu_block``    ``__init__.py:592-616``
``route_tokens``        ``distributed/moe.py:119-206`` (+ transport ABI
                        ``compiler/moe_transport.py:194-273``)
``moe_dispatch`` /      ``stdlib/moe.py:117-134``, ``runtime.py:1791-1824``
``moe_combine``
``moe_layer``           ``nn/functional.py:403-490``
``quantize_fp8``        ``__init__.py:3340-3374``
``quantize_int8_per_channel`` / ``w8a8_matmul``
                        ``compiler/smoothquant.py:79-84,115-124``
=====================  ==========================================================
"""
from __future__ import annotations

import ctypes
import math
from dataclasses import dataclass
from typing import NamedTuple, Optional

import numpy as np

from . import bf16 as _bf16
from . import lane as _lane
from .bf16 import BF16Array

GROUPED_KINDS = ("contiguous", "dense", "masked", "k_grouped")
_SUPPORTED_GROUPED_KINDS = ("contiguous", "dense")


# ---------------------------------------------------------------------------
# storage helpers
# ---------------------------------------------------------------------------


def _storage(a, b=None) -> str:
    """'f16' or 'bf16' — the 16-bit storage dtype of the operand(s)."""
    def one(x):
        if _bf16.is_bf16(x):
            return "bf16"
        if getattr(x, "dtype", None) == np.float16:
            return "f16"
        raise ValueError(
            f"gfx950 lane handles f16/bf16 storage (f32 accumulate); got {getattr(x, 'dtype', type(x))}")
    s = one(a)
    if b is not None and one(b) != s:
        raise ValueError("operands must share one 16-bit storage dtype")
    return s


def _bits(a) -> np.ndarray:
    if _bf16.is_bf16(a):
        return _bf16.as_bits(a)
    return np.ascontiguousarray(a, np.float16).view(np.uint16)


def _wrap(bits: np.ndarray, storage: str):
    return bits.view(BF16Array) if storage == "bf16" else bits.view(np.float16)


def _unbox(x):
    return x._data if hasattr(x, "_data") else x


# ---------------------------------------------------------------------------
# GEMM
# ---------------------------------------------------------------------------


#: activations of ``ops.fused_epilogue`` (``__init__.py:2665-2670``; anything else is the identity there)
_EPILOGUE_ACTIVATIONS = {"linear": "none", "none": "none", None: "none", "gelu": "gelu", "relu": "relu", "silu": "silu"}


def _gemm_with_epilogue(A, B, epilogue: dict, out: str):
    """``gemm(A, B, epilogue={...})`` (``__init__.py:239-248, 2658-2675``): bias add and
    activation on the f32 product, inside the GEMM kernel, before the storage rule rounds."""
    ep = dict(epilogue)
    bias = ep.pop("bias", None)
    act = ep.pop("activation", "linear")
    for key in ("residual", "cast_dtype"):
        if ep.pop(key, None) is not None:
            raise NotImplementedError(f"gemm(epilogue=): {key!r} is not fused on the gfx950 lane")
    if ep.pop("dropout_p", 0.0):
        raise NotImplementedError("gemm(epilogue=): dropout is not fused on the gfx950 lane")
    if act not in _EPILOGUE_ACTIVATIONS:
        act = "linear"                                  # the reference applies no activation for other names
    A, B = _unbox(A), _unbox(B)
    st = _storage(A, B)
    if _bits(B).ndim != 2:
        raise NotImplementedError("gemm(epilogue=) with a batched B is not fused on the gfx950 lane")
    a = _bits(A)
    N = _bits(B).shape[1]
    if bias is not None:
        bias = np.ascontiguousarray(np.broadcast_to(np.asarray(_unbox(bias), np.float32), (N,)))
    a2 = _wrap(np.ascontiguousarray(a.reshape(-1, a.shape[-1])), st)
    d = fused_gemm(a2, B, bias, _EPILOGUE_ACTIVATIONS[act]).reshape(a.shape[:-1] + (N,))
    if out == "f32":
        return d
    return _bf16.from_float32(d) if st == "bf16" else d.astype(np.float16)


def gemm(A, B, epilogue=None, *, out: str = "storage"):
    """``A @ B`` with f32 accumulate.  16-bit operands; leading dims of ``A`` (and
    of ``B`` when it is not rank 2) are batch dims and must match.

    ``out="storage"`` stores the result in the operands' storage dtype (the
    ``ops.gemm`` rule for reduced-precision operands); ``out="f32"`` returns the
    f32 accumulators (the executors' contract).  ``epilogue`` is the reference's
    ``fused_epilogue`` dict (``bias``, ``activation``), applied to the f32 product."""
    if out not in ("storage", "f32"):
        raise ValueError("out must be 'storage' or 'f32'")
    if epilogue:
        return _gemm_with_epilogue(A, B, epilogue, out)
    A, B = _unbox(A), _unbox(B)
    st = _storage(A, B)
    a, b = _bits(A), _bits(B)
    if a.ndim < 2 or b.ndim < 2:
        raise ValueError("gemm needs operands of rank >= 2")
    M, K = a.shape[-2:]
    if b.shape[-2] != K:
        raise ValueError(f"gemm: K mismatch — A {a.shape} @ B {b.shape}")
    N = b.shape[-1]
    lead = a.shape[:-2]
    batch = int(np.prod(lead)) if lead else 1
    if b.ndim > 2:
        if b.shape[:-2] != lead:
            raise ValueError(f"batched gemm: leading dims differ — A {a.shape} @ B {b.shape}")
    elif batch > 1:
        # one weight for every batch: fold the batch into M
        M = batch * M
        batch = 1
        a = a.reshape(M, K)
    if out not in ("storage", "f32"):
        raise ValueError("out must be 'storage' or 'f32'")
    lib = _lane.load()
    f32 = out == "f32"
    shape = tuple(A.shape[:-1]) + (N,)
    if batch == 1:
        d = np.empty((M, N), np.float32 if f32 else np.uint16)
        name = f"tessera_gfx950_gemm_{st}" + ("" if f32 else f"_{st}")
        _lane.check(getattr(lib, name)(a.ctypes.data, b.ctypes.data, d.ctypes.data, M, N, K), "gemm")
        return d.reshape(shape) if f32 else _wrap(d.reshape(shape), st)
    # the batched entry point keeps f32 accumulators; the storage rule rounds after
    d32 = np.empty((batch, M, N), np.float32)
    _lane.check(getattr(lib, f"tessera_gfx950_batched_gemm_{st}")(
        a.ctypes.data, b.ctypes.data, d32.ctypes.data, batch, M, N, K), "batched_gemm")
    if f32:
        return d32.reshape(shape)
    if st == "bf16":
        return _bf16.from_float32(d32).reshape(shape)
    return d32.astype(np.float16).reshape(shape)


matmul = gemm
batched_gemm = gemm

#: activation codes of the fused-epilogue entry points
ACTIVATIONS = {"none": 0, "relu": 1, "gelu": 2, "silu": 3, "sigmoid": 4, "tanh": 5}


def _activation_code(name) -> int:
    key = str(name or "none")
    if key not in ACTIVATIONS:
        raise ValueError(f"activation must be one of {sorted(ACTIVATIONS)}; got {name!r}")
    return ACTIVATIONS[key]


def fused_gemm(A, B, bias=None, activation: str = "none") -> np.ndarray:
    """``act(A @ B + bias)`` in one kernel → f32.  Rank-2 16-bit operands, ``bias``
    f32 ``[N]`` or None, ``activation`` from the reference's epilogue vocabulary
    (none / relu / gelu / silu / sigmoid / tanh)."""
    A, B = _unbox(A), _unbox(B)
    st = _storage(A, B)
    a, b = _bits(A), _bits(B)
    if a.ndim != 2 or b.ndim != 2 or a.shape[1] != b.shape[0]:
        raise ValueError(f"fused_gemm needs rank-2 operands with matching K; got {a.shape} @ {b.shape}")
    M, K = a.shape
    N = b.shape[1]
    act = _activation_code(activation)
    bias_arr = None
    if bias is not None:
        bias_arr = np.ascontiguousarray(bias, np.float32)
        if bias_arr.shape != (N,):
            raise ValueError(f"bias must have shape ({N},) (one per output column); got {bias_arr.shape}")
    d = np.empty((M, N), np.float32)
    fn = getattr(_lane.load(), f"tessera_gfx950_gemm_bias_act_{st}")
    _lane.check(fn(a.ctypes.data, b.ctypes.data, bias_arr.ctypes.data if bias_arr is not None else None, act,
                   d.ctypes.data, M, N, K), "fused_gemm")
    return d


def gated_gemm(A, Wg, Wu, gate_act: str = "silu") -> np.ndarray:
    """``act(A @ Wg) * (A @ Wu)`` in one kernel → f32 ``[M, H]`` (the gated MLP
    projection; ``silu`` gives the SwiGLU gate)."""
    A, Wg, Wu = _unbox(A), _unbox(Wg), _unbox(Wu)
    st = _storage(A, Wg)
    if _storage(A, Wu) != st:
        raise ValueError("operands must share one 16-bit storage dtype")
    a, g, u = _bits(A), _bits(Wg), _bits(Wu)
    if a.ndim != 2 or g.ndim != 2 or g.shape != u.shape or a.shape[1] != g.shape[0]:
        raise ValueError(f"gated_gemm needs A (M,K) and Wg, Wu (K,H); got {a.shape}, {g.shape}, {u.shape}")
    act = _activation_code(gate_act)
    if act == 0:
        raise ValueError("gate activation must be a unary pointwise op")
    M, K = a.shape
    H = g.shape[1]
    d = np.empty((M, H), np.float32)
    fn = getattr(_lane.load(), f"tessera_gfx950_gated_gemm_{st}")
    _lane.check(fn(a.ctypes.data, g.ctypes.data, u.ctypes.data, act, d.ctypes.data, M, H, K), "gated_gemm")
    return d


def gemm_i8(A, B) -> np.ndarray:
    """``int32(A) @ int32(B)`` for int8 operands — exact."""
    a = np.ascontiguousarray(_unbox(A))
    b = np.ascontiguousarray(_unbox(B))
    if a.dtype != np.int8 or b.dtype != np.int8:
        raise ValueError("gemm_i8 needs int8 operands")
    if a.ndim != 2 or b.ndim != 2 or a.shape[1] != b.shape[0]:
        raise ValueError(f"gemm_i8 needs rank-2 operands with matching K; got {a.shape} @ {b.shape}")
    M, K = a.shape
    N = b.shape[1]
    c = np.empty((M, N), np.int32)
    _lane.check(_lane.load().tessera_gfx950_gemm_i8_i32(a.ctypes.data, b.ctypes.data, c.ctypes.data, M, N, K),
                "gemm_i8")
    return c


# ---------------------------------------------------------------------------
# attention
# ---------------------------------------------------------------------------


def _attention(Q, K, V, scale, causal, return_lse, out, allow_gqa, window=0, logit_softcap=0.0, attn_bias=None):
    Q, K, V = _unbox(Q), _unbox(K), _unbox(V)
    st = _storage(Q, K)
    if _storage(V) != st:
        raise ValueError("Q, K, V must share one storage dtype")
    q, k, v = _bits(Q), _bits(K), _bits(V)
    if q.ndim < 2 or k.ndim < 2 or v.ndim < 2:
        raise ValueError("flash_attn Q/K/V must be at least rank 2 ([..., S, D])")
    D = q.shape[-1]
    if D <= 0 or D % 16 != 0:
        raise ValueError(f"gfx950 flash_attn lane needs head_dim a positive multiple of 16; got {D}")
    Sq, Sk = q.shape[-2], k.shape[-2]
    if v.shape != k.shape or k.shape[-1] != D:
        raise ValueError(f"flash_attn requires V to match K and Q's head dim; got Q{q.shape} K{k.shape} V{v.shape}")
    Hq = q.shape[-3] if q.ndim >= 3 else 1
    Hkv = k.shape[-3] if k.ndim >= 3 else 1
    Bq = int(np.prod(q.shape[:-3])) if q.ndim > 3 else 1
    Bk = int(np.prod(k.shape[:-3])) if k.ndim > 3 else 1
    if Bq != Bk:
        raise ValueError("flash_attn: batch dims of Q and K differ")
    if Hq != Hkv:
        if not allow_gqa:
            raise ValueError(f"flash_attn needs matching head counts; got {Hq} vs {Hkv} (use gqa_attention)")
        if Hkv <= 0 or Hq % Hkv != 0:
            raise ValueError(f"GQA needs query-heads ({Hq}) divisible by kv-heads ({Hkv})")
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    window = int(window or 0)
    softcap = float(logit_softcap or 0.0)
    if window < 0:
        raise ValueError(f"flash_attn window must be a non-negative width; got {window}")
    if softcap < 0:
        raise ValueError(f"flash_attn logit_softcap must be non-negative; got {softcap}")
    bias = None
    if attn_bias is not None:
        # host-broadcast to [..., Hq, Sq, Sk], as the reference's executor does (runtime.py:7341-7355)
        try:
            bias = np.broadcast_to(np.asarray(_unbox(attn_bias), dtype=np.float32), tuple(q.shape[:-2]) + (Sq, Sk))
        except ValueError:
            raise ValueError(f"flash_attn attn_bias {np.asarray(attn_bias).shape} is not broadcastable to "
                             f"{tuple(q.shape[:-2]) + (Sq, Sk)}") from None
        bias = np.ascontiguousarray(bias, dtype=np.float32)
    o = np.empty(q.shape, np.float32)
    lse = np.empty(q.shape[:-1], np.float32) if return_lse else None
    if bias is not None:
        fn = getattr(_lane.load(), f"tessera_gfx950_flash_attn_bias_{st}")
        rc = fn(q.ctypes.data, k.ctypes.data, v.ctypes.data, bias.ctypes.data, o.ctypes.data, _lane.ptr(lse),
                Bq, Hq, Hkv, Sq, Sk, D, float(scale), 1 if causal else 0, window, softcap)
    elif window or softcap:
        fn = getattr(_lane.load(), f"tessera_gfx950_flash_attn_ext_{st}")
        rc = fn(q.ctypes.data, k.ctypes.data, v.ctypes.data, o.ctypes.data, _lane.ptr(lse),
                Bq, Hq, Hkv, Sq, Sk, D, float(scale), 1 if causal else 0, window, softcap)
    else:
        fn = getattr(_lane.load(), f"tessera_gfx950_flash_attn_gqa_{st}")
        rc = fn(q.ctypes.data, k.ctypes.data, v.ctypes.data, o.ctypes.data, _lane.ptr(lse),
                Bq, Hq, Hkv, Sq, Sk, D, float(scale), 1 if causal else 0)
    _lane.check(rc, "flash_attn")
    if out == "storage":
        o = _bf16.from_float32(o) if st == "bf16" else o.astype(np.float16)
    elif out != "f32":
        raise ValueError("out must be 'storage' or 'f32'")
    return (o, lse) if return_lse else o


def flash_attn_backward(dO, Q, K, V, scale=None, causal: bool = False):
    """``(dQ, dK, dV)`` of ``softmax(scale * Q K^T, causal) V`` for the cotangent
    ``dO`` — f32 arrays shaped like ``Q``, ``K``, ``V``.  ``Q``/``dO``
    ``[..., Hq, Sq, D]``, ``K``/``V`` ``[..., Hkv, Sk, D]`` in one 16-bit storage
    dtype; with ``Hkv < Hq`` the gradients of a KV head sum over its query heads.
    The forward is recomputed on the device (nothing saved)."""
    dO, Q, K, V = _unbox(dO), _unbox(Q), _unbox(K), _unbox(V)
    st = _storage(Q, K)
    if _storage(V) != st or _storage(dO) != st:
        raise ValueError("dO, Q, K, V must share one storage dtype")
    g, q, k, v = _bits(dO), _bits(Q), _bits(K), _bits(V)
    for name, arr in (("dO", g), ("Q", q), ("K", k), ("V", v)):
        if arr.ndim < 2:
            raise ValueError(f"flash_attn backward {name} must be rank >= 2 ([..., S, D]); got {arr.shape}")
    D = q.shape[-1]
    if D <= 0 or D % 16 != 0:
        raise ValueError(f"gfx950 flash_attn backward needs head_dim a positive multiple of 16; got {D}")
    Hq = q.shape[-3] if q.ndim >= 3 else 1
    Hkv = k.shape[-3] if k.ndim >= 3 else 1
    if Hkv <= 0 or Hq % Hkv != 0:
        raise ValueError(f"flash_attn backward GQA needs query-heads ({Hq}) divisible by kv-heads ({Hkv})")
    if v.shape != k.shape or g.shape != q.shape or k.shape[-1] != D or q.shape[:-3] != k.shape[:-3]:
        raise ValueError("flash_attn backward requires V==K, dO==Q, matching batch dims and a shared head_dim; "
                         f"got Q{q.shape} K{k.shape} V{v.shape} dO{g.shape}")
    Bq = int(np.prod(q.shape[:-3])) if q.ndim > 3 else 1
    Sq, Sk = q.shape[-2], k.shape[-2]
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    dq = np.empty(q.shape, np.float32)
    dk = np.empty(k.shape, np.float32)
    dv = np.empty(k.shape, np.float32)
    fn = getattr(_lane.load(), f"tessera_gfx950_flash_attn_bwd_{st}")
    rc = fn(g.ctypes.data, q.ctypes.data, k.ctypes.data, v.ctypes.data, dq.ctypes.data, dk.ctypes.data,
            dv.ctypes.data, Bq, Hq, Hkv, Sq, Sk, D, float(scale), 1 if causal else 0)
    _lane.check(rc, "flash_attn_backward")
    return dq, dk, dv


def flash_attn(Q, K=None, V=None, scale=None, causal: bool = False, cache=None, dropout_p: float = 0.0, params=None,
               deterministic=None, seed=None, attn_bias=None, kv_state=None, *, return_lse: bool = False,
               out: str = "storage", window: int = 0, logit_softcap: float = 0.0):
    """``softmax(scale * Q K^T, causal) V``.  Q/K/V ``[..., H, S, D]`` 16-bit; the
    causal mask is bottom-right aligned (key ``j`` visible to query ``i`` iff
    ``j <= i + max(Sk - Sq, 0)``).  Head counts must match (as in the reference).
    ``attn_bias`` (f32, broadcastable to ``[..., H, Sq, Sk]``) is added to the scaled
    (and, with ``logit_softcap``, capped) scores before the softmax.  The positional
    parameters are the reference's (``__init__.py:1304-1317``); the kernel is
    deterministic and has no dropout, and paged KV state is another lane's."""
    if not 0.0 <= float(dropout_p) < 1.0:
        raise ValueError("dropout_p must be in [0.0, 1.0)")
    if dropout_p:
        raise NotImplementedError("flash_attn: dropout is not implemented on the gfx950 lane")
    if kv_state is not None or cache is not None:
        raise NotImplementedError("flash_attn: paged KV state / cache objects are not served by the gfx950 lane")
    if K is None or V is None:
        raise ValueError("flash_attn needs K and V")
    return _attention(Q, K, V, scale, causal, return_lse, out, False, window, logit_softcap, attn_bias)


def gqa_attention(Q, K, V, num_query_heads=None, num_kv_heads=None, *, scale=None, causal: bool = False,
                  return_lse: bool = False, out: str = "storage", window: int = 0, logit_softcap: float = 0.0,
                  attn_bias=None):
    """Grouped-query attention (``nn/functional.py:349-356``): kv head of query head ``h``
    is ``h // (Hq / Hkv)`` — identical to repeating K/V along the head axis, which is what
    the reference does with ``num_query_heads // num_kv_heads``.  The head counts may be left
    out (they are read off the operands); when given they must agree with the operands."""
    if num_query_heads is not None or num_kv_heads is not None:
        if num_query_heads is None or num_kv_heads is None:
            raise ValueError("gqa_attention: give both num_query_heads and num_kv_heads, or neither")
        nq, nkv = int(num_query_heads), int(num_kv_heads)
        if nkv <= 0 or nq % nkv != 0:
            raise ValueError("num_query_heads must be divisible by num_kv_heads")
        hq, hkv = _bits(_unbox(Q)).shape[-3], _bits(_unbox(K)).shape[-3]
        if hkv * (nq // nkv) != hq:
            raise ValueError(f"gqa_attention: K/V with {hkv} heads repeated {nq // nkv} times do not match "
                             f"Q's {hq} heads")
    return _attention(Q, K, V, scale, causal, return_lse, out, True, window, logit_softcap, attn_bias)


def mqa_attention(Q, K, V, **kwargs):
    """Multi-query attention (``nn/functional.py:359-360``): one K/V head shared by every query head."""
    return gqa_attention(Q, K, V, num_query_heads=_bits(_unbox(Q)).shape[-3], num_kv_heads=1, **kwargs)


# ---------------------------------------------------------------------------
# MoE
# ---------------------------------------------------------------------------


def _offsets(group_sizes, total: int, what: str) -> np.ndarray:
    gs = np.asarray(group_sizes).astype(np.int64).reshape(-1)
    if gs.size <= 0 or np.any(gs < 0) or int(gs.sum()) != total:
        raise ValueError(f"{what}: group_sizes sum {int(gs.sum()) if gs.size else 0} != T={total}")
    off = np.concatenate((np.zeros(1, np.int64), np.cumsum(gs)))
    if int(off[-1]) > np.iinfo(np.int32).max:
        raise ValueError("grouped expert offsets exceed the int32 device ABI")
    return np.ascontiguousarray(off, np.int32)


def grouped_gemm(x, weights, group_sizes, *, kind: str = "contiguous", alignment=None, quant=None,
                 out: str = "storage"):
    """Ragged grouped matmul: row block ``e`` of the result is
    ``x[block e] @ weights[e]``.  ``x`` ``(T, K)`` sorted by expert, ``weights``
    ``(E, K, N)``, ``group_sizes`` ``(E,)`` summing to ``T``."""
    if kind not in GROUPED_KINDS:
        raise ValueError(f"grouped_gemm: unknown kind {kind!r}; expected one of {GROUPED_KINDS}")
    if kind not in _SUPPORTED_GROUPED_KINDS:
        raise NotImplementedError(
            f"grouped_gemm: kind={kind!r} is not implemented — supported: "
            f"{', '.join(_SUPPORTED_GROUPED_KINDS)}")
    x, weights = _unbox(x), _unbox(weights)
    st = _storage(x, weights)
    xa, w = _bits(x), _bits(weights)
    gs = np.asarray(group_sizes).astype(np.int64).reshape(-1)
    if quant is not None:
        if st != "bf16":
            raise ValueError("grouped_gemm(quant=) on the gfx950 lane takes bf16 storage")
        scheme = GROUPED_QUANT_SCHEMES.get(str(quant).lower())
        if scheme is None:
            raise ValueError(f"grouped_gemm: quant {quant!r} has no grouped path; expected one of "
                             f"{tuple(GROUPED_QUANT_SCHEMES)}")
        if scheme == ("fp8_e4m3", "fp8_e4m3"):
            return _grouped_gemm_fp8(x, weights, xa, w, gs, quant, alignment, out)
        return _grouped_gemm_grid(x, weights, xa, w, gs, scheme, alignment, out)
    if alignment is not None:
        al = int(alignment)
        if al <= 0 or np.any(gs % al != 0):
            raise ValueError(f"grouped_gemm: every group size must be a multiple of alignment={alignment}")
    if xa.ndim != 2:
        raise ValueError(f"grouped_gemm: x must be (T, K); got {xa.shape}")
    if w.ndim != 3 or w.shape[0] != gs.shape[0]:
        raise ValueError(f"grouped_gemm: weights {w.shape} must be (E, K, N) with E == len(group_sizes)={gs.shape[0]}")
    if w.shape[1] != xa.shape[1]:
        raise ValueError(f"grouped_gemm: K mismatch — x K={xa.shape[1]}, weights K={w.shape[1]}")
    T, K = xa.shape
    E, _, N = w.shape
    off = _offsets(gs, T, "grouped_gemm")
    f32 = out == "f32"
    y = np.zeros((T, N), np.float32 if f32 else np.uint16)
    name = f"tessera_gfx950_grouped_gemm_{st}" + ("_f32" if f32 else "")
    _lane.check(getattr(_lane.load(), name)(xa.ctypes.data, w.ctypes.data, off.ctypes.data, y.ctypes.data, T, K, N, E),
                "grouped_gemm")
    return y if f32 else _wrap(y, st)


def _nvfp4_round(x32: np.ndarray, want_scales: bool = False):
    """x f32 (..., n) rounded onto the NVFP4 grid on the device → (dequantised f32,
    dequantised bf16 bits, scales or None)."""
    x32 = np.ascontiguousarray(x32, np.float32)
    n = x32.shape[-1]
    rows = int(x32.size // n) if n else 0
    if rows <= 0 or n <= 0:
        raise ValueError("quantize_nvfp4 needs a non-empty array")
    dq = np.empty(x32.shape, np.float32)
    dq16 = np.empty(x32.shape, np.uint16)
    scales = np.empty(x32.shape[:-1] + (-(-n // 16),), np.float32) if want_scales else None
    _lane.check(_lane.load().tessera_gfx950_fake_quantize_nvfp4_f32(
        x32.ctypes.data, rows, n, dq.ctypes.data, dq16.ctypes.data, scales.ctypes.data if want_scales else None),
        "quantize_nvfp4")
    return dq, dq16, scales


def quantize_nvfp4(x, *, block_size: int = 16):
    """NVFP4 — block-scaled E2M1 with one e4m3 scale per 16 elements of the last axis
    (``__init__.py:3472-3500``).  Returns ``(x_q_as_fp32, scales)`` like the reference:
    the values already dequantised, and the block scales as f32."""
    if int(block_size) != 16:
        raise NotImplementedError("the gfx950 lane rounds to NVFP4 in blocks of 16 (the format's block size)")
    x = _unbox(x)
    x32 = x.to_float32() if isinstance(x, BF16Array) else np.asarray(x, np.float32)
    if x32.shape[-1] % 16 != 0:
        raise ValueError(f"last dim {x32.shape[-1]} must be divisible by block_size 16 for NVFP4")
    dq, _, scales = _nvfp4_round(x32, want_scales=True)
    return dq, scales


def dequantize_nvfp4(x_q, scales=None, *, block_size: int = 16):
    """Inverse of :func:`quantize_nvfp4`, which already returns dequantised values
    (``__init__.py:3502-3504``)."""
    return np.asarray(x_q, np.float32)


#: (max_normal, mantissa_bits, min_exp) of the per-tensor float grids
#: (``runtime.py:16939-16946``): IEEE gradual underflow for fp8, the pure mantissa snap for
#: fp6 and fp4.
FP_FORMATS = {"e4m3": (448.0, 3, -6), "e5m2": (57344.0, 2, -14), "e2m3": (7.5, 3, -126), "e3m2": (28.0, 2, -126),
              "e2m1": (6.0, 1, -126)}


def _fp_round(x32: np.ndarray, fmt: str, scale=None, want_grid: bool = False):
    """x f32 snapped to a per-tensor float grid on the device → (dequantised f32, grid values
    as bf16 bits or None, scale f32)."""
    mx, mant, min_exp = FP_FORMATS[fmt]
    x32 = np.ascontiguousarray(x32, np.float32)
    if x32.size == 0:
        raise ValueError("quantize: empty array")
    dq = np.empty(x32.shape, np.float32)
    g16 = np.empty(x32.shape, np.uint16) if want_grid else None
    s_out = np.zeros(1, np.float32)
    _lane.check(_lane.load().tessera_gfx950_fake_quantize_fp_f32(
        x32.ctypes.data, x32.size, mx, mant, min_exp, 0.0 if scale is None else float(scale), dq.ctypes.data,
        g16.ctypes.data if want_grid else None, s_out.ctypes.data), "quantize_fp")
    return dq, g16, np.float32(s_out[0])


def fpquant(x, max_normal: float, mantissa_bits: int, min_exp: int) -> np.ndarray:
    """x f32 snapped to the float grid ``(max_normal, mantissa_bits, min_exp)``: the native
    lanes' grid kernel (``avx512_fpquant_f32.cpp:45-83``) on the device."""
    x32 = np.ascontiguousarray(_unbox(x), np.float32)
    out = np.empty(x32.shape, np.float32)
    if x32.size:
        _lane.check(_lane.load().tessera_gfx950_fpquant_f32(x32.ctypes.data, x32.size, float(max_normal), int(mantissa_bits),
                                                            int(min_exp), out.ctypes.data), "fpquant")
    return out


def _quantize_per_tensor(x, fmt: str, formats, scale):
    if fmt not in formats:
        raise ValueError("format must be " + " or ".join(repr(f) for f in formats) + f"; got {fmt!r}")
    x = _unbox(x)
    x32 = x.to_float32() if isinstance(x, BF16Array) else np.asarray(x, np.float32)
    dq, _, s = _fp_round(x32, fmt, scale)
    return dq, s


def quantize_fp6(x, *, format: str = "e3m2", scale=None):
    """Per-tensor symmetric fp6 quantisation (``__init__.py:3411-3435``) →
    ``(x_q_as_fp32, scale)``."""
    return _quantize_per_tensor(x, format, ("e2m3", "e3m2"), scale)


def quantize_fp4(x, *, format: str = "e2m1", scale=None):
    """Per-tensor symmetric fp4 quantisation (``__init__.py:3446-3464``) →
    ``(x_q_as_fp32, scale)``."""
    return _quantize_per_tensor(x, format, ("e2m1",), scale)


def dequantize_fp8(x_q, scale=None, *, format: str = "e4m3"):
    """The quantisers already return rescaled values (``__init__.py:3376-3392``)."""
    if format not in ("e4m3", "e5m2"):
        raise ValueError(f"format must be 'e4m3' or 'e5m2'; got {format!r}")
    return np.asarray(x_q, np.float32)


def dequantize_fp6(x_q, scale=None, *, format: str = "e3m2"):
    if format not in ("e2m3", "e3m2"):
        raise ValueError(f"format must be 'e2m3' or 'e3m2'; got {format!r}")
    return np.asarray(x_q, np.float32)


def dequantize_fp4(x_q, scale=None, *, format: str = "e2m1"):
    if format != "e2m1":
        raise ValueError(f"format must be 'e2m1'; got {format!r}")
    return np.asarray(x_q, np.float32)


#: ``quant=`` spellings of the grouped product → (activation format, weight format)
#: (``compiler/grouped_layout.py:320-332``)
GROUPED_QUANT_SCHEMES = {
    "fp8_e4m3": ("fp8_e4m3", "fp8_e4m3"), "fp8": ("fp8_e4m3", "fp8_e4m3"), "fp8_e5m2": ("fp8_e5m2", "fp8_e5m2"),
    "nvfp4": ("nvfp4", "nvfp4"), "fp8xfp4": ("fp8_e4m3", "nvfp4"), "fp8_e4m3xnvfp4": ("fp8_e4m3", "nvfp4"),
    "fp8_e5m2xnvfp4": ("fp8_e5m2", "nvfp4"),
}


def _grid_operand(a32: np.ndarray, dtype: str):
    """One 2-D operand rounded as the reference's ``_qdq_2d`` does
    (``compiler/grouped_layout.py:353-370``) → (values exact in bf16, as bits; the f32 factor
    that turns them into the dequantised operand)."""
    if dtype == "nvfp4":
        if a32.shape[-1] % 16 != 0:
            raise ValueError(f"last dim {a32.shape[-1]} must be divisible by block_size 16 for NVFP4")
        return _nvfp4_round(a32)[1], np.float32(1.0)
    _, g16, s = _fp_round(a32, "e5m2" if dtype == "fp8_e5m2" else "e4m3", want_grid=True)
    return g16, s


def _grouped_gemm_grid(x, weights, xa, w, gs, scheme, alignment, out):
    """The quantised grouped product for every scheme but plain e4m3: x is rounded as one
    tensor with the activation format and every expert's weight on its own with the weight
    format (``compiler/grouped_layout.py:373-392``), on the device.  The rounded values
    without their per-tensor scales are exact in bf16 (at most six significant bits), so one
    launch of the bf16 grouped kernel with f32 accumulation forms their product, and the
    scales (the activation's times expert e's) multiply the rows of group e afterwards: the
    reference's f32 product of the dequantised operands up to summation order and one
    rounding of the scale product."""
    act, wt = scheme
    if alignment is not None:
        al = int(alignment)
        if al <= 0 or np.any(gs % al != 0):
            raise ValueError(f"grouped_gemm: every group size must be a multiple of alignment={alignment}")
    if xa.ndim != 2 or w.ndim != 3 or w.shape[0] != gs.shape[0] or w.shape[1] != xa.shape[1]:
        raise ValueError(f"grouped_gemm: x {xa.shape} / weights {w.shape} / group_sizes {gs.shape} disagree")
    T, K = xa.shape
    E, _, N = w.shape
    off = _offsets(gs, T, "grouped_gemm")
    xf = x.to_float32() if isinstance(x, BF16Array) else _bf16.from_bits(xa).to_float32()
    wf = weights.to_float32() if isinstance(weights, BF16Array) else _bf16.from_bits(w).to_float32()
    xg, sx = _grid_operand(xf, act)
    if wt == "nvfp4":                                   # blocks along N within one expert's row: one call
        wg, sw = _grid_operand(wf, wt)[0], np.ones(E, np.float32)
    else:
        parts = [_grid_operand(wf[e], wt) for e in range(E)]
        wg = np.stack([p[0] for p in parts])
        sw = np.array([p[1] for p in parts], np.float32)
    f32 = out == "f32"
    lib = _lane.load()
    scales = (np.float32(sx) * sw).astype(np.float32)
    if np.all(scales == np.float32(1.0)):
        y = np.zeros((T, N), np.float32 if f32 else np.uint16)
        name = "tessera_gfx950_grouped_gemm_bf16" + ("_f32" if f32 else "")
        _lane.check(getattr(lib, name)(xg.ctypes.data, wg.ctypes.data, off.ctypes.data, y.ctypes.data, T, K, N, E),
                    "grouped_gemm")
        return y if f32 else y.view(BF16Array)
    acc = np.zeros((T, N), np.float32)
    _lane.check(lib.tessera_gfx950_grouped_gemm_bf16_f32(xg.ctypes.data, wg.ctypes.data, off.ctypes.data, acc.ctypes.data,
                                                         T, K, N, E), "grouped_gemm")
    y = np.zeros((T, N), np.float32 if f32 else np.uint16)
    if T:
        _lane.check(lib.tessera_gfx950_scale_groups_f32(acc.ctypes.data, off.ctypes.data, scales.ctypes.data, y.ctypes.data,
                                                        0 if f32 else 1, T, N, E), "grouped_gemm")
    return y if f32 else y.view(BF16Array)


def _grouped_gemm_fp8(x, weights, xa, w, gs, quant, alignment, out):
    """``quant="fp8_e4m3"``: x is quantised per tensor and every expert's weight per
    tensor (the reference's scale layout, ``compiler/grouped_layout.py:353-392``),
    and each group is one e4m3 GEMM with f32 accumulation, scaled by both scales.
    The reference dequantises on the host and multiplies in f32; the products of two
    e4m3 values are exact in f32, so the two differ only in summation order."""
    if alignment is not None:
        al = int(alignment)
        if al <= 0 or np.any(gs % al != 0):
            raise ValueError(f"grouped_gemm: every group size must be a multiple of alignment={alignment}")
    if xa.ndim != 2 or w.ndim != 3 or w.shape[0] != gs.shape[0] or w.shape[1] != xa.shape[1]:
        raise ValueError(f"grouped_gemm: x {xa.shape} / weights {w.shape} / group_sizes {gs.shape} disagree")
    T, K = xa.shape
    E, _, N = w.shape
    _offsets(gs, T, "grouped_gemm")
    xf = x.to_float32() if isinstance(x, BF16Array) else _bf16.from_bits(xa).to_float32()
    wf = weights.to_float32() if isinstance(weights, BF16Array) else _bf16.from_bits(w).to_float32()
    x_codes, sx = quantize_fp8_codes(xf)
    f32 = out == "f32"
    y = np.zeros((T, N), np.float32 if f32 else np.uint16)
    row = 0
    for e in range(E):
        n = int(gs[e])
        if n:
            w_codes, sw = quantize_fp8_codes(wf[e])
            y[row:row + n] = np.asarray(gemm_fp8(x_codes[row:row + n], w_codes, sx, sw, out="f32" if f32 else "bf16"),
                                        y.dtype)
        row += n
    return y if f32 else y.view(BF16Array)


def silu_mul(a, b):
    """``silu(a) * b`` elementwise (``__init__.py:559-574``) on 16-bit storage arrays of one
    shape; the result is rounded to the same storage dtype."""
    a, b = _unbox(a), _unbox(b)
    st = _storage(a, b)
    ab, bb = _bits(a), _bits(b)
    if ab.shape != bb.shape:
        raise ValueError(f"silu_mul: shapes differ — {ab.shape} vs {bb.shape}")
    outb = np.empty(ab.shape, np.uint16)
    if ab.size:
        _lane.check(getattr(_lane.load(), f"tessera_gfx950_silu_mul_{st}")(
            np.ascontiguousarray(ab).ctypes.data, np.ascontiguousarray(bb).ctypes.data, outb.ctypes.data, ab.size), "silu_mul")
    return _wrap(outb, st)


def moe_swiglu_block(x, w_gate, w_up, w_down, group_sizes, *, kind: str = "contiguous", alignment=None,
                     quant=None):
    """``gg(silu_mul(gg(x, Wg), gg(x, Wu)), Wd)`` over contiguous expert groups,
    every intermediate rounded to bf16 as the reference's storage rule does.  With
    ``quant`` every grouped product quantises its operands as ``grouped_gemm(quant=)``
    does, and the block is the reference's composition of the three products around
    ``silu_mul`` (``__init__.py:610-616``) instead of the fused kernel."""
    if kind not in GROUPED_KINDS:
        raise ValueError(f"moe_swiglu_block: unknown kind {kind!r}")
    if kind not in _SUPPORTED_GROUPED_KINDS:
        raise NotImplementedError("moe_swiglu_block: only contiguous/dense on the gfx950 lane")
    if quant is not None:
        gg = lambda a, w: grouped_gemm(a, w, group_sizes, kind=kind, alignment=alignment, quant=quant)
        return gg(silu_mul(gg(x, w_gate), gg(x, w_up)), w_down)
    x, w_gate, w_up, w_down = map(_unbox, (x, w_gate, w_up, w_down))
    for a in (x, w_gate, w_up, w_down):
        if _storage(a) != "bf16":
            raise ValueError("moe_swiglu_block on the gfx950 lane takes bf16 storage")
    xa, wg, wu, wd = map(_bits, (x, w_gate, w_up, w_down))
    if xa.ndim != 2 or wg.ndim != 3 or wu.shape != wg.shape or wd.ndim != 3:
        raise ValueError("moe_swiglu_block: x (T,K), w_gate/w_up (E,K,F), w_down (E,F,N)")
    T, K = xa.shape
    E, Kw, F = wg.shape
    if Kw != K or wd.shape[0] != E or wd.shape[1] != F:
        raise ValueError("moe_swiglu_block: weight shapes disagree")
    N = wd.shape[2]
    gs = np.asarray(group_sizes).astype(np.int64).reshape(-1)
    if gs.shape[0] != E:
        raise ValueError("moe_swiglu_block: len(group_sizes) != E")
    if alignment is not None and np.any(gs % int(alignment) != 0):
        raise ValueError(f"moe_swiglu_block: every group size must be a multiple of alignment={alignment}")
    off = _offsets(gs, T, "moe_swiglu_block")
    y = np.zeros((T, N), np.uint16)
    rc = _lane.load().tessera_gfx950_moe_swiglu_block_bf16(
        xa.ctypes.data, wg.ctypes.data, wu.ctypes.data, wd.ctypes.data, off.ctypes.data, y.ctypes.data, T, K, F, N, E)
    _lane.check(rc, "moe_swiglu_block")
    return y.view(BF16Array)


@dataclass
class MoETransport:
    """The int32 device ABI of the MoE transport descriptor
    (``compiler/moe_transport.py:194-273``)."""
    num_tokens: int
    top_k: int
    num_experts: int
    capacity: Optional[int]
    token_of_slot: np.ndarray      # int32[S]
    expert_of_slot: np.ndarray     # int32[S], non-decreasing
    combine_weights: np.ndarray    # f32[S]
    group_sizes: np.ndarray        # int32[E]
    group_offsets: np.ndarray      # int32[E+1]

    @property
    def num_slots(self) -> int:
        return int(self.token_of_slot.shape[0])


def expert_capacity(capacity_factor: float, num_tokens: int, num_experts: int) -> int:
    """Slots per expert, ``ceil(capacity_factor * (T / E))`` evaluated in that order
    (``MoEConfig.compute_capacity``, ``distributed/moe.py:79-92``): the quotient first,
    then the factor — ``(cf * T) / E`` rounds differently on a few (cf, T, E) triples
    (cf=1.1, T=540, E=3: 199, not 198) and one slot of capacity changes which slots drop."""
    return int(math.ceil(capacity_factor * (num_tokens / max(1, num_experts))))


def _capacity_arg(capacity: Optional[int], T: int, k: int) -> int:
    if capacity is None or capacity >= T * k:
        return 0            # cannot overflow
    if capacity < 1:
        raise ValueError("capacity must be >= 1")
    return int(capacity)


@dataclass(frozen=True)
class MoEConfig:
    """The reference's MoE configuration record (``distributed/moe.py:43-92``)."""
    num_experts: int
    top_k: int = 1
    expert_capacity: Optional[int] = None
    capacity_factor: float = 1.25
    jitter_noise: float = 0.0
    normalize_weights: bool = True

    def __post_init__(self) -> None:
        if self.num_experts < 1:
            raise ValueError(f"num_experts must be >= 1, got {self.num_experts}")
        if self.top_k < 1 or self.top_k > self.num_experts:
            raise ValueError(f"top_k must be in [1, num_experts={self.num_experts}], got {self.top_k}")
        if self.capacity_factor <= 0:
            raise ValueError(f"capacity_factor must be > 0, got {self.capacity_factor}")
        if not (0.0 <= self.jitter_noise < 1.0):
            raise ValueError(f"jitter_noise must be in [0, 1), got {self.jitter_noise}")

    def compute_capacity(self, num_tokens: int, num_ranks: int = 1) -> int:
        if self.expert_capacity is not None:
            return self.expert_capacity
        return expert_capacity(self.capacity_factor, num_tokens, max(1, self.num_experts // num_ranks))


class RoutingResult(NamedTuple):
    """What the reference's ``route_tokens`` returns (``distributed/moe.py:98-113``)."""
    assignment: np.ndarray   # (T, top_k) int64, -1 = dropped over capacity
    weights: np.ndarray      # (T, top_k) f32, 0 for a dropped slot
    load: np.ndarray         # (E,) int64, selections per expert before any drop
    overflow: int


def _route_tokens_result(scores, config, capacity) -> RoutingResult:
    """``route_tokens(scores, config, capacity=None)`` as the reference spells it
    (``distributed/moe.py:119-206``): the token-major view of the routing — selection, weights
    and the first-come capacity drop run on the device; ties between bit-equal probabilities
    go to the lowest expert id."""
    s = np.ascontiguousarray(_unbox(scores), np.float32)
    if s.ndim != 2:
        raise ValueError(f"scores must be 2D (num_tokens, num_experts), got shape {s.shape}")
    T, E = s.shape
    if E != config.num_experts:
        raise ValueError(f"scores has {E} expert columns but config.num_experts={config.num_experts}")
    if getattr(config, "jitter_noise", 0.0) > 0.0:
        raise NotImplementedError("route_tokens: jitter noise is not implemented on the gfx950 lane")
    k = int(config.top_k)
    if capacity is None:
        capacity = config.compute_capacity(T)
    capacity = int(capacity)
    cap = min(capacity, T * k) if capacity > 0 else None          # (0 or less: every slot drops, below)
    plan = _plan_call(s, None, None, T, E, k, 2 if config.normalize_weights else 3, cap)
    kept = plan.kept_mask if capacity > 0 else np.zeros((T, k), bool)
    assignment = np.where(kept, plan.expert_ids, -1).astype(np.int64)
    weights = np.where(kept, plan.weights, np.float32(0.0)).astype(np.float32)
    load = np.bincount(plan.expert_ids.reshape(-1), minlength=E).astype(np.int64)
    return RoutingResult(assignment, weights, load, int(kept.size - int(kept.sum())))


def route_tokens(scores, num_experts, top_k: Optional[int] = None, *, normalize_weights: bool = True,
                 capacity_factor: float = 1.25, capacity: Optional[int] = None):
    """Top-k routing + packing plan.  ``scores`` ``(T, E)`` f32 gate logits.
    capacity defaults to ``ceil(capacity_factor * (T / E))``; over-capacity slots are
    dropped first-come in token-major order.  Ties between equal probabilities go
    to the lowest expert id.  Returns the transport descriptor of the kept slots.

    Called as the reference spells it — ``route_tokens(scores, config, capacity=None)`` with
    a :class:`MoEConfig` (or any object with its fields) — it returns a
    :class:`RoutingResult` instead (assignment, weights, load, overflow)."""
    if hasattr(num_experts, "num_experts"):
        return _route_tokens_result(scores, num_experts, top_k if capacity is None else capacity)
    if top_k is None:
        raise TypeError("route_tokens(scores, num_experts, top_k) needs top_k")
    s = np.ascontiguousarray(_unbox(scores), np.float32)
    if s.ndim != 2:
        raise ValueError(f"scores must be 2D (num_tokens, num_experts), got shape {s.shape}")
    T, E = s.shape
    if E != num_experts:
        raise ValueError(f"scores has {E} expert columns but num_experts={num_experts}")
    if top_k < 1 or top_k > num_experts:
        raise ValueError(f"top_k must be in [1, num_experts={num_experts}], got {top_k}")
    if capacity is None:
        if capacity_factor <= 0:
            raise ValueError(f"capacity_factor must be > 0, got {capacity_factor}")
        capacity = expert_capacity(capacity_factor, T, E)
    cap = _capacity_arg(capacity, T, top_k)
    S = T * top_k
    tos = np.empty(S, np.int32)
    eos = np.empty(S, np.int32)
    cw = np.empty(S, np.float32)
    gs = np.empty(E, np.int32)
    go = np.empty(E + 1, np.int32)
    n = np.zeros(1, np.int32)
    rc = _lane.load().tessera_gfx950_moe_route_f32(
        s.ctypes.data, T, E, top_k, 1 if normalize_weights else 0, cap,
        tos.ctypes.data, eos.ctypes.data, cw.ctypes.data, gs.ctypes.data, go.ctypes.data, n.ctypes.data)
    _lane.check(rc, "route_tokens")
    k = int(n[0])
    return MoETransport(T, top_k, E, cap or None, tos[:k].copy(), eos[:k].copy(), cw[:k].copy(), gs, go)


@dataclass
class DispatchPlan:
    """The reference's packing plan in its token-major view
    (``stdlib/moe.py:58-77`` ``DispatchPlan``; ``models/moe_routing.py:33-51``
    ``RoutingPlan`` is the no-capacity case): which routed slots survive and the
    contiguous per-expert order of the survivors."""
    expert_ids: np.ndarray       # (T, k) int64 selected experts
    weights: np.ndarray          # (T, k) f32 route weights
    kept_mask: np.ndarray        # (T, k) bool, False = dropped over capacity
    sort_perm: np.ndarray        # (S,) int64 kept token-major slot ids, expert-sorted
    inverse_perm: np.ndarray     # (T*k,) int64 packed position of each slot, -1 = dropped
    group_sizes: np.ndarray      # (E,) int64 kept slots per expert
    num_tokens: int
    top_k: int
    capacity: Optional[int]
    transport: MoETransport      # the same plan as the int32 transport descriptor

    @property
    def num_kept(self) -> int:
        return int(self.sort_perm.shape[0])

    @property
    def drop_fraction(self) -> float:
        total = self.num_tokens * self.top_k
        return 0.0 if total == 0 else 1.0 - self.num_kept / total

    def round_trips(self) -> bool:
        """True iff nothing was dropped and ``sort_perm[inverse_perm]`` is the identity."""
        n = self.num_tokens * self.top_k
        return self.num_kept == n and bool(np.array_equal(self.sort_perm[self.inverse_perm], np.arange(n)))


def _plan_call(logits, given_ids, given_weights, T: int, E: int, k: int, normalize: bool,
               capacity: Optional[int]) -> DispatchPlan:
    S = T * k
    cap = 0 if capacity is None else int(capacity)
    ids = np.empty((T, k), np.int32)
    w = np.empty((T, k), np.float32)
    kept = np.empty((T, k), np.uint8)
    sp = np.empty(S, np.int32)
    ip = np.empty(S, np.int32)
    tos = np.empty(S, np.int32)
    eos = np.empty(S, np.int32)
    cw = np.empty(S, np.float32)
    gs = np.empty(E, np.int32)
    go = np.empty(E + 1, np.int32)
    n = np.zeros(1, np.int32)
    rc = _lane.load().tessera_gfx950_moe_plan_f32(
        _lane.ptr(logits), _lane.ptr(given_ids), _lane.ptr(given_weights), T, E, k, int(normalize), cap,
        ids.ctypes.data, w.ctypes.data, kept.ctypes.data, sp.ctypes.data, ip.ctypes.data, tos.ctypes.data,
        eos.ctypes.data, cw.ctypes.data, gs.ctypes.data, go.ctypes.data, n.ctypes.data)
    _lane.check(rc, "moe plan")
    m = int(n[0])
    if logits is None:
        ids = np.asarray(given_ids, np.int32).reshape(T, k)
        w = (np.zeros((T, k), np.float32) if given_weights is None
             else np.asarray(given_weights, np.float32).reshape(T, k))
    transport = MoETransport(T, k, E, capacity, tos[:m].copy(), eos[:m].copy(), cw[:m].copy(), gs, go)
    return DispatchPlan(ids.astype(np.int64), w, kept.astype(bool), sp[:m].astype(np.int64), ip.astype(np.int64),
                        gs.astype(np.int64), T, k, capacity, transport)


def route_top_k(router_logits, top_k: int, *, normalize: bool = True, compute_dtype=np.float32):
    """Exact top-k routing on the LOGITS → ``(expert_ids (T,k) int64, weights (T,k) f32)``:
    descending by logit, ties to the lowest expert id; ``normalize`` makes the weights a
    softmax over the selected logits, else each is ``1/k`` (``models/moe_routing.py:54-77``)."""
    if np.dtype(compute_dtype) != np.float32:
        raise NotImplementedError("route_top_k on the gfx950 lane computes in f32")
    lg = np.ascontiguousarray(_unbox(router_logits), np.float32)
    if lg.ndim != 2:
        raise ValueError("router_logits must be (T, num_experts)")
    T, E = lg.shape
    if not (1 <= top_k <= E):
        raise ValueError(f"top_k={top_k} out of [1, num_experts={E}]")
    plan = _plan_call(lg, None, None, T, E, int(top_k), normalize, None)
    return plan.expert_ids, plan.weights


def _check_ids(expert_ids, num_experts: int) -> np.ndarray:
    ids = np.asarray(_unbox(expert_ids))
    if ids.ndim != 2:
        raise ValueError("expert_ids must be (T, k)")
    if ids.size and (ids.min() < 0 or ids.max() >= num_experts):
        raise ValueError("expert id out of range")
    return np.ascontiguousarray(ids, np.int32)


def plan_packing(expert_ids, num_experts: int) -> DispatchPlan:
    """The per-expert packing plan of a routing, nothing dropped
    (``models/moe_routing.py:80-99``); ``weights`` is the reference's zero placeholder."""
    ids = _check_ids(expert_ids, num_experts)
    T, k = ids.shape
    return _plan_call(None, ids, None, T, num_experts, k, True, None)


def plan_dispatch(expert_ids, weights, num_experts: int, *, capacity: Optional[int] = None) -> DispatchPlan:
    """Capacity-aware plan from routing decisions: slots in token-major order, an expert
    keeps its first ``capacity`` (``None``: all), kept slots stable-sorted by expert
    (``stdlib/moe.py:79-115``)."""
    ids = _check_ids(expert_ids, num_experts)
    w = np.ascontiguousarray(_unbox(weights), np.float32)
    if w.shape != ids.shape:
        raise ValueError("weights must match expert_ids")
    T, k = ids.shape
    if capacity is not None and capacity < 1:
        raise ValueError("capacity must be >= 1 (or None)")
    return _plan_call(None, ids, w, T, num_experts, k, True, capacity)


def pack_tokens(x, plan: DispatchPlan):
    """Gather ``x`` (T, H) into packed per-expert slot order → ``(S, H)``
    (``models/moe_routing.py:102-106``, ``stdlib/moe.py:117-121``)."""
    return moe_dispatch(x, plan.transport)


def unpack_combine(y_packed, plan: DispatchPlan, weights) -> np.ndarray:
    """Scatter packed expert rows back to token order and sum each token's k slots in
    rank order with their route weights → ``(T, H)`` f32; dropped slots add nothing
    (``models/moe_routing.py:109-116``)."""
    y = _unbox(y_packed)
    w = np.ascontiguousarray(_unbox(weights), np.float32)
    T, k = plan.num_tokens, plan.top_k
    if w.shape != (T, k):
        raise ValueError(f"weights must be (T, k)=({T}, {k}); got {w.shape}")
    lib = _lane.load()
    if _bf16.is_bf16(y):
        ya, fn = _bf16.as_bits(y), lib.tessera_gfx950_moe_unpack_combine_bf16
    else:
        ya, fn = np.ascontiguousarray(y, np.float32), lib.tessera_gfx950_moe_unpack_combine_f32
    S = plan.num_kept
    if ya.ndim != 2 or ya.shape[0] != S:
        raise ValueError(f"packed rows must be (S, H) with S={S}; got {ya.shape}")
    ip = np.ascontiguousarray(plan.inverse_perm, np.int32)
    out = np.empty((T, ya.shape[1]), np.float32)
    _lane.check(fn(ya.ctypes.data, ip.ctypes.data, w.ctypes.data, out.ctypes.data, T, k, S, ya.shape[1]),
                "unpack_combine")
    return out


def moe_dispatch(x, plan: MoETransport):
    """Gather the token row of every kept, expert-sorted slot → ``(S, H)``."""
    x = _unbox(x)
    if _bf16.is_bf16(x):
        xa, wrap = _bf16.as_bits(x), (lambda b: b.view(BF16Array))
    else:
        xa = np.ascontiguousarray(x)
        if xa.dtype not in (np.float16, np.float32, np.float64):
            raise ValueError("moe_dispatch takes f16, bf16, f32 or f64 rows")
        wrap = lambda b: b
    if xa.ndim != 2:
        raise ValueError(f"moe_dispatch x must be 2-D (T,H); got {xa.shape}")
    T, H = xa.shape
    if T != plan.num_tokens:
        raise ValueError("moe_dispatch: x rows != plan.num_tokens")
    S = plan.num_slots
    outp = np.empty((S, H), xa.dtype)
    tos = np.ascontiguousarray(plan.token_of_slot, np.int32)
    rc = _lane.load().tessera_gfx950_moe_dispatch(xa.ctypes.data, tos.ctypes.data, outp.ctypes.data, T, S, H,
                                                  xa.dtype.itemsize)
    _lane.check(rc, "moe_dispatch")
    return wrap(outp)


def moe_combine(y_packed, plan: MoETransport) -> np.ndarray:
    """Weighted scatter-add of the packed expert rows back to ``(T, N)`` f32;
    dropped slots contribute zero."""
    y = _unbox(y_packed)
    S = plan.num_slots
    tos = np.ascontiguousarray(plan.token_of_slot, np.int32)
    w = np.ascontiguousarray(plan.combine_weights, np.float32)
    lib = _lane.load()
    if _bf16.is_bf16(y):
        ya = _bf16.as_bits(y)
        fn = lib.tessera_gfx950_moe_combine_bf16
    else:
        ya = np.ascontiguousarray(y, np.float32)
        fn = lib.tessera_gfx950_moe_combine_f32
    if ya.ndim != 2 or ya.shape[0] != S:
        raise ValueError(f"moe_combine partials must be 2-D (S,H) with S={S}; got {ya.shape}")
    N = ya.shape[1]
    outp = np.zeros((plan.num_tokens, N), np.float32)
    _lane.check(fn(ya.ctypes.data, tos.ctypes.data, w.ctypes.data, outp.ctypes.data, plan.num_tokens, S, N),
                "moe_combine")
    return outp


def _as_transport(plan) -> MoETransport:
    """The int32 descriptor of a plan: a :class:`MoETransport`, this module's
    :class:`DispatchPlan`, or any object with the fields of the reference's plans
    (``stdlib/moe.py:55-67``, ``models/moe_routing.py:35-45``)."""
    if isinstance(plan, MoETransport):
        return plan
    tr = getattr(plan, "transport", None)
    if isinstance(tr, MoETransport):
        return tr
    ids = np.asarray(plan.expert_ids)
    T, k = ids.shape
    perm = np.asarray(plan.sort_perm, np.int64).reshape(-1)
    groups = np.asarray(plan.group_sizes, np.int64).reshape(-1)
    if perm.size and (perm.min() < 0 or perm.max() >= T * k):
        raise ValueError("plan.sort_perm contains an invalid slot")
    if int(groups.sum()) != perm.size:
        raise ValueError("plan.group_sizes must sum to the number of kept slots")
    w = getattr(plan, "weights", None)
    w = np.zeros(T * k, np.float32) if w is None else np.asarray(w, np.float32).reshape(-1)
    offsets = np.concatenate((np.zeros(1, np.int64), np.cumsum(groups))).astype(np.int32)
    return MoETransport(int(T), int(k), int(groups.size), getattr(plan, "capacity", None), (perm // k).astype(np.int32),
                        ids.reshape(-1)[perm].astype(np.int32), w[perm].astype(np.float32), groups.astype(np.int32), offsets)


def compute_capacity(num_tokens: int, top_k: int, num_experts: int, capacity_factor: float) -> int:
    """Per-expert capacity ``ceil(factor * T * k / E)``, at least 1 (``stdlib/moe.py:41-52``)."""
    if num_tokens <= 0:
        return 0
    return max(1, int(math.ceil(capacity_factor * num_tokens * top_k / max(1, num_experts))))


def dispatch(x, plan):
    """``stdlib.moe.dispatch`` (``stdlib/moe.py:117-121``): token rows of the kept, expert-sorted
    slots → ``(S, H)``, gathered on the device."""
    return moe_dispatch(x, _as_transport(plan))


def combine(y_packed, plan) -> np.ndarray:
    """``stdlib.moe.combine`` (``stdlib/moe.py:124-134``): packed expert rows scattered back to
    ``(T, H)``, each weighted by its slot's route weight, added in packed order (f32 here)."""
    return moe_combine(y_packed, _as_transport(plan))


def grouped_swiglu(x_packed, w_gate, w_up, w_down, group_sizes):
    """``stdlib.moe.grouped_swiglu`` (``stdlib/moe.py:151-163``) on the fused expert-block
    kernels: bf16 storage in and out, f32 accumulation."""
    return moe_swiglu_block(x_packed, w_gate, w_up, w_down, group_sizes)


def _moe_layer_staged(x, W_router, W_gate, W_up, W_down, top_k, normalize_weights, capacity_factor, kind, alignment,
                      quant, router_logits, return_plan):
    """The layer as the reference composes it (``nn/functional.py:447-490``) — router product,
    routing, dispatch, expert block, combine — each stage one device op with host arrays in
    between: the form that carries ``quant`` and ``alignment`` into the expert block."""
    xa = _unbox(x)
    T = _bits(xa).shape[0]
    E = _bits(_unbox(W_gate)).shape[0]
    if router_logits is None:
        scores = gemm(xa, W_router)
        scores = scores.to_float32() if isinstance(scores, BF16Array) else np.asarray(scores, np.float32)
    else:
        scores = np.ascontiguousarray(router_logits, np.float32)
    plan = route_tokens(scores, E, top_k, normalize_weights=normalize_weights,
                        capacity_factor=capacity_factor if capacity_factor > 0 else 1e9)
    x_perm = moe_dispatch(xa, plan)
    y_perm = moe_swiglu_block(x_perm, W_gate, W_up, W_down, np.asarray(plan.group_sizes, np.int64), kind=kind,
                              alignment=alignment, quant=quant)
    out = moe_combine(y_perm, plan)
    return (out, plan) if return_plan else out


def moe_layer(x, W_router, W_gate, W_up, W_down, *, top_k: int = 1, normalize_weights: bool = True,
              capacity_factor: float = 0.0, kind: str = "contiguous", alignment=None, quant=None,
              router_logits=None, return_plan: bool = False):
    """Single-device top-k SwiGLU MoE layer: router → permute → expert FFN →
    combine.  ``x`` ``(T, K)``, ``W_router`` ``(K, E)``, ``W_gate``/``W_up``
    ``(E, K, F)``, ``W_down`` ``(E, F, N)`` in bf16; returns ``(T, N)`` f32.
    ``capacity_factor <= 0`` disables capacity drops.  ``router_logits``
    ``(T, E)`` f32 may be given instead of ``W_router``."""
    if kind not in _SUPPORTED_GROUPED_KINDS:
        raise NotImplementedError("moe_layer: contiguous / dense grouped layouts only on the gfx950 lane")
    if quant is not None or alignment is not None:
        return _moe_layer_staged(x, W_router, W_gate, W_up, W_down, top_k, normalize_weights, capacity_factor, kind,
                                 alignment, quant, router_logits, return_plan)
    x, W_gate, W_up, W_down = map(_unbox, (x, W_gate, W_up, W_down))
    for a in (x, W_gate, W_up, W_down):
        if _storage(a) != "bf16":
            raise ValueError("moe_layer on the gfx950 lane takes bf16 storage")
    xa, wg, wu, wd = map(_bits, (x, W_gate, W_up, W_down))
    if xa.ndim != 2 or wg.ndim != 3 or wu.shape != wg.shape or wd.ndim != 3:
        raise ValueError("moe_layer: x (T,K), W_gate/W_up (E,K,F), W_down (E,F,N)")
    T, H = xa.shape
    E, Kw, F = wg.shape
    if Kw != H or wd.shape[0] != E or wd.shape[1] != F:
        raise ValueError(f"moe_layer: weight shapes disagree: x {xa.shape}, W_gate/W_up {wg.shape}, W_down {wd.shape}")
    if top_k < 1 or top_k > E:
        raise ValueError(f"top_k must be in [1, num_experts={E}], got {top_k}")
    N = wd.shape[2]
    lib = _lane.load()
    cap = 0
    if capacity_factor > 0:
        cap = _capacity_arg(expert_capacity(capacity_factor, T, E), T, top_k)
    S = T * top_k
    outp = np.zeros((T, N), np.float32)
    tos = np.empty(S, np.int32)
    eos = np.empty(S, np.int32)
    cw = np.empty(S, np.float32)
    gs = np.empty(E, np.int32)
    go = np.empty(E + 1, np.int32)
    tail = (T, H, F, N, E, top_k, 1 if normalize_weights else 0, cap,
            tos.ctypes.data, eos.ctypes.data, cw.ctypes.data, gs.ctypes.data, go.ctypes.data)
    if router_logits is None:
        # scores = ops.gemm(x, W_router) on the device, stored in bf16 and read as f32 like every
        # reduced-precision product; the routing follows on the same stream without a host hop
        W_router = _unbox(W_router)
        if _storage(W_router) != "bf16":
            raise ValueError("moe_layer on the gfx950 lane takes a bf16 W_router")
        wr = _bits(W_router)
        if wr.shape != (H, E):
            raise ValueError(f"W_router must be (K, E)=({H}, {E}); got {wr.shape}")
        rc = lib.tessera_gfx950_moe_layer_router_bf16(
            xa.ctypes.data, wr.ctypes.data, wg.ctypes.data, wu.ctypes.data, wd.ctypes.data, outp.ctypes.data,
            *tail, None)
    else:
        logits = np.ascontiguousarray(router_logits, np.float32)
        if logits.shape != (T, E):
            raise ValueError(f"router logits must be (T, E)=({T}, {E}); got {logits.shape}")
        rc = lib.tessera_gfx950_moe_layer_bf16(
            xa.ctypes.data, logits.ctypes.data, wg.ctypes.data, wu.ctypes.data, wd.ctypes.data, outp.ctypes.data,
            *tail)
    _lane.check(rc, "moe_layer")
    if not return_plan:
        return outp
    n = int(go[E])
    return outp, MoETransport(T, top_k, E, cap or None, tos[:n].copy(), eos[:n].copy(), cw[:n].copy(), gs, go)


# ---------------------------------------------------------------------------
# quantisation
# ---------------------------------------------------------------------------

_E4M3_TABLE: Optional[np.ndarray] = None


def e4m3_table() -> np.ndarray:
    """The 256 OCP e4m3fn code values as f32."""
    global _E4M3_TABLE
    if _E4M3_TABLE is None:
        c = np.arange(256)
        e = (c >> 3) & 0xF
        m = (c & 7).astype(np.float64)
        v = np.where(e == 0, m * 2.0 ** -9, (1.0 + m / 8.0) * np.exp2(e.astype(np.float64) - 7.0))
        v = np.where((e == 15) & ((c & 7) == 7), np.nan, v)
        _E4M3_TABLE = np.where(c & 0x80, -v, v).astype(np.float32)
    return _E4M3_TABLE


def e5m2_table() -> np.ndarray:
    """The 256 OCP e5m2 code values as f32 (a code is the upper byte of an IEEE half)."""
    return (np.arange(256, dtype=np.uint16) << 8).view(np.float16).astype(np.float32)


def _fp8_format(format: str) -> str:
    if format not in ("e4m3", "e5m2"):
        raise ValueError(f"format must be 'e4m3' or 'e5m2'; got {format!r}")
    return format


def quantize_fp8_codes(x, *, scale=None, format: str = "e4m3"):
    """Per-tensor fp8 quantisation on the device → ``(codes uint8, scale f32)``; ``format``
    ``"e4m3"`` or ``"e5m2"`` (the operand formats of :func:`gemm_fp8`)."""
    xa = np.ascontiguousarray(_unbox(x), np.float32)
    codes = np.empty(xa.shape, np.uint8)
    s_out = ctypes.c_float(0)
    rc = getattr(_lane.load(), f"tessera_gfx950_quantize_{_fp8_format(format)}_f32")(
        xa.ctypes.data, xa.size, float(scale) if scale is not None else 0.0, codes.ctypes.data,
        ctypes.byref(s_out))
    _lane.check(rc, "quantize_fp8")
    return codes, np.float32(s_out.value)


def quantize_fp8(x, *, format: str = "e4m3", scale=None):
    """Per-tensor symmetric fp8 quantisation → ``(x_q_as_fp32, scale)`` where
    ``x_q_as_fp32`` is the fp8-rounded value cast back to f32 (``grid * scale``)."""
    return _quantize_per_tensor(x, format, ("e4m3", "e5m2"), scale)


def gemm_fp8(a_codes, b_codes, scale_a, scale_b, *, out: str = "bf16", format: str = "e4m3"):
    """``f32acc(Aq . Bq) * scale_a * scale_b`` over fp8 codes (both operands ``format``:
    ``"e4m3"`` or ``"e5m2"``); bf16 or f32 result."""
    fmt = _fp8_format(format)
    a = np.ascontiguousarray(a_codes, np.uint8)
    b = np.ascontiguousarray(b_codes, np.uint8)
    if a.ndim != 2 or b.ndim != 2 or a.shape[1] != b.shape[0]:
        raise ValueError(f"gemm_fp8 needs rank-2 operands with matching K; got {a.shape} @ {b.shape}")
    M, K = a.shape
    N = b.shape[1]
    if out == "bf16":
        d = np.empty((M, N), np.uint16)
        fn = getattr(_lane.load(), f"tessera_gfx950_gemm_{fmt}_bf16")
    elif out == "f32":
        d = np.empty((M, N), np.float32)
        fn = getattr(_lane.load(), f"tessera_gfx950_gemm_{fmt}_f32")
    else:
        raise ValueError("out must be 'bf16' or 'f32'")
    _lane.check(fn(a.ctypes.data, b.ctypes.data, float(scale_a), float(scale_b), d.ctypes.data, M, N, K), "gemm_fp8")
    return d.view(BF16Array) if out == "bf16" else d


def quantize_int8_per_channel(M, axis: int, *, smoothing=None):
    """Symmetric int8 quantise along the kept axis → ``(q int8, scale f32)`` with
    ``scale`` shaped like numpy's ``keepdims`` reduction over ``axis``.  ``smoothing``
    (f32 ``[C]``, ``axis=1`` only): every element is divided by its column's factor first,
    in the same pass (the smoothed activation of ``smoothquant_matmul``)."""
    a = np.ascontiguousarray(_unbox(M), np.float32)
    if a.ndim != 2 or axis not in (0, 1):
        raise ValueError("quantize_int8_per_channel takes a 2-D array and axis 0 or 1")
    R, C = a.shape
    q = np.empty((R, C), np.int8)
    sc = np.empty(R if axis == 1 else C, np.float32)
    if smoothing is not None:
        sm = np.ascontiguousarray(smoothing, np.float32).reshape(-1)
        if axis != 1 or sm.shape[0] != C:
            raise ValueError(f"smoothing needs axis=1 and one factor per column ({C}); got axis={axis}, {sm.shape}")
        _lane.check(_lane.load().tessera_gfx950_quantize_i8_smoothed_f32(a.ctypes.data, R, C, sm.ctypes.data, q.ctypes.data,
                                                                         sc.ctypes.data), "quantize_int8_per_channel")
        return q, sc.reshape(R, 1)
    _lane.check(_lane.load().tessera_gfx950_quantize_i8_f32(a.ctypes.data, R, C, axis, q.ctypes.data, sc.ctypes.data),
                "quantize_int8_per_channel")
    return q, (sc.reshape(R, 1) if axis == 1 else sc.reshape(1, C))


def quantize_int8(x, scale=None, zero_point: int = 0, *, symmetric: bool = True):
    """Per-tensor int8 quantisation → ``(q, scale, zero_point)`` (``quantization.py:31-44``);
    the symmetric form runs on the device."""
    if not symmetric:
        raise NotImplementedError("quantize_int8: only the symmetric form is implemented on the gfx950 lane")
    a = np.ascontiguousarray(_unbox(x), np.float32)
    q = np.empty(a.shape, np.int8)
    s_out = np.ones(1, np.float32)
    if scale is not None and not float(scale) > 0.0:
        raise ValueError("quantize_int8: scale must be positive")
    if a.size:
        _lane.check(_lane.load().tessera_gfx950_quantize_i8_tensor_f32(
            a.ctypes.data, a.size, 0.0 if scale is None else float(np.float32(scale)), q.ctypes.data, s_out.ctypes.data),
            "quantize_int8")
    elif scale is not None:
        s_out[0] = np.float32(scale)
    return q, np.float32(s_out[0]), 0


def dequantize_int8(q, scale, zero_point: int = 0) -> np.ndarray:
    """``(q - zero_point) * scale`` in f32 (``quantization.py:47-48``); a host-side view of codes."""
    return (np.asarray(_unbox(q)).astype(np.float32) - float(zero_point)) * np.float32(scale)


def smoothquant_matmul(X, migrated):
    """The W8A8 direct-consume path (``compiler/smoothquant.py:115-124``): the activation is
    smoothed (``X / migrated.smoothing``) and quantised per token on the device in one pass,
    multiplied with the int8 weight ``migrated.w_q`` on the int8 matrix cores, and the int32
    accumulators are rescaled by the token scales and ``migrated.w_scale``.  ``migrated`` is the
    reference's ``MigratedLinear`` or any object with its ``smoothing``, ``w_q``, ``w_scale``."""
    x = np.asarray(_unbox(X), np.float32)
    w_q = np.asarray(migrated.w_q)
    if x.ndim != 2 or w_q.ndim != 2 or x.shape[1] != w_q.shape[0]:
        raise ValueError(f"shape mismatch: X {x.shape} @ w_q {w_q.shape}")
    if w_q.dtype != np.int8:
        raise ValueError("smoothquant_matmul consumes the int8 weight operand as it is")
    x_q, a_scale = quantize_int8_per_channel(x, axis=1, smoothing=migrated.smoothing)
    return w8a8_gemm(x_q, w_q, a_scale, migrated.w_scale)


def w8a8_gemm(x_q, w_q, a_scale, w_scale, *, return_acc: bool = False):
    """``f32(int32(x_q) @ int32(w_q)) * a_scale[:, None] * w_scale[None, :]``."""
    a = np.ascontiguousarray(x_q, np.int8)
    b = np.ascontiguousarray(w_q, np.int8)
    if a.ndim != 2 or b.ndim != 2 or a.shape[1] != b.shape[0]:
        raise ValueError(f"w8a8_gemm needs rank-2 operands with matching K; got {a.shape} @ {b.shape}")
    M, K = a.shape
    N = b.shape[1]
    rs = np.ascontiguousarray(np.asarray(a_scale, np.float32).reshape(-1))
    cs = np.ascontiguousarray(np.asarray(w_scale, np.float32).reshape(-1))
    if rs.shape[0] != M or cs.shape[0] != N:
        raise ValueError("w8a8_gemm: a_scale must have M entries and w_scale N entries")
    d = np.empty((M, N), np.float32)
    acc = np.empty((M, N), np.int32) if return_acc else None
    rc = _lane.load().tessera_gfx950_gemm_w8a8_f32(a.ctypes.data, b.ctypes.data, rs.ctypes.data, cs.ctypes.data,
                                                   d.ctypes.data, _lane.ptr(acc), M, N, K)
    _lane.check(rc, "w8a8_gemm")
    return (d, acc) if return_acc else d


def w8a8_matmul(X, W):
    """The W8A8 direct-consume path without smoothing: quantise activations per
    row and weights per column on the device, integer GEMM, rescale."""
    x_q, a_scale = quantize_int8_per_channel(X, axis=1)
    w_q, w_scale = quantize_int8_per_channel(W, axis=0)
    return w8a8_gemm(x_q, w_q, a_scale, w_scale)
