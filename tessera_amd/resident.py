"""Device-resident operands for chains of ops.

The functions of :mod:`tessera_amd.ops` follow the reference's C-ABI convention —
host arrays in, host arrays out — and so pay an allocation, an upload and a download
per op (``tessera_rocm_gemm.cpp:450-475``).  A chain written with the functions
below keeps every intermediate in HBM and only enqueues kernels: a
:class:`DeviceArray` is a typed handle on a device buffer (the role of the reference's
device-operand lease, ``python/tessera/runtime.py:1549-1614``), each function takes and
returns such handles and calls the library's ``*_dev`` entry points on the default
stream, and nothing synchronises until :meth:`DeviceArray.to_host`.

    x = DeviceArray.from_host(x_bf16);  wq = DeviceArray.from_host(wq_bf16)  # once
    q = gemm(x, wq)                                  # stays on the device
    o = flash_attn(q.reshape(B, S, H, D), k4, v4, causal=True, layout="bshd")   # reads the projections in place
    y = moe_layer(h, w_router, wg, wu, wd, top_k=8)  # router product -> routing -> experts -> combine
    y.to_host()

Same names, argument meaning and results as the host-pointer functions of
:mod:`tessera_amd.ops` (the kernels are the same).
"""
from __future__ import annotations

import ctypes
import math
from dataclasses import dataclass
from typing import Optional

import numpy as np

from . import bf16 as _bf16
from . import lane as _lane
from . import ops as _ops

_ITEMSIZE = {"bf16": 2, "f16": 2, "f32": 4, "i32": 4, "i8": 1, "u8": 1}
_NUMPY = {"f16": np.float16, "f32": np.float32, "i32": np.int32, "i8": np.int8, "u8": np.uint8}


class DeviceArray:
    """A contiguous row-major array in device memory: buffer + shape + dtype tag
    (``bf16`` / ``f16`` / ``f32`` / ``i32`` / ``i8`` / ``u8``)."""

    def __init__(self, shape, dtype: str, buf: Optional[_lane.DeviceBuffer] = None):
        if dtype not in _ITEMSIZE:
            raise ValueError(f"unknown device dtype {dtype!r}")
        self.shape = tuple(int(d) for d in shape)
        self.dtype = dtype
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * _ITEMSIZE[dtype]
        self.buf = buf if buf is not None else _lane.DeviceBuffer(max(self.nbytes, 16))

    @property
    def ptr(self) -> int:
        return self.buf.ptr

    @property
    def ndim(self) -> int:
        return len(self.shape)

    @classmethod
    def from_host(cls, x) -> "DeviceArray":
        x = getattr(x, "_data", x)
        if _bf16.is_bf16(x):
            bits = np.ascontiguousarray(_bf16.as_bits(x))
            return cls(bits.shape, "bf16", _lane.DeviceBuffer.from_host(bits))
        a = np.ascontiguousarray(x)
        for tag, dt in _NUMPY.items():
            if a.dtype == dt:
                return cls(a.shape, tag, _lane.DeviceBuffer.from_host(a))
        raise ValueError(f"no device dtype for host dtype {a.dtype}")

    def to_host(self):
        """Synchronises, then downloads (bf16 comes back as a ``BF16Array``)."""
        _lane.synchronize()
        if self.dtype == "bf16":
            return _bf16.from_bits(self.buf.download(self.shape, np.uint16))
        return self.buf.download(self.shape, _NUMPY[self.dtype])

    def reshape(self, *shape) -> "DeviceArray":
        shape = shape[0] if len(shape) == 1 and not np.isscalar(shape[0]) else shape
        out = DeviceArray.__new__(DeviceArray)
        out.shape, out.dtype, out.nbytes, out.buf = tuple(int(d) for d in shape), self.dtype, self.nbytes, self.buf
        if int(np.prod(out.shape, dtype=np.int64)) * _ITEMSIZE[self.dtype] != self.nbytes:
            raise ValueError(f"cannot reshape {self.shape} to {out.shape}")
        return out


def synchronize() -> None:
    _lane.synchronize()


def _storage(*arrays: DeviceArray) -> str:
    tags = {a.dtype for a in arrays}
    if len(tags) != 1 or not tags <= {"bf16", "f16"}:
        raise ValueError(f"operands must share one 16-bit storage dtype (f16 or bf16); got {sorted(tags)}")
    return tags.pop()


def gemm(A: DeviceArray, B: DeviceArray, *, out: str = "storage") -> DeviceArray:
    """``A @ B``, f32 accumulate; leading dims of ``A`` are batch dims; a rank-2 ``B`` is
    shared by every product of the batch (the batch folds into the rows of one product).  ``out`` as
    in :func:`tessera_amd.ops.gemm`."""
    st = _storage(A, B)
    if A.ndim < 2 or B.ndim < 2 or A.shape[-1] != B.shape[-2]:
        raise ValueError(f"gemm: operands {A.shape} @ {B.shape} do not multiply")
    if out not in ("storage", "f32"):
        raise ValueError("out must be 'storage' or 'f32'")
    M, K = A.shape[-2:]
    N = B.shape[-1]
    lead = A.shape[:-2]
    batch = int(np.prod(lead)) if lead else 1
    if B.ndim > 2 and B.shape[:-2] != lead:
        raise ValueError(f"batched gemm: leading dims differ — A {A.shape} @ B {B.shape}")
    D = DeviceArray(lead + (M, N), "f32" if out == "f32" else st)
    lib = _lane.load()
    if batch == 1:
        name = f"tessera_gfx950_gemm_{st}" + ("" if out == "f32" else f"_{st}") + "_dev"
        rc = getattr(lib, name)(A.ptr, B.ptr, D.ptr, M, N, K, None)
    elif B.ndim == 2:
        # one weight for the whole batch: the batch folds into the rows of one product
        name = f"tessera_gfx950_gemm_{st}" + ("" if out == "f32" else f"_{st}") + "_dev"
        rc = getattr(lib, name)(A.ptr, B.ptr, D.ptr, batch * M, N, K, None)
    else:
        rc = getattr(lib, f"tessera_gfx950_batched_gemm_strided_{st}_dev")(
            A.ptr, B.ptr, D.ptr, batch, M, N, K, M * K, K * N, M * N, 0 if out == "f32" else 1, None)
    _lane.check(rc, "gemm")
    return D


matmul = gemm
batched_gemm = gemm


def _attention_call(st, q_ptr, k_ptr, v_ptr, O, L, B, Hq, Hkv, Sq, Sk, D, strides, sc, causal, window, softcap, out):
    arr = (ctypes.c_int64 * 12)(*strides)
    fn = getattr(_lane.load(), f"tessera_gfx950_flash_attn_strided_{st}_dev")
    _lane.check(fn(q_ptr, k_ptr, v_ptr, O.ptr, L.ptr if L else None, B, Hq, Hkv, Sq, Sk, D, arr, ctypes.c_float(sc),
                   1 if causal else 0, int(window), ctypes.c_float(softcap), 0 if out == "f32" else 1, None),
                "flash_attn")


def flash_attn(Q: DeviceArray, K: DeviceArray, V: DeviceArray, *, scale: Optional[float] = None,
               causal: bool = False, return_lse: bool = False, out: str = "storage", layout: str = "bhsd",
               window: int = 0, logit_softcap: float = 0.0):
    """Attention forward on device handles (GQA when ``Hq != Hkv``); ``out`` ``"storage"`` or
    ``"f32"``; the log-sum-exp ``[B, Hq, Sq]`` f32 on request.

    ``layout="bhsd"``: ``Q [B, Hq, Sq, D]``, ``K, V [B, Hkv, Sk, D]`` (the reference's layout).
    ``layout="bshd"``: ``Q [B, Sq, Hq, D]``, ``K, V [B, Sk, Hkv, D]`` — what a projection
    ``x[B, S, E] @ W[E, H * D]`` leaves in memory (reshape the handle, no copy); the output
    comes back in the same layout, ready for the output projection."""
    st = _storage(Q, K, V)
    if layout not in ("bhsd", "bshd"):
        raise ValueError("layout must be 'bhsd' or 'bshd'")
    if Q.ndim != 4 or K.ndim != 4 or V.shape != K.shape or K.shape[0] != Q.shape[0] or K.shape[3] != Q.shape[3]:
        raise ValueError(f"flash_attn: Q {Q.shape}, K {K.shape}, V {V.shape}")
    if layout == "bhsd":
        B, Hq, Sq, D = Q.shape
        Hkv, Sk = K.shape[1], K.shape[2]
        qst, kst = (Hq * Sq * D, Sq * D, D), (Hkv * Sk * D, Sk * D, D)
    else:
        B, Sq, Hq, D = Q.shape
        Sk, Hkv = K.shape[1], K.shape[2]
        qst, kst = (Sq * Hq * D, D, Hq * D), (Sk * Hkv * D, D, Hkv * D)
    if Hq % Hkv:
        raise ValueError("the number of query heads must be a multiple of the KV heads")
    sc = float(scale) if scale is not None else 1.0 / math.sqrt(D)
    O = DeviceArray(Q.shape, "f32" if out == "f32" else st)
    L = DeviceArray((B, Hq, Sq), "f32") if return_lse else None
    _attention_call(st, Q.ptr, K.ptr, V.ptr, O, L, B, Hq, Hkv, Sq, Sk, D, qst + kst + kst + qst, sc, causal, window,
                    logit_softcap, out)
    return (O, L) if return_lse else O


def flash_attn_fused_qkv(QKV: DeviceArray, num_q_heads: int, num_kv_heads: int, *, scale: Optional[float] = None,
                         causal: bool = False, return_lse: bool = False, out: str = "storage"):
    """Attention forward on the output of ONE fused projection ``x[B, S, E] @ Wqkv[E, (Hq + 2 Hkv) * D]``:
    ``QKV [B, S, (Hq + 2 Hkv) * D]`` holds, per token, the query heads, then the key heads, then
    the value heads.  The kernel reads the three column blocks in place through row strides;
    returns ``O [B, S, Hq, D]`` (and ``LSE [B, Hq, S]``)."""
    st = _storage(QKV)
    if QKV.ndim != 3 or QKV.shape[2] % (num_q_heads + 2 * num_kv_heads) or num_q_heads % num_kv_heads:
        raise ValueError(f"flash_attn_fused_qkv: QKV {QKV.shape} for {num_q_heads} + 2 x {num_kv_heads} heads")
    B, S, W = QKV.shape
    D = W // (num_q_heads + 2 * num_kv_heads)
    sc = float(scale) if scale is not None else 1.0 / math.sqrt(D)
    O = DeviceArray((B, S, num_q_heads, D), "f32" if out == "f32" else st)
    L = DeviceArray((B, num_q_heads, S), "f32") if return_lse else None
    inb, outb = (S * W, D, W), (S * num_q_heads * D, D, num_q_heads * D)
    k_ptr = QKV.ptr + num_q_heads * D * 2
    v_ptr = k_ptr + num_kv_heads * D * 2
    _attention_call(st, QKV.ptr, k_ptr, v_ptr, O, L, B, num_q_heads, num_kv_heads, S, S, D, inb + inb + inb + outb, sc,
                    causal, 0, 0.0, out)
    return (O, L) if return_lse else O


gqa_attention = flash_attn


@dataclass
class ResidentPlan:
    """The MoE transport descriptor in device memory (``compiler/moe_transport.py:194-273``);
    the arrays hold ``T * k`` entries of which the first ``num_slots`` (a device int) are valid."""
    num_tokens: int
    top_k: int
    num_experts: int
    token_of_slot: DeviceArray
    expert_of_slot: DeviceArray
    combine_weights: DeviceArray
    group_sizes: DeviceArray
    group_offsets: DeviceArray
    num_slots: DeviceArray

    @classmethod
    def empty(cls, T: int, k: int, E: int) -> "ResidentPlan":
        S = T * k
        return cls(T, k, E, DeviceArray((S,), "i32"), DeviceArray((S,), "i32"), DeviceArray((S,), "f32"),
                   DeviceArray((E,), "i32"), DeviceArray((E + 1,), "i32"), DeviceArray((1,), "i32"))


def route_tokens(scores: DeviceArray, num_experts: int, top_k: int, *, normalize_weights: bool = True,
                 capacity: Optional[int] = None) -> ResidentPlan:
    """Top-k routing + packing plan of ``(T, E)`` f32 logits, all on the device."""
    if scores.dtype != "f32" or scores.ndim != 2 or scores.shape[1] != num_experts:
        raise ValueError(f"scores must be f32 (T, {num_experts}); got {scores.dtype} {scores.shape}")
    T = scores.shape[0]
    plan = ResidentPlan.empty(T, top_k, num_experts)
    rc = _lane.load().tessera_gfx950_moe_route_f32_dev(
        scores.ptr, T, num_experts, top_k, 1 if normalize_weights else 0, int(capacity or 0),
        plan.token_of_slot.ptr, plan.expert_of_slot.ptr, plan.combine_weights.ptr, plan.group_sizes.ptr,
        plan.group_offsets.ptr, plan.num_slots.ptr, None)
    _lane.check(rc, "route_tokens")
    return plan


def moe_layer(x: DeviceArray, W_router: Optional[DeviceArray], W_gate: DeviceArray, W_up: DeviceArray,
              W_down: DeviceArray, *, top_k: int = 1, normalize_weights: bool = True, capacity_factor: float = 0.0,
              router_logits: Optional[DeviceArray] = None, return_plan: bool = False):
    """The whole top-k SwiGLU MoE layer on resident operands: router product (when
    ``W_router`` is given, else ``router_logits`` f32 ``(T, E)``) → routing → expert block →
    combine, enqueued back to back.  Returns ``(T, N)`` f32 (and the :class:`ResidentPlan`)."""
    if any(a.dtype != "bf16" for a in (x, W_gate, W_up, W_down)):
        raise ValueError("moe_layer on the gfx950 lane takes bf16 storage")
    if x.ndim != 2 or W_gate.ndim != 3 or W_up.shape != W_gate.shape or W_down.ndim != 3:
        raise ValueError("moe_layer: x (T,K), W_gate/W_up (E,K,F), W_down (E,F,N)")
    T, H = x.shape
    E, Kw, F = W_gate.shape
    if Kw != H or W_down.shape[:2] != (E, F):
        raise ValueError("moe_layer: weight shapes disagree")
    N = W_down.shape[2]
    if (W_router is None) == (router_logits is None):
        raise ValueError("give exactly one of W_router and router_logits")
    if W_router is not None and (W_router.dtype != "bf16" or W_router.shape != (H, E)):
        raise ValueError(f"W_router must be bf16 (K, E)=({H}, {E})")
    if router_logits is not None and (router_logits.dtype != "f32" or router_logits.shape != (T, E)):
        raise ValueError(f"router_logits must be f32 (T, E)=({T}, {E})")
    cap = _ops.expert_capacity(capacity_factor, T, E) if capacity_factor > 0 else 0
    lib = _lane.load()
    need = ctypes.c_size_t(0)
    _lane.check(lib.tessera_gfx950_moe_layer_workspace_bytes(T, H, F, N, E, top_k, ctypes.byref(need)), "moe_layer")
    ws = _lane.DeviceBuffer(need.value)
    out = DeviceArray((T, N), "f32")
    plan = ResidentPlan.empty(T, top_k, E)
    rc = lib.tessera_gfx950_moe_layer_bf16_dev(
        x.ptr, W_router.ptr if W_router is not None else None,
        router_logits.ptr if router_logits is not None else None, W_gate.ptr, W_up.ptr, W_down.ptr, out.ptr,
        ws.ptr, need.value, T, H, F, N, E, top_k, 1 if normalize_weights else 0, cap,
        plan.token_of_slot.ptr, plan.expert_of_slot.ptr, plan.combine_weights.ptr, plan.group_sizes.ptr,
        plan.group_offsets.ptr, plan.num_slots.ptr, None)
    _lane.check(rc, "moe_layer")
    out._workspace = ws          # the kernels just enqueued still use it: it lives as long as the result
    return (out, plan) if return_plan else out
