"""CPU oracle for the gfx950 dense-op lane.  TEST INFRASTRUCTURE ONLY.

This module restates, in plain numpy, the arithmetic of the reference's CPU
path for the ops the gfx950 lane accelerates.  It is the checker the parity
tests, the smoke test and the benchmark's ``cpu_baseline`` leg compare the HIP
kernels against.  Nothing in the shipped package imports it, and no product
code path may route through it.

Every function cites the reference file:line it follows (paths are relative to
the reference checkout).  How each function is pinned (the check that would fail
on a dropped term, wrong sign or transposed operand) is listed beside it and
implemented in ``tests/test_oracle_*.py``:

=========================  ====================================================
function                   pin
=========================  ====================================================
bf16 rounding              all 2^16 bf16 codes round-trip; RNE ties table;
                           torch.bfloat16 library cross-check
gemm / batched_gemm        f64 matmul of storage-rounded operands; identity /
                           ones / K-ramp closed forms; compiled reference twin
                           ``tessera_x86_reference_gemm_bf16``
flash_attn_backward        torch autograd of scaled_dot_product_attention (library);
                           central finite differences of the forward oracle
flash_attn (+GQA, +LSE)    dense textbook softmax in f64; row 0 -> V[0];
                           identical keys -> prefix mean; torch SDPA library
                           cross-check; compiled reference
                           ``tessera_x86_flash_attn_ext_lse_f32``
route_tokens / moe_layer   brute force on tiny inputs; partition invariants;
                           agreement of the two routers' expert sets
route_top_k / plan /       per-token python sort with (-logit, index) keys; softmax
unpack_combine             of the selected logits against scipy.special.softmax;
                           first-come capacity by an independent per-expert walk;
                           inverse_perm . sort_perm = identity; k = 1 and equal-weight
                           closed forms of the combine
fused epilogue / gated     torch.nn.functional relu / gelu(tanh) / silu / sigmoid /
                           tanh library cross-check; relu and zero-bias closed forms
grouped_gemm / swiglu      per-group matmul; E=1 reduces to dense SwiGLU
quantize_int8 / W8A8       exact integer arithmetic; compiled reference twin
                           ``tessera_x86_reference_gemm_u8s8_s32`` on the
                           non-negative half of the range
e4m3 grid                  OCP e4m3fn table of all 256 codes; torch
                           float8_e4m3fn library cross-check; compiled
                           reference ``scalar_fpquant`` closed form
=========================  ====================================================

Floating-point summation order is NOT pinned by anything in the reference
(BLAS sgemm and ``np.add.at`` order are build-dependent), so floating-point
parity is to tolerance; integer results (int8 accumulators, MoE indices) are
bit-exact.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import numpy as np

# ---------------------------------------------------------------------------
# storage rounding
# ---------------------------------------------------------------------------


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """f32 -> bf16 bit pattern (uint16), round-to-nearest-even.

    Follows the integer fallback in ``compiler/fusion_core.py:358-361``:
    ``(u + 0x7FFF + ((u >> 16) & 1)) >> 16``.  NaNs are kept quiet.
    """
    a = np.ascontiguousarray(x, np.float32)
    flat = a.reshape(-1)
    out = np.empty(flat.shape, np.uint16)
    step = 1 << 22                       # chunks keep the 64-bit temporaries small
    for i in range(0, flat.size, step):
        c = flat[i:i + step]
        u = c.view(np.uint32).astype(np.uint64)
        r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
        nan = np.isnan(c)
        if nan.any():
            r = np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), r)
        out[i:i + step] = r
    return out.reshape(a.shape)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    """bf16 bit pattern -> f32 (``<< 16``; avx512_gemm_bf16.cpp:6-11)."""
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


def round_to_storage(x: np.ndarray, dtype: str) -> np.ndarray:
    """Round f32 ``x`` to a 16-bit storage dtype and back to f32.

    ``compiler/fusion_core.py:348-362`` (``_round_to_storage``).
    """
    a = np.ascontiguousarray(x, np.float32)
    if dtype in ("float16", "f16", "fp16"):
        return a.astype(np.float16).astype(np.float32)
    if dtype in ("bfloat16", "bf16"):
        return bf16_bits_to_f32(f32_to_bf16_bits(a))
    if dtype in ("float32", "f32"):
        return a
    raise ValueError(f"unsupported storage dtype {dtype!r}")


# ---------------------------------------------------------------------------
# GEMM  (python/tessera/__init__.py:239-254, 5783-5855; fusion_core.py:398-405)
# ---------------------------------------------------------------------------


def gemm_f32(A: np.ndarray, B: np.ndarray, dtype: str = "bf16") -> np.ndarray:
    """``MatmulRegion.reference``: operands rounded to storage, f32 product.

    ``compiler/fusion_core.py:398-405``.  Leading dims broadcast like
    ``np.matmul`` (``ops.batched_gemm`` is the same function,
    ``__init__.py:250-254``).
    """
    Aq = round_to_storage(np.asarray(A, np.float32), dtype)
    Bq = round_to_storage(np.asarray(B, np.float32), dtype)
    return np.matmul(Aq, Bq).astype(np.float32)


def gemm_f64(A: np.ndarray, B: np.ndarray, dtype: str = "bf16") -> np.ndarray:
    """Same product with an f64 accumulate — the "fp32 reference or better"
    the tolerance in the parity tests is measured against."""
    Aq = round_to_storage(np.asarray(A, np.float32), dtype).astype(np.float64)
    Bq = round_to_storage(np.asarray(B, np.float32), dtype).astype(np.float64)
    return np.matmul(Aq, Bq)


def gemm_storage(A: np.ndarray, B: np.ndarray, dtype: str = "bf16") -> np.ndarray:
    """``ops.gemm`` on reduced-precision operands: promote to f32, matmul,
    store back in operand 0's storage dtype (returned here as f32 values that
    lie on the storage grid).  ``__init__.py:5771-5781,5824-5855``.
    """
    return round_to_storage(gemm_f32(A, B, dtype), dtype)


# ---------------------------------------------------------------------------
# fused matmul epilogue and gated projection
# ---------------------------------------------------------------------------


def _gelu_tanh(x: np.ndarray) -> np.ndarray:
    """``compiler/fusion_core.py:104-106``: tanh-form GELU, argument clamped to +-30."""
    t = np.clip(0.7978845608028654 * (x + 0.044715 * x ** 3), -30.0, 30.0)
    return 0.5 * x * (1.0 + np.tanh(t))


#: the pointwise epilogue vocabulary (``compiler/fusion_core.py:121-138``)
EPILOGUE_REFS = {
    "relu": lambda x: np.maximum(x, 0.0),
    "gelu": _gelu_tanh,
    "silu": lambda x: x / (1.0 + np.exp(-x)),
    "sigmoid": lambda x: 1.0 / (1.0 + np.exp(-x)),
    "tanh": np.tanh,
}


def fused_epilogue(A, B, bias=None, epilogue=()) -> np.ndarray:
    """Matmul then the ordered pointwise chain — ``FusedRegion.reference``
    (``compiler/fusion_core.py:318-345``) for regions without prologue, residual or
    reduction.  Computed in f64 on the given operands (round them to storage
    first), returned as f32."""
    out = np.asarray(A, np.float64) @ np.asarray(B, np.float64)
    for op in epilogue:
        if op == "bias":
            if bias is None:
                raise ValueError("region needs a bias")
            out = out + np.asarray(bias, np.float64)
        else:
            out = EPILOGUE_REFS[op](out)
    return out.astype(np.float32)


def gated_matmul(A, Wg, Wu, gate_act: str = "silu") -> np.ndarray:
    """``act(A @ Wg) * (A @ Wu)`` — ``GatedMatmulRegion.reference``
    (``compiler/fusion_core.py:776-782``), f64 inside, f32 out."""
    a = np.asarray(A, np.float64)
    gate = EPILOGUE_REFS[gate_act](a @ np.asarray(Wg, np.float64))
    return (gate * (a @ np.asarray(Wu, np.float64))).astype(np.float32)


# ---------------------------------------------------------------------------
# flash attention forward
# (__init__.py:1304-1356; nn/functional.py:349-356;
#  avx512_flash_attn_f32.cpp:75-107,180-196,379-422)
# ---------------------------------------------------------------------------


def _causal_limit(sq: int, sk: int) -> int:
    """Bottom-right alignment offset: key j visible to query i iff
    ``j <= i + max(sk - sq, 0)`` (``__init__.py:1344-1350``,
    ``avx512_flash_attn_f32.cpp:180-196``)."""
    return max(sk - sq, 0)


def key_bounds(i: int, sq: int, sk: int, causal: bool, window: int = 0):
    """First and last visible key of query row ``i`` — ``attention_bounds``
    (``avx512_flash_attn_f32.cpp:180-196``): the causal diagonal is bottom-right
    aligned; a window keeps ``window`` keys ending at the diagonal (causal) or
    ``window // 2`` keys either side of it."""
    off = _causal_limit(sq, sk)
    lo, hi = 0, (i + off if causal else sk - 1)
    if window > 0:
        if causal:
            lo, hi = i + off - window + 1, i + off
        else:
            lo, hi = i + off - window // 2, i + off + window // 2
    return max(lo, 0), min(hi, sk - 1)


def flash_attn_dense(Q, K, V, scale=None, causal=False, dtype=np.float64, window: int = 0,
                     softcap: float = 0.0, bias=None):
    """Dense ``softmax(scale*Q K^T, causal) V`` with GQA and LSE; optional sliding
    ``window`` (see :func:`key_bounds`), logit soft cap (scaled scores pass
    through ``cap * tanh(s / cap)``, ``avx512_flash_attn_f32.cpp:115,161``) and
    additive ``bias`` ``[B,Hq,Sq,Sk]`` added after the cap
    (``avx512_flash_attn_f32.cpp:198-208``).

    Q ``[B,Hq,Sq,D]``; K, V ``[B,Hkv,Sk,D]``.  kv head of q head ``h`` is
    ``h * Hkv // Hq`` (``avx512_flash_attn_f32.cpp:386``), which equals
    ``np.repeat(K, Hq//Hkv, axis=1)`` (``nn/functional.py:349-356``).
    Returns ``(O [B,Hq,Sq,D], LSE [B,Hq,Sq])`` with ``LSE = max + log(sum)``
    on the scaled logits (``avx512_flash_attn_f32.cpp:396-418``).  A fully
    masked row gives O = 0 (``tessera_rocm_flash_attn.cpp:137-143``) and
    LSE = -inf.
    """
    Q = np.asarray(Q, dtype)
    K = np.asarray(K, dtype)
    V = np.asarray(V, dtype)
    B, Hq, Sq, D = Q.shape
    _, Hkv, Sk, _ = K.shape
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    O = np.zeros((B, Hq, Sq, V.shape[-1]), dtype)
    LSE = np.full((B, Hq, Sq), -np.inf, dtype)
    off = _causal_limit(Sq, Sk)
    for b in range(B):
        for h in range(Hq):
            kh = h * Hkv // Hq
            s = (Q[b, h] @ K[b, kh].T) * dtype(scale)
            if softcap > 0:
                s = dtype(softcap) * np.tanh(s / dtype(softcap))
            if bias is not None:
                s = s + np.asarray(bias[b, h], dtype)
            if causal or window > 0:
                bounds = np.array([key_bounds(i, Sq, Sk, causal, window) for i in range(Sq)])
                j = np.arange(Sk)[None, :]
                s = np.where((j < bounds[:, :1]) | (j > bounds[:, 1:]), -np.inf, s)
            m = s.max(axis=-1, keepdims=True)
            msafe = np.where(np.isfinite(m), m, 0.0)
            e = np.exp(s - msafe)
            l = e.sum(axis=-1, keepdims=True)
            with np.errstate(divide="ignore", invalid="ignore"):
                p = np.where(l > 0, e / np.where(l > 0, l, 1.0), 0.0)
                LSE[b, h] = np.where(l[:, 0] > 0, msafe[:, 0] + np.log(l[:, 0]), -np.inf)
            O[b, h] = p @ V[b, kh]
    return O, LSE


def flash_attn_backward(dO, Q, K, V, scale=None, causal=False):
    """Adjoint of ``softmax(scale*Q K^T, causal) V`` — ``vjp_flash_attn``
    (``autodiff/vjp.py:1311-1377``) restated with GQA: ``dK`` / ``dV`` of a kv head
    are the sums over the query heads that share it
    (``runtime.py:7640-7649``).  f64 inside; returns ``(dQ, dK, dV)`` shaped like
    ``(Q, K, V)``.  Recomputes S and P; ``dS = (dP - rowsum(dP * P)) * P``."""
    Q = np.asarray(Q, np.float64)
    K = np.asarray(K, np.float64)
    V = np.asarray(V, np.float64)
    dO = np.asarray(dO, np.float64)
    B, Hq, Sq, D = Q.shape
    _, Hkv, Sk, _ = K.shape
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    dQ, dK, dV = np.zeros_like(Q), np.zeros_like(K), np.zeros_like(V)
    off = _causal_limit(Sq, Sk)
    for b in range(B):
        for h in range(Hq):
            kh = h * Hkv // Hq
            s = (Q[b, h] @ K[b, kh].T) * scale
            if causal:
                i = np.arange(Sq)[:, None]
                j = np.arange(Sk)[None, :]
                mask = j > i + off
                s = np.where(mask, -np.inf, s)
            m = s.max(axis=-1, keepdims=True)
            m = np.where(np.isfinite(m), m, 0.0)
            e = np.exp(s - m)
            l = e.sum(axis=-1, keepdims=True)
            p = np.where(l > 0, e / np.where(l > 0, l, 1.0), 0.0)
            dV[b, kh] += p.T @ dO[b, h]
            dp = dO[b, h] @ V[b, kh].T
            ds = (dp - (dp * p).sum(axis=-1, keepdims=True)) * p
            dQ[b, h] = (ds @ K[b, kh]) * scale
            dK[b, kh] += (ds.T @ Q[b, h]) * scale
    return dQ, dK, dV


def flash_attn_blockwise(Q, K, V, scale=None, causal=False, block=512,
                         dtype=np.float32, heads=None):
    """Same result computed one (batch, head) and ``block`` query rows at a
    time, so the S x S score tensor is never materialised (the dense reference
    would need 8.6 GB at B=4,H=32,S=4096).  ``heads`` optionally restricts to
    an iterable of (b, h) pairs (used by the bounded CPU baseline)."""
    Q = np.asarray(Q)
    K = np.asarray(K)
    V = np.asarray(V)
    B, Hq, Sq, D = Q.shape
    _, Hkv, Sk, _ = K.shape
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    off = _causal_limit(Sq, Sk)
    pairs = list(heads) if heads is not None else [(b, h) for b in range(B) for h in range(Hq)]
    O = np.zeros((B, Hq, Sq, V.shape[-1]), dtype)
    LSE = np.full((B, Hq, Sq), -np.inf, dtype)
    for (b, h) in pairs:
        kh = h * Hkv // Hq
        Kf = K[b, kh].astype(dtype)
        Vf = V[b, kh].astype(dtype)
        for i0 in range(0, Sq, block):
            i1 = min(i0 + block, Sq)
            jend = min(Sk, i1 + off) if causal else Sk
            if jend <= 0:
                continue
            s = (Q[b, h, i0:i1].astype(dtype) @ Kf[:jend].T) * dtype(scale)
            if causal:
                i = np.arange(i0, i1)[:, None]
                j = np.arange(jend)[None, :]
                s = np.where(j > i + off, -np.inf, s)
            m = s.max(axis=-1, keepdims=True)
            msafe = np.where(np.isfinite(m), m, 0.0)
            e = np.exp(s - msafe)
            l = e.sum(axis=-1, keepdims=True)
            ok = l[:, 0] > 0
            lsafe = np.where(l > 0, l, 1.0)
            O[b, h, i0:i1] = np.where(l > 0, (e @ Vf[:jend]) / lsafe, 0.0)
            with np.errstate(divide="ignore"):
                LSE[b, h, i0:i1] = np.where(ok, msafe[:, 0] + np.log(lsafe[:, 0]), -np.inf)
    return O, LSE


def attention_region_reference(Q, K, V, scale=1.0, causal=False):
    """``AttentionRegion.reference`` — the 2-D (M,D),(Nk,D) arbiter oracle;
    causal masks ``n > m`` (top-left aligned).  ``fusion_core.py:714-727``."""
    Q = np.asarray(Q, np.float32)
    K = np.asarray(K, np.float32)
    V = np.asarray(V, np.float32)
    s = (Q @ K.T) * np.float32(scale)
    if causal:
        m = np.arange(s.shape[0])[:, None]
        n = np.arange(s.shape[1])[None, :]
        s = np.where(n > m, np.float32(-np.inf), s)
    s = s - s.max(-1, keepdims=True)
    e = np.exp(s)
    p = e / e.sum(-1, keepdims=True)
    return (p @ V).astype(np.float32)


# ---------------------------------------------------------------------------
# MoE routing, permutation, grouped GEMM, SwiGLU, combine
# ---------------------------------------------------------------------------


@dataclass
class Routing:
    """Result of :func:`route_tokens` (``distributed/moe.py:95-116``)."""
    assignment: np.ndarray   # (T, k) int64, -1 = dropped
    weights: np.ndarray      # (T, k) f32
    load: np.ndarray         # (E,) int64
    overflow: int


def router_probs(scores: np.ndarray) -> np.ndarray:
    """f32 max-subtracted softmax over experts (``distributed/moe.py:163-165``)."""
    s = np.asarray(scores, np.float32)
    e = np.exp(s - s.max(axis=1, keepdims=True))
    return e / e.sum(axis=1, keepdims=True)


def topk_desc_lowest_index(p: np.ndarray, k: int) -> np.ndarray:
    """Top-k per row, descending by value, ties broken by LOWEST expert id.

    The reference takes ``np.argsort(probs, axis=1)[:, -k:][:, ::-1]`` with the
    default (unstable) sort kind (``distributed/moe.py:168``), whose order among
    bit-equal probabilities is numpy-build dependent.  The lane and this oracle
    fix the tie rule to the one the reference's stable router uses
    (``models/moe_routing.py:69-70``); on inputs with no bit-equal
    probabilities among a token's experts the two coincide exactly —
    :func:`has_routing_ties` detects the other case.
    """
    order = np.argsort(-np.asarray(p), axis=1, kind="stable")
    return order[:, :k]


def has_routing_ties(p: np.ndarray, k: int) -> bool:
    """True if some token has bit-equal probabilities among its top-(k+1)."""
    srt = -np.sort(-np.asarray(p), axis=1)
    kk = min(k + 1, p.shape[1])
    return bool(np.any(srt[:, : kk - 1] == srt[:, 1:kk]))


def compute_capacity(capacity_factor, num_tokens, num_experts):
    """MoEConfig.compute_capacity (distributed/moe.py:79-92) on one rank: the tokens-per-expert
    quotient is formed first, then scaled, then rounded up (numpy float64 throughout)."""
    tokens_per_expert = num_tokens / max(1, num_experts)
    return int(np.ceil(capacity_factor * tokens_per_expert))


def route_tokens(scores: np.ndarray, num_experts: int, top_k: int,
                 normalize_weights: bool = True,
                 capacity_factor: float = 1e9,
                 capacity: int | None = None) -> Routing:
    """``distributed/moe.py:119-206`` without jitter.

    capacity = ``ceil(capacity_factor * (T / E))`` when not given
    (``distributed/moe.py:79-92``).  Over-capacity slots are dropped in
    token-major, slot-minor order: assignment -1, weight 0.
    """
    s = np.asarray(scores, np.float32)
    if s.ndim != 2:
        raise ValueError("scores must be 2D (num_tokens, num_experts)")
    T, E = s.shape
    if E != num_experts:
        raise ValueError("expert count mismatch")
    p = router_probs(s)
    idx = topk_desc_lowest_index(p, top_k)
    w = np.take_along_axis(p, idx, axis=1)
    if normalize_weights and top_k > 1:
        ws = w.sum(axis=1, keepdims=True)
        ws = np.where(ws > 0, ws, 1.0)
        w = w / ws
    load = np.bincount(idx.reshape(-1), minlength=E).astype(np.int64)
    if capacity is None:
        capacity = compute_capacity(capacity_factor, T, E)
    assignment = idx.astype(np.int64).copy()
    weights = w.astype(np.float32).copy()
    overflow = 0
    fill = np.zeros(E, np.int64)
    if capacity < T:          # otherwise nothing can overflow
        for t in range(T):
            for s_ in range(top_k):
                e = idx[t, s_]
                if fill[e] >= capacity:
                    assignment[t, s_] = -1
                    weights[t, s_] = 0.0
                    overflow += 1
                else:
                    fill[e] += 1
    return Routing(assignment, weights, load, overflow)


@dataclass
class TransportDescriptor:
    """The int32 device ABI of ``compiler/moe_transport.py:194-273``."""
    token_of_slot: np.ndarray     # int32[S]
    expert_of_slot: np.ndarray    # int32[S], non-decreasing
    combine_weights: np.ndarray   # f32[S]
    group_sizes: np.ndarray       # int32[E]
    group_offsets: np.ndarray     # int32[E+1]
    sort_perm: np.ndarray         # int64[S] kept token-major slot ids, expert-sorted


def plan_dispatch(assignment: np.ndarray, weights: np.ndarray, num_experts: int
                  ) -> TransportDescriptor:
    """Steps 2 of ``moe_layer`` (``nn/functional.py:463-476``) expressed in the
    transport ABI (``compiler/moe_transport.py:221-227``): drop ``-1`` slots,
    stable-sort the kept token-major slots by expert."""
    a = np.asarray(assignment, np.int64)
    T, k = a.shape
    flat_e = a.reshape(-1)
    flat_w = np.asarray(weights, np.float32).reshape(-1)
    kept = np.nonzero(flat_e >= 0)[0]
    order = np.argsort(flat_e[kept], kind="stable")
    sort_perm = kept[order].astype(np.int64)
    sizes = np.bincount(flat_e[sort_perm], minlength=num_experts).astype(np.int64)
    offsets = np.concatenate(([0], np.cumsum(sizes)))
    return TransportDescriptor(
        token_of_slot=(sort_perm // k).astype(np.int32),
        expert_of_slot=flat_e[sort_perm].astype(np.int32),
        combine_weights=flat_w[sort_perm].astype(np.float32),
        group_sizes=sizes.astype(np.int32),
        group_offsets=offsets.astype(np.int32),
        sort_perm=sort_perm,
    )


def route_top_k_stable(logits: np.ndarray, top_k: int, normalize: bool = True):
    """The reference's second router (``models/moe_routing.py:54-77``): stable
    descending sort on the logits, weights = softmax over the SELECTED logits."""
    lg = np.asarray(logits, np.float32)
    order = np.argsort(-lg, axis=1, kind="stable")[:, :top_k]
    sel = np.take_along_axis(lg, order, axis=1)
    if normalize:
        sel = sel - sel.max(axis=1, keepdims=True)
        w = np.exp(sel)
        w = w / w.sum(axis=1, keepdims=True)
    else:
        w = np.ones_like(sel) / top_k
    return order.astype(np.int64), w.astype(np.float32)


@dataclass
class PackingPlan:
    """Token-major view of a packing plan (``stdlib/moe.py:58-77``)."""
    expert_ids: np.ndarray     # (T, k) int64
    weights: np.ndarray        # (T, k) f32
    kept_mask: np.ndarray      # (T, k) bool
    sort_perm: np.ndarray      # (S,) int64 kept token-major slot ids, expert-sorted
    inverse_perm: np.ndarray   # (T*k,) int64 packed position of each slot, -1 = dropped
    group_sizes: np.ndarray    # (E,) int64


def plan_dispatch_token_major(expert_ids, weights, num_experts: int, capacity: int | None = None) -> PackingPlan:
    """``stdlib.moe.plan_dispatch`` (``stdlib/moe.py:79-115``): slots in token-major
    order; once an expert has ``capacity`` slots the rest routed to it are dropped;
    kept slots stable-sorted by expert.  Without a capacity this is
    ``models.moe_routing.plan_packing`` (``models/moe_routing.py:80-99``), whose
    ``inverse_perm`` (``inverse_perm[sort_perm] = arange``) is extended here with -1 for
    dropped slots."""
    eids = np.asarray(expert_ids, np.int64)
    if eids.ndim != 2:
        raise ValueError("expert_ids must be (T, k)")
    T, k = eids.shape
    if eids.size and (eids.min() < 0 or eids.max() >= num_experts):
        raise ValueError("expert id out of range")
    flat = eids.reshape(-1)
    kept = np.ones(flat.shape[0], bool)
    if capacity is not None:
        seen = np.zeros(num_experts, np.int64)
        for s_ in range(flat.shape[0]):
            e = int(flat[s_])
            if seen[e] >= capacity:
                kept[s_] = False
            else:
                seen[e] += 1
    kept_slots = np.nonzero(kept)[0]
    order = np.argsort(flat[kept_slots], kind="stable")
    sort_perm = kept_slots[order].astype(np.int64)
    inverse = np.full(flat.shape[0], -1, np.int64)
    inverse[sort_perm] = np.arange(sort_perm.shape[0], dtype=np.int64)
    sizes = np.bincount(flat[sort_perm], minlength=num_experts).astype(np.int64)
    return PackingPlan(eids, np.asarray(weights, np.float32).reshape(T, k), kept.reshape(T, k), sort_perm, inverse,
                       sizes)


def unpack_combine(y_packed, inverse_perm, weights) -> np.ndarray:
    """``models.moe_routing.unpack_combine`` (``models/moe_routing.py:109-116``):
    ``(y_packed[inverse_perm].reshape(T, k, H) * w[:, :, None]).sum(axis=1)`` in f32;
    a dropped slot (``inverse_perm < 0``) contributes zero, the rule of
    ``stdlib.moe.combine`` (``stdlib/moe.py:124-134``)."""
    yp = np.asarray(y_packed, np.float32)
    w = np.asarray(weights, np.float32)
    T, k = w.shape
    inv = np.asarray(inverse_perm, np.int64).reshape(T, k)
    rows = np.where(inv[:, :, None] >= 0, yp[np.maximum(inv, 0)], np.float32(0))      # (T, k, H)
    return (rows * w[:, :, None]).sum(axis=1, dtype=np.float32)


def grouped_gemm(x, w, group_sizes, dtype: str = "bf16", store: bool = True):
    """``ops.grouped_gemm`` contiguous kind (``__init__.py:291-351``) /
    ``reference_grouped_gemm`` (``compiler/grouped_layout.py:396-414``).

    ``store=True`` applies the storage-dtype rule (result re-rounded to the
    operand storage dtype, ``__init__.py:5824-5855``); ``store=False`` keeps
    the f64 product of the storage-rounded operands.
    """
    xa = round_to_storage(np.asarray(x, np.float32), dtype)
    wa = round_to_storage(np.asarray(w, np.float32), dtype)
    gs = np.asarray(group_sizes).astype(np.int64).reshape(-1)
    if xa.ndim != 2 or wa.ndim != 3 or wa.shape[0] != gs.shape[0]:
        raise ValueError("grouped_gemm: x (T,K), w (E,K,N), group_sizes (E,)")
    if wa.shape[1] != xa.shape[1]:
        raise ValueError("grouped_gemm: K mismatch")
    if int(gs.sum()) != xa.shape[0]:
        raise ValueError("grouped_gemm: group_sizes must sum to T")
    out = np.zeros((xa.shape[0], wa.shape[2]), np.float64)
    off = 0
    for e in range(wa.shape[0]):
        n = int(gs[e])
        if n:
            out[off:off + n] = xa[off:off + n].astype(np.float64) @ wa[e].astype(np.float64)
        off += n
    if store:
        return round_to_storage(out.astype(np.float32), dtype)
    return out


def silu_mul(a, b):
    """``silu(a) * b`` with ``silu(a) = a / (1 + exp(-a))``
    (``__init__.py:559-574``), f32."""
    a = np.asarray(a, np.float32)
    b = np.asarray(b, np.float32)
    return (a / (1.0 + np.exp(-a))) * b


def moe_swiglu_block(x, w_gate, w_up, w_down, group_sizes, dtype: str = "bf16"):
    """``ops.moe_swiglu_block`` (``__init__.py:592-616``): every intermediate
    re-rounded to the storage dtype (gate, up, silu_mul, down)."""
    gate = grouped_gemm(x, w_gate, group_sizes, dtype)
    up = grouped_gemm(x, w_up, group_sizes, dtype)
    hidden = round_to_storage(silu_mul(gate, up), dtype)
    return grouped_gemm(hidden, w_down, group_sizes, dtype)


def moe_combine(y_perm, desc: TransportDescriptor, num_tokens: int, dtype: str = "bf16",
                accumulate: str = "f64"):
    """Step 4 of ``moe_layer`` (``nn/functional.py:487-490``): scatter-add of
    ``y_perm * weight`` into token rows.  The reference accumulates in slot
    order into an array of the storage dtype; that order is not pinned, so the
    oracle offers the exact (f64) sum, and the caller compares to tolerance."""
    y = np.asarray(y_perm, np.float32)
    acc = np.zeros((num_tokens, y.shape[1]), np.float64 if accumulate == "f64" else np.float32)
    np.add.at(acc, desc.token_of_slot.astype(np.int64),
              (y * desc.combine_weights[:, None]).astype(acc.dtype))
    return acc


def moe_layer(x, router_logits, w_gate, w_up, w_down, top_k: int,
              normalize_weights: bool = True, capacity_factor: float = 0.0,
              dtype: str = "bf16"):
    """``nn.functional.moe_layer`` (``nn/functional.py:403-490``) with the
    router logits given directly (the router GEMM is ``ops.gemm`` and is
    covered by :func:`gemm_storage`).  Returns (out f64 [T,N], descriptor)."""
    T = np.asarray(x).shape[0]
    E = np.asarray(w_gate).shape[0]
    cf = capacity_factor if capacity_factor > 0 else 1e9
    r = route_tokens(np.asarray(router_logits, np.float32), E, top_k,
                     normalize_weights=normalize_weights, capacity_factor=cf)
    desc = plan_dispatch(r.assignment, r.weights, E)
    xa = round_to_storage(np.asarray(x, np.float32), dtype)
    x_perm = xa[desc.token_of_slot.astype(np.int64)]
    y_perm = moe_swiglu_block(x_perm, w_gate, w_up, w_down, desc.group_sizes, dtype)
    return moe_combine(y_perm, desc, T, dtype), desc


# ---------------------------------------------------------------------------
# quantisation
# ---------------------------------------------------------------------------

E4M3_MAX = 448.0


def e4m3_decode_table() -> np.ndarray:
    """All 256 OCP e4m3fn codes -> f32 (bias 7, no inf, 0x7f/0xff = NaN,
    subnormal step 2^-9).  This is the published format definition, not a
    restatement of reference code; it anchors :func:`e4m3_encode`."""
    t = np.zeros(256, np.float32)
    for c in range(256):
        s = -1.0 if c & 0x80 else 1.0
        e = (c >> 3) & 0xF
        m = c & 7
        if e == 0xF and m == 7:
            t[c] = np.nan
        elif e == 0:
            t[c] = s * m * 2.0 ** -9
        else:
            t[c] = s * (1.0 + m / 8.0) * 2.0 ** (e - 7)
    return t


def fpquant_grid(v: np.ndarray, max_normal: float = 448.0, mantissa_bits: int = 3,
                 min_exp: int = -6) -> np.ndarray:
    """The native lanes' definition of the fp8 grid, elementwise f32 -> f32:
    ``ax=min(|x|,max)``; ``e=max(floor(log2 ax), min_exp)``; ``ulp=2^(e-mant)``;
    ``rounded=min(rne(ax/ulp)*ulp, max)``; NaN propagates.
    (``avx512_fpquant_f32.cpp:28-41``.)"""
    v = np.asarray(v, np.float32)
    ax = np.minimum(np.abs(v), np.float32(max_normal))
    with np.errstate(divide="ignore", invalid="ignore"):
        _, ex = np.frexp(ax)                    # ax = m * 2^ex, m in [0.5,1)
        e = np.maximum(ex.astype(np.int32) - 1, min_exp)
        ulp = np.ldexp(np.float32(1.0), e - mantissa_bits).astype(np.float32)
        r = np.minimum(np.rint(ax / ulp) * ulp, np.float32(max_normal))
    r = np.where(ax > 0, r, np.float32(0.0))
    out = np.where(v < 0, -r, r).astype(np.float32)
    return np.where(np.isnan(v), v, out)


def e4m3_encode(grid_values: np.ndarray) -> np.ndarray:
    """f32 values that already lie on the e4m3fn grid -> their byte codes."""
    v = np.asarray(grid_values, np.float32)
    a = np.abs(v)
    m, ex = np.frexp(a)                         # a = m * 2^ex, m in [0.5, 1)
    e = ex.astype(np.int32) - 1                 # floor(log2 a)
    normal = a >= 2.0 ** -6
    mant_n = np.rint((a / np.ldexp(1.0, np.where(normal, e, 0)) - 1.0) * 8).astype(np.int32)
    code_n = ((e + 7) << 3) | mant_n
    code_s = np.rint(a * 512.0).astype(np.int32)
    code = np.where(normal, code_n, code_s)
    code = np.where(a == 0, 0, code)
    code = code | np.where(np.signbit(v), 0x80, 0)
    return code.astype(np.uint8)


def quantize_fp8_e4m3(x: np.ndarray, scale: float | None = None):
    """``ops.quantize_fp8`` on the ml_dtypes branch (``__init__.py:3340-3374``):
    ``scale = max(amax/448, 1e-12)`` as a Python float; ``t = clip(x/scale,
    +-448)``; round to the e4m3fn grid (RNE, gradual underflow).  Returns
    ``(codes uint8, grid f32, scale np.float32)``; the reference's return value
    is ``grid * f32(scale)``."""
    x = np.asarray(x, np.float32)
    if scale is None:
        amax = np.max(np.abs(x)) if x.size else np.float32(0)
        scale = float(np.maximum(amax / E4M3_MAX, 1e-12))
    scaled = np.clip(x / scale, -E4M3_MAX, E4M3_MAX).astype(np.float32)
    grid = fpquant_grid(scaled)
    return e4m3_encode(grid), grid, np.float32(scale)


#: (max_normal, mantissa_bits, min_exp) of the per-tensor float grids: the native lanes'
#: format table (``runtime.py:16939-16946``).  The fp8 grids have IEEE gradual underflow;
#: fp6 and fp4 keep the pure mantissa snap (exponent floor -126, i.e. none in practice).
FP_FORMATS = {"e4m3": (448.0, 3, -6), "e5m2": (57344.0, 2, -14), "e2m3": (7.5, 3, -126), "e3m2": (28.0, 2, -126),
              "e2m1": (6.0, 1, -126)}


def quantize_fp(x: np.ndarray, fmt: str, scale: float | None = None):
    """``ops.quantize_fp8`` / ``quantize_fp6`` / ``quantize_fp4`` (``__init__.py:3340-3374``,
    ``3411-3464``): per-tensor ``scale = max(amax / max_normal, 1e-12)`` in f32 unless given,
    ``grid = fpquant(clip(x / scale))``, result ``grid * f32(scale)``.  Returns
    ``(dequantised f32, grid f32, scale np.float32)``."""
    mx, mant, min_exp = FP_FORMATS[fmt]
    x = np.asarray(x, np.float32)
    if scale is None:
        amax = np.max(np.abs(x)) if x.size else np.float32(0)
        scale = float(np.maximum(amax / np.float32(mx), np.float32(1e-12)))
    with np.errstate(invalid="ignore"):
        scaled = np.clip(x / np.float32(scale), -mx, mx).astype(np.float32)
    grid = fpquant_grid(scaled, mx, mant, min_exp)
    return (grid * np.float32(scale)).astype(np.float32), grid, np.float32(scale)


def quantize_nvfp4(x: np.ndarray, block_size: int = 16):
    """``ops.quantize_nvfp4`` (``__init__.py:3472-3500``), i.e. ``microscaling.quantize`` with
    the ``nvfp4`` format followed by ``dequantize`` (``compiler/microscaling.py:317-384``):
    blocks of ``block_size`` along the last axis (zero-padded to a whole block);
    ``raw = max(amax / 6, 1e-30)``; the block scale is ``raw`` cast to e4m3fn (round to
    nearest even; a scale that rounds to zero is replaced by 1); codes are
    ``block / scale`` cast to the E2M1 grid {0, .5, 1, 1.5, 2, 3, 4, 6} (round to nearest
    even, saturating); the dequantised value is ``code * scale`` in f32.  Returns
    ``(dequantised f32, scales f32)`` with ``scales.shape == x.shape[:-1] + (blocks,)``.
    (The reference's casts go through ``ml_dtypes``; a raw scale above 448, which that
    cast turns into NaN, saturates here.)"""
    x = np.asarray(x, np.float32)
    n = x.shape[-1]
    nb = -(-n // block_size)
    xp = np.zeros(x.shape[:-1] + (nb * block_size,), np.float32)
    xp[..., :n] = x
    blocks = xp.reshape(x.shape[:-1] + (nb, block_size))
    amax = np.abs(blocks).max(axis=-1)
    raw = np.maximum(amax / np.float32(6.0), np.float32(1e-30)).astype(np.float32)
    scale = fpquant_grid(raw)                                   # e4m3fn grid, RNE, gradual underflow
    sf = np.where(scale == 0.0, np.float32(1.0), scale).astype(np.float32)[..., None]
    codes = fpquant_grid((blocks / sf).astype(np.float32), max_normal=6.0, mantissa_bits=1, min_exp=0)
    dq = (codes * sf).astype(np.float32).reshape(x.shape[:-1] + (nb * block_size,))[..., :n]
    return np.ascontiguousarray(dq), scale.astype(np.float32)


def grouped_gemm_nvfp4(x, w, group_sizes):
    """``ops.grouped_gemm(..., quant="nvfp4")`` (``__init__.py:340-351``,
    ``compiler/grouped_layout.py:353-392``): x ``(T, K)`` and every expert's weight
    ``(K, N)`` are rounded onto the NVFP4 grid along their last axis, then the grouped
    product runs on the dequantised values (f64 here).  Returns ``(T, N)`` f64."""
    xq, _ = quantize_nvfp4(np.asarray(x, np.float32))
    w = np.asarray(w, np.float32)
    wq = np.stack([quantize_nvfp4(w[e])[0] for e in range(w.shape[0])])
    out = np.zeros((xq.shape[0], w.shape[2]), np.float64)
    off = 0
    for e, n in enumerate(np.asarray(group_sizes).astype(np.int64)):
        if n:
            out[off:off + n] = xq[off:off + n].astype(np.float64) @ wq[e].astype(np.float64)
        off += int(n)
    return out


#: quant= spellings of the grouped product -> (activation format, weight format)
#: (``compiler/grouped_layout.py:320-332``)
GROUPED_QUANT_SCHEMES = {
    "fp8_e4m3": ("fp8_e4m3", "fp8_e4m3"), "fp8": ("fp8_e4m3", "fp8_e4m3"), "fp8_e5m2": ("fp8_e5m2", "fp8_e5m2"),
    "nvfp4": ("nvfp4", "nvfp4"), "fp8xfp4": ("fp8_e4m3", "nvfp4"), "fp8_e4m3xnvfp4": ("fp8_e4m3", "nvfp4"),
    "fp8_e5m2xnvfp4": ("fp8_e5m2", "nvfp4"),
}


def _qdq(a: np.ndarray, dtype: str) -> np.ndarray:
    """One 2-D operand quantised and dequantised (``compiler/grouped_layout.py:353-370``)."""
    if dtype == "nvfp4":
        return quantize_nvfp4(a)[0]
    return quantize_fp(a, "e5m2" if dtype == "fp8_e5m2" else "e4m3")[0]


def grouped_gemm_quant(x, w, group_sizes, quant: str):
    """``ops.grouped_gemm(..., quant=)`` for every scheme of the reference
    (``compiler/grouped_layout.py:373-392``): x ``(T, K)`` is quantised as one tensor with
    the activation format, every expert's ``(K, N)`` weight on its own with the weight
    format, and the grouped product runs on the dequantised values (f64 here)."""
    act, wt = GROUPED_QUANT_SCHEMES[str(quant).lower()]
    xq = _qdq(np.asarray(x, np.float32), act)
    w = np.asarray(w, np.float32)
    wq = np.stack([_qdq(w[e], wt) for e in range(w.shape[0])])
    out = np.zeros((xq.shape[0], w.shape[2]), np.float64)
    off = 0
    for e, n in enumerate(np.asarray(group_sizes).astype(np.int64)):
        if n:
            out[off:off + n] = xq[off:off + n].astype(np.float64) @ wq[e].astype(np.float64)
        off += int(n)
    return out


def e5m2_decode_table() -> np.ndarray:
    """All 256 OCP e5m2 codes -> f32 (bias 15, two mantissa bits, subnormal step 2^-16, exponent 31
    = inf / NaN): the published format, i.e. the upper byte of IEEE half precision."""
    t = np.zeros(256, np.float32)
    for c in range(256):
        s = -1.0 if c & 0x80 else 1.0
        e = (c >> 2) & 0x1F
        m = c & 3
        if e == 0x1F:
            t[c] = s * np.inf if m == 0 else np.nan
        elif e == 0:
            t[c] = s * m * 2.0 ** -16
        else:
            t[c] = s * (1.0 + m / 4.0) * 2.0 ** (e - 15)
    return t


def e5m2_encode(grid_values: np.ndarray) -> np.ndarray:
    """f32 values that already lie on the e5m2 grid (finite) -> their byte codes."""
    v = np.asarray(grid_values, np.float32)
    h = v.astype(np.float16)                      # exact: every e5m2 value is a half
    assert np.array_equal(h.astype(np.float32), v, equal_nan=True)
    return (h.view(np.uint16) >> 8).astype(np.uint8)


def quantize_fp8_e5m2(x: np.ndarray, scale: float | None = None):
    """``ops.quantize_fp8(format="e5m2")`` (``__init__.py:3340-3374``) -> ``(codes uint8, grid f32,
    scale np.float32)``: per-tensor ``scale = max(amax / 57344, 1e-12)``, clip, the (57344, 2, -14) grid."""
    dq, grid, s = quantize_fp(x, "e5m2", scale)
    return e5m2_encode(grid), grid, s


def gemm_fp8_codes(a_codes, b_codes, scale_a, scale_b, fmt: str = "e4m3"):
    """The fp8 GEMM on codes of either format, f64 accumulate: ``(A @ B) * sA * sB``."""
    t = (e5m2_decode_table() if fmt == "e5m2" else e4m3_decode_table()).astype(np.float64)
    return (t[np.asarray(a_codes, np.uint8)] @ t[np.asarray(b_codes, np.uint8)]) * float(np.float32(scale_a)) * float(np.float32(scale_b))


def gemm_e4m3(a_codes, b_codes, scale_a, scale_b, out_dtype: str = "bf16"):
    """fp8 GEMM config: ``f32acc(Aq.Bq) * sA * sB`` stored in ``out_dtype``
    (f64 accumulate here).  Returns the f64 value before the final store; the
    caller rounds when comparing stored results."""
    t = e4m3_decode_table().astype(np.float64)
    A = t[np.asarray(a_codes, np.uint8)]
    B = t[np.asarray(b_codes, np.uint8)]
    return (A @ B) * float(np.float32(scale_a)) * float(np.float32(scale_b))


def quantize_int8_per_channel(M: np.ndarray, axis: int):
    """``compiler/smoothquant.py:79-84``: ``absmax = max(|M|.max(axis), 1e-12)``;
    ``scale = absmax/127``; ``q = clip(round_half_even(M/scale), +-127)``."""
    M = np.asarray(M, np.float32)
    absmax = np.maximum(np.abs(M).max(axis=axis, keepdims=True), 1e-12)
    scale = absmax / 127.0
    q = np.round(M / scale).clip(-127, 127).astype(np.int8)
    return q, scale.astype(np.float32)


def gemm_i8_i32(xq: np.ndarray, wq: np.ndarray) -> np.ndarray:
    """Exact ``int32(x_q) @ int32(w_q)`` (``compiler/smoothquant.py:122``).
    Computed blockwise in f64 BLAS where exact (|products| sum < 2^53), else in
    int64 — both give the exact integer, then wrap to int32 like numpy."""
    xq = np.asarray(xq)
    wq = np.asarray(wq)
    K = xq.shape[-1]
    if K * 127 * 127 < 2 ** 52:
        acc = np.rint(xq.astype(np.float64) @ wq.astype(np.float64)).astype(np.int64)
    else:  # pragma: no cover - not reached at any tested size
        acc = xq.astype(np.int64) @ wq.astype(np.int64)
    return acc.astype(np.int32)


def w8a8_matmul(X: np.ndarray, W: np.ndarray):
    """``smoothquant_matmul`` without smoothing == ``_naive_w8a8``
    (``compiler/smoothquant.py:115-124``;
    ``tests/unit/test_smoothquant_migration.py:68-74``): per-row activation
    scales, per-column weight scales, int32 accumulate, two f32 multiplies in
    the order ``acc * a_scale * w_scale``.  Returns (y f32, acc i32, x_q, a_scale
    [M,1], w_q, w_scale [N])."""
    x_q, a_scale = quantize_int8_per_channel(X, axis=1)
    w_q, w_scale = quantize_int8_per_channel(W, axis=0)
    acc = gemm_i8_i32(x_q, w_q)
    y = acc.astype(np.float32) * a_scale * w_scale.reshape(-1)[None, :]
    return y.astype(np.float32), acc, x_q, a_scale, w_q, w_scale.reshape(-1)


def quantize_int8_tensor(x: np.ndarray, scale: float | None = None):
    """``quantization.quantize_int8`` symmetric (``quantization.py:24-37``): one scale,
    ``f32(max|x| / 127)`` (1 when the tensor is all zero) unless given;
    ``q = clip(rint(x / scale), -127, 127)``.  Returns ``(q int8, scale np.float32)``."""
    x = np.asarray(x, np.float32)
    if scale is None:
        m = float(np.max(np.abs(x))) if x.size else 0.0
        s = np.float32(1.0) if m == 0.0 else np.float32(m / 127)
    else:
        s = np.float32(scale)
    return np.round(x / s).clip(-127, 127).astype(np.int8), s


def migrate_activation_scale(X_calib: np.ndarray, W: np.ndarray, alpha: float = 0.5, eps: float = 1e-5):
    """``compiler/smoothquant.py:69-76, 87-112``: per input channel
    ``s = max(max|X|^alpha / max|W|^(1-alpha), eps)`` (f64 powers of the eps-floored maxima,
    stored f32), ``W_s = s[:, None] * W``, quantised per output column.
    Returns ``(s f32 [C_in], w_q int8, w_scale f32 [C_out])``."""
    X_calib = np.asarray(X_calib, np.float32)
    W = np.asarray(W, np.float32)
    a = np.maximum(np.abs(X_calib).max(axis=0).astype(np.float64), eps)
    w = np.maximum(np.abs(W).max(axis=1).astype(np.float64), eps)
    s = np.maximum((a ** alpha) / (w ** (1.0 - alpha)), eps).astype(np.float32)
    w_q, w_scale = quantize_int8_per_channel(s[:, None] * W, axis=0)
    return s, w_q, w_scale.reshape(-1)


def smoothquant_matmul(X: np.ndarray, smoothing: np.ndarray, w_q: np.ndarray, w_scale: np.ndarray):
    """``compiler/smoothquant.py:115-124``: ``X_hat = f32(X) / s``; per-row int8 codes of
    ``X_hat``; exact integer product with the int8 weight; ``f32(acc) * a_scale * w_scale``.
    Returns ``(y f32, acc i32, x_q, a_scale [M,1])``."""
    X_hat = np.asarray(X, np.float32) / np.asarray(smoothing, np.float32)[None, :]
    x_q, a_scale = quantize_int8_per_channel(X_hat, axis=1)
    acc = gemm_i8_i32(x_q, np.asarray(w_q, np.int8))
    y = acc.astype(np.float32) * a_scale * np.asarray(w_scale, np.float32).reshape(-1)[None, :]
    return y.astype(np.float32), acc, x_q, a_scale


# ---------------------------------------------------------------------------
# error metrics used by the parity tests
# ---------------------------------------------------------------------------


def max_rel_err(x: np.ndarray, ref: np.ndarray) -> float:
    """Normwise max relative error ``max|x - ref| / max|ref|``."""
    x = np.asarray(x, np.float64)
    ref = np.asarray(ref, np.float64)
    d = float(np.max(np.abs(x - ref))) if x.size else 0.0
    s = float(np.max(np.abs(ref))) if ref.size else 0.0
    return d / s if s > 0 else d
