"""The measured-arbiter seam: gfx950 kernel candidates behind Tessera's
``Candidate`` plugin protocol.

Mirrors ``python/tessera/compiler/emit/candidate.py:41-48,110-236,339-451`` —
``Tier``, the op-kind tags, ``Candidate`` (``name / tier / target / op /
accuracy_atol / available() / applies_to() / run() / measure_device_latency()``),
``register_candidate``, ``arbitrate``, ``run_arbitrated``, the dispatch log and
histogram — so the classes below can be registered into the reference's own
registry unchanged.  The F4 gate (``verify_candidate``) runs a candidate on the
reference's probe shapes (``compiler/fusion_core.py:1067-1126``) and compares
with the region's numpy definition; that comparison is the only place the
region's ``reference`` executes.

One deliberate difference from the reference's ROCm candidates
(``compiler/emit/rocm_hip.py:701-806``): these never degrade to numpy.  A
candidate that cannot run reports ``available() == False`` / ``applies_to() ==
False`` and so never wins; a failure inside ``run`` propagates.  When no
candidate is viable :func:`run_arbitrated` raises :class:`ArbiterError` instead
of computing the region on the CPU.
"""
from __future__ import annotations

from abc import ABC, abstractmethod
from collections import deque
from dataclasses import dataclass
from enum import IntEnum
from typing import Any, Callable, Optional

import numpy as np

from . import bf16 as _bf16
from . import lane as _lane
from . import ops as _ops


class Tier(IntEnum):
    SYNTHESIZED = 1
    EMITTED = 2
    HAND_TUNED = 3


OP_FUSED_REGION = "fused_region"
OP_ATTENTION = "attention"
OP_GATED_MATMUL = "gated_matmul"
OP_POINTWISE = "pointwise"
OP_MATMUL = "matmul"
OP_GROUPED_GEMM = "grouped_gemm"          # registered through register_op_kind below

#: execution tags that mean "no kernel ran" (``kernel_emitter.py:248``)
REFERENCE_EXECUTIONS = frozenset({"reference", "fallback"})

TARGET = "rocm_gfx950"
GEMM_TAG = "gfx950_mfma_gemm"
ATTN_TAG = "gfx950_mfma_flash_attn"
GROUPED_TAG = "gfx950_mfma_grouped_gemm"
FUSED_TAG = "gfx950_mfma_fused_gemm"
GATED_TAG = "gfx950_mfma_gated_gemm"


class ArbiterError(RuntimeError):
    """A forced candidate is missing / unavailable, or no candidate is viable."""


# ---- regions (the slices of compiler/fusion_core.py the gate needs) ------------------

def _round_to_storage(x, dtype: str) -> np.ndarray:
    a = np.ascontiguousarray(x, np.float32)
    if dtype in ("float16", "f16"):
        return a.astype(np.float16).astype(np.float32)
    if dtype in ("bfloat16", "bf16"):
        return _bf16.from_float32(a).to_float32()
    raise ValueError(f"unsupported matmul storage dtype {dtype!r}")


@dataclass(frozen=True)
class MatmulRegion:
    """``fusion_core.MatmulRegion`` (``:365-405``): bare ``D = A @ B``, 16-bit
    storage, f32 accumulate; transpose flags orient the raw operands."""
    dtype: str = "bfloat16"
    transpose_a: bool = False
    transpose_b: bool = False

    def _natural(self, A, B, cast: bool = True):
        A = np.asarray(A, np.float32) if cast else np.asarray(A)
        B = np.asarray(B, np.float32) if cast else np.asarray(B)
        if self.transpose_a:
            A = np.ascontiguousarray(A.T)
        if self.transpose_b:
            B = np.ascontiguousarray(B.T)
        return A, B

    def reference(self, A, B) -> np.ndarray:
        A, B = self._natural(A, B)
        return (_round_to_storage(A, self.dtype) @ _round_to_storage(B, self.dtype)).astype(np.float32)


@dataclass(frozen=True)
class AttentionRegion:
    """``fusion_core.AttentionRegion`` (``:672-727``): 2-D ``softmax(scale Q K^T) V``;
    ``causal`` masks keys ``n > m``."""
    scale: float = 1.0
    causal: bool = False
    q_transposed: bool = False
    k_transposed: bool = False
    storage_dtype: str = "f16"

    def _natural(self, Q, K, cast: bool = True):
        Q = np.asarray(Q, np.float32) if cast else np.asarray(Q)
        K = np.asarray(K, np.float32) if cast else np.asarray(K)
        if self.q_transposed:
            Q = np.ascontiguousarray(Q.T)
        if self.k_transposed:
            K = np.ascontiguousarray(K.T)
        return Q, K

    def reference(self, Q, K, V) -> np.ndarray:
        Q, K = self._natural(Q, K)
        V = np.asarray(V, np.float32)
        s = (Q @ K.T) * np.float32(self.scale)
        if self.causal:
            m = np.arange(s.shape[0])[:, None]
            n = np.arange(s.shape[1])[None, :]
            s = np.where(n > m, np.float32(-np.inf), s)
        s = s - s.max(-1, keepdims=True)
        e = np.exp(s)
        return ((e / e.sum(-1, keepdims=True)) @ V).astype(np.float32)


def _gelu(x):
    t = np.clip(0.7978845608028654 * (x + 0.044715 * x ** 3), -30.0, 30.0)
    return 0.5 * x * (1.0 + np.tanh(t))


#: numpy side of the pointwise epilogue vocabulary (``fusion_core.py:121-138``)
EPILOGUE_REFS: dict = {
    "bias": None,
    "relu": lambda x: np.maximum(x, 0.0),
    "gelu": _gelu,
    "silu": lambda x: x / (1.0 + np.exp(-x)),
    "sigmoid": lambda x: 1.0 / (1.0 + np.exp(-x)),
    "tanh": np.tanh,
}


@dataclass(frozen=True)
class FusedRegion:
    """``fusion_core.FusedRegion`` (``:226-345``): a matmul root plus an ordered
    pointwise epilogue chain.  The fields the gfx950 candidate cannot honour
    (reduction, residual, prologue) are carried so it can decline them."""
    epilogue: tuple = ()
    reduction: Optional[str] = None
    residual: bool = False
    prologue: tuple = ()
    storage_dtype: str = "f16"

    def __post_init__(self) -> None:
        for op in self.epilogue:
            if op not in EPILOGUE_REFS:
                raise ValueError(f"E_FUSED_EPILOGUE_BAD_OP: unknown epilogue op {op!r}")
        if sum(1 for op in self.epilogue if op == "bias") > 1:
            raise ValueError("E_FUSED_EPILOGUE_BAD_ORDER: at most one bias op per region")

    @property
    def has_bias(self) -> bool:
        return "bias" in self.epilogue

    def reference(self, A, B, bias=None, residual=None) -> np.ndarray:
        out = np.asarray(A, np.float32) @ np.asarray(B, np.float32)
        for op in self.epilogue:
            if op == "bias":
                if bias is None:
                    raise ValueError("E_FUSED_EPILOGUE_MISSING_OPERAND: region needs a bias for 'bias'")
                out = out + np.asarray(bias, np.float32)
            else:
                out = EPILOGUE_REFS[op](out)
        if self.residual:
            if residual is None:
                raise ValueError("E_FUSED_EPILOGUE_MISSING_OPERAND: region needs a residual")
            out = out + np.asarray(residual, np.float32)
        return out.astype(np.float32)


@dataclass(frozen=True)
class GatedMatmulRegion:
    """``fusion_core.GatedMatmulRegion`` (``:747-782``): ``act(A Wg) * (A Wu)``."""
    gate_act: str = "silu"
    storage_dtype: str = "f16"

    def __post_init__(self) -> None:
        if self.gate_act not in EPILOGUE_REFS or self.gate_act == "bias":
            raise ValueError(f"gate activation must be a unary pointwise op, got {self.gate_act!r}")

    def reference(self, A, Wg, Wu) -> np.ndarray:
        a = np.asarray(A, np.float32)
        gate = EPILOGUE_REFS[self.gate_act](a @ np.asarray(Wg, np.float32))
        return (gate * (a @ np.asarray(Wu, np.float32))).astype(np.float32)


@dataclass(frozen=True)
class GroupedGemmRegion:
    """Contiguous grouped GEMM (``compiler/grouped_layout.py:396-414``): the
    region kind for the op-kind this lane adds."""
    group_sizes: tuple = ()
    dtype: str = "bfloat16"

    def reference(self, x, w) -> np.ndarray:
        xa = _round_to_storage(x, self.dtype).astype(np.float64)
        wa = _round_to_storage(w, self.dtype).astype(np.float64)
        out = np.zeros((xa.shape[0], wa.shape[2]), np.float64)
        off = 0
        for e, n in enumerate(self.group_sizes):
            if n:
                out[off:off + n] = xa[off:off + n] @ wa[e]
            off += n
        return out.astype(np.float32)


# ---- the protocol ------------------------------------------------------------------------

class Candidate(ABC):
    name: str = ""
    tier: Tier = Tier.SYNTHESIZED
    target: str = ""
    op: str = OP_FUSED_REGION
    accuracy_atol: Optional[float] = None
    accuracy_rtol: Optional[float] = None
    mma_target: Optional[str] = None
    mma_arch: Optional[str] = None
    mma_prefer_shape: Optional[tuple] = None

    def mma_dtype(self, region: Any) -> Optional[str]:
        raw = getattr(region, "dtype", None)
        if not isinstance(raw, str):
            return None
        return {"float16": "fp16", "f16": "fp16", "bfloat16": "bf16", "float32": "fp32", "f32": "fp32"}.get(raw, raw)

    def available(self) -> bool:
        return True

    def applies_to(self, region: Any) -> bool:
        return True

    def measure_device_latency(self, region: Any, *inputs: Any, reps: int = 100, warmup: int = 10) -> Optional[float]:
        return None

    @abstractmethod
    def run(self, region: Any, *inputs: Any, **kwargs: Any) -> tuple:
        """Execute ``region`` → ``(output, execution_tag)``."""


_CANDIDATES: dict[tuple, list] = {}
_OP_KIND_VERIFY: dict[str, Callable[..., bool]] = {}
_BUILTIN_OPS = (OP_FUSED_REGION, OP_ATTENTION, OP_GATED_MATMUL, OP_POINTWISE, OP_MATMUL)


def register_op_kind(op: str, verify_fn: Callable[..., bool]) -> None:
    """``candidate.py:81-87``: add an op-kind with its own reference-diff verifier."""
    _OP_KIND_VERIFY[op] = verify_fn


def register_candidate(candidate: Candidate) -> None:
    if not candidate.target or not candidate.name:
        raise ValueError("Candidate.target and Candidate.name must be non-empty")
    if candidate.op not in _BUILTIN_OPS and candidate.op not in _OP_KIND_VERIFY:
        raise ValueError(f"unknown Candidate.op {candidate.op!r}")
    bucket = _CANDIDATES.setdefault((candidate.target, candidate.op), [])
    for i, existing in enumerate(bucket):
        if existing.name == candidate.name:
            bucket[i] = candidate
            return
    bucket.append(candidate)


def candidates_for(target: str, op: str) -> list:
    return list(_CANDIDATES.get((target, op), ()))


def _effective_atol(c: Candidate, atol: float) -> float:
    return max(atol, c.accuracy_atol) if c.accuracy_atol is not None else atol


def verify_candidate(candidate: Candidate, region: Any, *, atol: float = 1e-3, seed: int = 0) -> bool:
    """F4 gate: True iff the candidate ran a real kernel on the probe and matched
    the region's numpy definition within its budget.  Probe shapes and scales are
    the reference's (``fusion_core.py:1081-1126``): matmul 32x16x32 * 0.4,
    attention 8x16 * 0.2."""
    if candidate.op in _OP_KIND_VERIFY:
        return bool(_OP_KIND_VERIFY[candidate.op](candidate, region, atol=atol, seed=seed))
    rng = np.random.default_rng(seed)
    if candidate.op == OP_MATMUL:
        A = (rng.standard_normal((32, 32)) * 0.4).astype(np.float32)
        B = (rng.standard_normal((32, 16)) * 0.4).astype(np.float32)
        if getattr(region, "transpose_a", False):
            A = np.ascontiguousarray(A.T)
        if getattr(region, "transpose_b", False):
            B = np.ascontiguousarray(B.T)
        out, tag = candidate.run(region, A, B)
        ref = region.reference(A, B)
    elif candidate.op == OP_ATTENTION:
        Q, K, V = ((rng.standard_normal((8, 16)) * .2).astype(np.float32) for _ in range(3))
        out, tag = candidate.run(region, Q, K, V)
        ref = region.reference(Q, K, V)
    elif candidate.op == OP_FUSED_REGION:
        # fusion_core.py:1046-1062
        A = (rng.standard_normal((8, 12)) * .2).astype(np.float32)
        B = (rng.standard_normal((12, 16)) * .2).astype(np.float32)
        bias = (rng.standard_normal((16,)) * .2).astype(np.float32) if region.has_bias else None
        out, tag = candidate.run(region, A, B, bias)
        ref = region.reference(A, B, bias)
    elif candidate.op == OP_GATED_MATMUL:
        # fusion_core.py:809-822
        A = (rng.standard_normal((8, 12)) * .2).astype(np.float32)
        Wg = (rng.standard_normal((12, 16)) * .2).astype(np.float32)
        Wu = (rng.standard_normal((12, 16)) * .2).astype(np.float32)
        out, tag = candidate.run(region, A, Wg, Wu)
        ref = region.reference(A, Wg, Wu)
    else:
        return False
    if tag in REFERENCE_EXECUTIONS:
        return False
    rtol = candidate.accuracy_rtol or 0.0
    return bool(np.allclose(np.asarray(out), ref, atol=_effective_atol(candidate, atol), rtol=rtol))


def _reg_index(c: Candidate) -> int:
    bucket = _CANDIDATES.get((c.target, c.op), [])
    for i, x in enumerate(bucket):
        if x is c:
            return i
    return len(bucket)


def arbitrate(region: Any, op: str, target: str, *, verify: bool = True, force: Optional[str] = None,
              measure: Optional[Callable[[Candidate], float]] = None) -> Optional[Candidate]:
    """``candidate.py:339-376``: applies ∧ available → (force) → F4 gate → lowest
    ``measure`` or highest tier (registration order breaks ties)."""
    cands = [c for c in candidates_for(target, op) if c.applies_to(region) and c.available()]
    if force is not None:
        forced = [c for c in cands if c.name == force]
        if not forced:
            names = [c.name for c in candidates_for(target, op)]
            raise ArbiterError(f"forced candidate {force!r} not available for ({target}, {op}); "
                               f"registered: {names or '<none>'}")
        cands = forced
    if verify:
        cands = [c for c in cands if verify_candidate(c, region)]
    if not cands:
        return None
    if measure is not None:
        return min(cands, key=measure)
    return max(cands, key=lambda c: (int(c.tier), -_reg_index(c)))


_ARBITER_LOG: deque = deque(maxlen=4096)


def arbiter_dispatch_log() -> list:
    return list(_ARBITER_LOG)


def reset_arbiter_dispatch_log() -> None:
    _ARBITER_LOG.clear()


def arbiter_dispatch_histogram(target: Optional[str] = None, op: Optional[str] = None) -> dict:
    """Per ``(target, op)`` counts of ``{won, degraded, no_candidate}``
    (``candidate.py:478-502``)."""
    hist: dict = {}
    for (t, o, selected, tag) in _ARBITER_LOG:
        if (target is not None and t != target) or (op is not None and o != op):
            continue
        b = hist.setdefault((t, o), {"won": 0, "degraded": 0, "no_candidate": 0})
        if selected is None:
            b["no_candidate"] += 1
        elif tag in REFERENCE_EXECUTIONS:
            b["degraded"] += 1
        else:
            b["won"] += 1
    return hist


def run_arbitrated(region: Any, op: str, target: str, *inputs: Any, verify: bool = True,
                   force: Optional[str] = None, measure: Optional[Callable[[Candidate], float]] = None) -> tuple:
    """Arbitrate then execute → ``(output, tag)``; every dispatch is logged.  With
    no viable candidate this raises (the lane has no numpy degrade path)."""
    winner = arbitrate(region, op, target, verify=verify, force=force, measure=measure)
    if winner is None:
        _ARBITER_LOG.append((target, op, None, "reference"))
        raise ArbiterError(f"no viable gfx950 candidate for ({target}, {op})")
    out, tag = winner.run(region, *inputs)
    _ARBITER_LOG.append((target, op, winner.name, tag))
    return out, tag


# ---- gfx950 candidates ---------------------------------------------------------------------

def _to_storage(x, dtype: str):
    a = np.ascontiguousarray(x, np.float32)
    return _bf16.from_float32(a) if dtype in ("bfloat16", "bf16") else a.astype(np.float16)


def _time_ms(fn, reps: int, warmup: int) -> float:
    for _ in range(max(warmup, 1)):
        fn()
    t = _lane.DeviceTimer()
    try:
        t.start()
        for _ in range(reps):
            fn()
        t.stop()
        return t.elapsed_ms() / reps
    finally:
        t.close()


class Gfx950MfmaGemmCandidate(Candidate):
    """Tier-3 bare matmul on the CDNA4 MFMA GEMM (16-bit storage, f32 accumulate)."""
    name = "gfx950_mfma_gemm"
    tier = Tier.HAND_TUNED
    target = TARGET
    op = OP_MATMUL
    accuracy_atol = 5e-3
    mma_target = "rocm"
    mma_arch = "gfx950"
    mma_prefer_shape = (32, 32, 16)

    def available(self) -> bool:
        return _lane.available()

    def applies_to(self, region: Any) -> bool:
        return getattr(region, "dtype", None) in ("bfloat16", "bf16", "float16", "f16")

    def run(self, region: Any, A: Any, B: Any, *a: Any, **k: Any) -> tuple:
        An, Bn = region._natural(A, B)
        return _ops.gemm(_to_storage(An, region.dtype), _to_storage(Bn, region.dtype), out="f32"), GEMM_TAG

    def measure_device_latency(self, region: Any, A: Any, B: Any, *a: Any, reps: int = 100, warmup: int = 10):
        An, Bn = region._natural(A, B)
        a16 = np.ascontiguousarray(np.asarray(_to_storage(An, region.dtype)).view(np.uint16))
        b16_ = np.ascontiguousarray(np.asarray(_to_storage(Bn, region.dtype)).view(np.uint16))
        M, K = a16.shape
        N = b16_.shape[1]
        da, db = _lane.DeviceBuffer.from_host(a16), _lane.DeviceBuffer.from_host(b16_)
        dd = _lane.DeviceBuffer(M * N * 4)
        st = "bf16" if region.dtype in ("bfloat16", "bf16") else "f16"
        fn = getattr(_lane.load(), f"tessera_gfx950_gemm_{st}_dev")
        try:
            return _time_ms(lambda: _lane.check(fn(da.ptr, db.ptr, dd.ptr, M, N, K, None), "gemm"), reps, warmup)
        finally:
            for b in (da, db, dd):
                b.close()


class Gfx950FlashAttnCandidate(Candidate):
    """Tier-3 attention on the CDNA4 MFMA FA-2 forward.  The 2-D region runs as
    one (batch, head); ``causal`` there masks ``n > m``, which is the lane's
    bottom-right alignment exactly when ``Sk <= Sq``."""
    name = "gfx950_flash_attn"
    tier = Tier.HAND_TUNED
    target = TARGET
    op = OP_ATTENTION
    accuracy_atol = 5e-3

    def available(self) -> bool:
        return _lane.available()

    def applies_to(self, region: Any) -> bool:
        return getattr(region, "storage_dtype", "f16") in ("f16", "bf16")

    def run(self, region: Any, Q: Any, K: Any, V: Any, *a: Any, **k: Any) -> tuple:
        Qn, Kn = region._natural(Q, K)
        Vn = np.asarray(V, np.float32)
        M, D = Qn.shape
        Nk = Kn.shape[0]
        if D % 16 != 0 or Kn.shape[1] != D or Vn.shape != (Nk, D):
            raise ValueError("gfx950 attention candidate needs head_dim % 16 == 0 and matching K/V")
        if region.causal and Nk > M:
            raise ValueError("top-left causal region with Sk > Sq is not the lane's mask")
        dt = "bf16" if region.storage_dtype == "bf16" else "f16"
        q, kk, v = (_to_storage(x.reshape(1, 1, *x.shape), dt) for x in (Qn, Kn, Vn))
        out = _ops.flash_attn(q, kk, v, scale=region.scale, causal=region.causal, out="f32")
        return out.reshape(M, D), ATTN_TAG


def _verify_grouped(candidate: Candidate, region: Any, *, atol: float, seed: int) -> bool:
    rng = np.random.default_rng(seed)
    sizes = (5, 0, 19, 8)
    K, N = 32, 24
    x = (rng.standard_normal((sum(sizes), K)) * .4).astype(np.float32)
    w = (rng.standard_normal((len(sizes), K, N)) * .4).astype(np.float32)
    probe = GroupedGemmRegion(sizes, getattr(region, "dtype", "bfloat16"))
    out, tag = candidate.run(probe, x, w)
    if tag in REFERENCE_EXECUTIONS:
        return False
    return bool(np.allclose(out, probe.reference(x, w), atol=_effective_atol(candidate, atol)))


register_op_kind(OP_GROUPED_GEMM, _verify_grouped)


class Gfx950GroupedGemmCandidate(Candidate):
    """Tier-3 contiguous grouped GEMM (the MoE expert-FFN core), bf16 -> f32."""
    name = "gfx950_grouped_gemm"
    tier = Tier.HAND_TUNED
    target = TARGET
    op = OP_GROUPED_GEMM
    accuracy_atol = 5e-3

    def available(self) -> bool:
        return _lane.available()

    def applies_to(self, region: Any) -> bool:
        return getattr(region, "dtype", None) in ("bfloat16", "bf16")

    def run(self, region: Any, x: Any, w: Any, *a: Any, **k: Any) -> tuple:
        out = _ops.grouped_gemm(_to_storage(x, "bf16"), _to_storage(w, "bf16"), list(region.group_sizes), out="f32")
        return out, GROUPED_TAG


#: Activations the MFMA epilogue fuses after the optional bias.
_MFMA_ACTS = ("relu", "gelu", "silu", "sigmoid", "tanh")


def mfma_epilogue(region: Any):
    """``(has_bias, activation)`` when ``region`` fits the kernel's epilogue — bias
    first, then at most one activation, no reduction / residual / prologue — else
    ``None``.  The rule of ``_wmma_epilogue`` (``emit/rocm_hip.py:679-699``)."""
    if not isinstance(region, FusedRegion):
        return None
    if region.reduction is not None or region.residual or region.prologue:
        return None
    epi = list(region.epilogue)
    has_bias = False
    if epi and epi[0] == "bias":
        has_bias = True
        epi = epi[1:]
    if not epi:
        return has_bias, "none"
    if len(epi) == 1 and epi[0] in _MFMA_ACTS:
        return has_bias, epi[0]
    return None


class Gfx950FusedGemmCandidate(Candidate):
    """Tier-3 matmul with the bias / activation epilogue fused on the MFMA GEMM."""
    name = "gfx950_mfma_fused_gemm"
    tier = Tier.HAND_TUNED
    target = TARGET
    op = OP_FUSED_REGION
    accuracy_atol = 5e-3
    mma_target = "rocm"
    mma_arch = "gfx950"

    def mma_dtype(self, region: Any) -> Optional[str]:
        return "bf16" if getattr(region, "storage_dtype", "f16") == "bf16" else "fp16"

    def available(self) -> bool:
        return _lane.available()

    def applies_to(self, region: Any) -> bool:
        return mfma_epilogue(region) is not None and getattr(region, "storage_dtype", "f16") in ("f16", "bf16")

    def run(self, region: Any, A: Any, B: Any, bias: Any = None, *a: Any, **k: Any) -> tuple:
        epi = mfma_epilogue(region)
        if epi is None:
            raise ValueError("region's epilogue is not representable on the gfx950 fused GEMM")
        has_bias, activation = epi
        if has_bias and bias is None:
            raise ValueError("E_FUSED_EPILOGUE_MISSING_OPERAND: region needs a bias")
        dt = region.storage_dtype
        out = _ops.fused_gemm(_to_storage(A, dt), _to_storage(B, dt), bias if has_bias else None, activation)
        return out, FUSED_TAG


class Gfx950GatedGemmCandidate(Candidate):
    """Tier-3 gated projection ``act(A Wg) * (A Wu)`` in one MFMA kernel."""
    name = "gfx950_mfma_gated_gemm"
    tier = Tier.HAND_TUNED
    target = TARGET
    op = OP_GATED_MATMUL
    accuracy_atol = 5e-3
    mma_target = "rocm"
    mma_arch = "gfx950"

    def available(self) -> bool:
        return _lane.available()

    def applies_to(self, region: Any) -> bool:
        return isinstance(region, GatedMatmulRegion) and region.storage_dtype in ("f16", "bf16")

    def run(self, region: Any, A: Any, Wg: Any, Wu: Any, *a: Any, **k: Any) -> tuple:
        dt = region.storage_dtype
        out = _ops.gated_gemm(_to_storage(A, dt), _to_storage(Wg, dt), _to_storage(Wu, dt), region.gate_act)
        return out, GATED_TAG


def register_all() -> None:
    """Plug the lane's candidates in (idempotent), as each backend module does at
    import (``compiler/emit/rocm_hip.py:809-818``)."""
    register_candidate(Gfx950MfmaGemmCandidate())
    register_candidate(Gfx950FlashAttnCandidate())
    register_candidate(Gfx950GroupedGemmCandidate())
    register_candidate(Gfx950FusedGemmCandidate())
    register_candidate(Gfx950GatedGemmCandidate())


register_all()
