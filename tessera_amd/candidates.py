"""gfx950 kernel candidates for Tessera's measured arbiter, written against an
*injected* host API.

The arbiter, its registry, the ``Candidate`` base class, the tier enum and the
region classes belong to the host (``python/tessera/compiler/emit/candidate.py``,
``python/tessera/compiler/fusion_core.py``); a plugin subclasses the host's base
class and registers through the host's functions, as the reference's own ROCm
lanes do (``python/tessera/compiler/emit/rocm_hip.py:701-818``).  Nothing of the
host is restated here: :func:`build_candidates` takes the host's candidate API
(any object with ``Candidate``, ``Tier`` and the ``OP_*`` tags — the module
``tessera.compiler.emit.candidate`` itself) and returns five candidate instances
whose classes derive from *that* ``Candidate``; :func:`register` hands them to
*that* ``register_candidate``.

Regions are read by attribute only (``dtype`` / ``transpose_a`` / ``transpose_b``
of a matmul region, ``scale`` / ``causal`` / ``q_transposed`` / ``k_transposed`` /
``storage_dtype`` of an attention region, ``epilogue`` / ``reduction`` / ``residual``
/ ``prologue`` / ``storage_dtype`` of a fused region, ``gate_act`` of a gated one),
so any host object with those fields is served.

Unlike the reference's ROCm candidates these never hand back the host's numpy
result: a candidate that cannot run says so through ``available()`` /
``applies_to()`` and otherwise raises from ``run``.

The grouped GEMM has no region class in the host, so the lane brings its op kind:
:data:`OP_GROUPED_GEMM`, the region :class:`GroupedGemmRegion` and the verifier
:func:`verify_grouped_gemm` for the host's ``register_op_kind``
(``emit/candidate.py:81-87``).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional

import numpy as np

from . import bf16 as _bf16
from . import lane as _lane
from . import ops as _ops

TARGET = "rocm_gfx950"
OP_GROUPED_GEMM = "grouped_gemm"

GEMM_TAG = "gfx950_mfma_gemm"
ATTN_TAG = "gfx950_mfma_flash_attn"
GROUPED_TAG = "gfx950_mfma_grouped_gemm"
FUSED_TAG = "gfx950_mfma_fused_gemm"
GATED_TAG = "gfx950_mfma_gated_gemm"

#: f16 / bf16 storage budget against the f32 definition (the figure of the
#: reference's half-precision ROCm candidates, ``emit/rocm_hip.py:735,780``)
HALF_ATOL = 5e-3

_BF16_NAMES = ("bfloat16", "bf16")
_F16_NAMES = ("float16", "f16")
#: activations the fused epilogue applies after the optional bias
_EPILOGUE_ACTIVATIONS = frozenset({"relu", "gelu", "silu", "sigmoid", "tanh"})


def _storage_of(name: Any) -> Optional[str]:
    """``"bf16"`` / ``"f16"`` for a host dtype string, else ``None``."""
    if name in _BF16_NAMES:
        return "bf16"
    if name in _F16_NAMES:
        return "f16"
    return None


def _store(x: Any, storage: str):
    """f32 host array -> the lane's 16-bit storage array."""
    a = np.ascontiguousarray(x, np.float32)
    return _bf16.from_float32(a) if storage == "bf16" else a.astype(np.float16)


def _oriented(x: Any, transposed: bool) -> np.ndarray:
    a = np.asarray(x, np.float32)
    return np.ascontiguousarray(a.T) if transposed else a


def fused_epilogue_plan(region: Any) -> Optional[tuple]:
    """``(has_bias, activation)`` when the kernel's epilogue can express the region's
    pointwise chain, else ``None``.  The kernel adds ``bias[n]`` first and then applies
    at most one activation, so the chain must be ``[]``, ``[bias]``, ``[act]`` or
    ``[bias, act]`` and the region may carry no reduction, residual or prologue (the
    representability rule of the reference's matrix-core candidate,
    ``emit/rocm_hip.py:679-699``, over this kernel's wider activation set)."""
    chain = getattr(region, "epilogue", None)
    if chain is None:
        return None
    if getattr(region, "reduction", None) is not None or getattr(region, "residual", False) or \
            tuple(getattr(region, "prologue", ()) or ()):
        return None
    chain = tuple(chain)
    has_bias = chain[:1] == ("bias",)
    rest = chain[1:] if has_bias else chain
    if len(rest) > 1 or any(op not in _EPILOGUE_ACTIVATIONS for op in rest):
        return None
    return has_bias, (rest[0] if rest else "none")


@dataclass(frozen=True)
class GroupedGemmRegion:
    """Contiguous grouped GEMM ``y[rows of group e] = x[rows of group e] @ w[e]``
    (``python/tessera/compiler/grouped_layout.py:396-414``): the region of the op kind
    this lane adds.  ``reference`` is its definition, evaluated only by the verifier."""
    group_sizes: tuple = ()
    dtype: str = "bfloat16"

    def reference(self, x: Any, w: Any) -> np.ndarray:
        xs = _bf16.from_float32(np.asarray(x, np.float32)).to_float32().astype(np.float64)
        ws = _bf16.from_float32(np.asarray(w, np.float32)).to_float32().astype(np.float64)
        bounds = np.concatenate(([0], np.cumsum(self.group_sizes))).astype(int)
        rows = [xs[lo:hi] @ ws[e] for e, (lo, hi) in enumerate(zip(bounds[:-1], bounds[1:]))]
        return np.concatenate(rows, axis=0).astype(np.float32) if rows else np.zeros((0, ws.shape[2]), np.float32)


def verify_grouped_gemm(candidate: Any, region: Any, *, atol: float = 1e-3, seed: int = 0) -> bool:
    """Verifier of the ``grouped_gemm`` op kind, in the signature ``register_op_kind``
    asks for (``emit/candidate.py:81-87``): run the candidate on a small ragged probe
    (an empty group included) and compare with the region's definition.  A result
    tagged as a host-side ("reference" / "fallback") execution does not count."""
    rng = np.random.default_rng(seed)
    sizes = (5, 0, 19, 8)
    x = (rng.standard_normal((sum(sizes), 32)) * 0.4).astype(np.float32)
    w = (rng.standard_normal((len(sizes), 32, 24)) * 0.4).astype(np.float32)
    probe = GroupedGemmRegion(sizes, getattr(region, "dtype", "bfloat16"))
    out, tag = candidate.run(probe, x, w)
    if tag in ("reference", "fallback"):
        return False
    budget = max(atol, getattr(candidate, "accuracy_atol", None) or 0.0)
    return bool(np.allclose(np.asarray(out), probe.reference(x, w), atol=budget))


def _time_ms(fn, reps: int, warmup: int) -> float:
    """Mean device time of ``fn`` (ms) between two events on the default stream."""
    for _ in range(max(warmup, 1)):
        fn()
    timer = _lane.DeviceTimer()
    try:
        timer.start()
        for _ in range(reps):
            fn()
        timer.stop()
        return timer.elapsed_ms() / reps
    finally:
        timer.close()


# ---- what each candidate does (plain functions; the classes below bind them) -------------

def _gemm_applies(self, region: Any) -> bool:
    return _storage_of(getattr(region, "dtype", None)) is not None


def _gemm_operands(region: Any, A: Any, B: Any):
    st = _storage_of(region.dtype)
    a = _store(_oriented(A, getattr(region, "transpose_a", False)), st)
    b = _store(_oriented(B, getattr(region, "transpose_b", False)), st)
    return st, a, b


def _gemm_run(self, region: Any, A: Any, B: Any, *rest: Any, **kw: Any) -> tuple:
    _, a, b = _gemm_operands(region, A, B)
    return _ops.gemm(a, b, out="f32"), GEMM_TAG


def _gemm_latency(self, region: Any, A: Any, B: Any, *rest: Any, reps: int = 100, warmup: int = 10):
    st, a, b = _gemm_operands(region, A, B)
    a_bits = np.ascontiguousarray(np.asarray(a).view(np.uint16))
    b_bits = np.ascontiguousarray(np.asarray(b).view(np.uint16))
    (M, K), N = a_bits.shape, b_bits.shape[1]
    bufs = [_lane.DeviceBuffer.from_host(a_bits), _lane.DeviceBuffer.from_host(b_bits), _lane.DeviceBuffer(M * N * 4)]
    entry = getattr(_lane.load(), f"tessera_gfx950_gemm_{st}_dev")
    try:
        return _time_ms(lambda: _lane.check(entry(bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, M, N, K, None), "gemm"),
                        reps, warmup)
    finally:
        for b_ in bufs:
            b_.close()


def _attn_applies(self, region: Any) -> bool:
    return _storage_of(getattr(region, "storage_dtype", "f16")) is not None


def _attn_run(self, region: Any, Q: Any, K: Any, V: Any, *rest: Any, **kw: Any) -> tuple:
    """The host's 2-D region runs as one (batch, head).  Its causal mask hides key
    ``n > m`` (top-left aligned); the lane's is bottom-right aligned, and the two agree
    exactly when ``Sk <= Sq``."""
    q = _oriented(Q, getattr(region, "q_transposed", False))
    k = _oriented(K, getattr(region, "k_transposed", False))
    v = np.asarray(V, np.float32)
    (M, D), Nk = q.shape, k.shape[0]
    if D % 16 != 0 or k.shape[1] != D or v.shape != (Nk, D):
        raise ValueError("gfx950 attention candidate needs head_dim % 16 == 0 and K, V shaped (Sk, head_dim)")
    causal = bool(getattr(region, "causal", False))
    if causal and Nk > M:
        raise ValueError("a top-left causal region with Sk > Sq is not the lane's bottom-right mask")
    st = _storage_of(getattr(region, "storage_dtype", "f16"))
    q4, k4, v4 = (_store(t.reshape(1, 1, *t.shape), st) for t in (q, k, v))
    out = _ops.flash_attn(q4, k4, v4, scale=float(getattr(region, "scale", 1.0)), causal=causal, out="f32")
    return out.reshape(M, D), ATTN_TAG


def _grouped_applies(self, region: Any) -> bool:
    return _storage_of(getattr(region, "dtype", None)) == "bf16"


def _grouped_run(self, region: Any, x: Any, w: Any, *rest: Any, **kw: Any) -> tuple:
    out = _ops.grouped_gemm(_store(x, "bf16"), _store(w, "bf16"), list(region.group_sizes), out="f32")
    return out, GROUPED_TAG


def _half_storage_dtype(self, region: Any) -> Optional[str]:
    """Storage dtype in the host's MMA footprint vocabulary (``fp16`` / ``bf16``)."""
    return "bf16" if _storage_of(getattr(region, "storage_dtype", "f16")) == "bf16" else "fp16"


def _fused_applies(self, region: Any) -> bool:
    return fused_epilogue_plan(region) is not None and _storage_of(getattr(region, "storage_dtype", "f16")) is not None


def _fused_run(self, region: Any, A: Any, B: Any, bias: Any = None, *rest: Any, **kw: Any) -> tuple:
    plan = fused_epilogue_plan(region)
    if plan is None:
        raise ValueError("the region's epilogue chain is not expressible on the gfx950 fused GEMM")
    has_bias, activation = plan
    if has_bias and bias is None:
        raise ValueError("the region's epilogue adds a bias but no bias operand was given")
    st = _storage_of(getattr(region, "storage_dtype", "f16"))
    return _ops.fused_gemm(_store(A, st), _store(B, st), bias if has_bias else None, activation), FUSED_TAG


def _gated_applies(self, region: Any) -> bool:
    return getattr(region, "gate_act", None) in _EPILOGUE_ACTIVATIONS and \
        _storage_of(getattr(region, "storage_dtype", "f16")) is not None


def _gated_run(self, region: Any, A: Any, Wg: Any, Wu: Any, *rest: Any, **kw: Any) -> tuple:
    st = _storage_of(getattr(region, "storage_dtype", "f16"))
    return _ops.gated_gemm(_store(A, st), _store(Wg, st), _store(Wu, st), region.gate_act), GATED_TAG


def _lane_available(self) -> bool:
    return _lane.available()


#: class name -> (op tag attribute of the host API or a literal op kind, class attributes)
_SPECS = (
    ("Gfx950MfmaGemmCandidate", "OP_MATMUL", dict(
        name="gfx950_mfma_gemm", mma_target="rocm", mma_arch="gfx950", mma_prefer_shape=(32, 32, 16),
        applies_to=_gemm_applies, run=_gemm_run, measure_device_latency=_gemm_latency,
        __doc__="Bare matmul on the CDNA4 MFMA GEMM: 16-bit storage, f32 accumulate, f32 result.")),
    ("Gfx950FlashAttnCandidate", "OP_ATTENTION", dict(
        name="gfx950_flash_attn", applies_to=_attn_applies, run=_attn_run,
        __doc__="Attention region on the CDNA4 MFMA flash-attention forward.")),
    ("Gfx950GroupedGemmCandidate", OP_GROUPED_GEMM, dict(
        name="gfx950_grouped_gemm", applies_to=_grouped_applies, run=_grouped_run,
        __doc__="Contiguous grouped GEMM (the MoE expert-FFN core), bf16 storage, f32 result.")),
    ("Gfx950FusedGemmCandidate", "OP_FUSED_REGION", dict(
        name="gfx950_mfma_fused_gemm", mma_target="rocm", mma_arch="gfx950", mma_dtype=_half_storage_dtype,
        applies_to=_fused_applies, run=_fused_run,
        __doc__="Matmul with the bias / activation epilogue fused into the MFMA GEMM.")),
    ("Gfx950GatedGemmCandidate", "OP_GATED_MATMUL", dict(
        name="gfx950_mfma_gated_gemm", mma_target="rocm", mma_arch="gfx950",
        applies_to=_gated_applies, run=_gated_run,
        __doc__="Gated projection act(A Wg) * (A Wu) in one MFMA kernel.")),
)


def candidate_classes(api: Any) -> dict:
    """The five candidate classes, each derived from ``api.Candidate`` with tier
    ``api.Tier.HAND_TUNED`` and the op tag the host defines.  Built per host API object
    (and cached on it) so that ``isinstance(c, api.Candidate)`` holds for the host that
    will arbitrate them."""
    cached = getattr(api, "_gfx950_candidate_classes", None)
    if cached is not None:
        return cached
    classes = {}
    for cls_name, op_ref, attrs in _SPECS:
        body = dict(attrs)
        body.update(target=TARGET, tier=api.Tier.HAND_TUNED, accuracy_atol=HALF_ATOL, available=_lane_available,
                    op=getattr(api, op_ref) if op_ref.startswith("OP_") else op_ref, __module__=__name__)
        classes[cls_name] = type(cls_name, (api.Candidate,), body)
    try:
        api._gfx950_candidate_classes = classes
    except (AttributeError, TypeError):          # a host API object that takes no attributes: rebuilt per call
        pass
    return classes


def build_candidates(api: Any) -> list:
    """One instance of every gfx950 candidate for the host API ``api``."""
    return [cls() for cls in candidate_classes(api).values()]


def register(api: Any) -> list:
    """Register the grouped-GEMM op kind and the five candidates with the host
    (``api.register_op_kind``, ``api.register_candidate``); returns the instances.
    Registering twice replaces by name in the host's registry, as a backend module
    re-imported by the host would (``emit/rocm_hip.py:809-818``)."""
    api.register_op_kind(OP_GROUPED_GEMM, verify_grouped_gemm)
    made = build_candidates(api)
    for c in made:
        api.register_candidate(c)
    return made
