"""A small stand-in for the parts of a Tessera host that the gfx950 lane plugs into.
TEST INFRASTRUCTURE ONLY — nothing under ``tessera_amd/`` imports it.

On the GPU box there is no Tessera checkout, so the plugin tests need *some* host to
register into.  This file provides one with the same surface the lane touches and
nothing more:

* :class:`CandidateHost` — what ``tessera.compiler.emit.candidate`` exposes to a
  backend: the ``OP_*`` tags, ``Tier``, a ``Candidate`` base to subclass,
  ``register_op_kind`` / ``register_candidate`` / ``candidates_for`` and an
  ``arbitrate(region, op, target, *, verify, force, measure)`` that filters by
  ``applies_to`` / ``available``, gates each survivor on a small probe against the
  region's numpy definition and picks by ``measure`` (lowest) or tier (highest, first
  registered on a tie);
* region classes with the attribute names of ``compiler/fusion_core.py`` (the lane
  reads regions by attribute) and a numpy ``reference`` each;
* :class:`MatrixHost` / :class:`RuntimeHost` — the execution matrix
  (``ExecutionRow``, ``_MATRIX``, ``KNOWN_EXECUTORS``) and the runtime's
  ``_executor_table()`` that :func:`tessera_amd.install.install` registers into.

It is written for these tests, not transcribed from the reference: only names that a
plugin must match are kept.
"""
from __future__ import annotations

import enum
from dataclasses import dataclass, field
from typing import Any, Callable, Optional

import numpy as np

from tessera_amd import bf16 as _bf16


class Tier(enum.IntEnum):
    SYNTHESIZED = 1
    EMITTED = 2
    HAND_TUNED = 3


class ArbiterError(RuntimeError):
    pass


class Candidate:
    """Base class a backend derives its candidates from."""
    name = ""
    tier = Tier.SYNTHESIZED
    target = ""
    op = "fused_region"
    accuracy_atol: Optional[float] = None
    accuracy_rtol: Optional[float] = None
    mma_target = mma_arch = mma_prefer_shape = None

    def mma_dtype(self, region):
        return None

    def available(self) -> bool:
        return True

    def applies_to(self, region) -> bool:
        return True

    def measure_device_latency(self, region, *inputs, reps=100, warmup=10):
        return None

    def run(self, region, *inputs, **kwargs):
        raise NotImplementedError


# ---- regions ---------------------------------------------------------------------------

def _storage_round(x, dtype: str) -> np.ndarray:
    a = np.ascontiguousarray(x, np.float32)
    if dtype in ("bfloat16", "bf16"):
        return _bf16.from_float32(a).to_float32()
    return a.astype(np.float16).astype(np.float32)


@dataclass(frozen=True)
class MatmulRegion:
    dtype: str = "bfloat16"
    transpose_a: bool = False
    transpose_b: bool = False

    def reference(self, A, B):
        a = np.asarray(A, np.float32).T if self.transpose_a else np.asarray(A, np.float32)
        b = np.asarray(B, np.float32).T if self.transpose_b else np.asarray(B, np.float32)
        return (_storage_round(a, self.dtype) @ _storage_round(b, self.dtype)).astype(np.float32)


@dataclass(frozen=True)
class AttentionRegion:
    scale: float = 1.0
    causal: bool = False
    q_transposed: bool = False
    k_transposed: bool = False
    storage_dtype: str = "f16"

    def reference(self, Q, K, V):
        q = np.asarray(Q, np.float64).T if self.q_transposed else np.asarray(Q, np.float64)
        k = np.asarray(K, np.float64).T if self.k_transposed else np.asarray(K, np.float64)
        s = self.scale * (q @ k.T)
        if self.causal:                                  # key n hidden from query m when n > m
            s = np.where(np.triu(np.ones(s.shape, bool), 1), -np.inf, s)
        p = np.exp(s - s.max(axis=-1, keepdims=True))
        return ((p / p.sum(axis=-1, keepdims=True)) @ np.asarray(V, np.float64)).astype(np.float32)


def _gelu_tanh(x):
    return 0.5 * x * (1.0 + np.tanh(np.clip(np.sqrt(2.0 / np.pi) * (x + 0.044715 * x ** 3), -30.0, 30.0)))


POINTWISE = {
    "relu": lambda x: np.maximum(x, 0.0),
    "gelu": _gelu_tanh,
    "silu": lambda x: x / (1.0 + np.exp(-x)),
    "sigmoid": lambda x: 1.0 / (1.0 + np.exp(-x)),
    "tanh": np.tanh,
}


@dataclass(frozen=True)
class FusedRegion:
    epilogue: tuple = ()
    reduction: Optional[str] = None
    residual: bool = False
    prologue: tuple = ()
    storage_dtype: str = "f16"

    def __post_init__(self):
        bad = [op for op in self.epilogue if op != "bias" and op not in POINTWISE]
        if bad or self.epilogue.count("bias") > 1:
            raise ValueError(f"bad epilogue chain {self.epilogue!r}")

    @property
    def has_bias(self) -> bool:
        return "bias" in self.epilogue

    def reference(self, A, B, bias=None, residual=None):
        y = np.asarray(A, np.float64) @ np.asarray(B, np.float64)
        for op in self.epilogue:
            if op == "bias":
                if bias is None:
                    raise ValueError("region adds a bias but none was given")
                y = y + np.asarray(bias, np.float64)
            else:
                y = POINTWISE[op](y)
        if self.residual:
            y = y + np.asarray(residual, np.float64)
        return y.astype(np.float32)


@dataclass(frozen=True)
class GatedMatmulRegion:
    gate_act: str = "silu"
    storage_dtype: str = "f16"

    def __post_init__(self):
        if self.gate_act not in POINTWISE:
            raise ValueError(f"gate activation {self.gate_act!r} is not a unary pointwise op")

    def reference(self, A, Wg, Wu):
        a = np.asarray(A, np.float64)
        return (POINTWISE[self.gate_act](a @ np.asarray(Wg, np.float64)) * (a @ np.asarray(Wu, np.float64))
                ).astype(np.float32)


class regions:                      # namespace handed to tessera_amd.autotune.measure_headline_corpus
    MatmulRegion = MatmulRegion
    AttentionRegion = AttentionRegion
    FusedRegion = FusedRegion
    GatedMatmulRegion = GatedMatmulRegion


# ---- the candidate host -------------------------------------------------------------------

def _probe_matmul(region, rng):
    a = (rng.standard_normal((32, 32)) * 0.4).astype(np.float32)
    b = (rng.standard_normal((32, 16)) * 0.4).astype(np.float32)
    return (a.T.copy() if region.transpose_a else a, b.T.copy() if region.transpose_b else b)


def _probe_attention(region, rng):
    return tuple((rng.standard_normal((16, 16)) * 0.2).astype(np.float32) for _ in range(3))


def _probe_fused(region, rng):
    a = (rng.standard_normal((8, 16)) * 0.2).astype(np.float32)
    b = (rng.standard_normal((16, 16)) * 0.2).astype(np.float32)
    bias = (rng.standard_normal(16) * 0.2).astype(np.float32) if region.has_bias else None
    return a, b, bias


def _probe_gated(region, rng):
    return tuple((rng.standard_normal(s) * 0.2).astype(np.float32) for s in ((8, 16), (16, 16), (16, 16)))


class CandidateHost:
    """One registry + arbiter.  A fresh instance per test keeps tests independent."""
    OP_FUSED_REGION = "fused_region"
    OP_ATTENTION = "attention"
    OP_GATED_MATMUL = "gated_matmul"
    OP_POINTWISE = "pointwise"
    OP_MATMUL = "matmul"
    NOT_A_KERNEL = frozenset({"reference", "fallback"})
    Tier = Tier
    Candidate = Candidate
    ArbiterError = ArbiterError

    def __init__(self):
        self._probes = {self.OP_MATMUL: _probe_matmul, self.OP_ATTENTION: _probe_attention,
                        self.OP_FUSED_REGION: _probe_fused, self.OP_GATED_MATMUL: _probe_gated}
        self._kind_verifiers: dict = {}
        self._registry: dict = {}
        self.log: list = []                    # (target, op, winner name or None, tag)

    def register_op_kind(self, op: str, verify_fn: Callable[..., bool]) -> None:
        self._kind_verifiers[op] = verify_fn

    def register_candidate(self, c) -> None:
        if not c.name or not c.target:
            raise ValueError("a candidate needs a name and a target")
        if c.op not in self._probes and c.op not in self._kind_verifiers:
            raise ValueError(f"no such op kind: {c.op!r}")
        bucket = self._registry.setdefault((c.target, c.op), {})
        bucket[c.name] = c                     # dicts keep first-insertion order; same name replaces in place

    def candidates_for(self, target: str, op: str) -> list:
        return list(self._registry.get((target, op), {}).values())

    def verify_candidate(self, c, region, *, atol: float = 1e-3, seed: int = 0) -> bool:
        if c.op in self._kind_verifiers:
            return bool(self._kind_verifiers[c.op](c, region, atol=atol, seed=seed))
        inputs = self._probes[c.op](region, np.random.default_rng(seed))
        out, tag = c.run(region, *inputs)
        if tag in self.NOT_A_KERNEL:
            return False
        want = region.reference(*inputs)
        return bool(np.allclose(out, want, atol=max(atol, c.accuracy_atol or 0.0), rtol=c.accuracy_rtol or 0.0))

    def arbitrate(self, region, op: str, target: str, *, verify: bool = True, force: Optional[str] = None,
                  measure: Optional[Callable[[Any], float]] = None):
        pool = [c for c in self.candidates_for(target, op) if c.applies_to(region) and c.available()]
        if force is not None:
            pool = [c for c in pool if c.name == force]
            if not pool:
                raise ArbiterError(f"forced candidate {force!r} cannot run for ({target}, {op})")
        if verify:
            pool = [c for c in pool if self.verify_candidate(c, region)]
        if not pool:
            return None
        if measure is not None:
            return min(pool, key=measure)
        best_tier = max(int(c.tier) for c in pool)
        return next(c for c in pool if int(c.tier) == best_tier)

    def run(self, region, op: str, target: str, *inputs, **kw):
        """Arbitrate and execute; raises when nothing is viable (this host has no numpy
        degrade path, so a lane that silently fell back would be seen)."""
        winner = self.arbitrate(region, op, target, **kw)
        if winner is None:
            self.log.append((target, op, None, "reference"))
            raise ArbiterError(f"no viable candidate for ({target}, {op})")
        out, tag = winner.run(region, *inputs)
        self.log.append((target, op, winner.name, tag))
        return out, tag


# ---- execution matrix / runtime -------------------------------------------------------------

@dataclass(frozen=True)
class ExecutionRow:
    target: str
    compiler_path: str
    execution_kind: str
    executable: bool
    executor_id: Optional[str]
    runtime_status: str
    reason: str = ""
    execution_mode: str = ""
    direction: str = "forward"
    op_family: str = ""
    device_proof: str = ""
    evidence_target: str = ""
    backward_aliases: tuple = ()


class MatrixHost:
    ExecutionRow = ExecutionRow

    def __init__(self):
        self._MATRIX: dict = {("cpu", "jit_cpu_numpy"): ExecutionRow("cpu", "jit_cpu_numpy", "reference_cpu", True,
                                                                     "jit_cpu_numpy", "success")}
        self.KNOWN_EXECUTORS: dict = {"jit_cpu_numpy": "numpy reference path"}


class RuntimeHost:
    """Resolves executor ids through ``_executor_table()``, a fresh dict per call, and
    launches the way the lane's executors expect: ``executor(artifact, args)``."""

    def __init__(self, matrix: MatrixHost):
        self.matrix = matrix

    def _executor_table(self) -> dict:
        return {"jit_cpu_numpy": lambda artifact, args: None}

    def launch(self, artifact, args):
        md = artifact.metadata or {}
        row = self.matrix._MATRIX.get((md.get("target"), md.get("compiler_path")))
        table = self._executor_table()
        if row is None or not row.executable or row.executor_id not in table or md.get("executable") is not True:
            return {"ok": False, "runtime_status": "unimplemented"}
        try:
            out = table[row.executor_id](artifact, args)
        except Exception as exc:                          # noqa: BLE001 - the envelope reports it
            return {"ok": False, "runtime_status": "invalid_artifact", "reason": str(exc)}
        kind = row.execution_kind
        if isinstance(out, tuple) and len(out) == 2 and isinstance(out[1], str):
            out, kind = out
        return {"ok": True, "runtime_status": "success", "execution_kind": kind, "output": out,
                "compiler_path": row.compiler_path}


# ---- typed native artifacts (stand-ins for the host's descriptor types) ---------------------

@dataclass(frozen=True)
class Binding:
    """A descriptor's buffer binding: a name and its position among the arguments."""
    name: str
    ordinal: int


@dataclass(frozen=True)
class Descriptor:
    abi_id: str
    entry_symbol: str
    buffers: tuple
    provenance: dict = field(default_factory=dict)


@dataclass(frozen=True)
class Image:
    target: str
    binary_format: str


class NativeLauncherHost:
    """Keeps one submit hook per exact target and drives it like the host's descriptor launch:
    a raise from the hook becomes a ``device_error`` result."""

    def __init__(self):
        self.hooks = {}

    def register_native_launcher(self, target, *, binary_formats, submit, replace=False):
        if target in self.hooks and not replace:
            raise ValueError(f"native launcher already registered for {target}")
        self.hooks[target] = (tuple(binary_formats), submit)

    def launch_descriptor(self, image, descriptor, buffers, scalars):
        hook = self.hooks.get(image.target)
        if hook is None or image.binary_format not in hook[0]:
            return {"ok": False, "runtime_status": "unimplemented"}
        try:
            out = hook[1](image, descriptor, buffers, scalars, None)
        except Exception as exc:                              # noqa: BLE001 - the envelope reports it
            return {"ok": False, "runtime_status": "device_error", "reason": str(exc)}
        return {"ok": True, "runtime_status": "success", "execution_kind": "native_gpu", "output": out}
