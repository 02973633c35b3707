"""Measured verdicts for the gfx950 candidates, kept as data.

The host's autotuner (``python/tessera/compiler/emit/autotune.py``) persists, per
workload, which candidate was fastest; other processes warm-start from that file.
This module owns only the lane's side of it:

* the *wire format* of such a file — the reference's corpus schema, version 3: a
  list of flat records with the key fields ``device, target, op, bucket, dtype,
  timing`` and the verdict fields ``winner, latency_ms, candidates, evidence``
  (``emit/autotune.py:40-75,170-202``) — so that ``autotune_corpus.json`` beside this
  file can be merged into Tessera's ``benchmarks/baselines/autotune_corpus.json``;
* :class:`Corpus`, a small table of those records with file I/O;
* :func:`tune`, which asks the *host's* arbiter (``api.arbitrate`` with its
  ``measure=`` hook) to pick the fastest verified candidate on a miss and records
  the verdict, and :func:`recommended`, which reads one back.

The arbiter, the verification gate and the candidate registry stay the host's; they
come in as the ``api`` argument (the object :mod:`tessera_amd.candidates` registers
into).
"""
from __future__ import annotations

import json
import os
import time
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, Iterator, Mapping, Optional

from . import candidates as _cand
from . import lane as _lane

SCHEMA_VERSION = 3
#: what a latency in a record means: wall clock around ``run`` or device events
TIMINGS = ("end_to_end", "device")
DEVICE_TAG = "rocm:gfx950"
PACKAGED = Path(__file__).resolve().parent / "autotune_corpus.json"


class NoCandidate(RuntimeError):
    """No registered candidate applies, is available and passes the host's gate.
    (The lane has no CPU path to degrade to.)"""


def pow2_bucket(dims) -> Optional[tuple]:
    """Every dim rounded up to a power of two — the reference's shape bucketing
    (``emit/kernel_emitter.py:72-80``), so records land in the buckets the host uses."""
    if dims is None:
        return None
    return tuple(1 << max(int(d) - 1, 0).bit_length() for d in dims)


@dataclass(frozen=True)
class Workload:
    """The key of one record."""
    device: str
    target: str
    op: str
    bucket: Optional[tuple]
    dtype: str
    timing: str = "end_to_end"

    def __post_init__(self) -> None:
        if self.timing not in TIMINGS:
            raise ValueError(f"timing must be one of {TIMINGS}, got {self.timing!r}")

    @classmethod
    def of(cls, device: str, target: str, op: str, dims, dtype: str, timing: str = "end_to_end") -> "Workload":
        return cls(device, target, op, pow2_bucket(dims), dtype, timing)


@dataclass
class Verdict:
    """The value of one record: the fastest candidate, its latency (ms), every timed
    candidate's latency, and free-form evidence."""
    winner: str
    latency_ms: float
    candidates: dict = field(default_factory=dict)
    evidence: dict = field(default_factory=dict)


def _record_to_wire(w: Workload, v: Verdict) -> dict:
    rec = {"device": w.device, "target": w.target, "op": w.op,
           "bucket": None if w.bucket is None else list(w.bucket), "dtype": w.dtype, "timing": w.timing,
           "winner": v.winner, "latency_ms": float(v.latency_ms),
           "candidates": {str(n): float(t) for n, t in v.candidates.items()}}
    if v.evidence:
        rec["evidence"] = dict(v.evidence)
    return rec


def _record_from_wire(rec: Mapping[str, Any]) -> tuple:
    bucket = rec.get("bucket")
    w = Workload(str(rec["device"]), str(rec["target"]), str(rec["op"]),
                 None if bucket is None else tuple(int(b) for b in bucket), str(rec["dtype"]),
                 str(rec.get("timing", "end_to_end")))          # records older than version 3 carry no timing
    v = Verdict(str(rec["winner"]), float(rec["latency_ms"]),
                {str(n): float(t) for n, t in dict(rec.get("candidates") or {}).items()},
                dict(rec.get("evidence") or {}))
    return w, v


class Corpus:
    """A table ``Workload -> Verdict``."""

    def __init__(self) -> None:
        self._table: dict = {}
        self.lookups = 0
        self.found = 0

    def __len__(self) -> int:
        return len(self._table)

    def __iter__(self) -> Iterator[tuple]:
        return iter(self._table.items())

    def lookup(self, w: Workload) -> Optional[Verdict]:
        self.lookups += 1
        v = self._table.get(w)
        self.found += v is not None
        return v

    def record(self, w: Workload, v: Verdict) -> None:
        self._table[w] = v

    def winners(self, device: str, target: str, op: str, bucket: Optional[tuple], timing: str,
                dtype: Optional[str] = None) -> set:
        """Names recorded as winner for this workload over every dtype (or one)."""
        return {v.winner for w, v in self._table.items()
                if (w.device, w.target, w.op, w.bucket, w.timing) == (device, target, op, bucket, timing)
                and dtype in (None, w.dtype)}

    def to_payload(self) -> dict:
        return {"version": SCHEMA_VERSION, "records": [_record_to_wire(w, v) for w, v in self._table.items()]}

    def absorb(self, payload: Mapping[str, Any], *, replace: bool = False) -> int:
        """Take in the records of a payload; returns how many were taken.  A record
        whose key is already present stays (what this process measured outranks a file)
        unless ``replace``.  A payload of an unknown schema version contributes nothing."""
        if payload.get("version") not in (1, 2, SCHEMA_VERSION):
            return 0
        taken = 0
        for rec in payload.get("records") or ():
            w, v = _record_from_wire(rec)
            if replace or w not in self._table:
                self._table[w] = v
                taken += 1
        return taken

    def save(self, path) -> Path:
        p = Path(path)
        p.parent.mkdir(parents=True, exist_ok=True)
        p.write_text(json.dumps(self.to_payload(), indent=2, sort_keys=True) + "\n")
        return p

    def absorb_file(self, path, *, replace: bool = False) -> int:
        """:meth:`absorb` from a JSON file; a missing or malformed file contributes
        nothing and does not raise."""
        try:
            payload = json.loads(Path(path).read_text())
            return self.absorb(payload, replace=replace)
        except (OSError, ValueError, KeyError, TypeError):
            return 0


def corpus_path() -> Path:
    """The corpus file: ``$TESSERA_AUTOTUNE_CORPUS`` (the reference's override variable,
    ``emit/autotune.py:226-230``) or the one packaged beside this module."""
    return Path(os.environ.get("TESSERA_AUTOTUNE_CORPUS") or PACKAGED)


_shared: Optional[Corpus] = None


def shared_corpus() -> Corpus:
    """The process-wide corpus, warm-started once from :func:`corpus_path` unless
    ``$TESSERA_AUTOTUNE_NO_WARMSTART`` is set."""
    global _shared
    if _shared is None:
        _shared = Corpus()
        if not os.environ.get("TESSERA_AUTOTUNE_NO_WARMSTART"):
            _shared.absorb_file(corpus_path())
    return _shared


def device_tag(target: str = _cand.TARGET) -> str:
    """``rocm:gfx950`` (the reference's ``<family>:<arch>`` form) when the lane runs
    here, else the bare target id, so nothing is keyed as a device it was not measured on."""
    return DEVICE_TAG if target == _cand.TARGET and _lane.available() else target


def problem_dims(op: str, inputs: tuple) -> Optional[tuple]:
    """``(Sq, Sk, D, Dv)`` for the 2-D operands ``(Q, K, V)`` of the ``attention`` op
    kind, ``(M, N, K)`` for the 2-D operands ``(A[M,K], B[K,N], ...)`` of any other;
    ``None`` when the operands are not 2-D arrays."""
    shapes = [tuple(getattr(x, "shape", ())) for x in inputs[:3]]
    if op == "attention":
        if len(shapes) == 3 and all(len(s) == 2 for s in shapes):
            return shapes[0][0], shapes[1][0], shapes[0][1], shapes[2][1]
        return None
    if len(shapes) >= 2 and len(shapes[0]) == 2 and len(shapes[1]) == 2:
        return shapes[0][0], shapes[1][1], shapes[0][1]
    return None


def _wall_ms(fn, reps: int, warmup: int) -> float:
    for _ in range(warmup):
        fn()
    laps = []
    for _ in range(max(reps, 1)):
        t0 = time.perf_counter()
        fn()
        laps.append((time.perf_counter() - t0) * 1e3)
    laps.sort()
    return laps[len(laps) // 2]


def _named(api: Any, target: str, op: str, name: str, region: Any):
    for c in api.candidates_for(target, op):
        if c.name == name and c.applies_to(region) and c.available():
            return c
    return None


def tune(api: Any, region: Any, op: str, target: str, *inputs: Any, corpus: Optional[Corpus] = None, dims=None,
         dtype: str = "f32", device: Optional[str] = None, timing: str = "end_to_end", reps: int = 20,
         warmup: int = 3):
    """The candidate to run for this workload, or ``None`` when none is viable.

    A recorded verdict whose winner is still registered, applicable and available is
    returned without timing anything.  Otherwise the host's arbiter verifies the
    candidates and calls back for a latency per survivor (device events through the
    candidate's ``measure_device_latency`` for ``timing="device"`` — a candidate
    without one is out of that race — else wall clock around ``run``); the fastest
    is recorded."""
    corpus = shared_corpus() if corpus is None else corpus
    key = Workload.of(device or device_tag(target), target, op, dims if dims is not None else problem_dims(op, inputs),
                      dtype, timing)
    known = corpus.lookup(key)
    if known is not None:
        c = _named(api, target, op, known.winner, region)
        if c is not None:
            return c
    timed: dict = {}

    def latency(c) -> float:
        if timing == "device":
            ms = c.measure_device_latency(region, *inputs, reps=reps, warmup=warmup)
            if ms is None:
                return float("inf")
        else:
            ms = _wall_ms(lambda: c.run(region, *inputs), reps, warmup)
        timed[c.name] = float(ms)
        return float(ms)

    best = api.arbitrate(region, op, target, verify=True, measure=latency)
    if best is None or best.name not in timed:
        return None
    corpus.record(key, Verdict(best.name, timed[best.name], dict(timed),
                               {"dims": None if key.bucket is None else list(dims or problem_dims(op, inputs)),
                                "reps": reps, "library": _lane.library_path().name}))
    return best


def recommended(api: Any, region: Any, op: str, target: str, *inputs: Any, corpus: Optional[Corpus] = None,
                dims=None, dtype: Optional[str] = None, device: Optional[str] = None,
                timing: str = "end_to_end") -> Optional[str]:
    """The recorded winner for this workload when the records agree on one name and
    that candidate is still viable here; a hint only — running it still goes through
    the host's gate."""
    corpus = shared_corpus() if corpus is None else corpus
    dims = dims if dims is not None else problem_dims(op, inputs)
    if dims is None:
        return None
    names = corpus.winners(device or device_tag(target), target, op, pow2_bucket(dims), timing, dtype)
    if len(names) != 1:
        return None
    (name,) = names
    return name if _named(api, target, op, name, region) is not None else None


def run_tuned(api: Any, region: Any, op: str, target: str, *inputs: Any, **kw: Any) -> tuple:
    """:func:`tune`, then run the winner -> ``(output, tag)``; :class:`NoCandidate`
    when nothing is viable."""
    best = tune(api, region, op, target, *inputs, **kw)
    if best is None:
        raise NoCandidate(f"no viable gfx950 candidate for ({target}, {op})")
    return best.run(region, *inputs)


def measure_headline_corpus(api: Any, regions: Any, corpus: Optional[Corpus] = None, *, reps: int = 10) -> Corpus:
    """Tune the lane's candidates on the shapes of the headline configurations.
    ``regions`` supplies the host's region classes (``MatmulRegion``, ``FusedRegion``,
    ``GatedMatmulRegion``, ``AttentionRegion`` of ``compiler/fusion_core.py``)."""
    import numpy as np
    corpus = Corpus() if corpus is None else corpus
    _cand.register(api)
    rng = np.random.default_rng(0)
    tgt = _cand.TARGET

    def randn(*shape, s=1.0):
        return rng.standard_normal(shape, dtype=np.float32) * np.float32(s)

    for M, N, K in ((8192, 8192, 8192), (4096, 8192, 8192), (128, 8192, 8192), (16, 8192, 8192), (1, 8192, 8192),
                    (512, 256, 64)):
        A, B = randn(M, K, s=K ** -0.5), randn(K, N, s=K ** -0.5)
        for dt in ("bfloat16", "float16"):
            tune(api, regions.MatmulRegion(dtype=dt), api.OP_MATMUL, tgt, A, B, dtype=dt, corpus=corpus, reps=reps,
                 warmup=2, timing="device")
    for M, N, K in ((4096, 4096, 4096), (8192, 1408, 4096)):
        A, B, bias = randn(M, K, s=K ** -0.5), randn(K, N), randn(N)
        for chain in (("bias", "gelu"), ("bias", "silu"), ("relu",)):
            tune(api, regions.FusedRegion(epilogue=chain, storage_dtype="bf16"), api.OP_FUSED_REGION, tgt, A, B, bias,
                 dtype="bf16:" + "+".join(chain), corpus=corpus, reps=max(3, reps // 3), warmup=1)
        tune(api, regions.GatedMatmulRegion(gate_act="silu", storage_dtype="bf16"), api.OP_GATED_MATMUL, tgt, A, B,
             randn(K, N), dtype="bf16", corpus=corpus, reps=max(3, reps // 3), warmup=1)
    for S, D in ((4096, 128), (1024, 64)):
        Q, Kk, V = randn(S, D), randn(S, D), randn(S, D)
        for causal in (False, True):
            tune(api, regions.AttentionRegion(scale=D ** -0.5, causal=causal, storage_dtype="bf16"), api.OP_ATTENTION,
                 tgt, Q, Kk, V, dims=(S, S, D, D), dtype="bf16:causal" if causal else "bf16", corpus=corpus,
                 reps=reps, warmup=2)
    return corpus
