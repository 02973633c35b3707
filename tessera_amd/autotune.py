"""Measured arbitration and the persisted autotune corpus for the gfx950 lane.

Mirrors ``python/tessera/compiler/emit/autotune.py``: a :class:`MeasureCache` of
:class:`MeasureRecord` keyed by ``(device, target, op, shape-bucket, dtype,
timing)`` (``:40-75,139-206``), measure-at-first-miss arbitration over the F4-gated
candidates (``:392-447``), and the committed JSON corpus that warm-starts other
processes (``:215-278``) in the reference's schema (``CORPUS_VERSION = 3``), so the
records written here can be merged into Tessera's own
``benchmarks/baselines/autotune_corpus.json``.  Device tags follow the reference's
``<family>:<arch>`` form (``rocm:gfx950``), so a record only warm-starts a matching
device.

``python -m tessera_amd.autotune [--out PATH]`` measures the lane's candidates on
the shapes of the headline configurations and writes the corpus.
"""
from __future__ import annotations

import json
import os
import statistics
import sys
import time
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, Mapping, Optional

import numpy as np

from . import candidates as _cand
from . import lane as _lane

CORPUS_VERSION = 3
TIMING_END_TO_END = "end_to_end"
TIMING_DEVICE = "device"
_TIMING_MODES = (TIMING_END_TO_END, TIMING_DEVICE)


@dataclass(frozen=True)
class MeasureRecord:
    """The measured verdict for one key: the fastest candidate, its median latency
    (ms), every timed candidate's latency and free-form evidence."""
    winner: str
    latency_ms: float
    candidates: dict = field(default_factory=dict)
    evidence: dict = field(default_factory=dict)
    candidate_descriptors: dict = field(default_factory=dict)

    def as_json(self) -> dict:
        out = {"winner": self.winner, "latency_ms": self.latency_ms, "candidates": dict(self.candidates)}
        if self.candidate_descriptors:
            out["candidate_descriptors"] = dict(self.candidate_descriptors)
        if self.evidence:
            out["evidence"] = dict(self.evidence)
        return out

    @classmethod
    def from_json(cls, d: Mapping[str, Any]) -> "MeasureRecord":
        return cls(winner=str(d["winner"]), latency_ms=float(d["latency_ms"]),
                   candidates={str(k): float(v) for k, v in dict(d.get("candidates", {})).items()},
                   candidate_descriptors={str(k): dict(v) for k, v in dict(d.get("candidate_descriptors", {})).items()
                                          if isinstance(v, dict)},
                   evidence=dict(d.get("evidence", {})))


def _dim_bucket(n: int) -> int:
    """Next power of two (``emit/kernel_emitter.py:72-80``)."""
    b = 1
    while b < n:
        b *= 2
    return b


def bucket_key(dims) -> Optional[tuple]:
    """Shape-bucket key: every dim coarsened to its power-of-two bucket."""
    return None if dims is None else tuple(_dim_bucket(int(d)) for d in dims)


def _normalize_key(key: tuple) -> tuple:
    if len(key) == 5:
        return (*key, TIMING_END_TO_END)
    if len(key) != 6 or key[5] not in _TIMING_MODES:
        raise ValueError(f"invalid autotune cache key {key!r}")
    return key


def _key_to_json(key: tuple) -> dict:
    dev, target, op, bucket, dtype, timing = _normalize_key(key)
    return {"device": dev, "target": target, "op": op, "bucket": list(bucket) if bucket is not None else None,
            "dtype": dtype, "timing": timing}


def _key_from_json(d: Mapping[str, Any]) -> tuple:
    b = d.get("bucket")
    return (d["device"], d["target"], d["op"], tuple(b) if b is not None else None, d["dtype"],
            d.get("timing", TIMING_END_TO_END))


class MeasureCache:
    """Content-keyed cache of measured verdicts — measure-at-first-miss."""

    def __init__(self) -> None:
        self._store: dict = {}
        self.hits = 0
        self.misses = 0

    def get(self, key: tuple) -> Optional[MeasureRecord]:
        rec = self._store.get(_normalize_key(key))
        if rec is not None:
            self.hits += 1
        else:
            self.misses += 1
        return rec

    def put(self, key: tuple, rec: MeasureRecord) -> None:
        self._store[_normalize_key(key)] = rec

    def clear(self) -> None:
        self._store.clear()
        self.hits = self.misses = 0

    @property
    def size(self) -> int:
        return len(self._store)

    def items(self):
        return self._store.items()

    def to_dict(self) -> dict:
        return {"version": CORPUS_VERSION,
                "records": [{**_key_to_json(k), **rec.as_json()} for k, rec in self._store.items()]}

    def load_dict(self, payload: Mapping[str, Any], *, overwrite: bool = False) -> int:
        """Merge a :meth:`to_dict` payload (warm start).  A key already present is
        kept (measured-on-this-box wins) unless ``overwrite``; a payload of another
        schema version loads nothing."""
        if int(payload.get("version", -1)) not in (1, 2, CORPUS_VERSION):
            return 0
        loaded = 0
        for r in payload.get("records", ()):
            key = _key_from_json(r)
            if not overwrite and key in self._store:
                continue
            self._store[key] = MeasureRecord.from_json(r)
            loaded += 1
        return loaded


_DEFAULT_CACHE = MeasureCache()
_CORPUS_PATH = Path(__file__).resolve().parent / "autotune_corpus.json"
_warm_started = False


def default_cache() -> MeasureCache:
    return _DEFAULT_CACHE


def corpus_path() -> Path:
    """``$TESSERA_AUTOTUNE_CORPUS`` overrides the packaged corpus (the reference's
    own override variable, ``emit/autotune.py:226-230``)."""
    env = os.environ.get("TESSERA_AUTOTUNE_CORPUS")
    return Path(env) if env else _CORPUS_PATH


def save_corpus(path=None, cache: Optional[MeasureCache] = None) -> Path:
    cache = cache if cache is not None else _DEFAULT_CACHE
    p = Path(path) if path is not None else corpus_path()
    p.parent.mkdir(parents=True, exist_ok=True)
    p.write_text(json.dumps(cache.to_dict(), indent=2, sort_keys=True) + "\n")
    return p


def load_corpus(path=None, cache: Optional[MeasureCache] = None, *, overwrite: bool = False) -> int:
    """Merge the corpus file into ``cache``; a missing, unreadable or stale file
    loads nothing and never raises."""
    cache = cache if cache is not None else _DEFAULT_CACHE
    p = Path(path) if path is not None else corpus_path()
    try:
        payload = json.loads(p.read_text())
    except (OSError, ValueError):
        return 0
    return cache.load_dict(payload, overwrite=overwrite)


def _maybe_warm_start(cache: MeasureCache) -> None:
    global _warm_started
    if _warm_started or cache is not _DEFAULT_CACHE:
        return
    _warm_started = True
    if os.environ.get("TESSERA_AUTOTUNE_NO_WARMSTART"):
        return
    load_corpus(cache=cache)


def measure_latency(run_fn, *, reps: int = 20, warmup: int = 3) -> float:
    """Median wall-clock latency (ms) of ``run_fn`` — end to end, what a caller pays
    (``emit/autotune.py:281-304``)."""
    for _ in range(warmup):
        run_fn()
    samples = []
    for _ in range(reps):
        t0 = time.perf_counter()
        run_fn()
        samples.append((time.perf_counter() - t0) * 1e3)
    return statistics.median(samples)


def device_id(target: str = _cand.TARGET) -> str:
    """``rocm:gfx950`` on the device; the bare target id when the lane is absent, so
    nothing measured on one device is keyed as another."""
    if target == _cand.TARGET and _lane.available():
        return "rocm:gfx950"
    return target


def _infer_dims(op: str, inputs: tuple) -> Optional[tuple]:
    try:
        if op in (_cand.OP_MATMUL, _cand.OP_FUSED_REGION, _cand.OP_GATED_MATMUL) and len(inputs) >= 2:
            a, b = inputs[0], inputs[1]
            if len(a.shape) == 2 and len(b.shape) == 2:
                return (int(a.shape[0]), int(b.shape[1]), int(a.shape[1]))
        if op == _cand.OP_ATTENTION and len(inputs) >= 3:
            q, k, v = inputs[:3]
            if len(q.shape) == len(k.shape) == len(v.shape) == 2:
                return (int(q.shape[0]), int(k.shape[0]), int(q.shape[1]), int(v.shape[1]))
    except (AttributeError, IndexError, TypeError, ValueError):
        pass
    return None


def measured_arbitrate(region: Any, op: str, target: str, *inputs: Any, dims=None, dtype: str = "f32",
                       cache: Optional[MeasureCache] = None, reps: int = 20, warmup: int = 3,
                       device: Optional[str] = None, timing: str = TIMING_END_TO_END):
    """The winning candidate by measured latency, or ``None`` when none applies and
    verifies.  A cache hit returns the recorded winner without re-timing; a miss
    F4-gates the candidates, times the survivors on ``inputs`` and records the
    fastest."""
    if timing not in _TIMING_MODES:
        raise ValueError(f"unknown autotune timing mode {timing!r}")
    cache = cache if cache is not None else _DEFAULT_CACHE
    _maybe_warm_start(cache)
    dims = dims if dims is not None else _infer_dims(op, inputs)
    key = (device or device_id(target), target, op, bucket_key(dims), dtype, timing)
    rec = cache.get(key)
    if rec is not None:
        for c in _cand.candidates_for(target, op):
            if c.name == rec.winner and c.applies_to(region) and c.available():
                return c
    latencies: dict = {}

    def _measure(c) -> float:
        if timing == TIMING_DEVICE:
            m = c.measure_device_latency(region, *inputs, reps=reps, warmup=warmup)
            if m is None:
                return float("inf")
            t = float(m)
        else:
            t = measure_latency(lambda: c.run(region, *inputs), reps=reps, warmup=warmup)
        latencies[c.name] = t
        return t

    winner = _cand.arbitrate(region, op, target, verify=True, measure=_measure)
    if winner is not None and winner.name in latencies:
        cache.put(key, MeasureRecord(winner=winner.name, latency_ms=latencies[winner.name],
                                     candidates=dict(latencies),
                                     evidence={"dims": list(dims) if dims is not None else None,
                                               "reps": reps, "library": Path(_lane.library_path()).name}))
        return winner
    return None


def corpus_winner(region: Any, op: str, target: str, *inputs: Any, dims=None, dtype: Optional[str] = None,
                  cache: Optional[MeasureCache] = None, device: Optional[str] = None,
                  timing: str = TIMING_END_TO_END) -> Optional[str]:
    """The persisted winner for this workload when it is unambiguous and still
    applicable — a selection hint; execution still passes the F4 gate."""
    cache = cache if cache is not None else _DEFAULT_CACHE
    _maybe_warm_start(cache)
    dims = dims if dims is not None else _infer_dims(op, inputs)
    if dims is None:
        return None
    dev = device or device_id(target)
    bucket = bucket_key(dims)
    winners = {rec.winner for (kd, kt, ko, kb, kdt, ktm), rec in cache.items()
               if kd == dev and kt == target and ko == op and kb == bucket and ktm == timing
               and (dtype is None or kdt == dtype)}
    if len(winners) != 1:
        return None
    name = next(iter(winners))
    for c in _cand.candidates_for(target, op):
        if c.name == name and c.applies_to(region) and c.available():
            return name
    return None


def run_measured_arbitrated(region: Any, op: str, target: str, *inputs: Any, **kw: Any) -> tuple:
    """:func:`measured_arbitrate` then run the winner → ``(output, tag)``.  With no
    viable candidate this raises :class:`~tessera_amd.candidates.ArbiterError`: the
    lane has no CPU degrade path."""
    winner = measured_arbitrate(region, op, target, *inputs, **kw)
    if winner is None:
        raise _cand.ArbiterError(f"no viable gfx950 candidate for ({target}, {op})")
    return winner.run(region, *inputs)


# ---- corpus generation on the device ----------------------------------------------------

def measure_headline_corpus(cache: Optional[MeasureCache] = None, *, reps: int = 10) -> MeasureCache:
    """Measure the lane's candidates on the shapes of the headline configurations and
    record the verdicts (device timing where a candidate offers it)."""
    cache = cache if cache is not None else MeasureCache()
    _cand.register_all()
    rng = np.random.default_rng(0)
    T = _cand.TARGET

    def randn(*shape, s=1.0):
        return (rng.standard_normal(shape, dtype=np.float32) * np.float32(s))

    for (M, N, K) in ((8192, 8192, 8192), (4096, 8192, 8192), (128, 8192, 8192), (16, 8192, 8192), (1, 8192, 8192),
                      (512, 256, 64)):
        A, B = randn(M, K, s=K ** -0.5), randn(K, N, s=K ** -0.5)
        for dt in ("bfloat16", "float16"):
            measured_arbitrate(_cand.MatmulRegion(dtype=dt), _cand.OP_MATMUL, T, A, B, dtype=dt, cache=cache,
                               reps=reps, warmup=2, timing=TIMING_DEVICE)
    for (M, N, K) in ((4096, 4096, 4096), (8192, 1408, 4096)):
        A, B, bias = randn(M, K, s=K ** -0.5), randn(K, N), randn(N)
        for epi in (("bias", "gelu"), ("bias", "silu"), ("relu",)):
            measured_arbitrate(_cand.FusedRegion(epilogue=epi, storage_dtype="bf16"), _cand.OP_FUSED_REGION, T, A, B,
                               bias, dtype="bf16:" + "+".join(epi), cache=cache, reps=max(3, reps // 3), warmup=1)
        measured_arbitrate(_cand.GatedMatmulRegion("silu", "bf16"), _cand.OP_GATED_MATMUL, T, A, B, randn(K, N),
                           dtype="bf16", cache=cache, reps=max(3, reps // 3), warmup=1)
    for (S, D) in ((4096, 128), (1024, 64)):
        Q, Kk, V = randn(S, D), randn(S, D), randn(S, D)
        for causal in (False, True):
            measured_arbitrate(_cand.AttentionRegion(scale=D ** -0.5, causal=causal, storage_dtype="bf16"),
                               _cand.OP_ATTENTION, T, Q, Kk, V, dtype="bf16:causal" if causal else "bf16",
                               cache=cache, reps=reps, warmup=2)
    return cache


def _main(argv: list) -> int:
    out = None
    if "--out" in argv:
        out = argv[argv.index("--out") + 1]
    if not _lane.available():
        print("gfx950 lane unavailable: the corpus is measured on the MI355X", file=sys.stderr)
        return 3
    cache = measure_headline_corpus()
    p = save_corpus(out, cache)
    print(f"wrote {cache.size} records to {p}")
    return 0


if __name__ == "__main__":
    sys.exit(_main(sys.argv[1:]))
