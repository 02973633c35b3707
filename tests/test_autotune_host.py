"""CPU checks of the measured-arbitration cache and corpus format (the schema of
python/tessera/compiler/emit/autotune.py), with stand-in candidates on a private
target so no device is needed."""
import json

import numpy as np
import pytest

from tessera_amd import autotune as at
from tessera_amd import candidates as cand

TGT = "unit_test_target"


class _Fake(cand.Candidate):
    target = TGT
    op = cand.OP_MATMUL
    tier = cand.Tier.EMITTED

    def __init__(self, name, delay_ms, wrong=False):
        self.name = name
        self.delay = delay_ms
        self.wrong = wrong
        self.calls = 0

    def run(self, region, A, B, *a, **k):
        self.calls += 1
        out = region.reference(A, B)
        return (out + 1.0 if self.wrong else out), self.name

    def measure_device_latency(self, region, *inputs, reps=100, warmup=10):
        return self.delay


@pytest.fixture()
def fakes():
    fast, slow, bad = _Fake("fast", 1.0), _Fake("slow", 5.0), _Fake("fast_but_wrong", 0.1, wrong=True)
    for c in (slow, fast, bad):
        cand.register_candidate(c)
    yield fast, slow, bad
    cand._CANDIDATES.pop((TGT, cand.OP_MATMUL), None)


def test_bucket_and_key_round_trip():
    assert at.bucket_key((8192, 100, 1)) == (8192, 128, 1)
    assert at.bucket_key(None) is None
    key = ("rocm:gfx950", "rocm_gfx950", "matmul", (8192, 8192, 8192), "bfloat16", "device")
    assert at._key_from_json(at._key_to_json(key)) == key
    assert at._normalize_key(key[:5])[5] == at.TIMING_END_TO_END
    with pytest.raises(ValueError):
        at._normalize_key(key[:4])


def test_measured_arbitrate_picks_fastest_verified_and_caches(fakes):
    fast, slow, bad = fakes
    region = cand.MatmulRegion(dtype="float16")
    A = np.random.default_rng(0).standard_normal((8, 8)).astype(np.float32)
    cache = at.MeasureCache()
    w = at.measured_arbitrate(region, cand.OP_MATMUL, TGT, A, A, dtype="float16", cache=cache, device="dev0",
                              timing=at.TIMING_DEVICE)
    assert w is fast                                      # the wrong one is gated out although fastest
    rec = cache.get(("dev0", TGT, cand.OP_MATMUL, (8, 8, 8), "float16", at.TIMING_DEVICE))
    assert rec.winner == "fast" and rec.candidates == {"fast": 1.0, "slow": 5.0}
    calls = (fast.calls, slow.calls)
    assert at.measured_arbitrate(region, cand.OP_MATMUL, TGT, A, A, dtype="float16", cache=cache, device="dev0",
                                 timing=at.TIMING_DEVICE) is fast
    assert (fast.calls, slow.calls) == calls              # cache hit: nothing re-run
    # another device or bucket is a different key
    assert cache.get(("dev1", TGT, cand.OP_MATMUL, (8, 8, 8), "float16", at.TIMING_DEVICE)) is None
    assert at.corpus_winner(region, cand.OP_MATMUL, TGT, A, A, cache=cache, device="dev0",
                            timing=at.TIMING_DEVICE) == "fast"
    assert at.corpus_winner(region, cand.OP_MATMUL, TGT, A, A, cache=cache, device="dev1",
                            timing=at.TIMING_DEVICE) is None
    out, tag = at.run_measured_arbitrated(region, cand.OP_MATMUL, TGT, A, A, dtype="float16", cache=cache,
                                          device="dev0", timing=at.TIMING_DEVICE)
    assert tag == "fast" and np.allclose(out, region.reference(A, A))


def test_no_candidate_raises_instead_of_cpu_fallback():
    region = cand.MatmulRegion(dtype="float16")
    A = np.zeros((4, 4), np.float32)
    with pytest.raises(cand.ArbiterError):
        at.run_measured_arbitrated(region, cand.OP_MATMUL, "no_such_target", A, A, cache=at.MeasureCache())


def test_corpus_file_round_trip_and_versioning(tmp_path, fakes):
    cache = at.MeasureCache()
    key = ("rocm:gfx950", "rocm_gfx950", "matmul", (8192, 8192, 8192), "bfloat16", "device")
    cache.put(key, at.MeasureRecord("gfx950_mfma_gemm", 0.93, {"gfx950_mfma_gemm": 0.93}, {"reps": 10}))
    p = at.save_corpus(tmp_path / "corpus.json", cache)
    payload = json.loads(p.read_text())
    assert payload["version"] == at.CORPUS_VERSION
    r = payload["records"][0]
    assert set(r) >= {"device", "target", "op", "bucket", "dtype", "timing", "winner", "latency_ms", "candidates"}
    fresh = at.MeasureCache()
    assert at.load_corpus(p, fresh) == 1 and fresh.get(key).latency_ms == 0.93
    # measured-on-this-box wins over the file unless overwrite
    fresh.put(key, at.MeasureRecord("other", 0.5))
    assert at.load_corpus(p, fresh) == 0 and fresh.get(key).winner == "other"
    assert at.load_corpus(p, fresh, overwrite=True) == 1 and fresh.get(key).winner == "gfx950_mfma_gemm"
    # stale schema and unreadable files load nothing, never raise
    p.write_text(json.dumps({"version": 99, "records": payload["records"]}))
    assert at.load_corpus(p, at.MeasureCache()) == 0
    assert at.load_corpus(tmp_path / "missing.json", at.MeasureCache()) == 0
    p.write_text("not json")
    assert at.load_corpus(p, at.MeasureCache()) == 0


def test_packaged_corpus_is_well_formed():
    """The committed corpus (measured on the MI355X) parses, is keyed to the gfx950
    device tag and names only candidates this lane registers."""
    cache = at.MeasureCache()
    n = at.load_corpus(at._CORPUS_PATH, cache)
    assert n > 0
    cand.register_all()
    names = {c.name for op in (cand.OP_MATMUL, cand.OP_ATTENTION, cand.OP_FUSED_REGION, cand.OP_GATED_MATMUL)
             for c in cand.candidates_for(cand.TARGET, op)}
    for (dev, target, op, bucket, dtype, timing), rec in cache.items():
        assert dev == "rocm:gfx950" and target == cand.TARGET and timing in (at.TIMING_DEVICE, at.TIMING_END_TO_END)
        assert rec.winner in names and rec.latency_ms > 0 and bucket is not None
