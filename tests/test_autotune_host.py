"""CPU checks of the lane's autotune corpus (the wire schema of
python/tessera/compiler/emit/autotune.py:40-75,170-202) and of tuning through a
host's arbiter, with stand-in candidates on a private target so no device is needed."""
import json

import numpy as np
import pytest

import standin_host as host
from tessera_amd import autotune as at
from tessera_amd import candidates as cand

TGT = "unit_test_target"


class _Fake(host.Candidate):
    target = TGT
    op = "matmul"
    tier = host.Tier.EMITTED

    def __init__(self, name, device_ms, wrong=False):
        self.name = name
        self.device_ms = device_ms
        self.wrong = wrong
        self.calls = 0

    def run(self, region, A, B, *a, **k):
        self.calls += 1
        out = region.reference(A, B)
        return (out + 1.0 if self.wrong else out), self.name

    def measure_device_latency(self, region, *inputs, reps=100, warmup=10):
        return self.device_ms


@pytest.fixture()
def api_and_fakes():
    api = host.CandidateHost()
    fast, slow, bad = _Fake("fast", 1.0), _Fake("slow", 5.0), _Fake("fast_but_wrong", 0.1, wrong=True)
    for c in (slow, fast, bad):
        api.register_candidate(c)
    return api, fast, slow, bad


def test_buckets_and_keys():
    assert at.pow2_bucket((8192, 100, 1)) == (8192, 128, 1)
    assert at.pow2_bucket((0, 3, 1025)) == (1, 4, 2048)
    assert at.pow2_bucket(None) is None
    w = at.Workload.of("rocm:gfx950", "rocm_gfx950", "matmul", (8000, 8192, 4097), "bfloat16", "device")
    assert w.bucket == (8192, 8192, 8192)
    assert at.Workload("d", "t", "matmul", None, "f32").timing == "end_to_end"
    with pytest.raises(ValueError):
        at.Workload("d", "t", "matmul", None, "f32", "cycles")
    assert at.problem_dims("matmul", (np.zeros((3, 5)), np.zeros((5, 7)), np.zeros(7))) == (3, 7, 5)
    assert at.problem_dims("attention", (np.zeros((9, 4)), np.zeros((6, 4)), np.zeros((6, 8)))) == (9, 6, 4, 8)
    assert at.problem_dims("matmul", (np.zeros(3), np.zeros((3, 2)))) is None


def test_tune_picks_fastest_verified_and_records_it(api_and_fakes):
    api, fast, slow, bad = api_and_fakes
    region = host.MatmulRegion(dtype="float16")
    A = np.random.default_rng(0).standard_normal((8, 8)).astype(np.float32)
    corpus = at.Corpus()
    kw = dict(dtype="float16", corpus=corpus, device="dev0", timing="device")
    assert at.tune(api, region, "matmul", TGT, A, A, **kw) is fast          # the wrong one is gated out although fastest
    v = corpus.lookup(at.Workload("dev0", TGT, "matmul", (8, 8, 8), "float16", "device"))
    assert v.winner == "fast" and v.latency_ms == 1.0 and v.candidates == {"fast": 1.0, "slow": 5.0}
    assert v.evidence["dims"] == [8, 8, 8]
    calls = (fast.calls, slow.calls, bad.calls)
    assert at.tune(api, region, "matmul", TGT, A, A, **kw) is fast
    assert (fast.calls, slow.calls, bad.calls) == calls                     # recorded verdict: nothing re-run
    assert corpus.lookup(at.Workload("dev1", TGT, "matmul", (8, 8, 8), "float16", "device")) is None
    assert at.recommended(api, region, "matmul", TGT, A, A, corpus=corpus, device="dev0", timing="device") == "fast"
    assert at.recommended(api, region, "matmul", TGT, A, A, corpus=corpus, device="dev1", timing="device") is None
    out, tag = at.run_tuned(api, region, "matmul", TGT, A, A, **kw)
    assert tag == "fast" and np.allclose(out, region.reference(A, A))
    # wall-clock timing runs the candidates themselves
    wall = at.Corpus()
    assert at.tune(api, region, "matmul", TGT, A, A, dtype="float16", corpus=wall, device="dev0", reps=2,
                   warmup=0) in (fast, slow)
    assert fast.calls > calls[0] and len(wall) == 1
    # a recorded winner that is no longer registered is measured again, not trusted
    stale = at.Corpus()
    stale.record(at.Workload("dev0", TGT, "matmul", (8, 8, 8), "float16", "device"), at.Verdict("gone", 0.1))
    assert at.tune(api, region, "matmul", TGT, A, A, dtype="float16", corpus=stale, device="dev0",
                   timing="device") is fast


def test_nothing_viable_raises_instead_of_running_on_the_cpu():
    api = host.CandidateHost()
    region = host.MatmulRegion(dtype="float16")
    A = np.zeros((4, 4), np.float32)
    assert at.tune(api, region, "matmul", "no_such_target", A, A, corpus=at.Corpus()) is None
    with pytest.raises(at.NoCandidate):
        at.run_tuned(api, region, "matmul", "no_such_target", A, A, corpus=at.Corpus())


def test_corpus_file_round_trip_and_versions(tmp_path):
    corpus = at.Corpus()
    key = at.Workload("rocm:gfx950", "rocm_gfx950", "matmul", (8192, 8192, 8192), "bfloat16", "device")
    corpus.record(key, at.Verdict("gfx950_mfma_gemm", 0.93, {"gfx950_mfma_gemm": 0.93}, {"reps": 10}))
    p = corpus.save(tmp_path / "corpus.json")
    payload = json.loads(p.read_text())
    assert payload["version"] == 3
    (r,) = payload["records"]
    assert set(r) == {"device", "target", "op", "bucket", "dtype", "timing", "winner", "latency_ms", "candidates",
                      "evidence"}
    assert r["bucket"] == [8192, 8192, 8192] and r["timing"] == "device"
    fresh = at.Corpus()
    assert fresh.absorb_file(p) == 1 and fresh.lookup(key).latency_ms == 0.93
    # what this process measured outranks the file unless replace
    fresh.record(key, at.Verdict("other", 0.5))
    assert fresh.absorb_file(p) == 0 and fresh.lookup(key).winner == "other"
    assert fresh.absorb_file(p, replace=True) == 1 and fresh.lookup(key).winner == "gfx950_mfma_gemm"
    # a record written before the timing field existed is an end-to-end one
    old = {"version": 2, "records": [{k: v for k, v in r.items() if k != "timing"}]}
    older = at.Corpus()
    assert older.absorb(old) == 1 and next(iter(older))[0].timing == "end_to_end"
    # unknown versions, missing and malformed files contribute nothing and do not raise
    p.write_text(json.dumps({"version": 99, "records": payload["records"]}))
    assert at.Corpus().absorb_file(p) == 0
    assert at.Corpus().absorb_file(tmp_path / "missing.json") == 0
    p.write_text("not json")
    assert at.Corpus().absorb_file(p) == 0
    p.write_text(json.dumps({"version": 3, "records": [{"device": "x"}]}))
    assert at.Corpus().absorb_file(p) == 0


def test_packaged_corpus_is_well_formed():
    """The committed corpus (measured on the MI355X) parses, is keyed to the gfx950
    device tag and names only candidates this lane registers."""
    corpus = at.Corpus()
    assert corpus.absorb_file(at.PACKAGED) > 0
    names = {c.name for c in cand.build_candidates(host.CandidateHost())}
    for w, v in corpus:
        assert w.device == at.DEVICE_TAG and w.target == cand.TARGET and w.timing in at.TIMINGS
        assert v.winner in names and v.latency_ms > 0 and w.bucket is not None
        assert set(v.candidates) <= names
