"""The reference's plugin seams on the MI355X: executors through ``launch`` and
candidates through the arbiter run real kernels (never a reference tag) and
match the oracle."""
import numpy as np
import pytest

import tessera_oracle as orc
from tessera_amd import bf16 as b16
from tessera_amd import candidates as cand
from tessera_amd import executors as ex
from tessera_amd import ops

pytestmark = pytest.mark.gpu


def test_launch_matmul_executor(lane):
    rng = np.random.default_rng(0)
    A = (rng.standard_normal((96, 160)) * .5).astype(np.float16)
    B = (rng.standard_normal((160, 72)) * .5).astype(np.float16)
    art = ex.make_artifact("tessera.matmul", ["a", "b"], ["a", "b"], "gfx950_gemm")
    assert art.metadata["executable"] is True
    res = ex.launch(art, (A, B))
    assert res["ok"] and res["execution_kind"] == "native_gpu" and res["execution_mode"] == "hip_runtime"
    assert res["output"].dtype == np.float32 and res["profile"]["cpu_wall_ms"] > 0
    ref = A.astype(np.float64) @ B.astype(np.float64)
    assert np.max(np.abs(res["output"] - ref)) <= 1e-2           # the reference test's f16 budget
    assert orc.max_rel_err(res["output"], ref) <= 1e-5
    a8 = rng.integers(-127, 128, (40, 64)).astype(np.int8)
    b8 = rng.integers(-127, 128, (64, 48)).astype(np.int8)
    res = ex.launch(art, {"a": a8, "b": b8})
    assert res["ok"] and res["output"].dtype == np.int32
    assert np.array_equal(res["output"], orc.gemm_i8_i32(a8, b8))


def test_launch_flash_attn_executor(lane):
    rng = np.random.default_rng(1)
    q = b16.from_float32(rng.standard_normal((2, 8, 130, 64)) * .5)
    k = b16.from_float32(rng.standard_normal((2, 2, 130, 64)) * .5)
    v = b16.from_float32(rng.standard_normal((2, 2, 130, 64)) * .5)
    art = ex.make_artifact("tessera.gqa_attention", ["q", "k", "v"], ["q", "k", "v"], "gfx950_flash_attn",
                           kwargs={"causal": True})
    res = ex.launch(art, (q, k, v))
    assert res["ok"] and res["output"].shape == (2, 8, 130, 64) and res["output"].dtype == np.float32
    ref, _ = orc.flash_attn_dense(q.to_float32(), k.to_float32(), v.to_float32(), causal=True)
    assert orc.max_rel_err(res["output"], ref) <= 2e-3
    bad = ex.make_artifact("tessera.flash_attn", ["q", "k", "v"], ["q", "k", "v"], "gfx950_flash_attn",
                           kwargs={"window": -16})
    assert ex.launch(bad, (q, k, v))["runtime_status"] == "invalid_artifact"
    drop = ex.make_artifact("tessera.flash_attn", ["q", "k", "v"], ["q", "k", "v"], "gfx950_flash_attn",
                            kwargs={"dropout_p": 0.1})
    assert ex.launch(drop, (q, k, v))["runtime_status"] == "invalid_artifact"


def test_launch_moe_transport_executor(lane):
    T, H, E, k = 200, 64, 8, 2
    lg = np.random.default_rng(2).standard_normal((T, E)).astype(np.float32)
    plan = ops.route_tokens(lg, E, k, capacity_factor=1e9)
    x = np.random.default_rng(3).standard_normal((T, H)).astype(np.float32)
    art = ex.make_artifact("tessera.moe_dispatch", ["x", "plan"], ["x", "plan"], "gfx950_moe_transport")
    res = ex.launch(art, {"x": x, "plan": plan})
    assert res["ok"] and res["execution_kind"] == "native_gpu"
    assert np.array_equal(res["output"], x[plan.token_of_slot])
    art = ex.make_artifact("tessera.moe_combine", ["partials", "plan"], ["partials", "plan"], "gfx950_moe_transport")
    res2 = ex.launch(art, {"partials": res["output"], "plan": plan})
    assert res2["ok"] and np.allclose(res2["output"], x, atol=1e-5)     # weights sum to 1 per token
    w = (np.random.default_rng(4).standard_normal((E, H, 48)) * .2).astype(np.float32)
    art = ex.make_artifact("tessera.grouped_gemm", ["x", "weights", "group_sizes"], ["x", "weights", "group_sizes"],
                           "gfx950_moe_transport")
    res3 = ex.launch(art, {"x": b16.from_float32(res["output"]), "weights": b16.from_float32(w),
                           "group_sizes": plan.group_sizes})
    assert res3["ok"] and res3["output"].dtype == np.float32
    assert orc.max_rel_err(res3["output"], orc.grouped_gemm(res["output"], w, plan.group_sizes, store=False)) <= 1e-5


def test_arbiter_picks_and_runs_real_kernels(lane):
    cand.reset_arbiter_dispatch_log()
    rng = np.random.default_rng(5)
    for dtype in ("bfloat16", "float16"):
        region = cand.MatmulRegion(dtype)
        assert cand.verify_candidate(cand.Gfx950MfmaGemmCandidate(), region)
        A = (rng.standard_normal((64, 96)) * .4).astype(np.float32)
        B = (rng.standard_normal((96, 40)) * .4).astype(np.float32)
        out, tag = cand.run_arbitrated(region, cand.OP_MATMUL, cand.TARGET, A, B)
        assert tag == cand.GEMM_TAG and tag not in cand.REFERENCE_EXECUTIONS
        assert np.allclose(out, region.reference(A, B), atol=1e-3)
    region = cand.MatmulRegion("bfloat16", transpose_a=True, transpose_b=True)
    A = (rng.standard_normal((96, 64)) * .4).astype(np.float32)       # raw (K, M)
    B = (rng.standard_normal((40, 96)) * .4).astype(np.float32)       # raw (N, K)
    out, tag = cand.run_arbitrated(region, cand.OP_MATMUL, cand.TARGET, A, B)
    assert tag == cand.GEMM_TAG and np.allclose(out, region.reference(A, B), atol=1e-3)
    for causal in (False, True):
        att = cand.AttentionRegion(scale=0.25, causal=causal, storage_dtype="bf16")
        Q, K, V = ((rng.standard_normal((48, 32)) * .5).astype(np.float32) for _ in range(3))
        out, tag = cand.run_arbitrated(att, cand.OP_ATTENTION, cand.TARGET, Q, K, V)
        assert tag == cand.ATTN_TAG and np.allclose(out, att.reference(Q, K, V), atol=5e-3)
    gg = cand.GroupedGemmRegion((10, 0, 30), "bfloat16")
    x = (rng.standard_normal((40, 64)) * .4).astype(np.float32)
    w = (rng.standard_normal((3, 64, 32)) * .4).astype(np.float32)
    out, tag = cand.run_arbitrated(gg, cand.OP_GROUPED_GEMM, cand.TARGET, x, w)
    assert tag == cand.GROUPED_TAG and np.allclose(out, gg.reference(x, w), atol=1e-3)
    hist = cand.arbiter_dispatch_histogram(target=cand.TARGET)
    assert all(v["degraded"] == 0 and v["no_candidate"] == 0 for v in hist.values())
    ms = cand.Gfx950MfmaGemmCandidate().measure_device_latency(cand.MatmulRegion("bfloat16"),
                                                               np.ones((256, 256), np.float32),
                                                               np.ones((256, 256), np.float32), reps=5, warmup=2)
    assert ms is not None and 0 < ms < 50


def test_bench_abi(lane):
    import ctypes
    ms = ctypes.c_double(0)
    lib = lane.load()
    assert lib.tessera_gfx950_gemm_bf16_bench(1024, 1024, 1024, 5, ctypes.byref(ms)) == 0
    assert 0 < ms.value < 100
    assert lib.tessera_gfx950_bench_last_timer_source() in (0, 1)
    assert "gfx950" in lane.device_name() and lane.device_cus() > 0


def test_measured_arbitration_on_device(lane):
    """Measure-at-first-miss on the real candidates: the verdict is keyed by the
    rocm:gfx950 device tag and reused from the cache on the second call."""
    from tessera_amd import autotune as at
    from tessera_amd import candidates as cand
    cand.register_all()
    rng = np.random.default_rng(0)
    A = (rng.standard_normal((256, 128)) * .1).astype(np.float32)
    B = (rng.standard_normal((128, 192)) * .1).astype(np.float32)
    region = cand.MatmulRegion(dtype="bfloat16")
    cache = at.MeasureCache()
    w = at.measured_arbitrate(region, cand.OP_MATMUL, cand.TARGET, A, B, dtype="bfloat16", cache=cache, reps=5,
                              warmup=1, timing=at.TIMING_DEVICE)
    assert w is not None and w.name == "gfx950_mfma_gemm"
    (key, rec), = cache.items()
    assert key[0] == "rocm:gfx950" and key[3] == (256, 256, 128) and rec.latency_ms > 0
    hits = cache.hits
    out, tag = at.run_measured_arbitrated(region, cand.OP_MATMUL, cand.TARGET, A, B, dtype="bfloat16", cache=cache,
                                          timing=at.TIMING_DEVICE)
    assert cache.hits == hits + 1 and tag == cand.GEMM_TAG
    assert np.allclose(out, region.reference(A, B), atol=5e-3)
    # the packaged corpus recommends the same winner for the headline GEMM bucket
    big = np.zeros((8192, 8192), np.float32)
    assert at.corpus_winner(region, cand.OP_MATMUL, cand.TARGET, big, big, dtype="bfloat16",
                            timing=at.TIMING_DEVICE) == "gfx950_mfma_gemm"
