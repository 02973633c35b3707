"""The reference's plugin seams on the MI355X: executors through ``launch`` and
candidates through the arbiter run real kernels (never a reference tag) and
match the oracle."""
import numpy as np
import pytest

import standin_host as host
import tessera_oracle as orc
from tessera_amd import bf16 as b16
from tessera_amd import candidates as cand
from tessera_amd import executors as ex
from tessera_amd import install as inst
from tessera_amd import native_launcher as nl
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
    """The candidates, registered into a host through install(), pass the host's gate
    on real kernels and win its arbitration; nothing is ever tagged as a host-side run."""
    api = host.CandidateHost()
    inst.install(api)
    rng = np.random.default_rng(5)
    gemm = api.candidates_for(cand.TARGET, api.OP_MATMUL)[0]
    for dtype in ("bfloat16", "float16"):
        region = host.MatmulRegion(dtype)
        assert api.verify_candidate(gemm, region)
        A = (rng.standard_normal((64, 96)) * .4).astype(np.float32)
        B = (rng.standard_normal((96, 40)) * .4).astype(np.float32)
        out, tag = api.run(region, api.OP_MATMUL, cand.TARGET, A, B)
        assert tag == cand.GEMM_TAG and np.allclose(out, region.reference(A, B), atol=1e-3)
    region = host.MatmulRegion("bfloat16", transpose_a=True, transpose_b=True)
    A = (rng.standard_normal((96, 64)) * .4).astype(np.float32)       # raw (K, M)
    B = (rng.standard_normal((40, 96)) * .4).astype(np.float32)       # raw (N, K)
    out, tag = api.run(region, api.OP_MATMUL, cand.TARGET, A, B)
    assert tag == cand.GEMM_TAG and np.allclose(out, region.reference(A, B), atol=1e-3)
    for causal in (False, True):
        att = host.AttentionRegion(scale=0.25, causal=causal, storage_dtype="bf16")
        Q, K, V = ((rng.standard_normal((48, 32)) * .5).astype(np.float32) for _ in range(3))
        out, tag = api.run(att, api.OP_ATTENTION, cand.TARGET, Q, K, V)
        assert tag == cand.ATTN_TAG and np.allclose(out, att.reference(Q, K, V), atol=5e-3)
    gg = cand.GroupedGemmRegion((10, 0, 30), "bfloat16")
    x = (rng.standard_normal((40, 64)) * .4).astype(np.float32)
    w = (rng.standard_normal((3, 64, 32)) * .4).astype(np.float32)
    out, tag = api.run(gg, cand.OP_GROUPED_GEMM, cand.TARGET, x, w)
    assert tag == cand.GROUPED_TAG and np.allclose(out, gg.reference(x, w), atol=1e-3)
    fr = host.FusedRegion(("bias", "gelu"), storage_dtype="bf16")
    a, b, bias = rng.standard_normal((40, 64)) * .3, rng.standard_normal((64, 48)) * .3, rng.standard_normal(48)
    out, tag = api.run(fr, api.OP_FUSED_REGION, cand.TARGET, a, b, bias)
    assert tag == cand.FUSED_TAG and np.allclose(out, fr.reference(a, b, bias), atol=2e-2)
    gr = host.GatedMatmulRegion("silu", "bf16")
    out, tag = api.run(gr, api.OP_GATED_MATMUL, cand.TARGET, a, b, b[:, ::-1].copy())
    assert tag == cand.GATED_TAG and np.allclose(out, gr.reference(a, b, b[:, ::-1]), atol=2e-2)
    assert len(api.log) == 8 and all(name is not None and t not in api.NOT_A_KERNEL for _, _, name, t in api.log)
    ms = gemm.measure_device_latency(host.MatmulRegion("bfloat16"), np.ones((256, 256), np.float32),
                                     np.ones((256, 256), np.float32), reps=5, warmup=2)
    assert ms is not None and 0 < ms < 50


def test_installed_lane_is_reached_through_the_hosts_launch(lane):
    matrix = host.MatrixHost()
    runtime = host.RuntimeHost(matrix)
    inst.install(execution_matrix=matrix, executor_table=runtime)
    rng = np.random.default_rng(9)
    A = (rng.standard_normal((70, 96)) * .5).astype(np.float16)
    B = (rng.standard_normal((96, 50)) * .5).astype(np.float16)
    art = ex.make_artifact("tessera.matmul", ["a", "b"], ["a", "b"], "gfx950_gemm")
    res = runtime.launch(art, (A, B))
    assert res["ok"] and res["execution_kind"] == "native_gpu" and res["compiler_path"] == "gfx950_gemm"
    assert orc.max_rel_err(res["output"], A.astype(np.float64) @ B.astype(np.float64)) <= 1e-5


def _typed(abi, entry, names, provenance=None):
    return host.Descriptor(abi, entry, tuple(host.Binding(n, i) for i, n in enumerate(names)), provenance or {})


def test_typed_descriptor_launches(lane):
    """The third seam: artifacts with a native image and a launch descriptor reach the lane
    through the hook install() registers for the exact target."""
    runtime = host.NativeLauncherHost()
    assert inst.install(native_launchers=runtime)["native_launcher"] == "rocm_gfx950"
    image = host.Image("rocm_gfx950", "shared_object")
    rng = np.random.default_rng(11)
    # matmul, f16 and bf16 -> f32
    A = (rng.standard_normal((70, 96)) * .5).astype(np.float16)
    B = (rng.standard_normal((96, 50)) * .5).astype(np.float16)
    out = np.zeros((70, 50), np.float32)
    res = runtime.launch_descriptor(image, _typed(nl.MATMUL_F16_F32_ABI, "tessera_gfx950_gemm_f16", ("A", "B", "O")),
                                    {"A": A, "B": B, "O": out}, {"M": 70, "N": 50, "K": 96})
    assert res["ok"] and res["output"] is out
    assert orc.max_rel_err(out, A.astype(np.float64) @ B.astype(np.float64)) <= 1e-5
    Ab, Bb = b16.from_float32(A.astype(np.float32)), b16.from_float32(B.astype(np.float32))
    res = runtime.launch_descriptor(image, _typed(nl.MATMUL_BF16_F32_ABI, "tessera_gfx950_gemm_bf16", ("A", "B", "O")),
                                    {"A": Ab, "B": Bb, "O": out}, {"M": 70, "N": 50, "K": 96})
    assert res["ok"]
    assert orc.max_rel_err(out, Ab.to_float32().astype(np.float64) @ Bb.to_float32().astype(np.float64)) <= 1e-5
    # a descriptor whose scalars disagree with the arrays is refused before the device is touched
    res = runtime.launch_descriptor(image, _typed(nl.MATMUL_F16_F32_ABI, "tessera_gfx950_gemm_f16", ("A", "B", "O")),
                                    {"A": A, "B": B, "O": out}, {"M": 70, "N": 50, "K": 95})
    assert not res["ok"] and res["runtime_status"] == "device_error" and "disagree" in res["reason"]
    # attention: GQA, causal, a left window of 23 keys (band width 24)
    b_, hq, hkv, sq, sk, d = 1, 4, 2, 80, 112, 64
    Q = (rng.standard_normal((b_, hq, sq, d)) * .5).astype(np.float16)
    K = (rng.standard_normal((b_, hkv, sk, d)) * .5).astype(np.float16)
    V = (rng.standard_normal((b_, hkv, sk, d)) * .5).astype(np.float16)
    O = np.zeros((b_, hq, sq, d), np.float32)
    prov = {"shape": [b_, hq, hkv, sq, sk, d, d], "scale": 0.125, "causal": True, "gqa": True, "kv_ratio": 2,
            "window_left": 23, "softcap": 0.0, "dropout_p": 0.0, "bias": False}
    res = runtime.launch_descriptor(image, _typed(nl.ATTN_F16_ABI, "tessera_gfx950_flash_attn_ext_f16",
                                                  ("Q", "K", "V", "O"), prov), {"Q": Q, "K": K, "V": V, "O": O}, {})
    assert res["ok"], res
    ref, _ = orc.flash_attn_dense(Q, K, V, 0.125, True, window=24)
    assert orc.max_rel_err(O, ref) <= 2e-3
    # MoE dispatch: an exact f32 gather
    x = rng.standard_normal((33, 40)).astype(np.float32)
    token = rng.integers(0, 33, 57).astype(np.int32)
    y = np.zeros((57, 40), np.float32)
    res = runtime.launch_descriptor(image, _typed(nl.MOE_DISPATCH_F32_ABI, "tessera_gfx950_moe_dispatch", ("X", "Token", "O")),
                                    {"X": x, "Token": token, "O": y}, {"T": 33, "S": 57, "H": 40})
    assert res["ok"] and np.array_equal(y, x[token])
    # another target's image, or another format, is not this lane's
    assert runtime.launch_descriptor(host.Image("rocm_gfx1151", "hsaco"), _typed(nl.MATMUL_F16_F32_ABI, "k", ("A",)),
                                     {}, {})["runtime_status"] == "unimplemented"


def test_bench_abi(lane):
    import ctypes
    ms = ctypes.c_double(0)
    lib = lane.load()
    assert lib.tessera_gfx950_gemm_bf16_bench(1024, 1024, 1024, 5, ctypes.byref(ms)) == 0
    assert 0 < ms.value < 100
    assert lib.tessera_gfx950_bench_last_timer_source() in (0, 1)
    # the f16 form carries the parameter list of tessera_rocm_wmma_gemm_f16_bench (mt, nt before avg_ms)
    assert lib.tessera_gfx950_gemm_f16_bench(1024, 1024, 1024, 5, 4, 2, ctypes.byref(ms)) == 0
    assert 0 < ms.value < 100 and lib.tessera_gfx950_bench_last_timer_source() in (0, 1)
    assert lib.tessera_gfx950_gemm_f16_bench(1024, 1024, 1024, 5, 0, 2, ctypes.byref(ms)) == 1
    assert lib.tessera_gfx950_bench_last_timer_source() == -1
    assert "gfx950" in lane.device_name() and lane.device_cus() > 0
    # the attention forward's bench entry: a failed call resets the timer source, a good one sets it
    assert lib.tessera_gfx950_flash_attn_bf16_bench(1, 4, 3, 64, 64, 128, 1, 3, ctypes.byref(ms)) == 1     # Hq % Hkv
    assert lib.tessera_gfx950_bench_last_timer_source() == -1
    assert lib.tessera_gfx950_flash_attn_bf16_bench(2, 8, 2, 1024, 1024, 128, 1, 5, ctypes.byref(ms)) == 0
    assert 0 < ms.value < 100 and lib.tessera_gfx950_bench_last_timer_source() in (0, 1)


def test_tuning_on_device(lane):
    """Measure at the first miss on the real candidates: the verdict is keyed by the
    rocm:gfx950 device tag and reused on the second call."""
    from tessera_amd import autotune as at
    api = host.CandidateHost()
    cand.register(api)
    rng = np.random.default_rng(0)
    A = (rng.standard_normal((256, 128)) * .1).astype(np.float32)
    B = (rng.standard_normal((128, 192)) * .1).astype(np.float32)
    region = host.MatmulRegion(dtype="bfloat16")
    corpus = at.Corpus()
    w = at.tune(api, region, api.OP_MATMUL, cand.TARGET, A, B, dtype="bfloat16", corpus=corpus, reps=5, warmup=1,
                timing="device")
    assert w is not None and w.name == "gfx950_mfma_gemm"
    ((key, verdict),) = list(corpus)
    assert key.device == "rocm:gfx950" and key.bucket == (256, 256, 128) and verdict.latency_ms > 0
    found = corpus.found
    out, tag = at.run_tuned(api, region, api.OP_MATMUL, cand.TARGET, A, B, dtype="bfloat16", corpus=corpus,
                            timing="device")
    assert corpus.found == found + 1 and tag == cand.GEMM_TAG
    assert np.allclose(out, region.reference(A, B), atol=5e-3)
    # the packaged corpus recommends the same winner for the headline GEMM bucket
    big = np.zeros((8192, 8192), np.float32)
    packaged = at.Corpus()
    packaged.absorb_file(at.PACKAGED)
    assert at.recommended(api, region, api.OP_MATMUL, cand.TARGET, big, big, corpus=packaged, dtype="bfloat16",
                          timing="device") == "gfx950_mfma_gemm"


def test_c_level_launcher_runs_the_kernels(lane):
    """The tsrGpuLauncherFn entry point (the C runtime's launch bridge,
    src/runtime/include/tessera/tessera_runtime.h:81-99): kernel names on target
    `rocm_gfx950` over ordered host buffers and dims; results equal the direct calls."""
    import ctypes
    from test_abi_and_host import launch_params
    lib = lane.load()
    fn = lib.tessera_gfx950_gpu_launcher
    rng = np.random.default_rng(77)
    M, N, K = 200, 328, 264
    a = np.asarray(b16.from_float32((rng.standard_normal((M, K)) * 0.5).astype(np.float32)), np.uint16)
    b = np.asarray(b16.from_float32((rng.standard_normal((K, N)) * 0.5).astype(np.float32)), np.uint16)
    d = np.zeros((M, N), np.float32)
    prm, keep = launch_params([a, b, d], [M, N, K])
    assert fn(b"rocm_gfx950", b"tessera_gfx950_gemm_bf16", ctypes.byref(prm), None) == 0
    want = ops.gemm(a.view(b16.BF16Array), b.view(b16.BF16Array), out="f32")
    assert np.array_equal(d, want)
    ref = a.view(b16.BF16Array).to_float32().astype(np.float64) @ b.view(b16.BF16Array).to_float32().astype(np.float64)
    assert orc.max_rel_err(d, ref) <= 1e-5
    # batched, f16
    Bt = 3
    af = (rng.standard_normal((Bt, 64, 40)) * 0.5).astype(np.float16)
    bf = (rng.standard_normal((Bt, 40, 72)) * 0.5).astype(np.float16)
    df = np.zeros((Bt, 64, 72), np.float32)
    prm, keep = launch_params([af, bf, df], [Bt, 64, 72, 40])
    assert fn(b"rocm", b"tessera_gfx950_batched_gemm_f16", ctypes.byref(prm), None) == 0
    assert orc.max_rel_err(df, af.astype(np.float64) @ bf.astype(np.float64)) <= 1e-5
    # attention with the default scale 1/sqrt(D), causal
    B, H, Sq, Sk, D = 1, 2, 96, 160, 64
    q, k, v = (np.asarray(b16.from_float32(rng.standard_normal(s).astype(np.float32)), np.uint16)
               for s in ((B, H, Sq, D), (B, H, Sk, D), (B, H, Sk, D)))
    o = np.zeros((B, H, Sq, D), np.float32)
    prm, keep = launch_params([q, k, v, o], [B, H, Sq, Sk, D, 1])
    assert fn(b"rocm_gfx950", b"tessera_gfx950_flash_attn_bf16", ctypes.byref(prm), None) == 0
    want = ops.flash_attn(q.view(b16.BF16Array), k.view(b16.BF16Array), v.view(b16.BF16Array), causal=True, out="f32")
    assert np.array_equal(o, np.asarray(want, np.float32))

