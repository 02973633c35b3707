"""Fused matmul epilogue (bias + activation) and gated projection on the MI355X,
through the C ABI, against the oracle's restatement of FusedRegion.reference /
GatedMatmulRegion.reference.  Tolerance: 2e-3 normwise against the f64 result on
the same 16-bit operands (f32 accumulate, f32 output)."""
import numpy as np
import pytest

import standin_host as host
import tessera_oracle as orc
from tessera_amd import bf16 as b16
from tessera_amd import candidates as cand
from tessera_amd import executors as ex
from tessera_amd import ops

pytestmark = pytest.mark.gpu
TOL = 2e-3
ACTS = ["none", "relu", "gelu", "silu", "sigmoid", "tanh"]


def _store(x, st):
    return b16.from_float32(x) if st == "bf16" else x.astype(np.float16)


def _f32(x):
    return x.to_float32() if isinstance(x, b16.BF16Array) else np.asarray(x, np.float32)


# tile kernel (aligned), split-K decode shape, single-split decode shape (epilogue in
# the streaming kernel itself), ragged generic path
SHAPES = [(512, 768, 256), (300, 520, 136), (16, 1024, 4096), (6, 16384, 512), (8, 1024, 2048), (8, 16, 12),
          (37, 29, 50)]


@pytest.mark.parametrize("M,N,K", SHAPES)
@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("with_bias", [False, True])
def test_fused_gemm_matches_oracle(lane, M, N, K, act, with_bias):
    rng = np.random.default_rng(M * 7 + N)
    st = "bf16" if (M + len(act)) % 2 else "f16"
    a = _store((rng.standard_normal((M, K)) * 2 / np.sqrt(K)).astype(np.float32), st)
    b = _store(rng.standard_normal((K, N)).astype(np.float32), st)
    bias = rng.standard_normal(N).astype(np.float32) if with_bias else None
    chain = (("bias",) if with_bias else ()) + ((act,) if act != "none" else ())
    ref = orc.fused_epilogue(_f32(a), _f32(b), bias, chain)
    got = ops.fused_gemm(a, b, bias, act)
    assert got.dtype == np.float32 and got.shape == (M, N)
    assert orc.max_rel_err(got, ref) <= TOL


def test_fused_gemm_closed_forms(lane):
    """relu of a non-positive product is exactly zero; a zero bias and no
    activation reproduce the bare product bit for bit."""
    rng = np.random.default_rng(3)
    a = b16.from_float32(np.abs(rng.standard_normal((64, 128))).astype(np.float32))
    b = b16.from_float32(-np.abs(rng.standard_normal((128, 256))).astype(np.float32))
    assert np.all(ops.fused_gemm(a, b, None, "relu") == 0.0)
    plain = ops.gemm(a, b, out="f32")
    assert np.array_equal(ops.fused_gemm(a, b, np.zeros(256, np.float32), "none"), plain)
    assert np.array_equal(ops.fused_gemm(a, b, np.full(256, 1.5, np.float32), "none"), plain + np.float32(1.5))


@pytest.mark.parametrize("M,H,K", [(512, 640, 256), (8, 16, 12), (130, 264, 72), (256, 128, 1024),
                                   # few rows: two weight-streaming products and a gate kernel
                                   (16, 2048, 4096), (128, 1024, 520), (1, 16384, 1024), (100, 264, 72)])
@pytest.mark.parametrize("act", ["silu", "gelu", "relu", "sigmoid", "tanh"])
def test_gated_gemm_matches_oracle(lane, M, H, K, act):
    rng = np.random.default_rng(H + K)
    st = "bf16" if (H + len(act)) % 2 else "f16"
    a = _store((rng.standard_normal((M, K)) / np.sqrt(K)).astype(np.float32), st)
    wg = _store(rng.standard_normal((K, H)).astype(np.float32), st)
    wu = _store(rng.standard_normal((K, H)).astype(np.float32), st)
    ref = orc.gated_matmul(_f32(a), _f32(wg), _f32(wu), act)
    got = ops.gated_gemm(a, wg, wu, act)
    assert got.shape == (M, H)
    assert orc.max_rel_err(got, ref) <= TOL


def test_gated_gemm_equals_two_products(lane):
    """The gated kernel's two accumulators are the bare products: with the up
    weight a 0/1 selector the result is silu(gate) gathered."""
    rng = np.random.default_rng(9)
    M, K, H = 256, 128, 256
    a = b16.from_float32(rng.standard_normal((M, K)).astype(np.float32) / 8)
    wg = b16.from_float32(rng.standard_normal((K, H)).astype(np.float32))
    gate = ops.gemm(a, wg, out="f32")
    ones_col = np.zeros((K, H), np.float32)
    ones_col[0, :] = 1.0
    a1 = a.to_float32().copy()
    a1[:, 0] = 1.0                                   # (A Wu) == 1 everywhere
    a1b = b16.from_float32(a1)
    gate1 = ops.gemm(a1b, wg, out="f32")
    got = ops.gated_gemm(a1b, wg, b16.from_float32(ones_col), "silu")
    ref = gate1 / (1.0 + np.exp(-gate1.astype(np.float64)))
    assert orc.max_rel_err(got, ref) <= 1e-5
    assert gate.shape == got.shape


def test_fused_and_gated_candidates_pass_the_gate(lane):
    api = host.CandidateHost()
    cand.register(api)
    for epi in [("bias", "relu"), ("gelu",), ("bias",), ("bias", "silu")]:
        region = host.FusedRegion(epilogue=epi, storage_dtype="bf16")
        winner = api.arbitrate(region, api.OP_FUSED_REGION, cand.TARGET)
        assert winner is not None and winner.name == "gfx950_mfma_fused_gemm"
    # not representable: activation before bias, residual
    assert api.arbitrate(host.FusedRegion(epilogue=("relu", "bias")), api.OP_FUSED_REGION, cand.TARGET) is None
    assert api.arbitrate(host.FusedRegion(epilogue=("relu",), residual=True), api.OP_FUSED_REGION,
                         cand.TARGET) is None
    g = host.GatedMatmulRegion("silu", "f16")
    winner = api.arbitrate(g, api.OP_GATED_MATMUL, cand.TARGET)
    assert winner is not None and winner.name == "gfx950_mfma_gated_gemm"
    rng = np.random.default_rng(0)
    A = (rng.standard_normal((64, 32)) * .3).astype(np.float32)
    Wg = (rng.standard_normal((32, 48)) * .3).astype(np.float32)
    Wu = (rng.standard_normal((32, 48)) * .3).astype(np.float32)
    out, tag = api.run(g, api.OP_GATED_MATMUL, cand.TARGET, A, Wg, Wu)
    assert tag == cand.GATED_TAG
    assert np.allclose(out, g.reference(A, Wg, Wu), atol=5e-3)


def test_executor_fused_epilogue_op(lane):
    rng = np.random.default_rng(1)
    a = (rng.standard_normal((48, 64)) / 8).astype(np.float16)
    b = rng.standard_normal((64, 40)).astype(np.float16)
    bias = rng.standard_normal(40).astype(np.float32)
    art = ex.make_artifact("tessera.fused_epilogue", ["a", "b", "bias"], ["a", "b", "bias"], "gfx950_gemm",
                           kwargs={"activation": "gelu"})
    res = ex.launch(art, (a, b, bias))
    assert res["ok"], res
    ref = orc.fused_epilogue(a.astype(np.float32), b.astype(np.float32), bias, ("bias", "gelu"))
    assert orc.max_rel_err(res["output"], ref) <= TOL
    bad = ex.make_artifact("tessera.fused_epilogue", ["a", "b"], ["a", "b"], "gfx950_gemm",
                           kwargs={"activation": "softmax"})
    res = ex.launch(bad, (a, b))
    assert not res["ok"] and res["runtime_status"] == "invalid_artifact"
    ai = np.ones((8, 16), np.int8)
    res = ex.launch(ex.make_artifact("tessera.matmul", ["a", "b"], ["a", "b"], "gfx950_gemm",
                                     kwargs={"activation": "relu"}), (ai, np.ones((16, 8), np.int8)))
    assert not res["ok"] and "float-only" in res["reason"]


@pytest.mark.parametrize("act", ["linear", "gelu", "relu", "silu"])
def test_gemm_epilogue_keyword(lane, act):
    """ops.gemm(A, B, epilogue={"bias", "activation"}): the reference applies the epilogue to the
    f32 product and rounds to the storage dtype afterwards."""
    rng = np.random.default_rng(len(act))
    a = b16.from_float32(rng.standard_normal((3, 70, 96)).astype(np.float32))       # leading dims fold into M
    b = b16.from_float32((rng.standard_normal((96, 136)) / 8).astype(np.float32))
    bias = rng.standard_normal(136).astype(np.float32)
    chain = ["bias"] + ([] if act == "linear" else [act])
    ref = orc.fused_epilogue(a.to_float32().reshape(-1, 96), b.to_float32(), bias, chain).reshape(3, 70, 136)
    got32 = ops.gemm(a, b, epilogue={"bias": bias, "activation": act}, out="f32")
    assert got32.shape == (3, 70, 136) and orc.max_rel_err(got32, ref) <= 2e-5
    got = ops.gemm(a, b, epilogue={"bias": bias, "activation": act})
    assert np.array_equal(got.to_float32(), orc.round_to_storage(got32, "bf16"))
    assert np.array_equal(np.asarray(ops.gemm(a, b, epilogue={}), np.uint16), np.asarray(ops.gemm(a, b), np.uint16))
    with pytest.raises(NotImplementedError):
        ops.gemm(a, b, epilogue={"residual": np.zeros((3, 70, 136), np.float32)})
