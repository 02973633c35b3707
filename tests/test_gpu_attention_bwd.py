"""Flash-attention backward on the MI355X (through the C ABI) against the oracle's
restatement of vjp_flash_attn.  Tolerance on dQ, dK, dV (max error over max
magnitude, against the f64 gradients of the same 16-bit inputs): 2e-3 for f16 and
5e-3 for bf16.  The kernels round P and dS to the storage dtype once before the
second products, an extra 2^-11 (f16) or 2^-9 (bf16) per term that the forward
does not have on dS; the reference's own budgets for this lane are 5e-3 (f16) and
3e-2 (bf16) (tests/unit/test_rocm_flash_attn_bwd_runtime_lane.py:126,147)."""
import numpy as np
import pytest

import tessera_oracle as orc
from tessera_amd import bf16 as b16
from tessera_amd import executors as ex
from tessera_amd import ops

pytestmark = pytest.mark.gpu
TOL = {"f16": 2e-3, "bf16": 5e-3}


def _store(x, st):
    return b16.from_float32(x) if st == "bf16" else x.astype(np.float16)


def _f32(x):
    return x.to_float32() if isinstance(x, b16.BF16Array) else np.asarray(x, np.float32)


def _inputs(B, Hq, Hkv, Sq, Sk, D, seed, st):
    rng = np.random.default_rng(seed)
    q = _store(rng.standard_normal((B, Hq, Sq, D)).astype(np.float32), st)
    k = _store(rng.standard_normal((B, Hkv, Sk, D)).astype(np.float32), st)
    v = _store(rng.standard_normal((B, Hkv, Sk, D)).astype(np.float32), st)
    do = _store(rng.standard_normal((B, Hq, Sq, D)).astype(np.float32), st)
    return do, q, k, v


CASES = [
    # B, Hq, Hkv, Sq, Sk, D, causal
    (1, 1, 1, 32, 32, 128, False), (1, 1, 1, 64, 64, 128, True),
    (2, 4, 2, 300, 300, 128, True), (1, 8, 2, 257, 511, 128, True),
    (1, 2, 2, 100, 77, 64, False), (1, 2, 1, 200, 333, 64, True), (1, 2, 2, 333, 200, 64, True),
    (1, 4, 4, 513, 129, 128, False), (1, 2, 2, 1, 129, 128, True),
    (1, 3, 3, 40, 40, 48, False), (1, 2, 1, 50, 60, 32, True),      # head dims served zero-padded to 64 / 128
    (1, 2, 1, 150, 203, 80, True), (1, 4, 2, 130, 130, 96, True), (2, 2, 2, 70, 90, 16, False),
    (1, 2, 2, 64, 64, 112, True),
    # above 128: dense products around an elementwise softmax kernel, per (batch, KV head) group
    (1, 2, 1, 40, 70, 160, True), (2, 4, 2, 200, 264, 256, True), (1, 6, 2, 130, 77, 192, False), (3, 2, 2, 65, 129, 256, True),
    (1, 8, 8, 333, 200, 144, True), (1, 4, 1, 1, 300, 256, True),
    # B * Hkv a multiple of 8: the XCD-aware workgroup order
    (2, 8, 4, 200, 264, 128, True), (1, 16, 8, 130, 130, 64, True), (2, 24, 8, 70, 330, 128, False),
]


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,causal", CASES)
@pytest.mark.parametrize("st", ["bf16", "f16"])
def test_attention_backward_matches_oracle(lane, B, Hq, Hkv, Sq, Sk, D, causal, st):
    do, q, k, v = _inputs(B, Hq, Hkv, Sq, Sk, D, 23, st)
    rq, rk, rv = orc.flash_attn_backward(_f32(do), _f32(q), _f32(k), _f32(v), causal=causal)
    dq, dk, dv = ops.flash_attn_backward(do, q, k, v, causal=causal)
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    for got, ref, name in ((dq, rq, "dQ"), (dk, rk, "dK"), (dv, rv, "dV")):
        assert not np.isnan(got).any(), name
        assert orc.max_rel_err(got, ref) <= TOL[st], name


@pytest.mark.parametrize("scale", [0.25, -0.05, 1e-3, 0.0])
def test_attention_backward_scales(lane, scale):
    """The kernels fold -LSE / scale into their accumulators; a negative or tiny
    scale goes the same way, a zero one (uniform P over the visible keys) is served
    by the kernels that do not divide by it."""
    do, q, k, v = _inputs(1, 4, 2, 130, 200, 128, 41, "f16")
    ref = orc.flash_attn_backward(_f32(do), _f32(q), _f32(k), _f32(v), scale=scale, causal=True)
    got = ops.flash_attn_backward(do, q, k, v, scale=scale, causal=True)
    for g, r, name in zip(got, ref, ("dQ", "dK", "dV")):
        assert not np.isnan(g).any(), name
        if np.abs(r).max() == 0:
            assert np.abs(g).max() <= 1e-6, name
        else:
            assert orc.max_rel_err(g, r) <= TOL["f16"], name


def test_attention_backward_closed_forms(lane):
    """One key: P = 1 for every query, so dV = sum of dO rows, dQ = dK = 0.
    dO = 0 gives all-zero gradients."""
    do, q, k, v = _inputs(1, 2, 2, 96, 1, 128, 3, "bf16")
    dq, dk, dv = ops.flash_attn_backward(do, q, k, v)
    assert np.allclose(dv[:, :, 0], do.to_float32().sum(axis=2), rtol=1e-3, atol=1e-3)
    assert np.abs(dq).max() <= 1e-6 and np.abs(dk).max() <= 1e-4
    do0 = b16.from_float32(np.zeros((1, 2, 96, 128), np.float32))
    _, qq, kk, vv = _inputs(1, 2, 2, 96, 80, 128, 4, "bf16")
    for g in ops.flash_attn_backward(do0, qq, kk, vv, causal=True):
        assert np.all(g == 0)


def test_gqa_backward_sums_over_the_group(lane):
    do, q, k, v = _inputs(1, 4, 2, 128, 128, 128, 31, "bf16")
    dq, dk, dv = ops.flash_attn_backward(do, q, k, v, causal=True)
    rep = lambda x: b16.from_float32(np.repeat(x.to_float32(), 2, axis=1))
    dq2, dk2, dv2 = ops.flash_attn_backward(do, q, rep(k), rep(v), causal=True)
    assert np.array_equal(dq, dq2)
    assert orc.max_rel_err(dk, dk2.reshape(1, 2, 2, 128, 128).sum(axis=2)) <= 1e-6
    assert orc.max_rel_err(dv, dv2.reshape(1, 2, 2, 128, 128).sum(axis=2)) <= 1e-6


def test_backward_headline_shape_properties(lane):
    """B4 Hq32 Hkv8 S4096 D128 causal: too large for a dense CPU gradient; check the
    batch/head slices a CPU can afford and linearity in dO."""
    B, Hq, Hkv, S, D = 4, 32, 8, 4096, 128
    do, q, k, v = _inputs(B, Hq, Hkv, S, S, D, 41, "bf16")
    dq, dk, dv = ops.flash_attn_backward(do, q, k, v, causal=True)
    assert not (np.isnan(dq).any() or np.isnan(dk).any() or np.isnan(dv).any())
    b, g = 2, 5                                           # one KV group: 4 query heads
    sl = slice(4 * g, 4 * g + 4)
    rq, rk, rv = orc.flash_attn_backward(_f32(do)[b:b + 1, sl], _f32(q)[b:b + 1, sl], _f32(k)[b:b + 1, g:g + 1],
                                         _f32(v)[b:b + 1, g:g + 1], causal=True)
    assert orc.max_rel_err(dq[b:b + 1, sl], rq) <= TOL["bf16"]
    assert orc.max_rel_err(dk[b:b + 1, g:g + 1], rk) <= TOL["bf16"]
    assert orc.max_rel_err(dv[b:b + 1, g:g + 1], rv) <= TOL["bf16"]
    # gradients are linear in dO: doubling dO doubles them exactly (power of two)
    do2 = b16.from_float32(2.0 * do.to_float32())
    dq2, dk2, dv2 = ops.flash_attn_backward(do2, q, k, v, causal=True)
    assert np.array_equal(dq2, 2 * dq) and np.array_equal(dk2, 2 * dk) and np.array_equal(dv2, 2 * dv)


@pytest.mark.parametrize("D", [48, 80, 128, 256])
def test_backward_with_saved_forward_results_equals_recompute(lane, D):
    """The device entry point fed the forward's own O and log-sum-exp gives the bits the
    recomputing host entry gives (the padded widths take the same path either way)."""
    import ctypes
    B, Hq, Hkv, Sq, Sk = 1, 4, 2, 150, 170
    do, q, k, v = _inputs(B, Hq, Hkv, Sq, Sk, D, 77, "bf16")
    want = ops.flash_attn_backward(do, q, k, v, causal=True)
    lib = lane.load()
    up = lambda a: lane.DeviceBuffer.from_host(np.ascontiguousarray(np.asarray(a, np.uint16)))
    ddo, dq_, dk_, dv_ = up(do), up(q), up(k), up(v)
    o, lse = lane.DeviceBuffer(B * Hq * Sq * D * 4), lane.DeviceBuffer(B * Hq * Sq * 4)
    gq, gk, gv = lane.DeviceBuffer(B * Hq * Sq * D * 4), lane.DeviceBuffer(B * Hkv * Sk * D * 4), lane.DeviceBuffer(B * Hkv * Sk * D * 4)
    sc = ctypes.c_float(D ** -0.5)
    lane.check(lib.tessera_gfx950_flash_attn_gqa_bf16_dev(dq_.ptr, dk_.ptr, dv_.ptr, o.ptr, lse.ptr, B, Hq, Hkv, Sq, Sk, D,
                                                          sc, 1, 0, None), "fwd")
    lane.check(lib.tessera_gfx950_flash_attn_bwd_bf16_dev(ddo.ptr, dq_.ptr, dk_.ptr, dv_.ptr, o.ptr, lse.ptr, gq.ptr, gk.ptr,
                                                          gv.ptr, B, Hq, Hkv, Sq, Sk, D, sc, 1, None), "bwd")
    lane.synchronize()
    got = (gq.download((B, Hq, Sq, D), np.float32), gk.download((B, Hkv, Sk, D), np.float32),
           gv.download((B, Hkv, Sk, D), np.float32))
    for g, w in zip(got, want):
        assert np.array_equal(g, w)


def test_backward_executor_and_bad_shapes(lane):
    do, q, k, v = _inputs(1, 2, 1, 64, 64, 64, 8, "f16")
    art = ex.make_artifact("tessera.flash_attn_bwd", ["dO", "Q", "K", "V"], ["dO", "Q", "K", "V"],
                           "gfx950_flash_attn_bwd", kwargs={"causal": True})
    res = ex.launch(art, (do, q, k, v))
    assert res["ok"], res
    dq, dk, dv = res["output"]
    rq, rk, rv = orc.flash_attn_backward(_f32(do), _f32(q), _f32(k), _f32(v), causal=True)
    t = TOL["f16"]
    assert orc.max_rel_err(dq, rq) <= t and orc.max_rel_err(dk, rk) <= t and orc.max_rel_err(dv, rv) <= t
    with pytest.raises(ValueError):
        ops.flash_attn_backward(do, q, k, v[:, :, :32])
    with pytest.raises(ValueError):
        ops.flash_attn_backward(do[..., :24], q[..., :24], k[..., :24], v[..., :24])
    bad = ex.make_artifact("tessera.flash_attn_bwd", ["dO", "Q", "K", "V"], ["dO", "Q", "K", "V"],
                           "gfx950_flash_attn_bwd", kwargs={"window": 16})
    assert not ex.launch(bad, (do, q, k, v))["ok"]
