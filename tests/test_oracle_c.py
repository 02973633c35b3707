"""Pins for the C restatement (oracle/oracle.c): it must agree with the numpy
oracle, with closed forms, and — where the reference's own x86 kernels were
compiled into oracle/_ref — with the reference itself.  No GPU."""
import numpy as np
import pytest

import c_oracle as co
import tessera_oracle as orc


def test_c_gemm_bf16_matches_numpy_and_reference():
    rng = np.random.default_rng(0)
    A = rng.standard_normal((37, 53)).astype(np.float32)
    B = rng.standard_normal((53, 29)).astype(np.float32)
    ab, bb = orc.f32_to_bf16_bits(A), orc.f32_to_bf16_bits(B)
    c = co.gemm_bf16_f32(ab, bb)
    assert orc.max_rel_err(c, orc.gemm_f64(A, B)) < 1e-6
    assert np.allclose(co.gemm_bf16_f64(ab, bb), orc.gemm_f64(A, B), rtol=1e-13)
    if co.ref() is not None:
        assert np.array_equal(c, co.ref_gemm_bf16(ab, bb))              # same k order -> same bits


def test_c_int8_gemm_exact():
    rng = np.random.default_rng(1)
    a = rng.integers(-128, 128, (19, 301)).astype(np.int8)
    b = rng.integers(-128, 128, (301, 23)).astype(np.int8)
    assert np.array_equal(co.gemm_s8s8_s32(a, b), a.astype(np.int64) @ b.astype(np.int64))
    if co.ref() is not None:
        a_pos = np.abs(a.astype(np.int16)).clip(0, 127).astype(np.int8)   # the u8 x s8 twin on the shared range
        assert np.array_equal(co.gemm_s8s8_s32(a_pos, b), co.ref_gemm_u8s8(a_pos.astype(np.uint8), b))


@pytest.mark.parametrize("Sq,Sk,causal", [(17, 17, True), (9, 30, True), (30, 9, True), (12, 20, False)])
def test_c_flash_attn_matches_numpy_and_reference(Sq, Sk, causal):
    rng = np.random.default_rng(2)
    q = rng.standard_normal((2, 4, Sq, 16)).astype(np.float32)
    k = rng.standard_normal((2, 2, Sk, 16)).astype(np.float32)
    v = rng.standard_normal((2, 2, Sk, 16)).astype(np.float32)
    o, lse = co.flash_attn_f32(q, k, v, 0.25, causal)
    ro, rl = orc.flash_attn_dense(q, k, v, scale=0.25, causal=causal)
    assert np.allclose(o, ro, atol=2e-6) and np.allclose(lse, rl, atol=2e-6)
    if co.ref() is not None:
        fo, fl = co.ref_flash_attn_lse(q, k, v, 0.25, causal)
        assert np.allclose(o, fo, atol=2e-6) and np.allclose(lse, fl, atol=2e-6)


def test_c_fpquant_matches_numpy_and_reference():
    rng = np.random.default_rng(3)
    x = np.concatenate([rng.standard_normal(50000) * 50, rng.standard_normal(50000) * 0.01,
                        [0.0, 448.0, -448.0, 1e9, 2.0 ** -9, 2.0 ** -10]]).astype(np.float32)
    g = co.fpquant_f32(x)
    assert np.array_equal(g, orc.fpquant_grid(x))
    if co.ref() is not None:
        assert np.array_equal(g, co.ref_fpquant(x))


@pytest.mark.parametrize("T,E,k,cap", [(200, 16, 4, 0), (333, 8, 2, 60), (64, 64, 8, 0)])
def test_c_router_matches_numpy(T, E, k, cap):
    lg = np.random.default_rng(T).standard_normal((T, E)).astype(np.float32)
    assert not orc.has_routing_ties(orc.router_probs(lg), k)
    tos, eos, cw, gs, go = co.moe_route(lg, k, True, cap)
    r = orc.route_tokens(lg, E, k, capacity=cap if cap > 0 else 10 ** 9)
    d = orc.plan_dispatch(r.assignment, r.weights, E)
    assert np.array_equal(tos, d.token_of_slot) and np.array_equal(eos, d.expert_of_slot)
    assert np.array_equal(gs, d.group_sizes) and np.array_equal(go, d.group_offsets)
    assert np.allclose(cw, d.combine_weights, rtol=2e-6)


def test_window_and_softcap_match_the_reference_kernel():
    """Sliding window (both forms) and logit soft cap of the numpy oracle against the
    reference's compiled CPU kernel."""
    if co.ref() is None:
        pytest.skip("compiled reference twins unavailable on this host")
    rng = np.random.default_rng(12)
    for (B, Hq, Hkv, Sq, Sk, D, causal, window, cap) in [
            (1, 2, 1, 40, 40, 16, True, 8, 0.0), (1, 2, 2, 24, 50, 16, True, 13, 0.0),
            (1, 1, 1, 33, 33, 8, False, 10, 0.0), (2, 4, 2, 20, 20, 16, True, 0, 3.0),
            (1, 2, 2, 31, 47, 16, True, 9, 5.0)]:
        q = rng.standard_normal((B, Hq, Sq, D)).astype(np.float32)
        k = rng.standard_normal((B, Hkv, Sk, D)).astype(np.float32)
        v = rng.standard_normal((B, Hkv, Sk, D)).astype(np.float32)
        o, lse = orc.flash_attn_dense(q, k, v, causal=causal, window=window, softcap=cap)
        ro, rl = co.ref_flash_attn_lse(q, k, v, 1.0 / np.sqrt(D), causal, window, cap)
        assert orc.max_rel_err(o, ro) <= 1e-5
        assert np.max(np.abs(lse - rl)) <= 1e-5


def test_additive_bias_matches_the_reference_kernel():
    """Additive attention bias of the numpy oracle (alone, with the causal mask, a
    window and a soft cap, where it is added after the cap) against the reference's
    compiled CPU kernel."""
    if co.ref() is None:
        pytest.skip("compiled reference twins unavailable on this host")
    rng = np.random.default_rng(13)
    for (B, Hq, Hkv, Sq, Sk, D, causal, window, cap) in [
            (1, 2, 1, 40, 40, 16, False, 0, 0.0), (2, 4, 2, 24, 50, 16, True, 0, 0.0),
            (1, 2, 2, 33, 33, 8, True, 10, 0.0), (1, 2, 2, 31, 47, 16, True, 0, 4.0)]:
        q = rng.standard_normal((B, Hq, Sq, D)).astype(np.float32)
        k = rng.standard_normal((B, Hkv, Sk, D)).astype(np.float32)
        v = rng.standard_normal((B, Hkv, Sk, D)).astype(np.float32)
        bias = (rng.standard_normal((B, Hq, Sq, Sk)) * 2).astype(np.float32)
        o, lse = orc.flash_attn_dense(q, k, v, causal=causal, window=window, softcap=cap, bias=bias)
        ro, rl = co.ref_flash_attn_lse(q, k, v, 1.0 / np.sqrt(D), causal, window, cap, bias=bias)
        assert orc.max_rel_err(o, ro) <= 1e-5
        assert np.max(np.abs(lse - rl)) <= 1e-5
        # a dropped bias would be seen: the biased result differs from the plain one
        assert orc.max_rel_err(o, orc.flash_attn_dense(q, k, v, causal=causal, window=window, softcap=cap)[0]) > 1e-2
