"""Chains of ops on device-resident handles (tessera_amd.resident): every intermediate
stays in HBM, the kernels are the ones the host-pointer ops run, so the results are the
same bits; each chain is also checked against the oracle."""
import numpy as np
import pytest

import tessera_oracle as orc
from tessera_amd import bf16 as b16
from tessera_amd import ops
from tessera_amd import resident as rs

pytestmark = pytest.mark.gpu


def test_projection_then_attention_chain(lane):
    """x @ Wq / Wk / Wv -> attention -> @ Wo with no host hop in between."""
    B, S, Hq, Hkv, D, E = 2, 192, 4, 2, 64, 256
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((B, S, E)) * 0.5).astype(np.float32)
    wq = (rng.standard_normal((E, Hq * D)) / 16).astype(np.float32)
    wk, wv = ((rng.standard_normal((E, Hkv * D)) / 16).astype(np.float32) for _ in range(2))
    wo = (rng.standard_normal((Hq * D, E)) / 16).astype(np.float32)
    xb, wqb, wkb, wvb, wob = (b16.from_float32(a) for a in (x, wq, wk, wv, wo))
    dx, dwq, dwk, dwv, dwo = (rs.DeviceArray.from_host(a) for a in (xb, wqb, wkb, wvb, wob))
    q = rs.gemm(dx, dwq)                                           # (B, S, Hq*D) bf16, resident
    k, v = rs.gemm(dx, dwk), rs.gemm(dx, dwv)
    assert q.shape == (B, S, Hq * D) and q.dtype == "bf16"
    # head split: the host-side reference does the same transposition on downloaded copies
    heads = lambda t, h: b16.from_bits(np.ascontiguousarray(
        np.asarray(t.to_host(), np.uint16).reshape(B, S, h, D).transpose(0, 2, 1, 3)))
    q4, k4, v4 = (rs.DeviceArray.from_host(heads(t, h)) for t, h in ((q, Hq), (k, Hkv), (v, Hkv)))
    o, lse = rs.flash_attn(q4, k4, v4, causal=True, return_lse=True)
    merged = rs.DeviceArray.from_host(b16.from_bits(np.ascontiguousarray(
        np.asarray(o.to_host(), np.uint16).transpose(0, 2, 1, 3).reshape(B, S, Hq * D))))
    y = rs.gemm(merged, dwo, out="f32").to_host()
    # the same chain through the host-pointer ops: identical bits
    hq, hk, hv = ops.gemm(xb, wqb), ops.gemm(xb, wkb), ops.gemm(xb, wvb)
    assert np.array_equal(np.asarray(hq, np.uint16), np.asarray(q.to_host(), np.uint16))
    t4 = lambda t, h: b16.from_bits(np.ascontiguousarray(np.asarray(t, np.uint16).reshape(B, S, h, D).transpose(0, 2, 1, 3)))
    ho, hl = ops.gqa_attention(t4(hq, Hq), t4(hk, Hkv), t4(hv, Hkv), causal=True, return_lse=True)
    assert np.array_equal(np.asarray(ho, np.uint16), np.asarray(o.to_host(), np.uint16))
    assert np.array_equal(hl, lse.to_host())
    # and the oracle on the attention stage
    ro, rl = orc.flash_attn_dense(t4(hq, Hq).to_float32(), t4(hk, Hkv).to_float32(), t4(hv, Hkv).to_float32(), causal=True)
    assert orc.max_rel_err(o.to_host().to_float32(), ro) <= 2e-3 + 2.0 ** -8
    assert y.shape == (B, S, E) and np.isfinite(y).all()
    ref_y = orc.gemm_f64(merged.to_host().to_float32().reshape(B * S, -1), wob.to_float32())
    assert orc.max_rel_err(y.reshape(B * S, E), ref_y) <= 1e-5


def test_batched_and_shared_weight_gemm(lane):
    rng = np.random.default_rng(4)
    a = (rng.standard_normal((3, 40, 64)) / 8).astype(np.float16)
    w3 = (rng.standard_normal((3, 64, 48)) / 8).astype(np.float16)
    w2 = w3[1].copy()
    da, dw3, dw2 = rs.DeviceArray.from_host(a), rs.DeviceArray.from_host(w3), rs.DeviceArray.from_host(w2)
    got3 = rs.gemm(da, dw3, out="f32").to_host()
    got2 = rs.gemm(da, dw2, out="f32").to_host()
    assert orc.max_rel_err(got3, np.matmul(a.astype(np.float64), w3.astype(np.float64))) <= 1e-5
    assert orc.max_rel_err(got2, np.matmul(a.astype(np.float64), w2.astype(np.float64))) <= 1e-5
    st = rs.gemm(da, dw3).to_host()
    assert st.dtype == np.float16 and np.array_equal(st, got3.astype(np.float16))
    with pytest.raises(ValueError):
        rs.gemm(da, rs.DeviceArray.from_host(np.zeros((2, 64, 48), np.float16)))
    with pytest.raises(ValueError):
        rs.gemm(da, rs.DeviceArray.from_host(np.zeros((64, 48), np.float32)))


def test_strided_batch_shares_an_operand_without_copies(lane):
    """stride 0 on B: every product of the batch reads the one weight."""
    rng = np.random.default_rng(5)
    a = b16.from_float32(rng.standard_normal((4, 300, 128)) / 8)
    w = b16.from_float32(rng.standard_normal((128, 264)) / 8)
    da, dw = rs.DeviceArray.from_host(a), rs.DeviceArray.from_host(w)
    d = rs.DeviceArray((4, 300, 264), "f32")
    rc = lane.load().tessera_gfx950_batched_gemm_strided_bf16_dev(da.ptr, dw.ptr, d.ptr, 4, 300, 264, 128,
                                                                  300 * 128, 0, 300 * 264, 0, None)
    lane.check(rc, "strided")
    ref = np.matmul(a.to_float32().astype(np.float64), w.to_float32().astype(np.float64))
    assert orc.max_rel_err(d.to_host(), ref) <= 1e-5
    # overlapping outputs are refused
    assert lane.load().tessera_gfx950_batched_gemm_strided_bf16_dev(da.ptr, dw.ptr, d.ptr, 4, 300, 264, 128,
                                                                    300 * 128, 0, 100, 0, None) == lane.BAD_SHAPE


def test_resident_moe_layer_matches_the_host_layer(lane):
    T, H, F, N, E, k = 384, 128, 256, 128, 8, 2
    for seed in range(50, 400):
        rng = np.random.default_rng(seed)
        x = rng.standard_normal((T, H)).astype(np.float32)
        wr = rng.standard_normal((H, E)).astype(np.float32)
        if not orc.has_routing_ties(orc.router_probs(orc.gemm_storage(x, wr, "bf16")), k):
            break
    wg, wu = ((rng.standard_normal((E, H, F)) * 0.1).astype(np.float32) for _ in range(2))
    wd = (rng.standard_normal((E, F, N)) * 0.1).astype(np.float32)
    hb = [b16.from_float32(a) for a in (x, wr, wg, wu, wd)]
    dx, dr, dg, du, dd = (rs.DeviceArray.from_host(a) for a in hb)
    out, plan = rs.moe_layer(dx, dr, dg, du, dd, top_k=k, return_plan=True)
    got = out.to_host()
    host = ops.moe_layer(*hb, top_k=k)
    assert np.array_equal(got.view(np.uint32), np.asarray(host, np.float32).view(np.uint32))
    ref, desc = orc.moe_layer(x, orc.gemm_storage(x, wr, "bf16"), wg, wu, wd, k)
    assert orc.max_rel_err(got, ref) <= 2e-3 + 2.0 ** -8
    n = int(plan.num_slots.to_host()[0])
    assert n == T * k and np.array_equal(plan.token_of_slot.to_host()[:n], desc.token_of_slot)
    # routing alone, from resident logits
    lg = rs.DeviceArray.from_host(orc.gemm_storage(x, wr, "bf16").astype(np.float32))
    p2 = rs.route_tokens(lg, E, k)
    assert np.array_equal(p2.group_offsets.to_host(), desc.group_offsets)
