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


def _heads_first(t, B, S, h, D):
    """[B, S, h*D] bits -> [B, h, S, D] BF16Array (host-side head split, for the reference chain)."""
    return b16.from_bits(np.ascontiguousarray(np.asarray(t, np.uint16).reshape(B, S, h, D).transpose(0, 2, 1, 3)))


def test_projection_then_attention_chain(lane):
    """x @ Wq / Wk / Wv -> attention -> @ Wo with NO host hop: the attention kernel reads the
    projections where the GEMMs left them ([B, S, H, D] through row strides) and writes its
    output in the layout the output projection consumes.  Nothing is downloaded before the
    chain's result; the intermediates are fetched afterwards only to check them."""
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
    o, lse = rs.flash_attn(q.reshape(B, S, Hq, D), k.reshape(B, S, Hkv, D), v.reshape(B, S, Hkv, D), causal=True,
                           return_lse=True, layout="bshd")
    assert o.shape == (B, S, Hq, D)
    y = rs.gemm(o.reshape(B, S, Hq * D), dwo, out="f32").to_host()  # the first download of the chain
    # the same chain through the host-pointer ops (which copy and transpose on the host): identical bits
    hq, hk, hv = ops.gemm(xb, wqb), ops.gemm(xb, wkb), ops.gemm(xb, wvb)
    assert np.array_equal(np.asarray(hq, np.uint16), np.asarray(q.to_host(), np.uint16))
    q4, k4, v4 = _heads_first(hq, B, S, Hq, D), _heads_first(hk, B, S, Hkv, D), _heads_first(hv, B, S, Hkv, D)
    ho, hl = ops.gqa_attention(q4, k4, v4, causal=True, return_lse=True)
    o_bits = np.asarray(o.to_host(), np.uint16)                    # [B, S, Hq, D]
    assert np.array_equal(np.asarray(ho, np.uint16), o_bits.transpose(0, 2, 1, 3))
    assert np.array_equal(hl, lse.to_host())
    # and the oracle on the attention stage and on the output projection
    ro, rl = orc.flash_attn_dense(q4.to_float32(), k4.to_float32(), v4.to_float32(), causal=True)
    got_o = b16.from_bits(np.ascontiguousarray(o_bits.transpose(0, 2, 1, 3))).to_float32()
    assert orc.max_rel_err(got_o, ro) <= 2e-3 + 2.0 ** -8
    assert np.max(np.abs(lse.to_host() - rl)) <= 2e-3
    assert y.shape == (B, S, E) and np.isfinite(y).all()
    ref_y = orc.gemm_f64(b16.from_bits(o_bits).to_float32().reshape(B * S, -1), wob.to_float32())
    assert orc.max_rel_err(y.reshape(B * S, E), ref_y) <= 1e-5
    host_y = ops.gemm(b16.from_bits(np.ascontiguousarray(o_bits.reshape(B * S, Hq * D))), wob, out="f32")
    assert np.array_equal(host_y.view(np.uint32), y.reshape(B * S, E).view(np.uint32))


def test_fused_qkv_projection_feeds_attention_in_place(lane):
    """ONE projection x @ [Wq | Wk | Wv]; the attention kernel reads its three column blocks
    through row strides (pointers offset to each block), f16 storage, D = 128."""
    B, S, Hq, Hkv, D, E = 1, 300, 4, 1, 128, 192
    rng = np.random.default_rng(8)
    x = (rng.standard_normal((B, S, E)) * 0.5).astype(np.float16)
    w = (rng.standard_normal((E, (Hq + 2 * Hkv) * D)) / 12).astype(np.float16)
    qkv = rs.gemm(rs.DeviceArray.from_host(x), rs.DeviceArray.from_host(w))
    o, lse = rs.flash_attn_fused_qkv(qkv, Hq, Hkv, causal=True, return_lse=True, out="f32")
    h = np.asarray(qkv.to_host()).reshape(B, S, Hq + 2 * Hkv, D).transpose(0, 2, 1, 3).astype(np.float32)
    ro, rl = orc.flash_attn_dense(h[:, :Hq], h[:, Hq:Hq + Hkv], h[:, Hq + Hkv:], causal=True)
    assert orc.max_rel_err(o.to_host().transpose(0, 2, 1, 3), ro) <= 2e-3
    assert np.max(np.abs(lse.to_host() - rl)) <= 2e-3
    # the contiguous entry point on host-transposed copies gives the same bits
    c = np.ascontiguousarray
    o2, l2 = ops.gqa_attention(c(h[:, :Hq]).astype(np.float16), c(h[:, Hq:Hq + Hkv]).astype(np.float16),
                               c(h[:, Hq + Hkv:]).astype(np.float16), causal=True, return_lse=True, out="f32")
    assert np.array_equal(o2, o.to_host().transpose(0, 2, 1, 3)) and np.array_equal(l2, lse.to_host())


def test_strided_attention_rejects_bad_strides(lane):
    import ctypes
    lib = lane.load()
    z = lane.DeviceBuffer(1 << 16)
    def call(strides, D=64):
        arr = (ctypes.c_int64 * 12)(*strides)
        return lib.tessera_gfx950_flash_attn_strided_bf16_dev(z.ptr, z.ptr, z.ptr, z.ptr, None, 1, 2, 2, 16, 16, D, arr,
                                                              ctypes.c_float(0.125), 1, 0, ctypes.c_float(0.0), 1, None)
    good = (2 * 16 * 64, 64, 128) * 4
    assert call(good) == 0
    lane.synchronize()
    assert call((2 * 16 * 64, 64, 32) + good[3:]) == lane.BAD_SHAPE          # row stride shorter than a row
    assert call((-1, 64, 128) + good[3:]) == lane.BAD_SHAPE
    assert lib.tessera_gfx950_flash_attn_strided_bf16_dev(z.ptr, z.ptr, z.ptr, z.ptr, None, 1, 2, 2, 16, 16, 64, None,
                                                          ctypes.c_float(0.125), 1, 0, ctypes.c_float(0.0), 1,
                                                          None) == lane.BAD_SHAPE


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
