"""Operands with more than 2^31 elements: every element offset the kernels form must be 64-bit.

A GEMM whose output has 2.15e9 elements and an attention forward whose Q and O have 2.15e9
elements each, checked on rows at the far end of the index range (where a 32-bit offset
would have wrapped) against numpy on the same 16-bit inputs.  Device-resident buffers; the
big operands are a small random block repeated, which the checks do not depend on.
"""
import ctypes

import numpy as np
import pytest

import tessera_oracle as orc

pytestmark = pytest.mark.gpu


def _bf16_bits(x):
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def _f32(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def test_gemm_output_beyond_2_31_elements(lane):
    M = N = 46400                                   # 2.153e9 outputs, 4.3 GB in bf16
    K = 64
    rng = np.random.default_rng(31)
    a = _bf16_bits(rng.standard_normal((M, K)) / 8)
    b = _bf16_bits(rng.standard_normal((K, N)))
    da, db = lane.DeviceBuffer.from_host(a), lane.DeviceBuffer.from_host(b)
    dd = lane.DeviceBuffer(M * N * 2)
    try:
        lane.check(lane.load().tessera_gfx950_gemm_bf16_bf16_dev(da.ptr, db.ptr, dd.ptr, M, N, K, None), "gemm")
        lane.synchronize()
        out = dd.download((M, N), np.uint16)
    finally:
        for buf in (da, db, dd):
            buf.close()
    rows = [0, 1, 255, 256, 23199, 46143, 46144, 46398, 46399]
    ref = _f32(a[rows]).astype(np.float64) @ _f32(b).astype(np.float64)
    got = _f32(out[rows])
    assert orc.max_rel_err(got, ref) <= 2e-3 + 2.0 ** -8
    assert np.array_equal(out[rows], _bf16_bits(ref.astype(np.float32))) or orc.max_rel_err(got, ref) <= 2.0 ** -8


def test_attention_operands_beyond_2_31_elements(lane):
    B, Hq, Hkv, S, D = 8, 40, 8, 65536, 128         # Q, O: 2.68e9 elements each; K, V a fifth of that
    rng = np.random.default_rng(32)
    blk = _bf16_bits(rng.standard_normal((1 << 22, D)))          # 4 Mi rows of random data, repeated
    reps_q = B * Hq * S // blk.shape[0]
    reps_kv = B * Hkv * S // blk.shape[0]
    q = np.tile(blk, (reps_q, 1)).reshape(B, Hq, S, D)
    k = np.tile(blk[::-1], (reps_kv, 1)).reshape(B, Hkv, S, D)
    v = np.tile(np.roll(blk, 12345, axis=0), (reps_kv, 1)).reshape(B, Hkv, S, D)
    assert q.size > 2 ** 31 and (B - 1) * Hq * S * D > 2 ** 31
    dq, dk, dv = (lane.DeviceBuffer.from_host(x) for x in (q, k, v))
    do = lane.DeviceBuffer(q.size * 2)
    dl = lane.DeviceBuffer(B * Hq * S * 4)
    try:
        lane.check(lane.load().tessera_gfx950_flash_attn_gqa_bf16_dev(
            dq.ptr, dk.ptr, dv.ptr, do.ptr, dl.ptr, B, Hq, Hkv, S, S, D, ctypes.c_float(D ** -0.5), 1, 1, None), "attn")
        lane.synchronize()
        out = do.download((B, Hq, S, D), np.uint16)
        lse = dl.download((B, Hq, S), np.float32)
    finally:
        for buf in (dq, dk, dv, do, dl):
            buf.close()
    # the last (batch, head) sits wholly beyond element 2^31; a row block in its middle and its last rows
    for (b, h, r0) in [(B - 1, Hq - 1, S - 32), (B - 1, Hq - 1, 40000), (0, 0, 100), (B // 2, 5, S - 64)]:
        rows = slice(r0, r0 + 32)
        qq = _f32(q[b, h, rows])[None, None]
        kk = _f32(k[b, h // (Hq // Hkv), : r0 + 32])[None, None]
        vv = _f32(v[b, h // (Hq // Hkv), : r0 + 32])[None, None]
        ro, rl = orc.flash_attn_dense(qq, kk, vv, causal=True)       # bottom-right aligned: row i sees keys <= r0 + i
        assert orc.max_rel_err(_f32(out[b, h, rows]), ro[0, 0]) <= 2e-3 + 2.0 ** -8, (b, h, r0)
        assert np.max(np.abs(lse[b, h, rows] - rl[0, 0])) <= 2e-3, (b, h, r0)
