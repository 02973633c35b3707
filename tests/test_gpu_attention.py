"""Flash-attention forward parity on the MI355X (through the C ABI) vs the oracle.

Tolerances (as stated for this path): O max relative error
<= 2e-3 normwise against an fp32-or-better reference of the same 16-bit inputs;
LSE absolute error <= 2e-3.  The reference's own test budgets are looser
(f16 2e-2, bf16 6e-2 absolute, tests/unit/test_rocm_flash_attn_runtime_symbol.py:90-132).
"""
import numpy as np
import pytest

import tessera_oracle as orc
from tessera_amd import bf16 as b16
from tessera_amd import ops

pytestmark = pytest.mark.gpu
TOL = 2e-3


def _qkv(B, Hq, Hkv, Sq, Sk, D, seed, st, scale=1.0):
    rng = np.random.default_rng(seed)
    q = (rng.standard_normal((B, Hq, Sq, D)) * scale).astype(np.float32)
    k = (rng.standard_normal((B, Hkv, Sk, D)) * scale).astype(np.float32)
    v = (rng.standard_normal((B, Hkv, Sk, D)) * scale).astype(np.float32)
    if st == "bf16":
        return tuple(b16.from_float32(x) for x in (q, k, v))
    return tuple(x.astype(np.float16) for x in (q, k, v))


def _f32(x):
    return x.to_float32() if isinstance(x, b16.BF16Array) else np.asarray(x, np.float32)


CASES = [
    # B, Hq, Hkv, Sq, Sk, D, causal
    (1, 1, 1, 16, 16, 16, False), (1, 1, 1, 16, 16, 16, True),
    (1, 2, 2, 64, 64, 128, False), (1, 2, 2, 64, 64, 128, True),
    (2, 4, 2, 300, 300, 128, True), (1, 8, 2, 257, 511, 128, True),
    (2, 4, 1, 256, 512, 128, True), (1, 2, 2, 100, 77, 64, False),
    (1, 2, 1, 200, 333, 64, True), (1, 2, 2, 333, 200, 64, True),
    (1, 1, 1, 50, 60, 32, True), (1, 3, 3, 40, 40, 48, False),
    (1, 2, 2, 1, 129, 128, True), (1, 4, 4, 513, 1, 128, False),
    (1, 2, 2, 700, 700, 256, True),
    # B * Hkv a multiple of 8: the XCD-aware workgroup order
    (2, 8, 4, 300, 520, 128, True), (1, 16, 8, 260, 260, 64, True), (2, 24, 8, 70, 330, 128, False),
]


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,causal", CASES)
@pytest.mark.parametrize("st", ["bf16", "f16"])
def test_attention_matches_oracle(lane, B, Hq, Hkv, Sq, Sk, D, causal, st):
    q, k, v = _qkv(B, Hq, Hkv, Sq, Sk, D, 17, st)
    ref_o, ref_lse = orc.flash_attn_dense(_f32(q), _f32(k), _f32(v), causal=causal)
    o, lse = ops.gqa_attention(q, k, v, causal=causal, return_lse=True, out="f32")
    assert o.shape == (B, Hq, Sq, D) and lse.shape == (B, Hq, Sq)
    assert not np.isnan(o).any()
    assert orc.max_rel_err(o, ref_o) <= TOL
    assert np.max(np.abs(lse - ref_lse)) <= TOL


# Few query rows per KV head — (Hq / Hkv) * Sq <= 32 at D = 256, 64 at 128, 128 at 64 — take the decode
# kernel: the rows of a GQA group share one MFMA tile, the key range is split over workgroups
# and waves, partials are merged.  One and many key splits, ratio 1 to 16, rows that fill the
# tile and that do not, ragged last tile, causal steps of several rows, a sliding window.
DECODE_CASES = [
    # B, Hq, Hkv, Sq, Sk, D, causal, window
    (2, 8, 2, 1, 777, 128, False, 0), (1, 32, 8, 1, 8192, 128, False, 0), (3, 16, 16, 1, 300, 64, False, 0),
    (2, 8, 1, 4, 1000, 128, True, 0), (1, 4, 4, 7, 129, 256, True, 0), (2, 6, 2, 3, 64, 64, True, 0),
    (1, 16, 1, 2, 4100, 128, True, 0), (1, 8, 2, 1, 5000, 128, True, 1024), (1, 2, 2, 16, 31, 128, False, 0),
    (40, 8, 2, 1, 2048, 128, False, 0), (1, 8, 8, 1, 33000, 64, False, 0), (2, 4, 1, 8, 20, 256, True, 0),
    # two and four query tiles per wave: up to 64 rows per KV head at D = 128, 128 at D = 64
    (1, 64, 8, 5, 3000, 128, True, 0), (2, 16, 2, 8, 777, 128, True, 0), (1, 8, 1, 7, 2100, 128, False, 0),
    (1, 16, 1, 8, 1500, 64, True, 0), (2, 12, 4, 33, 500, 64, True, 0), (1, 4, 2, 20, 4097, 64, False, 0),
]


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,causal,window", DECODE_CASES)
@pytest.mark.parametrize("st", ["bf16", "f16"])
def test_decode_shapes_match_oracle(lane, B, Hq, Hkv, Sq, Sk, D, causal, window, st):
    q, k, v = _qkv(B, Hq, Hkv, Sq, Sk, D, 23, st)
    ref_o, ref_lse = orc.flash_attn_dense(_f32(q), _f32(k), _f32(v), causal=causal, window=window)
    o, lse = ops.gqa_attention(q, k, v, causal=causal, return_lse=True, out="f32", window=window)
    assert not np.isnan(o).any()
    assert orc.max_rel_err(o, ref_o) <= TOL
    assert np.max(np.abs(lse - ref_lse)) <= TOL
    stored = ops.gqa_attention(q, k, v, causal=causal, window=window)
    assert orc.max_rel_err(_f32(stored), ref_o) <= TOL + (2.0 ** -8 if st == "bf16" else 2.0 ** -11)


def test_decode_kernel_reads_k_and_v_about_once(lane):
    """What the decode kernel is for: one query row per head against a long key range runs
    near the rate at which K and V can be read once, not once per query head."""
    import ctypes
    import time
    B, Hq, Hkv, Sk, D = 16, 32, 8, 4096, 128
    rng = np.random.default_rng(1)
    mk = lambda *shape: lane.DeviceBuffer.from_host((rng.standard_normal(shape).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16))
    q, k, v = mk(B, Hq, 1, D), mk(B, Hkv, Sk, D), mk(B, Hkv, Sk, D)
    o = lane.DeviceBuffer(B * Hq * D * 2)
    fn = lane.load().tessera_gfx950_flash_attn_gqa_bf16_dev
    call = lambda: lane.check(fn(q.ptr, k.ptr, v.ptr, o.ptr, None, B, Hq, Hkv, 1, Sk, D, ctypes.c_float(D ** -0.5), 0, 1, None), "decode")
    for _ in range(5):
        call()
    lane.synchronize()
    t0 = time.perf_counter()
    for _ in range(20):
        call()
    lane.synchronize()
    per_call = (time.perf_counter() - t0) / 20
    kv_bytes = 2 * B * Hkv * Sk * D * 2
    for b in (q, k, v, o):
        b.close()
    assert kv_bytes / per_call > 1.5e12, f"{kv_bytes / per_call / 1e12:.2f} TB/s"     # the general kernel: 2.1e12 / 4 heads


# Few workgroups against a long key range (a chunk of queries against a long context): the general
# kernel splits the key tiles over the grid and the partials are merged.  Causal (bottom-right
# aligned), non-causal, a window, GQA, head dims on the padded and the column-split kernels.
SPLIT_CASES = [
    # B, Hq, Hkv, Sq, Sk, D, causal, window
    (1, 8, 2, 128, 8192, 128, True, 0), (1, 4, 4, 300, 5000, 64, True, 0), (1, 16, 2, 16, 4100, 128, True, 0),
    (1, 2, 1, 257, 6000, 256, True, 0), (2, 4, 2, 64, 3000, 96, False, 0), (1, 8, 8, 200, 9000, 128, True, 2048),
    (1, 6, 2, 40, 2049, 160, True, 0),
]


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,causal,window", SPLIT_CASES)
@pytest.mark.parametrize("st", ["bf16", "f16"])
def test_key_split_shapes_match_oracle(lane, B, Hq, Hkv, Sq, Sk, D, causal, window, st):
    q, k, v = _qkv(B, Hq, Hkv, Sq, Sk, D, 29, st)
    ref_o, ref_lse = orc.flash_attn_dense(_f32(q), _f32(k), _f32(v), causal=causal, window=window)
    o, lse = ops.gqa_attention(q, k, v, causal=causal, return_lse=True, out="f32", window=window)
    assert not np.isnan(o).any()
    assert orc.max_rel_err(o, ref_o) <= TOL
    assert np.max(np.abs(lse - ref_lse)) <= TOL
    stored = ops.gqa_attention(q, k, v, causal=causal, window=window)
    assert orc.max_rel_err(_f32(stored), ref_o) <= TOL + (2.0 ** -8 if st == "bf16" else 2.0 ** -11)


@pytest.mark.parametrize("scale", [0.3, 1e-3, 0.0, -0.07])
def test_attention_scales(lane, scale):
    """Any finite scale: a negative one turns the row maximum of the raw scores into
    the minimum of the scaled ones, a zero one gives uniform weights."""
    q, k, v = _qkv(1, 4, 2, 130, 200, 128, 19, "f16")
    ref_o, ref_lse = orc.flash_attn_dense(_f32(q), _f32(k), _f32(v), scale=scale, causal=True)
    o, lse = ops.gqa_attention(q, k, v, scale=scale, causal=True, return_lse=True, out="f32")
    assert orc.max_rel_err(o, ref_o) <= TOL
    assert np.max(np.abs(lse - ref_lse)) <= TOL


def test_attention_special_cases(lane):
    """Closed forms: causal row 0 sees only key 0 -> O[0] = V[0], LSE[0] = s00;
    identical keys -> uniform weights -> prefix mean of V."""
    B, H, S, D = 1, 2, 192, 128
    q, k, v = _qkv(B, H, H, S, S, D, 3, "bf16")
    o, lse = ops.flash_attn(q, k, v, causal=True, return_lse=True, out="f32")
    qf, kf, vf = _f32(q), _f32(k), _f32(v)
    assert np.allclose(o[:, :, 0], vf[:, :, 0], rtol=0, atol=1e-6)
    s00 = (qf[:, :, 0] * kf[:, :, 0]).sum(-1) / np.sqrt(D)
    assert np.allclose(lse[:, :, 0], s00, atol=1e-4)
    k_same = b16.from_float32(np.broadcast_to(kf[:, :, :1], kf.shape).copy())
    o2 = ops.flash_attn(q, k_same, v, causal=True, out="f32")
    prefix_mean = np.cumsum(vf.astype(np.float64), axis=2) / np.arange(1, S + 1)[None, None, :, None]
    assert orc.max_rel_err(o2, prefix_mean) <= TOL


def test_gqa_equals_repeated_kv(lane):
    q, k, v = _qkv(2, 8, 2, 160, 160, 128, 5, "bf16")
    o_gqa = ops.gqa_attention(q, k, v, causal=True, out="f32")
    k_rep = b16.from_bits(np.repeat(np.asarray(k, np.uint16), 4, axis=1))
    v_rep = b16.from_bits(np.repeat(np.asarray(v, np.uint16), 4, axis=1))
    o_mha = ops.flash_attn(q, k_rep, v_rep, causal=True, out="f32")
    assert np.array_equal(o_gqa, o_mha)
    with pytest.raises(ValueError):
        ops.flash_attn(q, k, v)


def test_legacy_signature_and_storage_output(lane):
    """The MHA-only entry point (call-compatible with the shipped ROCm symbol)
    and the storage-dtype output."""
    q, k, v = _qkv(1, 2, 2, 96, 96, 64, 9, "f16")
    ref_o, _ = orc.flash_attn_dense(_f32(q), _f32(k), _f32(v), causal=True)
    o = np.empty(q.shape, np.float32)
    rc = lane.load().tessera_gfx950_flash_attn_f16(
        q.view(np.uint16).ctypes.data, k.view(np.uint16).ctypes.data, v.view(np.uint16).ctypes.data,
        o.ctypes.data, 1, 2, 96, 96, 64, float(1 / np.sqrt(64)), 1)
    assert rc == 0
    assert orc.max_rel_err(o, ref_o) <= TOL
    o16 = ops.flash_attn(q, k, v, causal=True)
    assert o16.dtype == np.float16 and np.array_equal(o16, o.astype(np.float16))


def test_headline_config_properties(lane):
    """B=4 Hq=32 Hkv=8 S=4096 D=128 causal: checked head-by-head against the
    blockwise oracle on a sample of (batch, head) pairs, plus the row-0 identity
    on every head."""
    B, Hq, Hkv, S, D = 4, 32, 8, 4096, 128
    q, k, v = _qkv(B, Hq, Hkv, S, S, D, 21, "bf16")
    o, lse = ops.gqa_attention(q, k, v, causal=True, return_lse=True, out="f32")
    assert not np.isnan(o).any()
    vf = _f32(v)
    assert np.allclose(o[:, :, 0], np.repeat(vf[:, :, 0], Hq // Hkv, axis=1), atol=1e-6)
    pairs = [(0, 0), (1, 13), (3, 31)]
    ref_o, ref_lse = orc.flash_attn_blockwise(_f32(q), _f32(k), _f32(v), causal=True, heads=pairs,
                                               dtype=np.float64)
    for (b, h) in pairs:
        assert orc.max_rel_err(o[b, h], ref_o[b, h]) <= TOL
        assert np.max(np.abs(lse[b, h] - ref_lse[b, h])) <= TOL


HEAD_DIMS = [16, 32, 48, 64, 80, 96, 112, 128, 144, 160, 192, 208, 256]


@pytest.mark.parametrize("D", HEAD_DIMS)
@pytest.mark.parametrize("st", ["bf16", "f16"])
def test_every_head_dim_on_the_matrix_path(lane, D, st):
    """Every head dimension that is a multiple of 16 runs the MFMA kernel (zero-padded to the
    next compiled width, as the reference's kernel serves every D % 16 == 0 on its matrix
    path, tessera_rocm_flash_attn.cpp:47-144): causal GQA with a ragged last tile, plus the
    soft-capped, windowed form."""
    B, Hq, Hkv, Sq, Sk = 1, 4, 2, 150, 203
    q, k, v = _qkv(B, Hq, Hkv, Sq, Sk, D, 100 + D, st)
    ref_o, ref_lse = orc.flash_attn_dense(_f32(q), _f32(k), _f32(v), causal=True)
    o, lse = ops.gqa_attention(q, k, v, causal=True, return_lse=True, out="f32")
    assert not np.isnan(o).any()
    assert orc.max_rel_err(o, ref_o) <= TOL
    assert np.max(np.abs(lse - ref_lse)) <= TOL
    o16 = ops.gqa_attention(q, k, v, causal=True)
    want16 = b16.from_float32(o) if st == "bf16" else o.astype(np.float16)
    assert np.array_equal(np.asarray(o16, np.uint16) if st == "bf16" else o16.view(np.uint16),
                          np.asarray(want16, np.uint16) if st == "bf16" else want16.view(np.uint16))
    ref_o, ref_lse = orc.flash_attn_dense(_f32(q), _f32(k), _f32(v), causal=True, window=70, softcap=4.0)
    o, lse = ops.gqa_attention(q, k, v, causal=True, return_lse=True, out="f32", window=70, logit_softcap=4.0)
    assert orc.max_rel_err(o, ref_o) <= TOL
    assert np.max(np.abs(lse - ref_lse)) <= TOL


def test_mfma_kernel_is_the_one_that_runs_for_padded_head_dims(lane):
    """The per-row kernel serves unaligned operands only: at S = 2048 it would take tens of
    milliseconds per launch, the MFMA kernel well under one."""
    import ctypes, time
    B, Hq, Hkv, S, D = 1, 16, 4, 2048, 96
    q, k, v = _qkv(B, Hq, Hkv, S, S, D, 5, "bf16")
    dq, dk, dv = (lane.DeviceBuffer.from_host(np.asarray(x, np.uint16)) for x in (q, k, v))
    do = lane.DeviceBuffer(B * Hq * S * D * 2)
    fn = lane.load().tessera_gfx950_flash_attn_gqa_bf16_dev
    run = lambda: fn(dq.ptr, dk.ptr, dv.ptr, do.ptr, None, B, Hq, Hkv, S, S, D, ctypes.c_float(D ** -0.5), 1, 1, None)
    for _ in range(3):
        assert run() == 0
    lane.synchronize()
    t0 = time.perf_counter()
    for _ in range(10):
        run()
    lane.synchronize()
    ms = (time.perf_counter() - t0) / 10 * 1e3
    flop = 4.0 * B * Hq * (S * (S + 1) / 2) * D
    assert flop / ms / 1e9 > 20.0, f"{ms:.3f} ms per launch: not the matrix path"


def test_strided_operands_that_are_not_16_byte_aligned_take_the_per_row_kernel(lane):
    """Row strides that are not multiples of 8 elements cannot be read 16 bytes at a time: the
    per-row kernel serves them through the same strides, to the same bounds."""
    import ctypes
    B, Hq, Hkv, Sq, Sk, D = 1, 2, 1, 40, 55, 32
    q, k, v = _qkv(B, Hq, Hkv, Sq, Sk, D, 41, "f16")
    ref_o, ref_lse = orc.flash_attn_dense(_f32(q), _f32(k), _f32(v), causal=True)
    pad = 4                                                           # rows of D + 4 elements
    def rows(x):
        out = np.zeros(x.shape[:-1] + (D + pad,), np.float16)
        out[..., :D] = x
        return lane.DeviceBuffer.from_host(np.ascontiguousarray(out.view(np.uint16)))
    dq, dk, dv = rows(q), rows(k), rows(v)
    do, dl = lane.DeviceBuffer(B * Hq * Sq * (D + pad) * 4), lane.DeviceBuffer(B * Hq * Sq * 4)
    W = D + pad
    strides = (ctypes.c_int64 * 12)(Hq * Sq * W, Sq * W, W, Hkv * Sk * W, Sk * W, W, Hkv * Sk * W, Sk * W, W,
                                    Hq * Sq * W, Sq * W, W)
    rc = lane.load().tessera_gfx950_flash_attn_strided_f16_dev(dq.ptr, dk.ptr, dv.ptr, do.ptr, dl.ptr, B, Hq, Hkv, Sq, Sk, D,
                                                               strides, ctypes.c_float(D ** -0.5), 1, 0, ctypes.c_float(0.0),
                                                               0, None)
    assert rc == 0
    lane.synchronize()
    o = do.download((B, Hq, Sq, W), np.float32)[..., :D]
    assert orc.max_rel_err(o, ref_o) <= TOL
    assert np.max(np.abs(dl.download((B, Hq, Sq), np.float32) - ref_lse)) <= TOL


def test_attention_rejects_bad_shapes(lane):
    lib = lane.load()
    z = np.zeros(1024, np.uint16)
    o = np.zeros(1024, np.float32)
    f = lib.tessera_gfx950_flash_attn_bf16
    assert f(z.ctypes.data, z.ctypes.data, z.ctypes.data, o.ctypes.data, 1, 1, 8, 8, 20, 1.0, 0) == 1   # D % 16
    assert f(z.ctypes.data, z.ctypes.data, z.ctypes.data, o.ctypes.data, 1, 1, 0, 8, 16, 1.0, 0) == 1
    g = lib.tessera_gfx950_flash_attn_gqa_bf16
    assert g(z.ctypes.data, z.ctypes.data, z.ctypes.data, o.ctypes.data, None, 1, 3, 2, 8, 8, 16, 1.0, 0) == 1


WINDOW_CASES = [
    # B, Hq, Hkv, Sq, Sk, D, causal, window, softcap
    (1, 2, 2, 300, 300, 128, True, 64, 0.0), (1, 4, 2, 700, 700, 128, True, 200, 0.0),
    (1, 2, 1, 257, 511, 128, True, 33, 0.0), (1, 2, 2, 513, 513, 64, True, 128, 0.0),
    (1, 2, 2, 300, 300, 128, False, 90, 0.0), (1, 2, 2, 400, 250, 64, False, 40, 0.0),
    (1, 2, 2, 300, 300, 128, True, 0, 5.0), (1, 4, 1, 257, 300, 64, True, 0, 2.5),
    (1, 2, 2, 520, 520, 128, True, 100, 8.0), (1, 2, 2, 100, 100, 48, True, 20, 3.0),
]


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,causal,window,cap", WINDOW_CASES)
def test_sliding_window_and_softcap(lane, B, Hq, Hkv, Sq, Sk, D, causal, window, cap):
    q, k, v = _qkv(B, Hq, Hkv, Sq, Sk, D, 29, "bf16")
    ref_o, ref_lse = orc.flash_attn_dense(_f32(q), _f32(k), _f32(v), causal=causal, window=window, softcap=cap)
    o, lse = ops.gqa_attention(q, k, v, causal=causal, return_lse=True, out="f32", window=window, logit_softcap=cap)
    assert not np.isnan(o).any()
    assert orc.max_rel_err(o, ref_o) <= TOL
    finite = np.isfinite(ref_lse)
    assert np.array_equal(np.isfinite(lse), finite)
    assert np.max(np.abs(lse[finite] - ref_lse[finite])) <= TOL


def test_window_closed_forms(lane):
    """window = 1 (causal): every query sees exactly its diagonal key -> O = V row,
    LSE = that score.  A window wider than the sequence equals plain causal."""
    q, k, v = _qkv(1, 2, 2, 200, 200, 128, 5, "bf16")
    o, lse = ops.flash_attn(q, k, v, causal=True, window=1, return_lse=True, out="f32")
    assert np.allclose(o, _f32(v), atol=1e-6)
    s = np.einsum("bhqd,bhqd->bhq", _f32(q).astype(np.float64), _f32(k).astype(np.float64)) / np.sqrt(128)
    assert np.max(np.abs(lse - s)) <= 2e-3
    wide = ops.flash_attn(q, k, v, causal=True, window=4096, out="f32")
    assert np.array_equal(wide, ops.flash_attn(q, k, v, causal=True, out="f32"))


def test_sliding_window_executor_op(lane):
    from tessera_amd import executors as ex
    q, k, v = (np.asarray(_f32(x), np.float16) for x in _qkv(1, 2, 2, 128, 128, 64, 7, "f16"))
    art = ex.make_artifact("tessera.attn_sliding_window", ["q", "k", "v"], ["q", "k", "v"], "gfx950_flash_attn",
                           kwargs={"window": 32})
    res = ex.launch(art, (q, k, v))
    assert res["ok"], res
    ref, _ = orc.flash_attn_dense(q.astype(np.float32), k.astype(np.float32), v.astype(np.float32), causal=True,
                                  window=32)
    assert orc.max_rel_err(res["output"], ref) <= TOL
    bad = ex.make_artifact("tessera.attn_sliding_window", ["q", "k", "v"], ["q", "k", "v"], "gfx950_flash_attn")
    assert not ex.launch(bad, (q, k, v))["ok"]


BIAS_CASES = [
    # B, Hq, Hkv, Sq, Sk, D, causal, window, softcap, storage
    (1, 2, 2, 300, 300, 128, False, 0, 0.0, "bf16"), (2, 4, 2, 257, 511, 128, True, 0, 0.0, "f16"),
    (1, 4, 1, 513, 513, 64, True, 0, 0.0, "bf16"), (1, 2, 2, 520, 520, 128, True, 100, 0.0, "bf16"),
    (1, 2, 2, 300, 300, 128, True, 0, 5.0, "bf16"), (1, 2, 1, 100, 130, 48, True, 0, 0.0, "f16"),
    (1, 2, 2, 64, 1000, 128, False, 0, 3.0, "f16"),
]


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,causal,window,cap,st", BIAS_CASES)
def test_additive_bias(lane, B, Hq, Hkv, Sq, Sk, D, causal, window, cap, st):
    q, k, v = _qkv(B, Hq, Hkv, Sq, Sk, D, 31, st)
    bias = (np.random.default_rng(32).standard_normal((B, Hq, Sq, Sk)) * 2).astype(np.float32)
    ref_o, ref_lse = orc.flash_attn_dense(_f32(q), _f32(k), _f32(v), causal=causal, window=window, softcap=cap,
                                          bias=bias)
    o, lse = ops.gqa_attention(q, k, v, causal=causal, return_lse=True, out="f32", window=window,
                               logit_softcap=cap, attn_bias=bias)
    assert not np.isnan(o).any()
    assert orc.max_rel_err(o, ref_o) <= TOL
    assert np.max(np.abs(lse - ref_lse)) <= TOL


def test_bias_broadcast_and_closed_forms(lane):
    """A bias constant along the keys leaves O unchanged and shifts LSE by it; a
    (Sq, Sk) bias broadcasts over batch and heads; a -inf bias acts as a mask
    (the causal mask written as a bias equals the causal kernel)."""
    q, k, v = _qkv(2, 4, 2, 200, 200, 128, 9, "bf16")
    plain_o, plain_lse = ops.gqa_attention(q, k, v, return_lse=True, out="f32")
    row = np.linspace(-3, 3, 200, dtype=np.float32)[:, None] * np.ones((1, 200), np.float32)
    o, lse = ops.gqa_attention(q, k, v, return_lse=True, out="f32", attn_bias=row)
    assert orc.max_rel_err(o, plain_o) <= 1e-5
    assert np.max(np.abs(lse - (plain_lse + row[:, 0]))) <= 1e-4
    tri = np.where(np.tril(np.ones((200, 200), bool)), 0.0, -np.inf).astype(np.float32)
    masked = ops.gqa_attention(q, k, v, out="f32", attn_bias=tri)
    assert orc.max_rel_err(masked, ops.gqa_attention(q, k, v, causal=True, out="f32")) <= 1e-5
    with pytest.raises(ValueError):
        ops.gqa_attention(q, k, v, attn_bias=np.zeros((3, 200), np.float32))


def test_bias_executor_operand(lane):
    from tessera_amd import executors as ex
    q, k, v = (np.asarray(_f32(x), np.float16) for x in _qkv(1, 2, 2, 130, 130, 64, 11, "f16"))
    bias = np.random.default_rng(3).standard_normal((130, 130)).astype(np.float32)
    art = ex.make_artifact("tessera.flash_attn", ["q", "k", "v", "b"], ["q", "k", "v", "b"], "gfx950_flash_attn",
                           kwargs={"causal": True})
    res = ex.launch(art, (q, k, v, bias))
    assert res["ok"], res
    ref, _ = orc.flash_attn_dense(q.astype(np.float32), k.astype(np.float32), v.astype(np.float32), causal=True,
                                  bias=np.broadcast_to(bias, (1, 2, 130, 130)))
    assert orc.max_rel_err(res["output"], ref) <= TOL
    bad = ex.launch(art, (q, k, v, np.zeros((7, 130), np.float32)))
    assert bad["runtime_status"] == "invalid_artifact"


def test_gqa_and_mqa_take_the_reference_head_count_arguments(lane):
    """nn.functional.gqa_attention(Q, K, V, num_query_heads, num_kv_heads, **kwargs) and mqa_attention."""
    rng = np.random.default_rng(5)
    q = b16.from_float32(rng.standard_normal((2, 8, 40, 64)).astype(np.float32))
    k = b16.from_float32(rng.standard_normal((2, 2, 40, 64)).astype(np.float32))
    v = b16.from_float32(rng.standard_normal((2, 2, 40, 64)).astype(np.float32))
    a = ops.gqa_attention(q, k, v, 8, 2, causal=True, out="f32")
    assert np.array_equal(a, ops.gqa_attention(q, k, v, causal=True, out="f32"))
    ref, _ = orc.flash_attn_dense(q.to_float32(), k.to_float32(), v.to_float32(), causal=True)
    assert orc.max_rel_err(a, ref) <= 2e-3
    k1, v1 = b16.from_float32(k.to_float32()[:, :1]), b16.from_float32(v.to_float32()[:, :1])
    m = ops.mqa_attention(q, k1, v1, out="f32")
    ref1, _ = orc.flash_attn_dense(q.to_float32(), k1.to_float32(), v1.to_float32())
    assert orc.max_rel_err(m, ref1) <= 2e-3
