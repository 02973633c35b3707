"""Quantised GEMM parity on the MI355X: int8 accumulators bit-exact; W8A8 output
exact to f32 rounding; fp8-e4m3 within 2e-3 of the fp32-or-better product of the
dequantised operands (the kernel's own error) and within the e4m3 format's
quantisation error (~3.3e-2 normwise) of the unquantised fp32 product."""
import numpy as np
import pytest

import tessera_oracle as orc
from tessera_amd import bf16 as b16
from tessera_amd import ops

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M,N,K", [(16, 16, 16), (32, 48, 64), (256, 256, 128), (300, 528, 400),
                                   (7, 13, 5), (100, 36, 1000), (512, 1024, 2048),
                                   # few tiles, long K: split along K (2, 4, 8, 16 slices; a ragged last slice)
                                   (16, 2048, 4096), (300, 1024, 8192), (128, 512, 16384), (1, 256, 40000), (40, 528, 2304),
                                   # at most 32 rows, K a multiple of 64 from 2048 up: the streaming kernel (strips of 128
                                   # columns, a ragged last strip and last K split, one row, 32 rows)
                                   (1, 8192, 8192), (32, 144, 2048), (3, 8208, 4160), (31, 4096, 12352), (17, 272, 2112),
                                   (33, 8208, 2112), (64, 272, 4096), (50, 1024, 8192),       # 33 to 64 rows: two row blocks a wave
                                   # K or N off the 16-byte grid, large: aligned zero-padded copies and the tile kernel
                                   (517, 1003, 771), (300, 2050, 4100), (64, 5000, 1001)])
def test_int8_gemm_bit_exact(lane, M, N, K):
    rng = np.random.default_rng(K + M)
    a = rng.integers(-127, 128, (M, K)).astype(np.int8)
    b = rng.integers(-127, 128, (K, N)).astype(np.int8)
    assert np.array_equal(ops.gemm_i8(a, b), orc.gemm_i8_i32(a, b))


def test_int8_extremes(lane):
    a = np.full((64, 4096), -127, np.int8)
    b = np.full((4096, 64), -127, np.int8)
    assert np.all(ops.gemm_i8(a, b) == 127 * 127 * 4096)
    b[:] = 127
    assert np.all(ops.gemm_i8(a, b) == -127 * 127 * 4096)
    a[:] = -128
    b[:] = -128
    assert np.all(ops.gemm_i8(a, b) == 128 * 128 * 4096)


@pytest.mark.parametrize("M,N,K", [(64, 128, 256), (200, 304, 144), (33, 20, 17),
                                   # row lengths on each side of the register-resident row quantiser's limits
                                   (9, 16, 4096), (7, 16, 8192), (6, 16, 16384), (3, 16, 16400), (4, 16, 4104),
                                   # column counts that do / do not take the four-column weight quantiser
                                   (10, 18, 200), (12, 1028, 130)])
def test_quantize_int8_matches_oracle(lane, M, N, K):
    rng = np.random.default_rng(3)
    X = rng.standard_normal((M, K)).astype(np.float32)
    W = rng.standard_normal((K, N)).astype(np.float32)
    X[5 % M] = 0.0                                   # an all-zero row -> absmax floor 1e-12
    xq, xs = ops.quantize_int8_per_channel(X, axis=1)
    wq, ws = ops.quantize_int8_per_channel(W, axis=0)
    oxq, oxs = orc.quantize_int8_per_channel(X, axis=1)
    owq, ows = orc.quantize_int8_per_channel(W, axis=0)
    assert np.array_equal(xq, oxq) and np.array_equal(xs, oxs)
    assert np.array_equal(wq, owq) and np.array_equal(ws, ows)


@pytest.mark.parametrize("M,K,N", [(320, 512, 272), (48, 4096, 2048), (200, 8192, 512),    # the last two: K split
                                   (1, 4096, 4096), (24, 2112, 400),                      # the few-row streaming kernel
                                   (333, 1001, 1030)])                                       # unaligned, large
def test_w8a8_matmul(lane, M, K, N):
    rng = np.random.default_rng(8)
    X = rng.standard_normal((M, K)).astype(np.float32)
    W = rng.standard_normal((K, N)).astype(np.float32)
    y_ref, acc_ref, xq, a_scale, wq, w_scale = orc.w8a8_matmul(X, W)
    y, acc = ops.w8a8_gemm(xq, wq, a_scale, w_scale, return_acc=True)
    assert np.array_equal(acc, acc_ref)
    assert np.array_equal(y, y_ref)                  # two f32 multiplies in the reference's order
    assert np.array_equal(ops.w8a8_matmul(X, W), y_ref)
    # the quantised product approximates the f32 product (sanity on the scales' orientation)
    assert orc.max_rel_err(y, X.astype(np.float64) @ W.astype(np.float64)) < 3e-2


@pytest.mark.parametrize("M", [1, 48, 200, 1024])
def test_int8_every_kernel_against_one_big_weight(lane, M):
    """N = K = 8192 with 1, 48, 200 and 1024 rows — the streaming kernel with one and with two row blocks, the
    128-row tile with K split and the 128-row tile on a full chip: sampled rows exact, and the checksum
    of checksums of the whole result in exact integer arithmetic."""
    N = K = 8192
    rng = np.random.default_rng(M)
    xq = rng.integers(-127, 128, (M, K)).astype(np.int8)
    wq = rng.integers(-127, 128, (K, N)).astype(np.int8)
    acc = ops.gemm_i8(xq, wq)
    rows = rng.choice(M, min(M, 8), replace=False)
    assert np.array_equal(acc[rows], orc.gemm_i8_i32(xq[rows], wq))
    assert int(acc.astype(np.int64).sum()) == int(xq.astype(np.int64).sum(0) @ wq.astype(np.int64).sum(1))
    assert np.array_equal(acc.astype(np.int64).sum(0), xq.astype(np.int64).sum(0) @ wq.astype(np.int64))


@pytest.mark.parametrize("M,N,K", [(64, 12288, 12288), (256, 8192, 8192), (48, 18432, 6144), (512, 8192, 8192)])
def test_int8_schedules_the_fitted_estimate_picks(lane, M, N, K):
    """16 to 1024 rows under a wide weight matrix: where the fitted estimate promises a clear gain the
    launcher leaves its rule (128-row tiles with 2 to 4 K parts, also in place of the streaming kernel).
    Sampled rows exact, column sums of the whole result in exact integer arithmetic."""
    from tessera_amd.schedule import select_gfx950_gemm_schedule as sel
    sch = sel(M, N, K, dtype="int8")
    assert sch.workgroup_tile == (128, 256, 128) and sch.split_k in (2, 3, 4)
    rng = np.random.default_rng(M + N)
    xq = rng.integers(-127, 128, (M, K)).astype(np.int8)
    wq = rng.integers(-127, 128, (K, N)).astype(np.int8)
    acc = ops.gemm_i8(xq, wq)
    rows = rng.choice(M, 8, replace=False)
    assert np.array_equal(acc[rows], orc.gemm_i8_i32(xq[rows], wq))
    assert np.array_equal(acc.astype(np.int64).sum(0), xq.astype(np.int64).sum(0) @ wq.astype(np.int64))


def test_w8a8_headline_shape_properties(lane):
    """M=4096, N=K=8192: accumulators checked exactly on sampled rows/columns."""
    M, N, K = 4096, 8192, 8192
    rng = np.random.default_rng(12)
    xq = rng.integers(-127, 128, (M, K)).astype(np.int8)
    wq = rng.integers(-127, 128, (K, N)).astype(np.int8)
    acc = ops.gemm_i8(xq, wq)
    rows = rng.choice(M, 16, replace=False)
    cols = rng.choice(N, 16, replace=False)
    assert np.array_equal(acc[rows], orc.gemm_i8_i32(xq[rows], wq))
    assert np.array_equal(acc[:, cols], orc.gemm_i8_i32(xq, wq[:, cols]))
    # checksum of checksums in exact integer arithmetic
    assert int(acc.astype(np.int64).sum()) == int(xq.astype(np.int64).sum(0) @ wq.astype(np.int64).sum(1))


def test_e4m3_quantiser_matches_oracle(lane):
    rng = np.random.default_rng(4)
    x = rng.standard_normal(1 << 16).astype(np.float32)
    x[:64] = np.linspace(-1e-3, 1e-3, 64, dtype=np.float32)     # subnormal range after scaling
    x[64] = 0.0
    codes, scale = ops.quantize_fp8_codes(x)
    ocodes, ogrid, oscale = orc.quantize_fp8_e4m3(x)
    assert scale == oscale
    assert np.array_equal(codes, ocodes)
    xq, s2 = ops.quantize_fp8(x)
    assert np.array_equal(xq, ogrid * oscale)
    # every grid point maps to itself; saturation at +-448
    table = orc.e4m3_decode_table()
    finite = ~np.isnan(table)
    c2, _ = ops.quantize_fp8_codes(table[finite], scale=1.0)
    assert np.array_equal(table[c2], table[finite])
    c3, _ = ops.quantize_fp8_codes(np.array([1e9, -1e9, 449.0, 0.0], np.float32), scale=1.0)
    assert list(c3) == [0x7E, 0xFE, 0x7E, 0x00]
    # rounding boundaries: the midpoint of every pair of neighbouring grid values and the
    # f32 on either side of it (ties to even), both signs, through the 16-wide path and
    # the element-wise tail alike
    grid = np.sort(np.unique(np.abs(table[finite]))).astype(np.float32)
    mid = ((grid[:-1].astype(np.float64) + grid[1:].astype(np.float64)) / 2).astype(np.float32)
    probe = np.concatenate([mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf))])
    probe = np.concatenate([probe, -probe]).astype(np.float32)
    assert probe.size % 16 != 0
    c4, _ = ops.quantize_fp8_codes(probe, scale=1.0)
    o4, _, _ = orc.quantize_fp8_e4m3(probe, scale=1.0)
    assert np.array_equal(c4, o4)


@pytest.mark.parametrize("M,N,K", [(64, 64, 64), (256, 512, 1024), (130, 272, 208), (9, 21, 13),
                                   (16, 2048, 4096), (300, 1024, 8192), (128, 512, 16400),    # these three: K split
                                   (1, 8192, 8192), (32, 144, 2048), (3, 8208, 4160), (17, 272, 2112),   # the few-row streaming kernel
                                   (33, 8208, 2112), (64, 272, 4096),
                                   (517, 1003, 771), (300, 2050, 4100)])                      # unaligned, large
def test_fp8_gemm(lane, M, N, K):
    rng = np.random.default_rng(6)
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((K, N)).astype(np.float32)
    ac, _, sa = orc.quantize_fp8_e4m3(A)
    bc, _, sb = orc.quantize_fp8_e4m3(B)
    ref = orc.gemm_e4m3(ac, bc, sa, sb)
    got32 = ops.gemm_fp8(ac, bc, sa, sb, out="f32")
    assert orc.max_rel_err(got32, ref) <= 2e-3       # vs f32 product of the dequantised operands
    # Against the UNQUANTISED product the error is the e4m3 format's own: 3 mantissa
    # bits give each operand up to 2^-4 relative error, the K-term sums of signal and
    # of error both grow like sqrt(K), so the normwise figure sits near 3.3e-2 at
    # every K for N(0,1) data with per-tensor scales — it measures the format, not
    # the kernel (whose own error is the 2e-3 line above).  Bound it loosely.
    if K >= 1024:
        assert orc.max_rel_err(got32, A.astype(np.float64) @ B.astype(np.float64)) <= 5e-2
    got16 = ops.gemm_fp8(ac, bc, sa, sb, out="bf16")
    assert np.array_equal(got16.to_float32(), orc.round_to_storage(got32, "bf16"))


def test_fp8_headline_shape_properties(lane):
    M, N, K = 4096, 8192, 8192
    rng = np.random.default_rng(14)
    ac = rng.integers(0, 256, (M, K)).astype(np.uint8)
    bc = rng.integers(0, 256, (K, N)).astype(np.uint8)
    ac[(ac & 0x7F) == 0x7F] = 0x3C                    # keep NaN codes out
    bc[(bc & 0x7F) == 0x7F] = 0x3C
    ac = ((ac & 0x80) | np.minimum(ac & 0x7F, 0x47)).astype(np.uint8)   # |value| <= 15 keeps f32 sums tame
    bc = ((bc & 0x80) | np.minimum(bc & 0x7F, 0x47)).astype(np.uint8)
    got = ops.gemm_fp8(ac, bc, 0.5, 0.25, out="f32")
    rows = rng.choice(M, 8, replace=False)
    ref = orc.gemm_e4m3(ac[rows], bc, 0.5, 0.25)
    assert orc.max_rel_err(got[rows], ref) <= 2e-3


def test_config5_chain_at_full_size_on_normal_data(lane):
    """The quantised-GEMM configuration end to end on its own data path: N(0,1)
    operands (M = 4096, N = K = 8192) quantised by the lane's quantisers, multiplied,
    rescaled; checked against the oracle's chain on sampled rows — (b) W8A8: codes,
    scales and int32 accumulators bit-exact, y equal to f32 rounding; (a) e4m3: codes
    equal as values (-0 and +0 are two codes of one value), result within 2e-3 of the
    f32 product of the dequantised operands and within the format's own error of the
    unquantised product."""
    M, N, K = 4096, 8192, 8192
    rng = np.random.default_rng(55)
    X = rng.standard_normal((M, K), dtype=np.float32)
    W = rng.standard_normal((K, N), dtype=np.float32)
    rows = np.sort(rng.choice(M, 12, replace=False))
    # (b) int8 W8A8
    xq, a_scale = ops.quantize_int8_per_channel(X, axis=1)
    wq, w_scale = ops.quantize_int8_per_channel(W, axis=0)
    y, acc = ops.w8a8_gemm(xq, wq, a_scale, w_scale, return_acc=True)
    ry, racc, rxq, ras, rwq, rws = orc.w8a8_matmul(X[rows], W)
    assert np.array_equal(xq[rows], rxq) and np.array_equal(wq, rwq)
    assert np.array_equal(a_scale[rows], ras) and np.array_equal(w_scale.reshape(-1), rws)
    assert np.array_equal(acc[rows], racc)
    assert np.array_equal(y[rows], ry)
    # (a) fp8 e4m3 with per-tensor scales
    xc, sx = ops.quantize_fp8_codes(X)
    wc, sw = ops.quantize_fp8_codes(W)
    oxc, _, osx = orc.quantize_fp8_e4m3(X)
    owc, _, osw = orc.quantize_fp8_e4m3(W)
    table = orc.e4m3_decode_table()
    assert sx == osx and sw == osw
    assert np.array_equal(table[xc], table[oxc]) and np.array_equal(table[wc], table[owc])
    got = ops.gemm_fp8(xc, wc, sx, sw, out="f32")[rows]
    assert orc.max_rel_err(got, orc.gemm_e4m3(oxc[rows], owc, osx, osw)) <= 2e-3
    assert orc.max_rel_err(got, X[rows].astype(np.float64) @ W.astype(np.float64)) <= 5e-2
    stored = ops.gemm_fp8(xc, wc, sx, sw, out="bf16")[rows]
    assert np.array_equal(stored.to_float32(), orc.round_to_storage(got, "bf16"))


def test_nvfp4_rounding_matches_oracle_bit_for_bit(lane):
    """Device NVFP4 rounding (block scale in e4m3, E2M1 codes) against the oracle: dequantised
    values and scales bit for bit, on data spanning 12 orders of magnitude, exact ties, zero
    blocks, a short last block and an unaligned row length."""
    from tessera_amd import lane as ln
    lib = ln.load()
    rng = np.random.default_rng(41)
    cases = [(rng.standard_normal((300, 256)) * np.exp(rng.standard_normal((300, 1)) * 6)).astype(np.float32),
             np.tile(np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0, -0.25, -0.75, -1.25, -1.75, -2.5, -3.5, -5.0, -6.0],
                              np.float32), (4, 3)),
             np.zeros((3, 48), np.float32),
             rng.standard_normal((7, 40)).astype(np.float32),             # 2.5 blocks a row
             rng.standard_normal((5, 19)).astype(np.float32) * 1e-8]       # scales in the e4m3 subnormals / zero
    for x in cases:
        rows, cols = x.shape
        dq = np.empty_like(x)
        dq16 = np.empty(x.shape, np.uint16)
        sc = np.empty((rows, -(-cols // 16)), np.float32)
        ln.check(lib.tessera_gfx950_fake_quantize_nvfp4_f32(x.ctypes.data, rows, cols, dq.ctypes.data, dq16.ctypes.data,
                                                            sc.ctypes.data), "nvfp4")
        odq, osc = orc.quantize_nvfp4(x)
        assert np.array_equal(dq.view(np.uint32), odq.view(np.uint32))
        assert np.array_equal(sc.view(np.uint32), osc.view(np.uint32))
        assert np.array_equal((dq16.astype(np.uint32) << 16).view(np.float32), odq)     # the bf16 form is exact
    dq, scales = ops.quantize_nvfp4(cases[0])
    assert np.array_equal(dq, orc.quantize_nvfp4(cases[0])[0]) and scales.shape == (300, 16)
    with pytest.raises(ValueError):
        ops.quantize_nvfp4(cases[3])                                        # 40 % 16 != 0, as the reference


@pytest.mark.parametrize("gs", [[5, 3, 4], [16, 16, 32], [300, 0, 77, 1000]])
def test_grouped_gemm_nvfp4(lane, gs):
    """quant="nvfp4": the product of the NVFP4-rounded operands (the reference rounds on the host
    and multiplies in f32).  Against the oracle's f64 product of the same rounded operands, and
    inside the reference's own 20 % budget against the unquantised product."""
    rng = np.random.default_rng(sum(gs))
    small = sum(gs) < 100
    T, K, N, E = sum(gs), (64 if small else 512), (16 if small else 256), len(gs)
    x = b16.from_float32(rng.standard_normal((T, K)).astype(np.float32))
    w = b16.from_float32(rng.standard_normal((E, K, N)).astype(np.float32))
    ref = orc.grouped_gemm_nvfp4(x.to_float32(), w.to_float32(), gs)
    got = ops.grouped_gemm(x, w, gs, quant="nvfp4", out="f32")
    assert got.shape == (T, N) and orc.max_rel_err(got, ref) <= 1e-5
    stored = ops.grouped_gemm(x, w, gs, quant="nvfp4")
    assert np.array_equal(stored.to_float32(), orc.round_to_storage(got, "bf16"))
    full = np.zeros((T, N))
    off = 0
    for e, n in enumerate(gs):
        full[off:off + n] = x.to_float32()[off:off + n].astype(np.float64) @ w.to_float32()[e].astype(np.float64)
        off += n
    assert np.linalg.norm(got - full) / np.linalg.norm(full) < 0.20
    with pytest.raises(ValueError):
        ops.grouped_gemm(b16.from_float32(np.zeros((T, 24), np.float32)),        # K = 24 is not whole blocks
                         b16.from_float32(np.zeros((E, 24, N), np.float32)), gs, quant="nvfp4")


FP_FORMATS = {"e4m3": (448.0, 3, -6), "e5m2": (57344.0, 2, -14), "e2m3": (7.5, 3, -126), "e3m2": (28.0, 2, -126),
              "e2m1": (6.0, 1, -126)}


@pytest.mark.parametrize("fmt", sorted(FP_FORMATS))
def test_float_grid_kernel_matches_oracle_bit_for_bit(lane, fmt):
    """The device grid rounding against the oracle (itself pinned on the reference's compiled
    kernel for every one of these formats): magnitudes from the denormals to beyond
    saturation, every tie, NaN and both zeros; through the 16-byte path and the element tail."""
    mx, mant, min_exp = FP_FORMATS[fmt]
    rng = np.random.default_rng(mant * 100 - min_exp)
    lo = max(min_exp, -20)
    pts = np.array(sorted({np.ldexp(1.0 + m / 2.0 ** mant, e) for e in range(lo - 2, int(np.log2(mx)) + 1)
                           for m in range(2 ** mant)}), np.float64)
    pts = pts[pts <= mx]
    mids = ((pts[1:] + pts[:-1]) / 2).astype(np.float32)
    mag = np.exp(rng.uniform(np.log(1e-42), np.log(mx * 8), 1 << 16))
    vals = np.concatenate([pts, mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(np.inf)), mag,
                           [0.0, -0.0, np.nan, mx, mx * 1.01, 1e30, np.inf, 1e-40, 2.0 ** -126, 2.0 ** -149]])
    x = (vals * rng.choice([-1.0, 1.0], vals.size)).astype(np.float32)
    for xs in (x, x[1:], x[:7]):                                       # aligned, unaligned, tail only
        got = ops.fpquant(xs, mx, mant, min_exp)
        assert np.array_equal(got, orc.fpquant_grid(xs, mx, mant, min_exp), equal_nan=True)
    # a snapped value is a fixed point
    g = ops.fpquant(x, mx, mant, min_exp)
    assert np.array_equal(ops.fpquant(g, mx, mant, min_exp), g, equal_nan=True)


@pytest.mark.parametrize("tag", ["e5m2", "e2m3", "e3m2", "e2m1", "e2m1_floor0"])
def test_float_grid_kernel_golden(lane, tag):
    from pathlib import Path
    gold = np.load(Path(__file__).parent / "golden" / "ref_vectors.npz")
    mx, mant, min_exp = gold[f"fpq_{tag}_fmt"]
    got = ops.fpquant(gold[f"fpq_{tag}_x"], float(mx), int(mant), int(min_exp))
    assert np.array_equal(got, gold[f"fpq_{tag}_y"], equal_nan=True)


@pytest.mark.parametrize("fmt", sorted(FP_FORMATS))
def test_per_tensor_float_quantisers_match_oracle(lane, fmt):
    """ops.quantize_fp8 / fp6 / fp4: automatic and given scale, values and scale bit for bit;
    the bf16 form of the unscaled grid values is exact."""
    from tessera_amd import lane as ln
    q = {"e4m3": ops.quantize_fp8, "e5m2": ops.quantize_fp8, "e2m3": ops.quantize_fp6, "e3m2": ops.quantize_fp6,
         "e2m1": ops.quantize_fp4}[fmt]
    rng = np.random.default_rng(len(fmt) + FP_FORMATS[fmt][1])
    x = (rng.standard_normal((257, 129)) * np.exp(rng.standard_normal((257, 1)) * 3)).astype(np.float32)
    for scale in (None, 0.037):
        dq, s = q(x, format=fmt, scale=scale)
        odq, ogrid, os_ = orc.quantize_fp(x, fmt, scale)
        assert s == os_ and dq.shape == x.shape
        assert np.array_equal(dq.view(np.uint32) & 0x7FFFFFFF, odq.view(np.uint32) & 0x7FFFFFFF) and np.array_equal(dq, odq)
        mx, mant, min_exp = FP_FORMATS[fmt]
        g16 = np.empty(x.shape, np.uint16)
        ln.check(ln.load().tessera_gfx950_fake_quantize_fp_f32(x.ctypes.data, x.size, mx, mant, min_exp, float(s), None,
                                                               g16.ctypes.data, None), "grid")
        assert np.array_equal((g16.astype(np.uint32) << 16).view(np.float32), ogrid)
    assert np.array_equal(ops.quantize_fp8(np.zeros(5, np.float32), format="e5m2")[0], np.zeros(5, np.float32))
    with pytest.raises(ValueError):
        q(x, format="e9m9")


@pytest.mark.parametrize("quant", ["fp8_e5m2", "fp8xfp4", "fp8_e4m3xnvfp4", "fp8_e5m2xnvfp4", "fp8", "nvfp4"])
@pytest.mark.parametrize("gs", [[5, 3, 4], [300, 0, 77, 1000]])
def test_grouped_gemm_quant_schemes(lane, quant, gs):
    """Every quant= scheme of the reference's grouped product against the oracle's f64 product of
    the same quantised operands."""
    rng = np.random.default_rng(sum(gs) + len(quant))
    small = sum(gs) < 100
    T, K, N, E = sum(gs), (64 if small else 512), (16 if small else 256), len(gs)
    x = b16.from_float32((rng.standard_normal((T, K)) * 3).astype(np.float32))
    w = b16.from_float32((rng.standard_normal((E, K, N)) * np.array([0.1, 1.0, 7.0, 0.5][:E])[:, None, None]).astype(np.float32))
    ref = orc.grouped_gemm_quant(x.to_float32(), w.to_float32(), gs, quant)
    got = ops.grouped_gemm(x, w, gs, quant=quant, out="f32")
    # (plain e4m3 runs on the fp8 matrix instruction, whose sum over one instruction's 64
    # products keeps fewer bits than an f32 sum; the other schemes run on the bf16 one)
    tol = 1e-4 if quant == "fp8" else 1e-5
    assert got.shape == (T, N) and orc.max_rel_err(got, ref) <= tol
    stored = ops.grouped_gemm(x, w, gs, quant=quant)
    assert orc.max_rel_err(stored.to_float32(), ref) <= 2.0 ** -8 + tol
    full = np.zeros((T, N))
    off = 0
    for e, n in enumerate(gs):
        full[off:off + n] = x.to_float32()[off:off + n].astype(np.float64) @ w.to_float32()[e].astype(np.float64)
        off += n
    assert np.linalg.norm(got - full) / np.linalg.norm(full) < 0.25
    with pytest.raises(ValueError):
        ops.grouped_gemm(x, w, gs, quant="int3")


def test_float_grid_and_group_scaling_on_device_buffers(lane):
    """The device-pointer forms: e5m2 with the automatic scale into f32 and bf16-grid outputs, the
    bare grid kernel, and the per-group scaling with f32 and bf16 results."""
    import ctypes
    from tessera_amd import lane as ln
    lib = ln.load()
    rng = np.random.default_rng(77)
    x = (rng.standard_normal(50003) * 11).astype(np.float32)
    dx = ln.DeviceBuffer.from_host(x)
    ddq, dg, dsc, dout = ln.DeviceBuffer(x.size * 4), ln.DeviceBuffer(x.size * 2), ln.DeviceBuffer(4), ln.DeviceBuffer(x.size * 4)
    try:
        ln.check(lib.tessera_gfx950_fake_quantize_fp_f32_dev(dx.ptr, x.size, ctypes.c_float(57344.0), 2, -14, ctypes.c_float(0.0),
                                                             ddq.ptr, dg.ptr, dsc.ptr, None), "fake_quantize_fp")
        ln.check(lib.tessera_gfx950_fpquant_f32_dev(dx.ptr, x.size, ctypes.c_float(6.0), 1, 0, dout.ptr, None), "fpquant")
        ln.synchronize()
        odq, ogrid, oscale = orc.quantize_fp(x, "e5m2")
        assert dsc.download((1,), np.float32)[0] == oscale
        assert np.array_equal(ddq.download(x.shape, np.float32), odq)
        assert np.array_equal((dg.download(x.shape, np.uint16).astype(np.uint32) << 16).view(np.float32), ogrid)
        assert np.array_equal(dout.download(x.shape, np.float32), orc.fpquant_grid(x, 6.0, 1, 0))
        # bad formats are refused before anything is launched
        assert lib.tessera_gfx950_fpquant_f32_dev(dx.ptr, x.size, ctypes.c_float(6.0), 24, 0, dout.ptr, None) == 1
        assert lib.tessera_gfx950_fpquant_f32_dev(dx.ptr, x.size, ctypes.c_float(-1.0), 1, 0, dout.ptr, None) == 1
        assert lib.tessera_gfx950_fpquant_f32_dev(dx.ptr, x.size, ctypes.c_float(6.0), 1, -127, dout.ptr, None) == 1
    finally:
        for b in (dx, ddq, dg, dsc, dout):
            b.close()
    S, N, E = 37, 24, 5
    y = rng.standard_normal((S, N)).astype(np.float32)
    off = np.array([0, 10, 10, 11, 30, 37], np.int32)
    sc = rng.uniform(0.1, 3.0, E).astype(np.float32)
    ref = y * np.repeat(sc, np.diff(off))[:, None]
    dy, dof, dsc2 = ln.DeviceBuffer.from_host(y), ln.DeviceBuffer.from_host(off), ln.DeviceBuffer.from_host(sc)
    d32, d16 = ln.DeviceBuffer(S * N * 4), ln.DeviceBuffer(S * N * 2)
    try:
        ln.check(lib.tessera_gfx950_scale_groups_f32_dev(dy.ptr, dof.ptr, dsc2.ptr, d32.ptr, 0, S, N, E, None), "scale_groups")
        ln.check(lib.tessera_gfx950_scale_groups_f32_dev(dy.ptr, dof.ptr, dsc2.ptr, d16.ptr, 1, S, N, E, None), "scale_groups")
        ln.synchronize()
        assert np.array_equal(d32.download((S, N), np.float32), ref)
        assert np.array_equal(d16.download((S, N), np.uint16), b16.from_float32(ref).view(np.uint16).reshape(S, N))
    finally:
        for b in (dy, dof, dsc2, d32, d16):
            b.close()
    out = np.empty((S, N), np.float32)
    bad = off.copy(); bad[2] = 12                        # offsets must not decrease
    assert lib.tessera_gfx950_scale_groups_f32(y.ctypes.data, bad.ctypes.data, sc.ctypes.data, out.ctypes.data, 0, S, N, E) == 1


@pytest.mark.parametrize("M,K,N", [(64, 256, 128), (33, 100, 72), (300, 4096, 512), (8, 16400, 64)])
def test_smoothquant_matmul_bit_for_bit(lane, M, K, N):
    """smoothquant_matmul on a migrated layer: smoothed activation codes, token scales and int32
    accumulators bit for bit, the rescaled f32 result exactly as numpy's two multiplies give it."""
    from types import SimpleNamespace
    rng = np.random.default_rng(M + K + N)
    X = (rng.standard_normal((M, K)) * np.exp(rng.standard_normal(K))).astype(np.float32)     # outlier channels
    W = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32)
    s, w_q, w_scale = orc.migrate_activation_scale(X, W)
    x_q, a_scale = ops.quantize_int8_per_channel(X, 1, smoothing=s)
    ry, racc, rxq, ras = orc.smoothquant_matmul(X, s, w_q, w_scale)
    assert np.array_equal(x_q, rxq) and np.array_equal(a_scale, ras)
    got = ops.smoothquant_matmul(X, SimpleNamespace(smoothing=s, w_q=w_q, w_scale=w_scale))
    assert got.dtype == np.float32 and np.array_equal(got, ry)
    # the point of the migration: closer to the f32 product than plain W8A8 on data with outlier channels
    full = X.astype(np.float64) @ W.astype(np.float64)
    plain = ops.w8a8_matmul(X, W)
    assert np.linalg.norm(got - full) <= np.linalg.norm(plain - full) * 1.05
    with pytest.raises(ValueError):
        ops.quantize_int8_per_channel(X, 0, smoothing=s)
    with pytest.raises(ValueError):
        ops.smoothquant_matmul(X, SimpleNamespace(smoothing=s, w_q=w_q.astype(np.int32), w_scale=w_scale))


def test_per_tensor_int8_quantiser(lane):
    """quantization.quantize_int8 (symmetric): codes and scale bit for bit; every half-way point of
    the code grid rounds to the even code; an all-zero tensor gets scale 1."""
    rng = np.random.default_rng(12)
    x = (rng.standard_normal((513, 257)) * 3).astype(np.float32)
    q, s, zp = ops.quantize_int8(x)
    oq, os_ = orc.quantize_int8_tensor(x)
    assert zp == 0 and s == os_ and q.dtype == np.int8 and np.array_equal(q, oq)
    q2, s2, _ = ops.quantize_int8(x, scale=0.05)
    assert s2 == np.float32(0.05) and np.array_equal(q2, orc.quantize_int8_tensor(x, 0.05)[0])
    ties = (np.arange(-260, 261, dtype=np.float32) / 2)                      # scale 1: k + 0.5 -> even
    qt, _, _ = ops.quantize_int8(ties, scale=1.0)
    assert np.array_equal(qt, np.clip(np.rint(ties), -127, 127).astype(np.int8))
    qz, sz, _ = ops.quantize_int8(np.zeros(40, np.float32))
    assert sz == np.float32(1.0) and not qz.any()
    assert np.allclose(ops.dequantize_int8(q, s), x, atol=float(s) / 2 * 1.0001)
    with pytest.raises(NotImplementedError):
        ops.quantize_int8(x, symmetric=False)


@pytest.mark.parametrize("fmt,bound", [("e4m3", 0.15), ("e5m2", 0.30)])
def test_fp8_facts_the_reference_tests_hold(lane, fmt, bound):
    """The statements of the reference's own fp8 tests (tests/unit/test_phase_e_f.py:474-516):
    round-trip error bound per format, dequantize is the identity on x_q, an explicit scale
    saturates at the format's max_normal, zeros stay zeros, an unknown format is a ValueError."""
    rng = np.random.RandomState(0)
    x = (rng.randn(64) * 50.0).astype(np.float32)
    x_q, scale = ops.quantize_fp8(x, format=fmt)
    assert float((np.abs(x - x_q) / (np.abs(x) + 1e-6)).max()) <= bound
    assert np.array_equal(ops.dequantize_fp8(x_q, scale, format=fmt), x_q)
    huge = np.array([1e6, -1e6], np.float32)
    top = 448.0 if fmt == "e4m3" else 57344.0
    assert np.array_equal(ops.quantize_fp8(huge, format=fmt, scale=1.0)[0], [top, -top])
    assert np.array_equal(ops.quantize_fp8(np.zeros(4, np.float32), format=fmt)[0], np.zeros(4))
    with pytest.raises(ValueError, match="format"):
        ops.quantize_fp8(np.array([1.0], np.float32), format="e3m4")
    with pytest.raises(ValueError, match="format"):
        ops.dequantize_fp8(x_q, scale, format="e3m4")


@pytest.mark.parametrize("quant,bound", [("fp8_e4m3", 0.06), ("fp8_e5m2", 0.30), ("nvfp4", 0.20), ("fp8xfp4", 0.20)])
def test_quantised_grouped_gemm_inside_the_reference_budgets(lane, quant, bound):
    """The normwise error budgets the reference's own tests give each scheme against the
    unquantised grouped product (tests/unit/test_grouped_gemm_contract.py:223-229)."""
    rng = np.random.default_rng(11)
    gs = [16, 16, 32]
    x32 = rng.standard_normal((sum(gs), 64)).astype(np.float32)
    w32 = rng.standard_normal((len(gs), 64, 16)).astype(np.float32)
    x, w = b16.from_float32(x32), b16.from_float32(w32)
    ref = orc.grouped_gemm(x.to_float32(), w.to_float32(), gs, store=False)
    got = ops.grouped_gemm(x, w, gs, quant=quant, out="f32")
    rel = np.linalg.norm(got - ref) / (np.linalg.norm(ref) + 1e-9)
    assert rel < bound, f"{quant}: {rel:.4f}"


def test_e5m2_quantiser_matches_oracle(lane):
    """e5m2 codes: scale and codes bit for bit on random data, every grid point a fixed point, saturation
    at +-57344, every midpoint between neighbours and its two f32 neighbours (ties to even), through
    the 16-wide hardware-conversion path and the element tail alike."""
    rng = np.random.default_rng(14)
    x = (rng.standard_normal(1 << 16) * np.exp(rng.standard_normal(1 << 16) * 3)).astype(np.float32)
    x[:64] = np.linspace(-1e-6, 1e-6, 64, dtype=np.float32)
    codes, scale = ops.quantize_fp8_codes(x, format="e5m2")
    ocodes, ogrid, oscale = orc.quantize_fp8_e5m2(x)
    table = orc.e5m2_decode_table()
    assert scale == oscale and np.array_equal(table[codes], ogrid)          # (-0 and +0 are two codes of one value)
    assert np.array_equal(ops.e5m2_table(), table, equal_nan=True)
    finite = np.isfinite(table)
    c2, _ = ops.quantize_fp8_codes(table[finite], scale=1.0, format="e5m2")
    assert np.array_equal(table[c2], table[finite])
    c3, _ = ops.quantize_fp8_codes(np.array([1e9, -1e9, 60000.0, 0.0], np.float32), scale=1.0, format="e5m2")
    assert list(c3) == [0x7B, 0xFB, 0x7B, 0x00]
    grid = np.sort(np.unique(np.abs(table[finite]))).astype(np.float32)
    mid = ((grid[:-1].astype(np.float64) + grid[1:].astype(np.float64)) / 2).astype(np.float32)
    probe = np.concatenate([mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf))])
    probe = np.concatenate([probe, -probe])
    for xs in (probe, probe[:13]):
        got, _ = ops.quantize_fp8_codes(xs, scale=1.0, format="e5m2")
        assert np.array_equal(table[got], orc.fpquant_grid(xs, 57344.0, 2, -14))
    with pytest.raises(ValueError):
        ops.quantize_fp8_codes(x, format="e3m4")


@pytest.mark.parametrize("M,N,K", [(64, 64, 64), (256, 512, 1024), (130, 272, 208), (9, 21, 13), (300, 1024, 8192),
                                   (1, 8192, 8192), (48, 272, 2112), (1024, 2048, 1024), (517, 1003, 771)])
def test_fp8_e5m2_gemm(lane, M, N, K):
    """The e5m2 operand format on every 8-bit kernel (both tile heights, K split, streaming, per-element,
    repitched) against the oracle's f64 product of the decoded codes."""
    rng = np.random.default_rng(60 + M)
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((K, N)).astype(np.float32)
    ac, _, sa = orc.quantize_fp8_e5m2(A)
    bc, _, sb = orc.quantize_fp8_e5m2(B)
    ref = orc.gemm_fp8_codes(ac, bc, sa, sb, "e5m2")
    got32 = ops.gemm_fp8(ac, bc, sa, sb, out="f32", format="e5m2")
    assert orc.max_rel_err(got32, ref) <= 2e-3
    if K >= 1024:      # two mantissa bits: the format's own error against the unquantised product
        assert orc.max_rel_err(got32, A.astype(np.float64) @ B.astype(np.float64)) <= 1e-1
    got16 = ops.gemm_fp8(ac, bc, sa, sb, out="bf16", format="e5m2")
    assert np.array_equal(got16.to_float32(), orc.round_to_storage(got32, "bf16"))
    with pytest.raises(ValueError):
        ops.gemm_fp8(ac, bc, sa, sb, format="e2m5")
