"""Seeded random-shape parity sweeps on the MI355X (through the C ABI) against the oracle.

The hand-picked cases of the other GPU test files pin the shapes that are known to be
delicate; these sweeps draw shapes nobody picked — ragged and unaligned sizes, every
kernel family behind each entry point (square-tile, skinny, split-K, generic fallback) —
with the same bounds: bit-exact for integer and index results, <= 2e-3 (normwise) for 16-bit
floating point with f32 accumulation, exact RNE of the f32 accumulators for stored results.
Every draw prints nothing and is reproducible from its seed.

``TESSERA_FUZZ_SCALE=n`` in the environment multiplies the number of seeds of every sweep
(default 1: the suite's normal run; a soak run uses 8 or more).
"""
import os

import numpy as np
import pytest

import tessera_oracle as orc
from tessera_amd import bf16 as b16
from tessera_amd import ops

pytestmark = pytest.mark.gpu
TOL = 2e-3
SCALE = max(1, int(os.environ.get("TESSERA_FUZZ_SCALE", "1")))


def _store(x, st):
    return b16.from_float32(x) if st == "bf16" else x.astype(np.float16)


def _f32(x):
    return x.to_float32() if isinstance(x, b16.BF16Array) else np.asarray(x, np.float32)


def _dim(rng, hi, aligned):
    """A size in [1, hi]; `aligned` makes it a multiple of 8 (the vector-load kernels)."""
    n = int(rng.integers(1, hi + 1))
    return max(8, n // 8 * 8) if aligned else n


@pytest.mark.parametrize("seed", range(6 * SCALE))
def test_gemm_random_shapes(lane, seed):
    rng = np.random.default_rng(1000 + seed)
    for _ in range(60):
        aligned = bool(rng.integers(0, 4))               # one draw in four takes the any-shape kernel
        M = int(rng.choice([1, 2, 5, 8, 9, 16, 33, 64, 100, 129, 257, 300]))
        N, K = _dim(rng, 520, aligned), _dim(rng, 1100, aligned)
        if rng.integers(0, 5) == 0:
            K = int(rng.choice([512, 1024, 2048, 4096]))  # long K: the split-K and streaming paths
        st = "bf16" if rng.integers(0, 2) else "f16"
        A = _store(rng.standard_normal((M, K)).astype(np.float32) * 0.5, st)
        B = _store(rng.standard_normal((K, N)).astype(np.float32) * 0.5, st)
        ref = _f32(A).astype(np.float64) @ _f32(B).astype(np.float64)
        got = ops.gemm(A, B, out="f32")
        assert got.shape == (M, N)
        assert orc.max_rel_err(got, ref) <= 1e-5, (seed, M, N, K, st)
        stored = ops.gemm(A, B)
        want = _store(got, st)                              # the storage rule: RNE of the f32 accumulators
        assert np.array_equal(np.asarray(stored).view(np.uint16), np.asarray(want).view(np.uint16)), (seed, M, N, K, st)


@pytest.mark.parametrize("seed", range(2 * SCALE))
def test_big_tile_gemm_random_shapes(lane, seed):
    """Shapes large enough for the 256 x 256 tile (its 16-wide MFMA step, peeled first and last
    K steps, ragged rows and columns), both storage types, short and odd K."""
    from tessera_amd.schedule import select_gfx950_gemm_schedule
    rng = np.random.default_rng(1500 + seed)
    for _ in range(6):
        M, N = (int(rng.integers(440, 513)) * 8 for _ in range(2))          # 3520 .. 4096, multiples of 8
        K = int(rng.integers(1, 90)) * 8
        st = "bf16" if rng.integers(0, 2) else "f16"
        assert select_gfx950_gemm_schedule(M, N, K, dtype=st).workgroup_tile[:2] == (256, 256)
        A = _store(rng.standard_normal((M, K)).astype(np.float32) * 0.5, st)
        B = _store(rng.standard_normal((K, N)).astype(np.float32) * 0.5, st)
        ref = _f32(A).astype(np.float64) @ _f32(B).astype(np.float64)
        got = ops.gemm(A, B, out="f32")
        assert orc.max_rel_err(got, ref) <= 1e-5, (seed, M, N, K, st)
        stored = ops.gemm(A, B)
        assert np.array_equal(np.asarray(stored).view(np.uint16), np.asarray(_store(got, st)).view(np.uint16)), (seed, M, N, K, st)


@pytest.mark.parametrize("seed", range(3 * SCALE))
def test_batched_gemm_random_shapes(lane, seed):
    rng = np.random.default_rng(2000 + seed)
    for _ in range(30):
        Bt = int(rng.integers(1, 7))
        aligned = bool(rng.integers(0, 3))
        M, N, K = _dim(rng, 200, False), _dim(rng, 300, aligned), _dim(rng, 300, aligned)
        st = "bf16" if rng.integers(0, 2) else "f16"
        A = _store(rng.standard_normal((Bt, M, K)).astype(np.float32) * 0.5, st)
        W = _store(rng.standard_normal((Bt, K, N)).astype(np.float32) * 0.5, st)
        ref = np.matmul(_f32(A).astype(np.float64), _f32(W).astype(np.float64))
        got = ops.gemm(A, W, out="f32")
        assert got.shape == (Bt, M, N)
        assert orc.max_rel_err(got, ref) <= 1e-5, (seed, Bt, M, N, K, st)


@pytest.mark.parametrize("seed", range(3 * SCALE))
def test_int8_gemm_random_shapes_bit_exact(lane, seed):
    rng = np.random.default_rng(3000 + seed)
    for _ in range(40):
        aligned = bool(rng.integers(0, 4))
        M, N, K = _dim(rng, 300, False), _dim(rng, 400, aligned), _dim(rng, 900, aligned)
        a = rng.integers(-128, 128, (M, K)).astype(np.int8)
        b = rng.integers(-128, 128, (K, N)).astype(np.int8)
        got = ops.gemm_i8(a, b)
        assert got.dtype == np.int32
        assert np.array_equal(got, orc.gemm_i8_i32(a, b)), (seed, M, N, K)


@pytest.mark.parametrize("seed", range(3 * SCALE))
def test_quantised_chains_random_shapes(lane, seed):
    """quantise -> GEMM -> dequantise on random shapes: int8 accumulators, codes and scales
    bit-exact; e4m3 codes equal as values, product within 2e-3 of the dequantised product."""
    rng = np.random.default_rng(4000 + seed)
    tbl = orc.e4m3_decode_table()
    for _ in range(15):
        M, N, K = _dim(rng, 200, False), _dim(rng, 320, True), _dim(rng, 640, True)
        X = rng.standard_normal((M, K)).astype(np.float32)
        W = rng.standard_normal((K, N)).astype(np.float32)
        xq, a_s = ops.quantize_int8_per_channel(X, axis=1)
        wq, w_s = ops.quantize_int8_per_channel(W, axis=0)
        ry, racc, rxq, ras, rwq, rws = orc.w8a8_matmul(X, W)
        assert np.array_equal(xq, rxq) and np.array_equal(wq, rwq), (seed, M, N, K)
        assert np.array_equal(np.asarray(a_s).reshape(-1), ras.reshape(-1))
        assert np.array_equal(np.asarray(w_s).reshape(-1), rws.reshape(-1))
        y, acc = ops.w8a8_gemm(xq, wq, a_s, w_s, return_acc=True)
        assert np.array_equal(acc, racc), (seed, M, N, K)
        assert np.array_equal(y, ry), (seed, M, N, K)
        ac, sa = ops.quantize_fp8_codes(X)
        bc, sb = ops.quantize_fp8_codes(W)
        ra, _, rsa = orc.quantize_fp8_e4m3(X)
        rb, _, rsb = orc.quantize_fp8_e4m3(W)
        assert np.array_equal(tbl[ac], tbl[ra]) and np.array_equal(tbl[bc], tbl[rb]), (seed, M, N, K)
        assert np.float32(sa) == np.float32(rsa) and np.float32(sb) == np.float32(rsb)
        got = ops.gemm_fp8(ac, bc, sa, sb, out="f32")
        ref = (tbl[ra].astype(np.float64) * float(rsa)) @ (tbl[rb].astype(np.float64) * float(rsb))
        assert orc.max_rel_err(got, ref) <= TOL, (seed, M, N, K)


@pytest.mark.parametrize("seed", range(6 * SCALE))
def test_attention_random_shapes(lane, seed):
    rng = np.random.default_rng(5000 + seed)
    for _ in range(30):
        B = int(rng.integers(1, 3))
        Hkv = int(rng.integers(1, 4))
        ratio = int(rng.choice([1, 1, 2, 4]))
        if rng.integers(0, 4) == 0:                       # the XCD-grouped workgroup order: B * Hkv % 8 == 0
            B, Hkv = 1, 8
        D = int(rng.choice([16, 32, 48, 64, 64, 80, 96, 128, 128, 128, 160, 192, 256]))
        Sq, Sk = int(rng.integers(1, 420)), int(rng.integers(1, 420))
        causal = bool(rng.integers(0, 2))
        window = int(rng.choice([0, 0, 0, 1, 7, 64, 130]))
        softcap = float(rng.choice([0.0, 0.0, 0.0, 5.0, 30.0]))
        st = "bf16" if rng.integers(0, 2) else "f16"
        amp = float(rng.choice([0.5, 1.0, 2.0]))
        q = _store(rng.standard_normal((B, Hkv * ratio, Sq, D)).astype(np.float32) * amp, st)
        k = _store(rng.standard_normal((B, Hkv, Sk, D)).astype(np.float32) * amp, st)
        v = _store(rng.standard_normal((B, Hkv, Sk, D)).astype(np.float32), st)
        ref_o, ref_lse = orc.flash_attn_dense(_f32(q), _f32(k), _f32(v), causal=causal, window=window, softcap=softcap)
        o, lse = ops.gqa_attention(q, k, v, causal=causal, return_lse=True, out="f32", window=window,
                                   logit_softcap=softcap)
        case = (seed, B, Hkv, ratio, Sq, Sk, D, causal, window, softcap, st, amp)
        assert not np.isnan(o).any(), case
        # The kernel, like the reference's (tessera_rocm_flash_attn.cpp:105-121), rounds P to the
        # storage dtype for the second product and keeps the normaliser in f32; the oracle rounds
        # nothing.  f16 P (2^-11) leaves the 2e-3 bound of the headline tests untouched; bf16 P has a
        # unit roundoff of 2^-9 = 1.95e-3, the bound itself, and a short key range can land a hair
        # over it (seed 4 draws one at 2.03e-3, which a numpy emulation of that rounding reproduces
        # to seven digits): random bf16 draws get 3e-3.
        assert orc.max_rel_err(o, ref_o) <= (TOL if st == "f16" else 3e-3), case
        live = np.isfinite(ref_lse)
        assert np.array_equal(np.isfinite(lse), live), case                  # rows with no visible key: -inf
        assert np.max(np.abs(lse[live] - ref_lse[live]), initial=0.0) <= TOL, case


@pytest.mark.parametrize("seed", range(3 * SCALE))
def test_strided_attention_random_layouts(lane, seed):
    """The strided entry point on operands that live inside wider rows (a fused projection's
    column blocks, with random gaps between the heads' blocks) gives the bits the contiguous
    entry point gives on compacted copies: only the addressing differs."""
    import ctypes
    lib = lane.load()
    rng = np.random.default_rng(5500 + seed)
    for _ in range(12):
        B, Hkv = int(rng.integers(1, 3)), int(rng.integers(1, 4))
        Hq = Hkv * int(rng.choice([1, 2, 4]))
        D = int(rng.choice([16, 48, 64, 96, 128, 256]))
        Sq, Sk = int(rng.integers(1, 300)), int(rng.integers(1, 300))
        causal = int(rng.integers(0, 2))
        f32_out = int(rng.integers(0, 2))
        st = "bf16" if rng.integers(0, 2) else "f16"
        # rows of width W hold [gap | q heads | gap | k heads | v heads | gap], gaps multiples of 8 elements
        g0, g1, g2 = (8 * int(rng.integers(0, 3)) for _ in range(3))
        Wq, Wk = g0 + Hq * D + g1, Hkv * D * 2 + g2
        q_rows = _store(rng.standard_normal((B, Sq, Wq)).astype(np.float32), st)
        kv_rows = _store(rng.standard_normal((B, Sk, Wk)).astype(np.float32), st)
        bits = lambda a: np.ascontiguousarray(np.asarray(a).view(np.uint16) if st == "f16" else np.asarray(a, np.uint16))
        qb, kvb = bits(q_rows), bits(kv_rows)
        dq, dkv = lane.DeviceBuffer.from_host(qb), lane.DeviceBuffer.from_host(kvb)
        esz = 4 if f32_out else 2
        Wo = Hq * D + g1
        do, dl = lane.DeviceBuffer(B * Sq * Wo * esz), lane.DeviceBuffer(B * Hq * Sq * 4)
        do.zero()
        strides = (ctypes.c_int64 * 12)(Sq * Wq, D, Wq, Sk * Wk, D, Wk, Sk * Wk, D, Wk, Sq * Wo, D, Wo)
        fn = getattr(lib, f"tessera_gfx950_flash_attn_strided_{st}_dev")
        rc = fn(dq.ptr + g0 * 2, dkv.ptr, dkv.ptr + Hkv * D * 2, do.ptr, dl.ptr, B, Hq, Hkv, Sq, Sk, D, strides,
                ctypes.c_float(D ** -0.5), causal, 0, ctypes.c_float(0.0), 0 if f32_out else 1, None)
        case = (seed, B, Hq, Hkv, Sq, Sk, D, causal, f32_out, st, g0, g1, g2)
        assert rc == 0, case
        lane.synchronize()
        got = do.download((B, Sq, Wo), np.float32 if f32_out else np.uint16)[:, :, :Hq * D].reshape(B, Sq, Hq, D)
        got_lse = dl.download((B, Hq, Sq), np.float32)
        # compacted [B, H, S, D] copies through the contiguous entry point
        q4 = np.ascontiguousarray(qb[:, :, g0:g0 + Hq * D].reshape(B, Sq, Hq, D).transpose(0, 2, 1, 3))
        k4 = np.ascontiguousarray(kvb[:, :, :Hkv * D].reshape(B, Sk, Hkv, D).transpose(0, 2, 1, 3))
        v4 = np.ascontiguousarray(kvb[:, :, Hkv * D:2 * Hkv * D].reshape(B, Sk, Hkv, D).transpose(0, 2, 1, 3))
        wrap = (lambda a: b16.from_bits(a)) if st == "bf16" else (lambda a: a.view(np.float16))
        ref, ref_lse = ops.gqa_attention(wrap(q4), wrap(k4), wrap(v4), causal=bool(causal), return_lse=True,
                                         out="f32" if f32_out else "storage")
        ref_bits = np.asarray(ref, np.float32) if f32_out else bits(ref)
        assert np.array_equal(got.transpose(0, 2, 1, 3), ref_bits), case
        assert np.array_equal(got_lse, ref_lse), case
        for buf in (dq, dkv, do, dl):
            buf.close()


def _tie_free_logits(rng, T, E, k):
    for _ in range(50):
        lg = rng.standard_normal((T, E)).astype(np.float32)
        if not orc.has_routing_ties(orc.router_probs(lg), k):
            return lg
    raise AssertionError("could not draw tie-free logits")


@pytest.mark.parametrize("seed", range(4 * SCALE))
def test_routing_random_shapes_bit_exact(lane, seed):
    rng = np.random.default_rng(6000 + seed)
    for _ in range(40):
        T = int(rng.integers(1, 700))
        E = int(rng.choice([1, 2, 3, 8, 17, 64, 65, 130]))
        k = int(rng.integers(1, min(E, 8) + 1))
        normalize = bool(rng.integers(0, 2))
        cf = float(rng.choice([1e9, 1e9, 0.5, 1.0, 1.25]))
        lg = _tie_free_logits(rng, T, E, k)
        r = orc.route_tokens(lg, E, k, normalize_weights=normalize, capacity_factor=cf)
        desc = orc.plan_dispatch(r.assignment, r.weights, E)
        plan = ops.route_tokens(lg, E, k, normalize_weights=normalize, capacity_factor=cf)
        case = (seed, T, E, k, normalize, cf)
        assert plan.num_slots == T * k - r.overflow, case
        assert np.array_equal(plan.token_of_slot, desc.token_of_slot), case
        assert np.array_equal(plan.expert_of_slot, desc.expert_of_slot), case
        assert np.array_equal(plan.group_sizes, desc.group_sizes), case
        assert np.array_equal(plan.group_offsets, desc.group_offsets), case
        np.testing.assert_allclose(plan.combine_weights, desc.combine_weights, rtol=2e-6, atol=1e-9)
        # the second router on the same logits: selection on the logits, weights over the selected ones
        ids, w = ops.route_top_k(lg, k, normalize=normalize)
        rids, rw = orc.route_top_k_stable(lg, k, normalize=normalize)
        assert np.array_equal(ids, rids), case
        np.testing.assert_allclose(w, rw, rtol=2e-6, atol=1e-9)


@pytest.mark.parametrize("seed", range(3 * SCALE))
def test_grouped_gemm_random_groups(lane, seed):
    rng = np.random.default_rng(7000 + seed)
    for _ in range(15):
        E = int(rng.integers(1, 24))
        sizes = rng.integers(0, 300, E) * rng.integers(0, 2, E)      # about half the groups empty
        if rng.integers(0, 3) == 0:
            sizes[int(rng.integers(0, E))] += int(rng.integers(250, 700))   # one long group: several row tiles
        T = int(sizes.sum())
        if T == 0:
            sizes[0] = T = 5
        K, N = _dim(rng, 520, True), _dim(rng, 520, True)
        x = b16.from_float32(rng.standard_normal((T, K)).astype(np.float32) * 0.5)
        w = b16.from_float32(rng.standard_normal((E, K, N)).astype(np.float32) * 0.5)
        ref = orc.grouped_gemm(x.to_float32(), w.to_float32(), sizes, store=False)
        got = ops.grouped_gemm(x, w, sizes, out="f32")
        assert orc.max_rel_err(got, ref) <= 1e-5, (seed, E, T, K, N)
        stored = ops.grouped_gemm(x, w, sizes)
        assert np.array_equal(np.asarray(stored).view(np.uint16), np.asarray(b16.from_float32(got)).view(np.uint16))


@pytest.mark.parametrize("seed", range(4 * SCALE))
def test_attention_backward_random_shapes(lane, seed):
    """dQ, dK, dV against the f64 gradients of the same 16-bit inputs; bounds as in the
    hand-picked backward tests (2e-3 f16, 5e-3 bf16: P and dS are rounded to the storage dtype
    once before the second products)."""
    rng = np.random.default_rng(8000 + seed)
    bound = {"f16": 2e-3, "bf16": 5e-3}
    for _ in range(12):
        B = int(rng.integers(1, 3))
        Hkv = int(rng.integers(1, 4))
        ratio = int(rng.choice([1, 1, 2, 4]))
        if rng.integers(0, 4) == 0:
            B, Hkv = 1, 8
        D = int(rng.choice([32, 48, 64, 64, 128, 128]))
        Sq, Sk = int(rng.integers(1, 330)), int(rng.integers(1, 330))
        causal = bool(rng.integers(0, 2))
        st = "bf16" if rng.integers(0, 2) else "f16"
        q = _store(rng.standard_normal((B, Hkv * ratio, Sq, D)).astype(np.float32), st)
        k = _store(rng.standard_normal((B, Hkv, Sk, D)).astype(np.float32), st)
        v = _store(rng.standard_normal((B, Hkv, Sk, D)).astype(np.float32), st)
        do = _store(rng.standard_normal((B, Hkv * ratio, Sq, D)).astype(np.float32), st)
        ref = orc.flash_attn_backward(_f32(do), _f32(q), _f32(k), _f32(v), causal=causal)
        got = ops.flash_attn_backward(do, q, k, v, causal=causal)
        case = (seed, B, Hkv, ratio, Sq, Sk, D, causal, st)
        for g, r, name in zip(got, ref, ("dQ", "dK", "dV")):
            assert g.shape == r.shape and not np.isnan(g).any(), (name, case)
            assert orc.max_rel_err(g, r) <= bound[st], (name, case)


@pytest.mark.parametrize("seed", range(3 * SCALE))
def test_moe_layer_random_shapes(lane, seed):
    """The whole layer (router product, routing, expert block, combine) on random sizes: the
    plan's indices bit-exact, the output within the bf16 stage-rounding bound of the layer tests."""
    rng = np.random.default_rng(9000 + seed)
    for _ in range(5):
        T = int(rng.integers(1, 400))
        H = _dim(rng, 200, True)
        F = _dim(rng, 260, True)
        E = int(rng.choice([1, 2, 4, 8, 17, 64]))
        k = int(rng.integers(1, min(E, 4) + 1))
        x = rng.standard_normal((T, H)).astype(np.float32)
        wr = (rng.standard_normal((H, E)) / np.sqrt(H)).astype(np.float32)
        wg, wu = ((rng.standard_normal((E, H, F)) / np.sqrt(H)).astype(np.float32) for _ in range(2))
        wd = (rng.standard_normal((E, F, H)) / np.sqrt(F)).astype(np.float32)
        xb, wrb, wgb, wub, wdb = (b16.from_float32(a) for a in (x, wr, wg, wu, wd))
        # the router product as the layer computes it: bf16 result of the f32-accumulated GEMM
        logits = ops.gemm(xb, wrb).to_float32()
        if orc.has_routing_ties(orc.router_probs(logits), k):
            continue
        ref, desc = orc.moe_layer(xb.to_float32(), logits, wgb.to_float32(), wub.to_float32(), wdb.to_float32(), k)
        got, plan = ops.moe_layer(xb, wrb, wgb, wub, wdb, top_k=k, return_plan=True)
        case = (seed, T, H, F, E, k)
        assert got.shape == (T, H) and got.dtype == np.float32
        assert np.array_equal(plan.token_of_slot, desc.token_of_slot), case
        assert np.array_equal(plan.expert_of_slot, desc.expert_of_slot), case
        assert np.array_equal(plan.group_offsets, desc.group_offsets), case
        assert orc.max_rel_err(got, ref) <= TOL + 2.0 ** -8, case
