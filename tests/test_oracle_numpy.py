"""Pins for the numpy oracle: library routines, closed forms, brute force and
the published format tables — chosen so that a dropped term, a wrong sign or a
transposed operand in the oracle fails one of them.  No GPU."""
import math

import numpy as np
import pytest
import torch

import tessera_oracle as orc


# ---- bf16 rounding ------------------------------------------------------------------

def test_bf16_round_trip_and_ties():
    codes = np.arange(1 << 16, dtype=np.uint16)
    vals = orc.bf16_bits_to_f32(codes)
    finite = np.isfinite(vals)
    assert np.array_equal(orc.f32_to_bf16_bits(vals[finite]), codes[finite])
    # ties: 1 + 2^-8 is halfway between 1 (even mantissa) and 1 + 2^-7 -> rounds to 1;
    # 1 + 3*2^-8 is halfway between 1+2^-7 (odd) and 1+2^-6 (even) -> rounds up.
    x = np.array([1 + 2.0 ** -8, 1 + 3 * 2.0 ** -8, -(1 + 2.0 ** -8), 1 + 2.0 ** -8 + 2.0 ** -20], np.float32)
    got = orc.bf16_bits_to_f32(orc.f32_to_bf16_bits(x))
    assert list(got) == [1.0, 1 + 2.0 ** -6, -1.0, 1 + 2.0 ** -7]


def test_bf16_matches_torch():
    rng = np.random.default_rng(0)
    x = (rng.standard_normal(200000) * np.exp(rng.uniform(-30, 30, 200000))).astype(np.float32)
    ours = orc.round_to_storage(x, "bf16")
    theirs = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(ours, theirs)
    assert np.array_equal(orc.round_to_storage(x, "f16"), x.astype(np.float16).astype(np.float32))


# ---- GEMM -----------------------------------------------------------------------------

def test_gemm_closed_forms_and_orientation():
    A = (np.arange(6 * 4) % 5).astype(np.float32).reshape(6, 4)
    B = (np.arange(4 * 3) % 7).astype(np.float32).reshape(4, 3)
    brute = np.array([[sum(A[i, k] * B[k, j] for k in range(4)) for j in range(3)] for i in range(6)])
    assert np.array_equal(orc.gemm_f32(A, B), brute)
    assert np.array_equal(orc.gemm_f64(A, B), brute)
    # operands are rounded to storage BEFORE the product
    a = np.array([[1 + 2.0 ** -10]], np.float32)
    assert orc.gemm_f32(a, np.array([[1024.0]], np.float32))[0, 0] == 1024.0
    assert orc.gemm_f32(a, np.array([[1024.0]], np.float32), "f16")[0, 0] == 1025.0
    # storage rule re-rounds the result; batched leading dims broadcast like np.matmul
    x = np.array([[1.0, 2.0 ** -9]], np.float32)
    y = np.array([[1.0], [1.0]], np.float32)
    assert orc.gemm_f32(x, y)[0, 0] == 1 + 2.0 ** -9
    assert orc.gemm_storage(x, y)[0, 0] == 1.0
    rng = np.random.default_rng(1)
    Ab = rng.standard_normal((4, 8, 16)).astype(np.float32)
    Bb = rng.standard_normal((4, 16, 8)).astype(np.float32)
    got = orc.gemm_f32(Ab, Bb, "f16")
    for i in range(4):
        assert np.allclose(got[i], orc.gemm_f32(Ab[i], Bb[i], "f16"))


# ---- attention --------------------------------------------------------------------------

def _brute_attention(q, k, v, scale, causal):
    B, Hq, Sq, D = q.shape
    Hkv, Sk = k.shape[1], k.shape[2]
    off = max(Sk - Sq, 0)
    O = np.zeros((B, Hq, Sq, D))
    L = np.zeros((B, Hq, Sq))
    for b in range(B):
        for h in range(Hq):
            kh = h // (Hq // Hkv)
            for i in range(Sq):
                js = [j for j in range(Sk) if (not causal) or j <= i + off]
                s = [scale * float(np.dot(q[b, h, i].astype(np.float64), k[b, kh, j])) for j in js]
                m = max(s)
                e = [math.exp(x - m) for x in s]
                z = sum(e)
                O[b, h, i] = sum(ei / z * v[b, kh, j].astype(np.float64) for ei, j in zip(e, js))
                L[b, h, i] = m + math.log(z)
    return O, L


@pytest.mark.parametrize("Sq,Sk,causal", [(5, 5, False), (5, 5, True), (3, 7, True), (7, 3, True)])
def test_attention_against_brute_force(Sq, Sk, causal):
    rng = np.random.default_rng(2)
    q = rng.standard_normal((2, 4, Sq, 8)).astype(np.float32)
    k = rng.standard_normal((2, 2, Sk, 8)).astype(np.float32)
    v = rng.standard_normal((2, 2, Sk, 8)).astype(np.float32)
    bo, bl = _brute_attention(q, k, v, 0.3, causal)
    o, lse = orc.flash_attn_dense(q, k, v, scale=0.3, causal=causal)
    assert np.allclose(o, bo, atol=1e-12) and np.allclose(lse, bl, atol=1e-12)
    o2, lse2 = orc.flash_attn_blockwise(q, k, v, scale=0.3, causal=causal, block=2, dtype=np.float64)
    assert np.allclose(o2, bo, atol=1e-12) and np.allclose(lse2, bl, atol=1e-12)


def test_attention_matches_torch_sdpa_and_gqa_repeat():
    rng = np.random.default_rng(3)
    q = rng.standard_normal((2, 8, 33, 16)).astype(np.float32)
    k = rng.standard_normal((2, 2, 33, 16)).astype(np.float32)
    v = rng.standard_normal((2, 2, 33, 16)).astype(np.float32)
    o, _ = orc.flash_attn_dense(q, k, v, causal=True)
    kr, vr = np.repeat(k, 4, axis=1), np.repeat(v, 4, axis=1)        # nn/functional.py:349-356
    o_rep, _ = orc.flash_attn_dense(q, kr, vr, causal=True)
    assert np.array_equal(o, o_rep)
    t = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q).double(), torch.from_numpy(kr).double(), torch.from_numpy(vr).double(), is_causal=True)
    assert np.allclose(o, t.numpy(), atol=1e-10)
    o_nc, _ = orc.flash_attn_dense(q, kr, vr, causal=False, scale=0.5)
    t2 = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q).double(), torch.from_numpy(kr).double(), torch.from_numpy(vr).double(), scale=0.5)
    assert np.allclose(o_nc, t2.numpy(), atol=1e-10)


def test_attention_region_reference_is_top_left_causal():
    rng = np.random.default_rng(4)
    Q, K, V = (rng.standard_normal((8, 16)).astype(np.float32) * .2 for _ in range(3))
    ref = orc.attention_region_reference(Q, K, V, scale=0.7, causal=True)
    o, _ = orc.flash_attn_dense(Q[None, None], K[None, None], V[None, None], scale=0.7, causal=True)
    assert np.allclose(ref, o[0, 0], atol=1e-6)


# ---- MoE --------------------------------------------------------------------------------

def _brute_route(scores, k, normalize, capacity):
    T, E = scores.shape
    slots = []
    fill = [0] * E
    for t in range(T):
        s = scores[t].astype(np.float32)
        e = np.exp(s - s.max())
        p = e / e.sum()
        order = sorted(range(E), key=lambda i: (-float(p[i]), i))[:k]
        w = np.array([p[i] for i in order], np.float32)
        if normalize and k > 1:
            w = w / w.sum()
        for j, ex in enumerate(order):
            if capacity is not None and fill[ex] >= capacity:
                continue
            fill[ex] += 1
            slots.append((ex, t, float(w[j])))
    slots.sort(key=lambda x: x[0])                       # stable by expert
    return slots


@pytest.mark.parametrize("T,E,k,cap", [(6, 4, 2, None), (9, 3, 3, None), (12, 4, 2, 3), (5, 5, 1, 1)])
def test_routing_against_brute_force(T, E, k, cap):
    rng = np.random.default_rng(T * 7 + E)
    lg = rng.standard_normal((T, E)).astype(np.float32)
    r = orc.route_tokens(lg, E, k, capacity=cap if cap is not None else 10 ** 9)
    d = orc.plan_dispatch(r.assignment, r.weights, E)
    brute = _brute_route(lg, k, True, cap)
    assert [s[1] for s in brute] == list(d.token_of_slot)
    assert [s[0] for s in brute] == list(d.expert_of_slot)
    assert np.allclose([s[2] for s in brute], d.combine_weights, rtol=1e-6)
    assert r.overflow == T * k - len(brute)
    assert np.array_equal(d.group_offsets, np.concatenate(([0], np.cumsum(d.group_sizes))))
    assert np.array_equal(r.load, np.bincount(orc.topk_desc_lowest_index(orc.router_probs(lg), k).ravel(), minlength=E))


def test_the_two_routers_pick_the_same_experts():
    """softmax is monotonic, so top-k of the probabilities (route_tokens) and
    top-k of the logits (route_top_k) select the same expert set absent ties;
    with normalisation both weight vectors are the softmax over the selection."""
    rng = np.random.default_rng(5)
    lg = rng.standard_normal((500, 16)).astype(np.float32)
    assert not orc.has_routing_ties(orc.router_probs(lg), 4)
    r = orc.route_tokens(lg, 16, 4)
    ids, w = orc.route_top_k_stable(lg, 4)
    assert np.array_equal(np.sort(r.assignment, 1), np.sort(ids, 1))
    assert np.array_equal(r.assignment, ids)
    assert np.allclose(r.weights, w, rtol=2e-6)
    assert np.allclose(r.weights.sum(1), 1.0, atol=1e-6)


def test_packing_invariants_and_round_trip():
    rng = np.random.default_rng(6)
    lg = rng.standard_normal((300, 8)).astype(np.float32)
    r = orc.route_tokens(lg, 8, 2)
    d = orc.plan_dispatch(r.assignment, r.weights, 8)
    assert int(d.group_sizes.sum()) == 600
    assert np.all(np.diff(d.expert_of_slot) >= 0)
    for e in range(8):
        seg = d.token_of_slot[d.group_offsets[e]:d.group_offsets[e + 1]]
        assert np.all(np.diff(seg) > 0)
    inv = np.empty_like(d.sort_perm)
    inv[d.sort_perm] = np.arange(600)
    assert np.array_equal(d.sort_perm[inv], np.arange(600))          # models/moe_routing.py:47-51
    # dispatch then combine with unit expert (identity FFN) returns sum_k w * x = x
    x = rng.standard_normal((300, 5)).astype(np.float32)
    y = x[d.token_of_slot]
    back = orc.moe_combine(y, d, 300)
    assert np.allclose(back, x, atol=1e-6)


def test_grouped_gemm_and_swiglu_reductions():
    rng = np.random.default_rng(7)
    x = rng.standard_normal((10, 6)).astype(np.float32)
    w = rng.standard_normal((3, 6, 4)).astype(np.float32)
    sizes = [4, 0, 6]
    got = orc.grouped_gemm(x, w, sizes, store=False)
    xq, wq = orc.round_to_storage(x, "bf16"), orc.round_to_storage(w, "bf16")
    assert np.allclose(got[:4], xq[:4].astype(np.float64) @ wq[0])
    assert np.allclose(got[4:], xq[4:].astype(np.float64) @ wq[2])
    with pytest.raises(ValueError):
        orc.grouped_gemm(x, w, [4, 1, 6])
    # E = 1 reduces to the dense SwiGLU MLP with the same storage roundings
    wg, wu = rng.standard_normal((1, 6, 8)).astype(np.float32), rng.standard_normal((1, 6, 8)).astype(np.float32)
    wd = rng.standard_normal((1, 8, 5)).astype(np.float32)
    blk = orc.moe_swiglu_block(x, wg, wu, wd, [10])
    g, u = orc.gemm_storage(x, wg[0]), orc.gemm_storage(x, wu[0])
    h = orc.round_to_storage(orc.silu_mul(g, u), "bf16")
    assert np.array_equal(blk, orc.gemm_storage(h, wd[0]))
    a = np.array([0.0, 1.0, -2.0], np.float32)
    assert np.allclose(orc.silu_mul(a, np.ones(3, np.float32)), a / (1 + np.exp(-a)))


# ---- quantisation -------------------------------------------------------------------------

def test_e4m3_table_matches_torch_and_spec():
    table = orc.e4m3_decode_table()
    t = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    assert np.array_equal(np.isnan(table), np.isnan(t))
    assert np.array_equal(table[~np.isnan(table)], t[~np.isnan(t)])
    assert table[0x7E] == 448.0 and table[0x01] == 2.0 ** -9 and table[0x08] == 2.0 ** -6 and table[0x38] == 1.0


def test_e4m3_rounding_matches_torch_cast():
    rng = np.random.default_rng(8)
    x = np.concatenate([rng.standard_normal(100000) * 100, rng.standard_normal(100000) * 0.01,
                        np.linspace(-448, 448, 50001), [0.0, -0.0, 2.0 ** -10, 3 * 2.0 ** -10, 447.9, 448.0]])
    x = np.clip(x, -448, 448).astype(np.float32)
    grid = orc.fpquant_grid(x)
    tq = torch.from_numpy(x).to(torch.float8_e4m3fn)
    assert np.array_equal(grid, tq.to(torch.float32).numpy())
    assert np.array_equal(orc.e4m3_encode(grid) & 0x7F, tq.view(torch.uint8).numpy() & 0x7F)
    table = orc.e4m3_decode_table()
    assert np.array_equal(table[orc.e4m3_encode(grid)], grid)


def test_quantize_fp8_scale_and_saturation():
    x = np.array([0.5, -2.0, 896.0, 1e-9], np.float32)
    codes, grid, scale = orc.quantize_fp8_e4m3(x)
    assert scale == np.float32(2.0) and grid[2] == 448.0 and grid[1] == -1.0
    z_codes, z_grid, z_scale = orc.quantize_fp8_e4m3(np.zeros(4, np.float32))
    assert z_scale == np.float32(1e-12) and not z_grid.any()          # amax floor
    c, g, s = orc.quantize_fp8_e4m3(np.array([1e6, -1e6], np.float32), scale=1.0)
    assert list(c) == [0x7E, 0xFE]                                     # tests/unit/test_phase_e_f.py:498-511


def test_nvfp4_grid_scales_and_error_bound():
    """The NVFP4 rounding (block-scaled E2M1) pinned by the format itself and by the bound the
    reference's own tests hold it to: the E2M1 grid by brute force (nearest value, ties to the
    even code), the block scale against torch's e4m3fn cast, closed forms for a zero block
    and a short last block, and the 20 % relative-error budget of
    tests/unit/test_grouped_gemm_contract.py:158-169 on a grouped product."""
    grid = np.array([0, 0.5, 1, 1.5, 2, 3, 4, 6], np.float64)          # E2M1: codes 0..7 in order
    xs = np.concatenate([np.linspace(-7, 7, 56001), (grid[:-1] + grid[1:]) / 2, -(grid[:-1] + grid[1:]) / 2])
    want = np.empty_like(xs)
    for i, v in enumerate(np.abs(xs)):
        d = np.abs(grid - v)
        near = np.flatnonzero(d == d.min())
        code = near[0] if near.size == 1 else (near[0] if near[0] % 2 == 0 else near[1])   # tie: even code
        want[i] = grid[code]
    want = np.copysign(want, xs)
    got = orc.fpquant_grid(xs.astype(np.float32), max_normal=6.0, mantissa_bits=1, min_exp=0)
    exact = xs.astype(np.float32).astype(np.float64) == xs              # only points f32 holds exactly are ties
    assert np.array_equal(got[exact], want[exact].astype(np.float32))
    assert np.max(np.abs(got - want)) <= 1.0                            # (a point f32 rounds across a midpoint lands on the neighbour)
    assert np.mean(got == want.astype(np.float32)) > 0.9999
    # a block whose amax is 6 * s for an e4m3-exact s quantises with scale s: values on the grid come back exactly
    blk = np.array([6, -4, 3, 2, 1.5, 1, 0.5, 0, -0.5, -1, -1.5, -2, -3, 4, -6, 0], np.float32)
    for sc in (1.0, 0.375, 2.0 ** -9, 448.0 / 8):
        dq, scales = orc.quantize_nvfp4((blk * np.float32(sc))[None])
        assert scales.shape == (1, 1) and scales[0, 0] == np.float32(sc)
        assert np.array_equal(dq[0], blk * np.float32(sc))
    # the block scale is the e4m3fn cast of amax / 6
    rng = np.random.default_rng(12)
    X = (rng.standard_normal((500, 64)) * np.exp(rng.standard_normal((500, 1)) * 3)).astype(np.float32)
    dq, scales = orc.quantize_nvfp4(X)
    raw = np.maximum(np.abs(X.reshape(500, 4, 16)).max(-1) / np.float32(6.0), np.float32(1e-30)).astype(np.float32)
    tq = torch.from_numpy(np.minimum(raw, np.float32(448.0))).to(torch.float8_e4m3fn).to(torch.float32).numpy()
    assert np.array_equal(scales, tq)
    # every value is code * scale with the code on the grid
    sf = np.where(scales == 0, 1, scales)[..., None]
    codes = np.abs(dq.reshape(500, 4, 16) / sf)
    assert np.isin(codes, grid.astype(np.float32)).all()
    # zero block -> zeros, scale as the cast of the floor (0 in e4m3); short last block == zero-padded block
    z, zs = orc.quantize_nvfp4(np.zeros((2, 32), np.float32))
    assert not z.any() and not zs.any()
    a, sa = orc.quantize_nvfp4(X[:, :40])
    b, sb = orc.quantize_nvfp4(np.concatenate([X[:, :40], np.zeros((500, 8), np.float32)], 1))
    assert np.array_equal(a, b[:, :40]) and np.array_equal(sa, sb)
    # the reference's budget for the grouped product on its own test's shapes
    for gs in ([5, 3, 4], [16, 16, 32]):
        r = np.random.default_rng(9)
        T = sum(gs)
        x = r.standard_normal((T, 64)).astype(np.float32)
        w = r.standard_normal((len(gs), 64, 16)).astype(np.float32)
        full = np.zeros((T, 16)); off = 0
        for e, n in enumerate(gs):
            full[off:off + n] = x[off:off + n].astype(np.float64) @ w[e].astype(np.float64); off += n
        got = orc.grouped_gemm_nvfp4(x, w, gs)
        assert np.linalg.norm(got - full) / np.linalg.norm(full) < 0.20


def test_int8_quantiser_and_w8a8():
    M = np.array([[1.0, -2.0, 0.5], [0.0, 0.0, 0.0], [127.0, 63.5, -64.5]], np.float32)
    q, s = orc.quantize_int8_per_channel(M, axis=1)
    assert np.allclose(s[:, 0], [2 / 127, 1e-12 / 127, 1.0])
    assert list(q[0]) == [64, -127, 32] and list(q[2]) == [127, 64, -64]   # half-to-even
    qc, sc = orc.quantize_int8_per_channel(M, axis=0)
    assert sc.shape == (1, 3) and np.allclose(sc[0], [1.0, 63.5 / 127, 64.5 / 127])
    rng = np.random.default_rng(9)
    X = rng.standard_normal((7, 11)).astype(np.float32)
    W = rng.standard_normal((11, 5)).astype(np.float32)
    y, acc, xq, a_s, wq, w_s = orc.w8a8_matmul(X, W)
    brute = np.array([[sum(int(xq[i, k]) * int(wq[k, j]) for k in range(11)) for j in range(5)] for i in range(7)])
    assert np.array_equal(acc, brute)
    assert np.array_equal(y, acc.astype(np.float32) * a_s * w_s[None, :])
    assert orc.max_rel_err(y, X @ W) < 0.05
    big = np.full((2, 70000), 127, np.int8)
    assert orc.gemm_i8_i32(big, big.T.copy())[0, 0] == 127 * 127 * 70000


def test_flash_attn_backward_matches_torch_autograd_and_finite_differences():
    import torch
    rng = np.random.default_rng(5)
    for (B, Hq, Hkv, Sq, Sk, D, causal) in [(1, 2, 2, 5, 5, 4, False), (2, 4, 2, 6, 9, 8, True), (1, 3, 1, 7, 7, 4, True)]:
        q = rng.standard_normal((B, Hq, Sq, D))
        k = rng.standard_normal((B, Hkv, Sk, D))
        v = rng.standard_normal((B, Hkv, Sk, D))
        do = rng.standard_normal((B, Hq, Sq, D))
        dq, dk, dv = orc.flash_attn_backward(do, q, k, v, causal=causal)
        # library: autograd through torch's attention with K/V repeated along heads
        tq, tk, tv = (torch.tensor(a, requires_grad=True) for a in (q, k, v))
        rep = Hq // Hkv
        kk, vv = tk.repeat_interleave(rep, dim=1), tv.repeat_interleave(rep, dim=1)
        mask = None
        if causal:
            i = torch.arange(Sq)[:, None]
            j = torch.arange(Sk)[None, :]
            mask = j <= i + max(Sk - Sq, 0)
        out = torch.nn.functional.scaled_dot_product_attention(tq, kk, vv, attn_mask=mask)
        out.backward(torch.tensor(do))
        assert np.allclose(dq, tq.grad.numpy(), atol=1e-10)
        assert np.allclose(dk, tk.grad.numpy(), atol=1e-10)
        assert np.allclose(dv, tv.grad.numpy(), atol=1e-10)
        # finite differences of the forward oracle on a few coordinates
        def loss(qq, kk_, vv_):
            o, _ = orc.flash_attn_dense(qq, kk_, vv_, causal=causal)
            return float((o * do).sum())
        eps = 1e-6
        for arr, grad in ((q, dq), (k, dk), (v, dv)):
            idx = tuple(rng.integers(0, n) for n in arr.shape)
            hi, lo = arr.copy(), arr.copy()
            hi[idx] += eps
            lo[idx] -= eps
            args_hi = [hi if a is arr else a for a in (q, k, v)]
            args_lo = [lo if a is arr else a for a in (q, k, v)]
            fd = (loss(*args_hi) - loss(*args_lo)) / (2 * eps)
            assert abs(fd - grad[idx]) <= 1e-6 * max(1.0, abs(fd))


def test_route_tokens_non_finite_rows_keep_indices_in_range():
    """A NaN or +inf logit, or a row of -inf, turns the whole row's probabilities into
    NaN (distributed/moe.py:163-165: the max-subtracted softmax).  numpy's argsort still
    returns valid indices for such a row; the oracle's stable sort orders the NaNs by
    index, so the row takes experts 0..k-1 with NaN weights and finite rows are untouched."""
    rng = np.random.default_rng(11)
    s = rng.standard_normal((6, 8)).astype(np.float32)
    s[1, 3] = np.nan
    s[2, 5] = np.inf
    s[4, :] = -np.inf
    with np.errstate(invalid="ignore"):
        r = orc.route_tokens(s, 8, 3)
    assert r.assignment.min() >= 0 and r.assignment.max() < 8
    for t in (1, 2, 4):
        assert list(r.assignment[t]) == [0, 1, 2]
        assert np.isnan(r.weights[t]).all()
    clean = orc.route_tokens(s[[0, 3, 5]], 8, 3)
    assert np.array_equal(r.assignment[[0, 3, 5]], clean.assignment)
    assert np.array_equal(r.weights[[0, 3, 5]], clean.weights)
    with np.errstate(invalid="ignore"):
        d = orc.plan_dispatch(r.assignment, r.weights, 8)
    assert d.group_offsets[-1] == 18 and np.array_equal(np.sort(d.token_of_slot), np.repeat(np.arange(6), 3))


def test_route_top_k_against_a_per_token_sort_and_library_softmax():
    """models/moe_routing.py:54-77: top-k of the LOGITS, descending, ties to the lowest
    id; weights = softmax over the selected logits (scipy's) or 1/k."""
    from scipy.special import softmax
    rng = np.random.default_rng(5)
    lg = rng.standard_normal((40, 12)).astype(np.float32)
    lg[3, 4] = lg[3, 9] = lg[3].max() + 1.0          # a tie at the top: lower id first
    lg[7, :] = 0.25                                   # a whole row of ties
    ids, w = orc.route_top_k_stable(lg, 3)
    for t in range(40):
        want = sorted(range(12), key=lambda e: (-float(lg[t, e]), e))[:3]
        assert list(ids[t]) == want
        np.testing.assert_allclose(w[t], softmax(lg[t, want].astype(np.float64)), rtol=1e-6)
    assert list(ids[3][:2]) == [4, 9] and list(ids[7]) == [0, 1, 2]
    _, wu = orc.route_top_k_stable(lg, 4, normalize=False)
    assert np.all(wu == np.float32(0.25))


def test_packing_plan_against_an_independent_walk():
    """stdlib/moe.py:79-115 and models/moe_routing.py:80-99, checked by walking each
    expert's slots separately (not the oracle's own argsort)."""
    rng = np.random.default_rng(6)
    T, k, E, cap = 50, 3, 7, 15
    ids = np.stack([rng.permutation(E)[:k] for _ in range(T)])
    w = rng.random((T, k)).astype(np.float32)
    plan = orc.plan_dispatch_token_major(ids, w, E, capacity=cap)
    flat = ids.reshape(-1)
    pos = 0
    for e in range(E):
        slots = [s for s in range(T * k) if flat[s] == e]           # token-major order
        keep, drop = slots[:cap], slots[cap:]
        assert plan.group_sizes[e] == len(keep)
        assert list(plan.sort_perm[pos:pos + len(keep)]) == keep
        assert all(plan.inverse_perm[s] == pos + i for i, s in enumerate(keep))
        assert all(plan.inverse_perm[s] == -1 and not plan.kept_mask.reshape(-1)[s] for s in drop)
        pos += len(keep)
    assert pos == plan.sort_perm.size == int(plan.kept_mask.sum()) < T * k
    full = orc.plan_dispatch_token_major(ids, w, E)
    assert np.array_equal(full.sort_perm[full.inverse_perm], np.arange(T * k)) and full.kept_mask.all()
    # the transport descriptor of route_tokens' plan is the same permutation
    d = orc.plan_dispatch(np.where(plan.kept_mask, ids, -1), w, E)
    assert np.array_equal(d.sort_perm, plan.sort_perm) and np.array_equal(d.token_of_slot, plan.sort_perm // k)
    with pytest.raises(ValueError):
        orc.plan_dispatch_token_major(np.array([[0, 7]]), np.ones((1, 2)), 7)


def test_unpack_combine_closed_forms():
    """models/moe_routing.py:109-116.  k = 1 with weight 1 undoes the packing; equal
    weights 1/k over identical rows give the row back; dropped slots add nothing."""
    rng = np.random.default_rng(8)
    T, k, E, H = 30, 2, 5, 6
    ids = np.stack([rng.permutation(E)[:k] for _ in range(T)])
    plan = orc.plan_dispatch_token_major(ids, np.ones((T, k)), E)
    x = rng.standard_normal((T, H)).astype(np.float32)
    packed = x[plan.sort_perm // k]                                  # every slot carries its token's row
    half = np.full((T, k), 0.5, np.float32)
    assert np.array_equal(orc.unpack_combine(packed, plan.inverse_perm, half), x)
    one = orc.plan_dispatch_token_major(ids[:, :1], np.ones((T, 1)), E)
    assert np.array_equal(orc.unpack_combine(x[one.sort_perm], one.inverse_perm, np.ones((T, 1), np.float32)), x)
    capped = orc.plan_dispatch_token_major(ids, np.ones((T, k)), E, capacity=4)
    got = orc.unpack_combine(x[capped.sort_perm // k], capped.inverse_perm, np.ones((T, k), np.float32))
    assert np.array_equal(got, x * capped.kept_mask.sum(axis=1, keepdims=True).astype(np.float32))
    # against the reference's own slot-order combine (stdlib/moe.py:124-134) on a random case
    y = rng.standard_normal((capped.sort_perm.size, H)).astype(np.float32)
    wts = rng.random((T, k)).astype(np.float32)
    ref = np.zeros((T, H), np.float64)
    for i, slot in enumerate(capped.sort_perm):
        ref[slot // k] += float(wts.reshape(-1)[slot]) * y[i]
    np.testing.assert_allclose(orc.unpack_combine(y, capped.inverse_perm, wts), ref, rtol=1e-5, atol=1e-6)


def test_smoothquant_restatement_closed_forms():
    """migrate_activation_scale / smoothquant_matmul: hand-worked factors at alpha 0, 0.5 and 1, the
    eps floor, reduction to the plain W8A8 path at s = 1, and the migration's defining identity
    (X / s) (s W) = X W within the int8 error."""
    X = np.array([[2.0, -8.0, 0.0], [1.0, 4.0, 0.0]], np.float32)
    W = np.array([[1.0, -0.5], [4.0, 2.0], [0.25, 0.125]], np.float32)
    s, w_q, w_scale = orc.migrate_activation_scale(X, W, alpha=0.5, eps=1e-5)
    # channel maxima: activations (2, 8, 0 -> eps), weights (1, 4, 0.25)
    want = np.array([np.sqrt(2.0 / 1.0), np.sqrt(8.0 / 4.0), np.sqrt(1e-5 / 0.25)])
    assert np.allclose(s, want, rtol=1e-6)
    assert np.allclose(orc.migrate_activation_scale(X, W, alpha=1.0)[0], [2.0, 8.0, 1e-5], rtol=1e-6)
    assert np.allclose(orc.migrate_activation_scale(X, W, alpha=0.0)[0], [1.0, 0.25, 4.0], rtol=1e-6)
    # the weight operand is the column-quantised smoothed weight
    ws = s[:, None] * W
    assert np.array_equal(w_q, np.rint(ws / (np.abs(ws).max(axis=0) / 127)).astype(np.int8))
    assert np.allclose(w_scale, np.abs(ws).max(axis=0) / 127, rtol=1e-6)
    rng = np.random.default_rng(3)
    X = (rng.standard_normal((40, 96)) * np.exp(rng.standard_normal(96))).astype(np.float32)
    W = (rng.standard_normal((96, 24)) / 10).astype(np.float32)
    # s = 1: exactly the unsmoothed path
    wq1, ws1 = orc.quantize_int8_per_channel(W, axis=0)
    y1, acc1, xq1, as1 = orc.smoothquant_matmul(X, np.ones(96, np.float32), wq1, ws1)
    ry, racc, rxq, ras, _, _ = orc.w8a8_matmul(X, W)
    assert np.array_equal(y1, ry) and np.array_equal(acc1, racc) and np.array_equal(xq1, rxq) and np.array_equal(as1, ras)
    # migrated: the product survives, and beats the unsmoothed path on outlier channels
    s, w_q, w_scale = orc.migrate_activation_scale(X, W)
    y, acc, x_q, a_scale = orc.smoothquant_matmul(X, s, w_q, w_scale)
    full = X.astype(np.float64) @ W.astype(np.float64)
    assert np.linalg.norm(y - full) / np.linalg.norm(full) < 0.02
    assert np.linalg.norm(y - full) < np.linalg.norm(ry - full)
    # codes are those of X / s, row scales its row maxima / 127
    xh = X / s[None, :]
    assert np.array_equal(a_scale.reshape(-1), np.abs(xh).max(axis=1) / np.float32(127.0))
    assert np.array_equal(acc, x_q.astype(np.int64) @ w_q.astype(np.int64))


def test_per_tensor_int8_closed_forms():
    """quantize_int8_tensor: a ramp of exact multiples of the scale maps to its own indices, half-way
    points go to the even code, the scale is max|x| / 127, zeros get scale 1, saturation at +-127."""
    ramp = np.arange(-127, 128, dtype=np.float32) * np.float32(0.25)
    q, s = orc.quantize_int8_tensor(ramp)
    assert s == np.float32(127 * 0.25 / 127) and np.array_equal(q, np.arange(-127, 128).astype(np.int8))
    q, _ = orc.quantize_int8_tensor(np.array([0.5, 1.5, 2.5, -0.5, -1.5, 300.0, -300.0], np.float32), scale=1.0)
    assert list(q) == [0, 2, 2, 0, -2, 127, -127]
    q, s = orc.quantize_int8_tensor(np.zeros(5, np.float32))
    assert s == np.float32(1.0) and not q.any()


def test_e5m2_tables_against_the_library_and_the_format():
    """The e5m2 decode table against torch.float8_e5m2 for all 256 codes and against the half-precision
    identity; encode(decode(c)) = c on every finite code; the grid function lands on table values only."""
    import torch
    t = orc.e5m2_decode_table()
    lib = torch.arange(256, dtype=torch.uint8).view(torch.float8_e5m2).to(torch.float32).numpy()
    assert np.array_equal(t, lib, equal_nan=True)
    assert np.array_equal(t, (np.arange(256, dtype=np.uint16) << 8).view(np.float16).astype(np.float32), equal_nan=True)
    finite = np.isfinite(t)
    codes = np.arange(256, dtype=np.uint8)[finite]
    back = orc.e5m2_encode(t[finite])
    assert np.array_equal(back & 0x7F, codes & 0x7F) and np.array_equal(t[back], t[codes])
    rng = np.random.default_rng(9)
    x = (rng.standard_normal(4000) * np.exp(rng.standard_normal(4000) * 4)).astype(np.float32)
    c, grid, s = orc.quantize_fp8_e5m2(x)
    assert np.array_equal(t[c], grid) and np.all(np.abs(grid) <= 57344)
    want = torch.from_numpy(np.clip(x / s, -57344, 57344)).to(torch.float8_e5m2).to(torch.float32).numpy()
    assert np.array_equal(grid, want)                    # the library's own rounding of the same scaled values
