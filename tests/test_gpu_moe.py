"""MoE parity on the MI355X: routing / permutation indices bit-exact against the
oracle; grouped GEMM, SwiGLU block and the whole layer within 2e-3 (normwise)
of the oracle computed with the reference's storage-rounding rule."""
import numpy as np
import pytest

import tessera_oracle as orc
from tessera_amd import bf16 as b16
from tessera_amd import ops

pytestmark = pytest.mark.gpu
TOL = 2e-3


def _logits(T, E, seed, k):
    """Seeded N(0,1) router logits with no bit-equal probabilities inside any
    token's top-(k+1) (the one case where the reference's unstable argsort leaves
    the order unspecified); re-seed until that holds."""
    for s in range(seed, seed + 50):
        lg = np.random.default_rng(s).standard_normal((T, E)).astype(np.float32)
        if not orc.has_routing_ties(orc.router_probs(lg), k):
            return lg
    raise AssertionError("could not draw tie-free logits")


def _check_plan(plan, desc):
    assert np.array_equal(plan.token_of_slot, desc.token_of_slot)
    assert np.array_equal(plan.expert_of_slot, desc.expert_of_slot)
    assert np.array_equal(plan.group_sizes, desc.group_sizes)
    assert np.array_equal(plan.group_offsets, desc.group_offsets)
    assert plan.token_of_slot.dtype == np.int32 and plan.group_offsets.dtype == np.int32
    np.testing.assert_allclose(plan.combine_weights, desc.combine_weights, rtol=2e-6, atol=1e-9)


@pytest.mark.parametrize("T,E,k", [(128, 8, 2), (1000, 64, 8), (37, 5, 5), (512, 130, 3), (8192, 64, 8), (64, 16, 1)])
@pytest.mark.parametrize("normalize", [True, False])
def test_routing_indices_bit_exact(lane, T, E, k, normalize):
    lg = _logits(T, E, 100 + T, k)
    r = orc.route_tokens(lg, E, k, normalize_weights=normalize)
    desc = orc.plan_dispatch(r.assignment, r.weights, E)
    plan = ops.route_tokens(lg, E, k, normalize_weights=normalize, capacity_factor=1e9)
    assert plan.num_slots == T * k
    _check_plan(plan, desc)
    # invariants of the packing (models/moe_routing.py:47-51)
    assert int(plan.group_sizes.sum()) == T * k
    assert np.all(np.diff(plan.expert_of_slot) >= 0)
    for e in range(E):
        seg = plan.token_of_slot[plan.group_offsets[e]:plan.group_offsets[e + 1]]
        assert np.all(np.diff(seg) > 0)


@pytest.mark.parametrize("T,E,k,cf", [(256, 8, 2, 1.0), (1000, 16, 4, 0.5), (300, 4, 2, 1.25)])
def test_routing_with_capacity_drops(lane, T, E, k, cf):
    lg = _logits(T, E, 7, k)
    r = orc.route_tokens(lg, E, k, capacity_factor=cf)
    assert r.overflow > 0
    desc = orc.plan_dispatch(r.assignment, r.weights, E)
    plan = ops.route_tokens(lg, E, k, capacity_factor=cf)
    assert plan.num_slots == T * k - r.overflow
    _check_plan(plan, desc)


def test_routing_ties_go_to_lowest_expert(lane):
    lg = np.zeros((16, 8), np.float32)                      # every probability equal
    plan = ops.route_tokens(lg, 8, 3, capacity_factor=1e9)
    assert np.array_equal(plan.group_sizes, [16, 16, 16, 0, 0, 0, 0, 0])
    assert np.allclose(plan.combine_weights, 1.0 / 3.0)


def test_routing_non_finite_rows_stay_in_range(lane):
    """Rows whose softmax is NaN (a NaN or +inf logit, a row of -inf) take experts
    0..k-1 with NaN weights, as the oracle's stable sort gives them; every index of the
    plan stays inside its range and finite rows route as they would alone."""
    T, E, k = 300, 64, 8
    lg = _logits(T, E, 31, k)
    lg[5, 17] = np.nan
    lg[77, 0] = np.inf
    lg[123, :] = -np.inf
    lg[299, 63] = np.nan
    with np.errstate(invalid="ignore"):
        r = orc.route_tokens(lg, E, k)
        desc = orc.plan_dispatch(r.assignment, r.weights, E)
    plan = ops.route_tokens(lg, E, k, capacity_factor=1e9)
    assert plan.num_slots == T * k
    assert np.array_equal(plan.token_of_slot, desc.token_of_slot)
    assert np.array_equal(plan.expert_of_slot, desc.expert_of_slot)
    assert np.array_equal(plan.group_offsets, desc.group_offsets)
    assert np.array_equal(np.isnan(plan.combine_weights), np.isnan(desc.combine_weights))
    ok = ~np.isnan(desc.combine_weights)
    np.testing.assert_allclose(plan.combine_weights[ok], desc.combine_weights[ok], rtol=2e-6, atol=1e-9)
    assert int(np.isnan(plan.combine_weights).sum()) == 4 * k


@pytest.mark.parametrize("T,E,k", [(257, 64, 8), (1000, 40, 6), (64, 8, 1), (33, 5, 5)])
@pytest.mark.parametrize("normalize", [True, False])
def test_route_top_k_and_packing_plan(lane, T, E, k, normalize):
    """The reference's second router (top-k of the logits, softmax over the selected
    ones or 1/k) and its packing plan: expert ids, sort_perm, inverse_perm, kept_mask and
    group sizes bit for bit against the oracle, weights to f32 rounding."""
    lg = np.random.default_rng(900 + T).standard_normal((T, E)).astype(np.float32)
    lg[T // 2, 1] = lg[T // 2, 3] = 9.0                   # a tie at the top: lower id first
    lg[T // 3, :] = -0.5                                   # a row of ties takes experts 0..k-1
    ids, w = ops.route_top_k(lg, k, normalize=normalize)
    rids, rw = orc.route_top_k_stable(lg, k, normalize=normalize)
    assert ids.dtype == np.int64 and np.array_equal(ids, rids)
    np.testing.assert_allclose(w, rw, rtol=3e-6, atol=1e-9)
    if k >= 2:
        assert list(ids[T // 2][:2]) == [1, 3]
    assert list(ids[T // 3]) == list(range(k))
    for cap in (None, max(1, (T * k) // (2 * E))):
        plan = ops.plan_dispatch(ids, w, E, capacity=cap)
        want = orc.plan_dispatch_token_major(rids, w, E, capacity=cap)
        assert np.array_equal(plan.kept_mask, want.kept_mask)
        assert np.array_equal(plan.sort_perm, want.sort_perm)
        assert np.array_equal(plan.inverse_perm, want.inverse_perm)
        assert np.array_equal(plan.group_sizes, want.group_sizes)
        assert np.array_equal(plan.transport.token_of_slot, want.sort_perm // k)
        assert np.array_equal(plan.transport.combine_weights, w.reshape(-1)[want.sort_perm])
        assert (cap is None) == plan.round_trips()
        if cap is not None:
            assert plan.num_kept < T * k and plan.drop_fraction > 0
    pk = ops.plan_packing(ids, E)
    assert pk.round_trips() and np.array_equal(pk.sort_perm, orc.plan_dispatch_token_major(rids, w, E).sort_perm)
    with pytest.raises(ValueError):
        ops.plan_packing(np.full((4, 2), E), E)


def test_pack_and_unpack_combine(lane):
    """pack_tokens / unpack_combine (models/moe_routing.py:102-116): the packed rows are
    an exact gather, and the token-major k-sum equals the oracle's bit for bit in f32."""
    T, E, k, H = 300, 16, 4, 72
    rng = np.random.default_rng(77)
    lg = rng.standard_normal((T, E)).astype(np.float32)
    ids, w = ops.route_top_k(lg, k)
    x = rng.standard_normal((T, H)).astype(np.float32)
    for cap in (None, 50):
        plan = ops.plan_dispatch(ids, w, E, capacity=cap)
        packed = ops.pack_tokens(x, plan)
        assert np.array_equal(packed, x[plan.sort_perm // k])
        y = rng.standard_normal(packed.shape).astype(np.float32)
        got = ops.unpack_combine(y, plan, w)
        assert np.array_equal(got, orc.unpack_combine(y, plan.inverse_perm, w))
        yb = b16.from_float32(y)
        assert np.array_equal(ops.unpack_combine(yb, plan, w), orc.unpack_combine(yb.to_float32(), plan.inverse_perm, w))
    H2 = 37                                                # rows that are not 16-byte multiples
    y2 = rng.standard_normal((plan.num_kept, H2)).astype(np.float32)
    assert np.array_equal(ops.unpack_combine(y2, plan, w), orc.unpack_combine(y2, plan.inverse_perm, w))


def test_dispatch_and_combine(lane):
    T, H, E, k = 300, 96, 8, 2
    lg = _logits(T, E, 1, k)
    plan = ops.route_tokens(lg, E, k, capacity_factor=1e9)
    x = np.random.default_rng(2).standard_normal((T, H)).astype(np.float32)
    xb = b16.from_float32(x)
    xp = ops.moe_dispatch(xb, plan)
    assert np.array_equal(np.asarray(xp, np.uint16), np.asarray(xb, np.uint16)[plan.token_of_slot])
    assert np.array_equal(ops.moe_dispatch(x, plan), x[plan.token_of_slot])
    y = np.random.default_rng(3).standard_normal((plan.num_slots, H)).astype(np.float32)
    desc = orc.TransportDescriptor(plan.token_of_slot, plan.expert_of_slot, plan.combine_weights,
                                   plan.group_sizes, plan.group_offsets, None)
    ref = orc.moe_combine(y, desc, T)
    got = ops.moe_combine(y, plan)
    assert orc.max_rel_err(got, ref) <= 1e-6
    # slot-order accumulation in f32 == a sequential np.add.at in f32
    seq = np.zeros((T, H), np.float32)
    np.add.at(seq, plan.token_of_slot, y * plan.combine_weights[:, None])
    assert np.array_equal(got, seq)
    yb = b16.from_float32(y)
    got_b = ops.moe_combine(yb, plan)
    assert orc.max_rel_err(got_b, orc.moe_combine(yb.to_float32(), desc, T)) <= 1e-6


@pytest.mark.parametrize("sizes,K,N", [
    ([5, 0, 300, 1, 64, 0, 257, 13], 128, 256),
    ([1024], 512, 384),
    ([0, 0, 7], 64, 72),
    ([100, 200, 300, 400], 1408, 512),
    ([3, 5], 24, 40),
    # last row tiles of 64 / 65 rows: either side of the short last-tile form
    ([64, 65, 320, 321, 0, 256], 200, 328),
    # groups of about a tile of rows: last tiles of 65 to 128 rows take the 128-row form, 129 the full one
    ([128, 129, 127, 66, 384, 385, 0, 100], 264, 520),
])
def test_grouped_gemm(lane, sizes, K, N):
    E, T = len(sizes), int(sum(sizes))
    rng = np.random.default_rng(K + N)
    x = rng.standard_normal((T, K)).astype(np.float32)
    w = (rng.standard_normal((E, K, N)) / np.sqrt(K)).astype(np.float32)
    ref = orc.grouped_gemm(x, w, sizes, store=False)
    got = ops.grouped_gemm(b16.from_float32(x), b16.from_float32(w), sizes, out="f32")
    assert orc.max_rel_err(got, ref) <= 1e-5
    stored = ops.grouped_gemm(b16.from_float32(x), b16.from_float32(w), sizes)
    assert np.array_equal(stored.to_float32(), orc.round_to_storage(got, "bf16"))
    with pytest.raises(ValueError):
        ops.grouped_gemm(b16.from_float32(x), b16.from_float32(w), [s + 1 for s in sizes])
    with pytest.raises(NotImplementedError):
        ops.grouped_gemm(b16.from_float32(x), b16.from_float32(w), sizes, kind="masked")


@pytest.mark.parametrize("sizes,K,N", [
    ([5, 0, 300, 1, 64, 0, 257, 13], 128, 256),
    ([100, 200, 300, 400], 1408, 512),
    ([3, 5], 24, 40),
    ([2, 1, 4], 30, 18),                                  # off the 16-byte grid: the per-element kernel
])
def test_grouped_gemm_f16_storage(lane, sizes, K, N):
    """The grouped product on f16 storage: f32 accumulation, result stored back as f16."""
    E, T = len(sizes), int(sum(sizes))
    rng = np.random.default_rng(K * N + 1)
    x = rng.standard_normal((T, K)).astype(np.float16)
    w = (rng.standard_normal((E, K, N)) / np.sqrt(K)).astype(np.float16)
    ref = orc.grouped_gemm(x.astype(np.float32), w.astype(np.float32), sizes, dtype="f16", store=False)
    got = ops.grouped_gemm(x, w, sizes, out="f32")
    assert got.dtype == np.float32 and orc.max_rel_err(got, ref) <= 1e-5
    stored = ops.grouped_gemm(x, w, sizes)
    assert stored.dtype == np.float16 and np.array_equal(stored, got.astype(np.float16))
    with pytest.raises(ValueError):
        ops.grouped_gemm(x, b16.from_float32(w.astype(np.float32)), sizes)        # mixed storage
    with pytest.raises(ValueError):
        ops.grouped_gemm(x, w, sizes, quant="fp8")                                # the quantised paths take bf16


def test_grouped_gemm_more_than_64_experts(lane):
    """The tile kernel looks its expert up 64 groups at a time: 150 experts of 0..300
    rows cross that boundary twice, with empty groups and short last tiles among them."""
    rng = np.random.default_rng(150)
    sizes = [int(v) for v in rng.integers(0, 301, size=150)]
    sizes[3] = sizes[64] = sizes[129] = 0
    E, T, K, N = len(sizes), int(sum(sizes)), 192, 264
    assert T >= 64 * E                      # the 256-row tile form is the one chosen
    x = rng.standard_normal((T, K)).astype(np.float32)
    w = (rng.standard_normal((E, K, N)) / np.sqrt(K)).astype(np.float32)
    ref = orc.grouped_gemm(x, w, sizes, store=False)
    got = ops.grouped_gemm(b16.from_float32(x), b16.from_float32(w), sizes, out="f32")
    assert orc.max_rel_err(got, ref) <= 1e-5


def _swiglu_inputs(sizes, K, F, N, seed):
    E, T = len(sizes), int(sum(sizes))
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((T, K)).astype(np.float32)
    wg = (rng.standard_normal((E, K, F)) * 0.05).astype(np.float32)
    wu = (rng.standard_normal((E, K, F)) * 0.05).astype(np.float32)
    wd = (rng.standard_normal((E, F, N)) * 0.05).astype(np.float32)
    return x, wg, wu, wd


@pytest.mark.parametrize("sizes,K,F,N", [
    ([40, 0, 300, 7], 256, 384, 128),
    ([512], 128, 128, 256),
    ([9, 200], 64, 1408, 320),
    ([3, 5, 0], 24, 40, 56),
    ([64, 65, 320, 321, 0, 256], 200, 328, 136),
    ([128, 129, 127, 66, 384, 385, 0, 100], 264, 520, 200),
])
def test_moe_swiglu_block(lane, sizes, K, F, N):
    x, wg, wu, wd = _swiglu_inputs(sizes, K, F, N, 5)
    ref = orc.moe_swiglu_block(x, wg, wu, wd, sizes)
    got = ops.moe_swiglu_block(*(b16.from_float32(a) for a in (x, wg, wu, wd)), sizes).to_float32()
    # every stage is re-rounded to bf16 in both; accumulation-order differences flip
    # the occasional rounding, so compare to tolerance with the store's roundoff.
    assert orc.max_rel_err(got, ref) <= TOL + 2.0 ** -8
    assert np.mean(got != ref) < 0.05


@pytest.mark.parametrize("T,K,F,N,E,k", [(300, 256, 384, 128, 8, 2), (1024, 128, 1408, 256, 16, 4),
                                          (77, 64, 128, 64, 4, 1)])
def test_swiglu_block_reading_through_the_dispatch_map(lane, T, K, F, N, E, k):
    """The block with the dispatch fused into its first operand load equals
    dispatch followed by the block, bit for bit (the gather is exact)."""
    rng = np.random.default_rng(T)
    plan = ops.route_tokens(_logits(T, E, 3, k), E, k, capacity_factor=1e9)
    S = plan.num_slots
    xb = b16.from_float32(rng.standard_normal((T, K)).astype(np.float32))
    wg, wu = (b16.from_float32((rng.standard_normal((E, K, F)) * 0.1).astype(np.float32)) for _ in range(2))
    wd = b16.from_float32((rng.standard_normal((E, F, N)) * 0.1).astype(np.float32))
    want = ops.moe_swiglu_block(ops.moe_dispatch(xb, plan), wg, wu, wd, plan.group_sizes)
    bufs = [lane.DeviceBuffer.from_host(np.asarray(a, np.uint16)) for a in (xb, wg, wu, wd)]
    dtos = lane.DeviceBuffer.from_host(np.ascontiguousarray(plan.token_of_slot, np.int32))
    doff = lane.DeviceBuffer.from_host(np.ascontiguousarray(plan.group_offsets, np.int32))
    dy = lane.DeviceBuffer(S * N * 2)
    rc = lane.load().tessera_gfx950_moe_swiglu_block_gather_bf16_dev(
        bufs[0].ptr, dtos.ptr, bufs[1].ptr, bufs[2].ptr, bufs[3].ptr, doff.ptr, dy.ptr, None, T, S, K, F, N, E, None)
    lane.check(rc, "swiglu_gather")
    lane.synchronize()
    got = dy.download((S, N), np.uint16)
    assert np.array_equal(got, np.asarray(want, np.uint16))
    for b in bufs + [dtos, doff, dy]:
        b.close()


def test_swiglu_block_with_no_slots_is_a_no_op(lane):
    """No slots (every token dropped, or an empty batch): the block entries return success without
    reading the activation, the dispatch map or the output — null pointers included."""
    K, F, N, E = 64, 128, 64, 4
    w = [lane.DeviceBuffer.from_host(np.zeros((E, a, b), np.uint16)) for a, b in ((K, F), (K, F), (F, N))]
    doff = lane.DeviceBuffer.from_host(np.zeros(E + 1, np.int32))
    lib = lane.load()
    lane.check(lib.tessera_gfx950_moe_swiglu_block_bf16_dev(None, w[0].ptr, w[1].ptr, w[2].ptr, doff.ptr, None, None,
                                                            0, K, F, N, E, None), "swiglu block, no slots")
    lane.check(lib.tessera_gfx950_moe_swiglu_block_gather_bf16_dev(None, None, w[0].ptr, w[1].ptr, w[2].ptr, doff.ptr,
                                                                   None, None, 5, 0, K, F, N, E, None),
               "gathering swiglu block, no slots")
    lane.synchronize()
    for b in w + [doff]:
        b.close()


def test_grouped_gemm_fp8_quant(lane):
    """quant="fp8_e4m3": per-tensor e4m3 for x and for every expert's weight, then the
    grouped product (compiler/grouped_layout.py:353-392).  Checked against the oracle's
    quantise-dequantise followed by the f64 grouped product."""
    sizes, K, N = [40, 0, 130, 7], 128, 96
    rng = np.random.default_rng(17)
    x = b16.from_float32(rng.standard_normal((sum(sizes), K)).astype(np.float32))
    w = b16.from_float32((rng.standard_normal((len(sizes), K, N)) * 0.2).astype(np.float32))
    got = ops.grouped_gemm(x, w, sizes, quant="fp8_e4m3", out="f32")
    def qdq(a):
        _, grid, scale = orc.quantize_fp8_e4m3(a)
        return grid.astype(np.float64) * np.float64(scale)
    xq = qdq(x.to_float32())
    ref = np.zeros((sum(sizes), N))
    row = 0
    for e, n in enumerate(sizes):
        ref[row:row + n] = xq[row:row + n] @ qdq(w.to_float32()[e])
        row += n
    assert orc.max_rel_err(got, ref) <= 1e-4              # f32 accumulation of exact products
    # and within the fp8 budget of the unquantised product
    assert orc.max_rel_err(got, orc.grouped_gemm(x.to_float32(), w.to_float32(), sizes, store=False)) <= 3e-2 * 4
    stored = ops.grouped_gemm(x, w, sizes, quant="fp8")
    assert np.array_equal(np.asarray(stored, np.uint16), np.asarray(b16.from_float32(got), np.uint16))
    with pytest.raises(ValueError):
        ops.grouped_gemm(x, w, sizes, quant="fp9")                # not one of the reference's schemes


def test_single_expert_reduces_to_dense_swiglu(lane):
    """E = 1 is the dense SwiGLU MLP (tests/unit/test_moe_layer.py:74-79)."""
    x, wg, wu, wd = _swiglu_inputs([200], 128, 256, 128, 9)
    xb, gb, ub, db = (b16.from_float32(a) for a in (x, wg, wu, wd))
    blk = ops.moe_swiglu_block(xb, gb, ub, db, [200]).to_float32()
    gate = ops.gemm(xb, b16.from_bits(np.asarray(gb, np.uint16)[0])).to_float32()
    up = ops.gemm(xb, b16.from_bits(np.asarray(ub, np.uint16)[0])).to_float32()
    hidden = b16.from_float32(orc.silu_mul(gate, up))
    dense = ops.gemm(hidden, b16.from_bits(np.asarray(db, np.uint16)[0])).to_float32()
    assert orc.max_rel_err(blk, dense) <= TOL + 2.0 ** -8


@pytest.mark.parametrize("T,H,F,N,E,k,cf", [(256, 128, 256, 128, 8, 2, 0.0), (500, 64, 128, 96, 4, 1, 0.0),
                                            (300, 128, 128, 128, 8, 2, 1.0)])
def test_moe_layer(lane, T, H, F, N, E, k, cf):
    rng = np.random.default_rng(31)
    x = rng.standard_normal((T, H)).astype(np.float32)
    lg = _logits(T, E, 40, k)
    wg = (rng.standard_normal((E, H, F)) * 0.1).astype(np.float32)
    wu = (rng.standard_normal((E, H, F)) * 0.1).astype(np.float32)
    wd = (rng.standard_normal((E, F, N)) * 0.1).astype(np.float32)
    ref, desc = orc.moe_layer(x, lg, wg, wu, wd, k, capacity_factor=cf)
    out, plan = ops.moe_layer(*(b16.from_float32(a) for a in (x,)), None,
                              *(b16.from_float32(a) for a in (wg, wu, wd)),
                              top_k=k, capacity_factor=cf, router_logits=lg, return_plan=True)
    _check_plan(plan, desc)
    assert orc.max_rel_err(out, ref) <= TOL + 2.0 ** -8


def test_moe_layer_with_router_gemm(lane):
    """Router logits from the lane's own GEMM (bf16-rounded, so equal probabilities
    are common): seeds are tried until one has no tie inside any token's top-(k+1),
    the only case in which the reference's expert order is defined."""
    T, H, F, N, E, k = 128, 64, 64, 64, 8, 2
    for seed in range(77, 77 + 400):
        rng = np.random.default_rng(seed)
        x = rng.standard_normal((T, H)).astype(np.float32)
        wr = rng.standard_normal((H, E)).astype(np.float32)
        if not orc.has_routing_ties(orc.router_probs(orc.gemm_storage(x, wr, "bf16")), k):
            break
    else:
        pytest.fail("no tie-free seed found")
    wg, wu = ((rng.standard_normal((E, H, F)) * 0.1).astype(np.float32) for _ in range(2))
    wd = (rng.standard_normal((E, F, N)) * 0.1).astype(np.float32)
    xb, rb = b16.from_float32(x), b16.from_float32(wr)
    scores = ops.gemm(xb, rb).to_float32()                       # storage-rounded router logits
    assert orc.max_rel_err(scores, orc.gemm_storage(x, wr, "bf16")) <= 2.0 ** -7
    assert not orc.has_routing_ties(orc.router_probs(scores), k)
    ref, desc = orc.moe_layer(x, scores, wg, wu, wd, k)
    out, plan = ops.moe_layer(xb, rb, *(b16.from_float32(a) for a in (wg, wu, wd)), top_k=k, return_plan=True)
    _check_plan(plan, desc)
    assert orc.max_rel_err(out, ref) <= TOL + 2.0 ** -8


@pytest.mark.parametrize("cf,use_router", [(0.0, True), (0.75, False), (0.0, False)])
def test_moe_layer_device_resident_entry(lane, cf, use_router):
    """tessera_gfx950_moe_layer_bf16_dev through the C ABI: router product, routing,
    expert block and combine on one stream with every operand resident; a capacity
    leaves the number of kept slots on the device.  Checked against the oracle and,
    bit for bit, against the host-pointer layer (the same kernels)."""
    import ctypes
    T, H, F, N, E, k = 320, 128, 192, 96, 8, 2
    for seed in range(900, 1300):
        rng = np.random.default_rng(seed)
        x = rng.standard_normal((T, H)).astype(np.float32)
        wr = rng.standard_normal((H, E)).astype(np.float32)
        lg = orc.gemm_storage(x, wr, "bf16") if use_router else rng.standard_normal((T, E)).astype(np.float32)
        if not orc.has_routing_ties(orc.router_probs(lg), k):
            break
    else:
        pytest.fail("no tie-free seed found")
    wg, wu = ((rng.standard_normal((E, H, F)) * 0.1).astype(np.float32) for _ in range(2))
    wd = (rng.standard_normal((E, F, N)) * 0.1).astype(np.float32)
    lib = lane.load()
    bits = lambda a: np.ascontiguousarray(np.asarray(b16.from_float32(a), np.uint16))
    dx, dr, dg, du, dd = (lane.DeviceBuffer.from_host(bits(a)) for a in (x, wr, wg, wu, wd))
    dl = lane.DeviceBuffer.from_host(np.ascontiguousarray(lg, np.float32))
    S = T * k
    need = ctypes.c_size_t(0)
    assert lib.tessera_gfx950_moe_layer_workspace_bytes(T, H, F, N, E, k, ctypes.byref(need)) == 0
    dws = lane.DeviceBuffer(need.value)
    dout = lane.DeviceBuffer(T * N * 4)
    dtos, deos, dcw = (lane.DeviceBuffer(S * 4) for _ in range(3))
    dgs, dgo, dn = lane.DeviceBuffer(E * 4), lane.DeviceBuffer((E + 1) * 4), lane.DeviceBuffer(4)
    cap = int(np.ceil(cf * T / E)) if cf > 0 else 0
    rc = lib.tessera_gfx950_moe_layer_bf16_dev(
        dx.ptr, dr.ptr if use_router else None, None if use_router else dl.ptr, dg.ptr, du.ptr, dd.ptr, dout.ptr,
        dws.ptr, need.value, T, H, F, N, E, k, 1, cap, dtos.ptr, deos.ptr, dcw.ptr, dgs.ptr, dgo.ptr, dn.ptr, None)
    lane.check(rc, "moe_layer_dev")
    lane.synchronize()
    n = int(dn.download((1,), np.int32)[0])
    got = dout.download((T, N), np.float32)
    ref, desc = orc.moe_layer(x, lg, wg, wu, wd, k, capacity_factor=cf)
    assert n == desc.token_of_slot.size and (cf == 0.0) == (n == S)
    assert np.array_equal(dtos.download((S,), np.int32)[:n], desc.token_of_slot)
    assert np.array_equal(deos.download((S,), np.int32)[:n], desc.expert_of_slot)
    assert np.array_equal(dgo.download((E + 1,), np.int32), desc.group_offsets)
    assert orc.max_rel_err(got, ref) <= TOL + 2.0 ** -8
    host = ops.moe_layer(b16.from_float32(x), b16.from_float32(wr) if use_router else None,
                         *(b16.from_float32(a) for a in (wg, wu, wd)), top_k=k, capacity_factor=cf,
                         router_logits=None if use_router else lg)
    assert np.array_equal(got.view(np.uint32), np.asarray(host, np.float32).view(np.uint32))
    # a workspace that is too small is refused before anything is launched
    assert lib.tessera_gfx950_moe_layer_bf16_dev(
        dx.ptr, None, dl.ptr, dg.ptr, du.ptr, dd.ptr, dout.ptr, dws.ptr, need.value - 256, T, H, F, N, E, k, 1, 0,
        dtos.ptr, deos.ptr, dcw.ptr, dgs.ptr, dgo.ptr, dn.ptr, None) == lane.BAD_SHAPE


def test_moe_headline_config(lane):
    """The full MoE configuration (8192 tokens, hidden 4096, 64 experts, top-8,
    F = 1408): routing / permutation indices bit-exact, and the layer output of a
    sample of tokens against the oracle's expert FFN on exactly those rows.  The
    expert weights are one seeded N(0, 0.02) block per matrix, re-used for every
    expert with a different row rotation and sign pattern (drawing 1.1e9 normals
    would dominate the test)."""
    T, H, F, E, k = 8192, 4096, 1408, 64, 8
    rng = np.random.default_rng(2024)
    x = b16.from_float32(rng.standard_normal((T, H), dtype=np.float32))
    lg = _logits(T, E, 500, k)

    def expert_weights(rows, cols, seed):
        r = np.random.default_rng(seed)
        base = np.asarray(b16.from_float32(0.02 * r.standard_normal((rows, cols), dtype=np.float32)), np.uint16)
        flip = (r.integers(0, 2, (rows, cols), dtype=np.uint16) << 15).astype(np.uint16)
        w = np.empty((E, rows, cols), np.uint16)
        for e in range(E):
            w[e] = np.roll(base, 17 * e + 3, axis=0) ^ np.roll(flip, 5 * e + 1, axis=1)
        return b16.from_bits(w)

    wg, wu, wd = expert_weights(H, F, 1), expert_weights(H, F, 2), expert_weights(F, H, 3)
    out, plan = ops.moe_layer(x, None, wg, wu, wd, top_k=k, router_logits=lg, return_plan=True)
    r = orc.route_tokens(lg, E, k)
    desc = orc.plan_dispatch(r.assignment, r.weights, E)
    _check_plan(plan, desc)
    assert out.shape == (T, H) and not np.isnan(np.asarray(out, np.float32)).any()

    tokens = np.sort(rng.choice(T, 20, replace=False))
    slots = np.flatnonzero(np.isin(desc.token_of_slot, tokens))           # slot order: expert-major
    tok_of = desc.token_of_slot[slots].astype(np.int64)
    exp_of = desc.expert_of_slot[slots].astype(np.int64)
    xs = x.to_float32()[tok_of]
    y = np.zeros((slots.size, H), np.float32)
    for e in np.unique(exp_of):
        rows = np.flatnonzero(exp_of == e)
        y[rows] = orc.moe_swiglu_block(xs[rows], wg[e:e + 1].to_float32(), wu[e:e + 1].to_float32(),
                                       wd[e:e + 1].to_float32(), [rows.size])
    ref = np.zeros((T, H), np.float64)
    np.add.at(ref, tok_of, y.astype(np.float64) * desc.combine_weights[slots][:, None].astype(np.float64))
    got = np.asarray(out, np.float32)[tokens]
    assert orc.max_rel_err(got, ref[tokens]) <= TOL + 2.0 ** -8


def test_silu_mul_on_the_storage_grid(lane):
    """ops.silu_mul: silu(a) * b on 16-bit storage, rounded to the same storage; odd length and
    both dtypes; the unquantised block equals grouped products around it."""
    rng = np.random.default_rng(61)
    for n in (1, 7, 4096, 100003):
        a = (rng.standard_normal(n) * 3).astype(np.float32)
        b = rng.standard_normal(n).astype(np.float32)
        for st in ("bf16", "f16"):
            aa = b16.from_float32(a) if st == "bf16" else a.astype(np.float16)
            bb = b16.from_float32(b) if st == "bf16" else b.astype(np.float16)
            af = aa.to_float32() if st == "bf16" else aa.astype(np.float32)
            bf = bb.to_float32() if st == "bf16" else bb.astype(np.float32)
            got = ops.silu_mul(aa, bb)
            gf = got.to_float32() if st == "bf16" else got.astype(np.float32)
            ref = (af.astype(np.float64) / (1 + np.exp(-af.astype(np.float64)))) * bf
            assert np.max(np.abs(gf - ref) / (np.abs(ref) + 1e-3)) <= (2.0 ** -8 if st == "bf16" else 2.0 ** -11) + 1e-5
    sizes = [40, 0, 300, 7]
    x, wg, wu, wd = _swiglu_inputs(sizes, 256, 384, 128, 3)
    xb, g, u, d = (b16.from_float32(t) for t in (x, wg, wu, wd))
    fused = ops.moe_swiglu_block(xb, g, u, d, sizes).to_float32()
    staged = ops.grouped_gemm(ops.silu_mul(ops.grouped_gemm(xb, g, sizes), ops.grouped_gemm(xb, u, sizes)), d, sizes).to_float32()
    assert orc.max_rel_err(staged, fused) <= 2.0 ** -7          # the same roundings; exp differs in its last bits


@pytest.mark.parametrize("quant,budget", [("nvfp4", 0.30), ("fp8_e4m3", 0.10)])
def test_quantised_swiglu_block_and_layer(lane, quant, budget):
    """moe_swiglu_block(quant=) is the reference's composition — three quantised grouped products
    around silu_mul — and moe_layer(quant=) carries it through routing, dispatch and combine.
    Against the unquantised block inside a format budget, against the oracle's composition
    normwise (a hidden value that sits on a rounding boundary may fall either way), and the
    layer against its own stages."""
    sizes = [48, 0, 304, 16]
    x, wg, wu, wd = _swiglu_inputs(sizes, 256, 384, 128, 5)
    xb, g, u, d = (b16.from_float32(t) for t in (x, wg, wu, wd))
    full = ops.moe_swiglu_block(xb, g, u, d, sizes).to_float32()
    got = ops.moe_swiglu_block(xb, g, u, d, sizes, quant=quant).to_float32()
    assert got.shape == full.shape
    assert np.linalg.norm(got - full) / np.linalg.norm(full) < budget
    if quant == "nvfp4":
        f = lambda t: t.to_float32()
        st = lambda t: orc.round_to_storage(np.asarray(t, np.float32), "bf16")
        gate = st(orc.grouped_gemm_nvfp4(f(xb), f(g), sizes))
        up = st(orc.grouped_gemm_nvfp4(f(xb), f(u), sizes))
        hid = st(orc.silu_mul(gate, up))
        ref = st(orc.grouped_gemm_nvfp4(hid, f(d), sizes))
        assert np.linalg.norm(got - ref) / np.linalg.norm(ref) < 2e-2
    with pytest.raises(ValueError):
        ops.moe_swiglu_block(xb, g, u, d, sizes, quant=quant, alignment=32)       # 48 and 304 are multiples of 16 only
    assert ops.moe_swiglu_block(xb, g, u, d, sizes, quant=quant, alignment=16).shape == full.shape
    # the layer
    T, H, F, N, E, k = 200, 256, 384, 128, 4, 2
    rng = np.random.default_rng(8)
    xl = b16.from_float32(rng.standard_normal((T, H)).astype(np.float32))
    lg = _logits(T, E, 41, k)
    plain, plan0 = ops.moe_layer(xl, None, g, u, d, top_k=k, router_logits=lg, return_plan=True)
    out, plan = ops.moe_layer(xl, None, g, u, d, top_k=k, router_logits=lg, quant=quant, return_plan=True)
    assert np.array_equal(plan.token_of_slot, plan0.token_of_slot) and np.array_equal(plan.group_sizes, plan0.group_sizes)
    assert np.linalg.norm(out - plain) / np.linalg.norm(plain) < budget
    staged = ops.moe_combine(ops.moe_swiglu_block(ops.moe_dispatch(xl, plan), g, u, d, np.asarray(plan.group_sizes),
                                                  quant=quant), plan)
    assert np.array_equal(out, staged)
    aligned = ops.moe_layer(xl, None, g, u, d, top_k=k, router_logits=lg, alignment=1)
    assert orc.max_rel_err(aligned, plain) <= 2.0 ** -6         # the staged unquantised form against the fused layer


@pytest.mark.parametrize("T,E,k,normalize,capacity", [
    (200, 8, 2, True, None), (200, 8, 2, False, None), (517, 64, 8, True, None), (517, 64, 8, True, 40),
    (64, 4, 1, True, 3), (300, 160, 70, True, None), (50, 6, 3, True, 0),
])
def test_route_tokens_with_the_reference_signature(lane, T, E, k, normalize, capacity):
    """route_tokens(scores, MoEConfig, capacity) -> RoutingResult(assignment, weights, load, overflow):
    indices and drops bit-exact, weights to the last bit of the f32 softmax."""
    rng = np.random.default_rng(T + E + k)
    scores = rng.standard_normal((T, E)).astype(np.float32)
    assert not orc.has_routing_ties(orc.router_probs(scores), k)
    cfg = ops.MoEConfig(num_experts=E, top_k=k, normalize_weights=normalize)
    got = ops.route_tokens(scores, cfg, capacity)
    ref = orc.route_tokens(scores, E, k, normalize_weights=normalize, capacity_factor=cfg.capacity_factor, capacity=capacity)
    assert got.assignment.dtype == np.int64 and got.weights.dtype == np.float32 and got.load.dtype == np.int64
    assert np.array_equal(got.assignment, ref.assignment)
    assert np.array_equal(got.load, ref.load) and got.overflow == ref.overflow
    assert np.allclose(got.weights, ref.weights, rtol=2e-6, atol=1e-9)
    assert np.array_equal(got.weights == 0, ref.weights == 0)
    # the same routing as the packed form
    if capacity != 0:
        tr = ops.route_tokens(scores, E, k, normalize_weights=normalize, capacity_factor=cfg.capacity_factor,
                              capacity=capacity)
        assert tr.num_slots == T * k - got.overflow
        assert np.array_equal(np.bincount(got.assignment[got.assignment >= 0], minlength=E), tr.group_sizes)
    with pytest.raises(ValueError):
        ops.route_tokens(scores, ops.MoEConfig(num_experts=E + 1, top_k=k))
    with pytest.raises(ValueError):
        ops.MoEConfig(num_experts=4, top_k=5)
    with pytest.raises(NotImplementedError):
        ops.route_tokens(scores, ops.MoEConfig(num_experts=E, top_k=k, jitter_noise=0.1))


def test_stdlib_moe_spellings(lane):
    """stdlib.moe's dispatch / combine / grouped_swiglu / compute_capacity on a plan object that only
    has the reference's fields (no device descriptor attached)."""
    from types import SimpleNamespace
    rng = np.random.default_rng(21)
    T, E, k, H, F = 96, 6, 2, 64, 48
    logits = rng.standard_normal((T, E)).astype(np.float32)
    ids, w = ops.route_top_k(logits, k, compute_dtype=np.float32)
    cap = ops.compute_capacity(T, k, E, 1.0)
    assert cap == 32 and ops.compute_capacity(0, k, E, 1.0) == 0 and ops.compute_capacity(3, 1, 64, 0.5) == 1
    plan = ops.plan_dispatch(ids, w, E, capacity=cap)
    bare = SimpleNamespace(expert_ids=plan.expert_ids, weights=plan.weights, kept_mask=plan.kept_mask,
                           sort_perm=plan.sort_perm, group_sizes=plan.group_sizes, num_tokens=T, top_k=k, capacity=cap)
    x = b16.from_float32(rng.standard_normal((T, H)).astype(np.float32))
    xp = ops.dispatch(x, bare)
    tok = plan.sort_perm // k
    assert np.array_equal(np.asarray(xp, np.uint16), np.asarray(x, np.uint16)[tok])
    assert np.array_equal(np.asarray(ops.dispatch(x, plan), np.uint16), np.asarray(xp, np.uint16))
    wg, wu = (b16.from_float32((rng.standard_normal((E, H, F)) / 8).astype(np.float32)) for _ in range(2))
    wd = b16.from_float32((rng.standard_normal((E, F, H)) / 7).astype(np.float32))
    yp = ops.grouped_swiglu(xp, wg, wu, wd, plan.group_sizes)
    ref = orc.moe_swiglu_block(xp.to_float32(), wg.to_float32(), wu.to_float32(), wd.to_float32(), plan.group_sizes)
    assert orc.max_rel_err(yp.to_float32(), ref) <= 2e-3 + 2.0 ** -8
    out = ops.combine(yp, bare)
    want = np.zeros((T, H), np.float64)
    flat_w = plan.weights.reshape(-1)
    for i, slot in enumerate(plan.sort_perm):                        # stdlib.moe.combine, as written there
        want[int(slot) // k] += float(flat_w[int(slot)]) * yp.to_float32()[i].astype(np.float64)
    assert out.shape == (T, H) and np.allclose(out, want, rtol=1e-5, atol=1e-6)
    with pytest.raises(NotImplementedError):
        ops.route_top_k(logits, k, compute_dtype=np.float64)
    with pytest.raises(ValueError):
        bad = SimpleNamespace(**{**bare.__dict__, "group_sizes": plan.group_sizes + 1})
        ops.dispatch(x, bad)


def test_route_tokens_facts_the_reference_tests_hold(lane):
    """The statements of the reference's own routing tests (tests/unit/test_moe.py:46-103)."""
    rng = np.random.default_rng(0)
    scores = rng.standard_normal((128, 8)).astype(np.float32)
    res = ops.route_tokens(scores, ops.MoEConfig(num_experts=8, top_k=2))
    assert res.assignment.shape == (128, 2) and res.weights.shape == (128, 2)
    res = ops.route_tokens(scores[:64], ops.MoEConfig(num_experts=8, top_k=2, normalize_weights=True))
    valid = (res.assignment >= 0).all(axis=1)
    assert np.allclose(res.weights.sum(axis=1)[valid], 1.0, atol=1e-5)
    res = ops.route_tokens(scores[:32], ops.MoEConfig(num_experts=8, top_k=1))
    a = res.assignment[:, 0]
    assert ((a[a >= 0] >= 0) & (a[a >= 0] < 8)).all() and res.load.sum() <= 32
    with pytest.raises(ValueError, match="num_experts"):
        ops.route_tokens(np.zeros((32, 4), np.float32), ops.MoEConfig(num_experts=8, top_k=1))
    with pytest.raises(ValueError, match="2D"):
        ops.route_tokens(np.zeros((32,), np.float32), ops.MoEConfig(num_experts=1, top_k=1))
    # equal scores: every token ties; a capacity of one slot per expert overflows
    res = ops.route_tokens(np.ones((16, 4), np.float32), ops.MoEConfig(num_experts=4, top_k=1, expert_capacity=1), capacity=1)
    assert res.overflow > 0 and res.overflow == int((res.assignment < 0).sum())
    assert ops.MoEConfig(num_experts=8, expert_capacity=50).compute_capacity(num_tokens=128) == 50
    assert ops.MoEConfig(num_experts=8, capacity_factor=1.25).compute_capacity(num_tokens=128) == 20


def test_dispatch_combine_round_trip_with_unit_weights(lane):
    """combine(dispatch(x)) with unit weights and no capacity is k times x
    (tests/unit/test_stdlib_moe.py:68-79), on f64 rows as the reference's test feeds them."""
    rng = np.random.default_rng(2)
    H, E, k, T = 8, 5, 2, 10
    x = rng.standard_normal((T, H)).astype(np.float64)
    eids = rng.integers(0, E, size=(T, k)).astype(np.int64)
    plan = ops.plan_dispatch(eids, np.ones((T, k), np.float32), E, capacity=None)
    packed = ops.dispatch(x, plan)
    assert packed.dtype == np.float64 and np.array_equal(packed, x[plan.sort_perm // k])
    np.testing.assert_allclose(ops.combine(packed, plan), x * k, rtol=1e-6, atol=1e-6)
    assert ops.compute_capacity(16, 2, 8, 1.5) == 6 and ops.compute_capacity(16, 2, 8, 1.0) == 4
