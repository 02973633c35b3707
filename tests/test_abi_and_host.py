"""No-GPU checks: the C-ABI library loads and exports every symbol the header
declares; shape validation happens before the device is touched; the host-side
mirrors of the reference's plugin interfaces behave as the reference's do."""
import ctypes
import re
from pathlib import Path

import numpy as np
import pytest

from tessera_amd import bf16 as b16
from tessera_amd import candidates as cand
from tessera_amd import executors as ex
from tessera_amd import lane, ops, tile_table

ROOT = Path(__file__).resolve().parents[1]


def _header_symbols():
    text = (ROOT / "include" / "tessera_gfx950.h").read_text()
    return sorted(set(re.findall(r"\bint\s+(tessera_gfx950_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = lane.load()
    declared = _header_symbols()
    assert len(declared) >= 60
    for name in declared:
        assert hasattr(lib, name), f"library lacks {name}"
    assert sorted(lane.exported_symbols()) == declared, "ctypes signature table out of step with the header"
    assert lib.tessera_gfx950_abi_version() == 1


def test_header_cites_the_reference_interface_it_replaces():
    text = (ROOT / "include" / "tessera_gfx950.h").read_text()
    for cite in ("tessera_rocm_gemm.cpp:843-856", "tessera_rocm_flash_attn.cpp:259-278", "runtime.py:26657-26715",
                 "moe_transport.py:194-273", "smoothquant.py:115-124", "__init__.py:3340-3374"):
        assert cite in text


def test_shape_validation_precedes_the_device():
    """rc == 1 for a bad shape even with no GPU present (the reference orders its
    checks the same way, tests/unit/test_rocm_wmma_runtime_symbol.py:216-224)."""
    lib = lane.load()
    z = np.zeros(64, np.uint16)
    d = np.zeros(64, np.float32)
    p = lambda a: a.ctypes.data
    assert lib.tessera_gfx950_gemm_bf16(p(z), p(z), p(d), 0, 4, 4) == 1
    assert lib.tessera_gfx950_gemm_f16(p(z), p(z), p(d), 4, 4, -2) == 1
    assert lib.tessera_gfx950_batched_gemm_f16(p(z), p(z), p(d), 0, 4, 4, 4) == 1
    assert lib.tessera_gfx950_gemm_i8_i32(p(z), p(z), p(d), 4, 0, 4) == 1
    assert lib.tessera_gfx950_gemm_bf16(None, p(z), p(d), 4, 4, 4) == 1
    assert lib.tessera_gfx950_flash_attn_bf16(p(z), p(z), p(z), p(d), 1, 1, 4, 4, 24, 1.0, 0) == 1
    assert lib.tessera_gfx950_flash_attn_gqa_f16(p(z), p(z), p(z), p(d), None, 1, 4, 3, 4, 4, 16, 1.0, 0) == 1
    off = np.array([0, 3, 2], np.int32)                        # decreasing offsets
    assert lib.tessera_gfx950_grouped_gemm_bf16(p(z), p(z), p(off), p(z), 2, 8, 8, 2) == 1
    assert lib.tessera_gfx950_moe_route_f32(p(d), 4, 4, 5, 1, 0, p(z), p(z), p(d), p(z), p(z), None) == 1
    tos = np.array([0, 9], np.int32)                           # token index out of range
    assert lib.tessera_gfx950_moe_dispatch(p(z), p(tos), p(z), 4, 2, 8, 2) == 1
    assert lib.tessera_gfx950_quantize_i8_f32(p(d), 4, 4, 2, p(z), p(d)) == 1
    assert lib.tessera_gfx950_bench_last_timer_source() == -1


def test_no_device_is_reported_not_faked():
    if lane.available():
        pytest.skip("a gfx950 device is present")
    lib = lane.load()
    z = np.zeros(256, np.uint16)
    d = np.zeros(256, np.float32)
    assert lib.tessera_gfx950_probe() == 2
    assert lib.tessera_gfx950_gemm_bf16(z.ctypes.data, z.ctypes.data, d.ctypes.data, 16, 16, 16) == 2
    with pytest.raises(lane.LaneUnavailable):
        ops.gemm(b16.from_float32(np.zeros((16, 16))), b16.from_float32(np.zeros((16, 16))))
    with pytest.raises(lane.LaneUnavailable):
        ops.route_tokens(np.zeros((4, 4), np.float32), 4, 2)
    assert not cand.Gfx950MfmaGemmCandidate().available()
    assert cand.arbitrate(cand.MatmulRegion(), cand.OP_MATMUL, cand.TARGET) is None
    with pytest.raises(cand.ArbiterError):
        cand.run_arbitrated(cand.MatmulRegion(), cand.OP_MATMUL, cand.TARGET, np.zeros((32, 32)), np.zeros((32, 16)))


def test_python_side_argument_errors():
    f16 = np.zeros((4, 8), np.float16)
    with pytest.raises(ValueError):
        ops.gemm(f16, np.zeros((9, 4), np.float16))
    with pytest.raises(ValueError):
        ops.gemm(np.zeros((4, 8), np.float32), np.zeros((8, 4), np.float32))       # not 16-bit storage
    with pytest.raises(ValueError):
        ops.gemm(f16, b16.from_float32(np.zeros((8, 4))))                          # mixed storage
    q = np.zeros((1, 4, 8, 24), np.float16)
    with pytest.raises(ValueError):
        ops.flash_attn(q, q, q)                                                    # head_dim % 16
    q = np.zeros((1, 4, 8, 16), np.float16)
    k = np.zeros((1, 3, 8, 16), np.float16)
    with pytest.raises(ValueError):
        ops.gqa_attention(q, k, k)                                                 # 4 % 3
    x = b16.from_float32(np.zeros((6, 8)))
    w = b16.from_float32(np.zeros((2, 8, 8)))
    with pytest.raises(ValueError):
        ops.grouped_gemm(x, w, [3, 4])
    with pytest.raises(ValueError):
        ops.grouped_gemm(x, w, [3, 3], kind="bogus")
    with pytest.raises(NotImplementedError):
        ops.grouped_gemm(x, w, [3, 3], kind="k_grouped")
    with pytest.raises(ValueError):
        ops.grouped_gemm(x, w, [3, 3], alignment=2)
    with pytest.raises(ValueError):
        ops.route_tokens(np.zeros((4, 4), np.float32), 5, 2)
    with pytest.raises(ValueError):
        ops.route_tokens(np.zeros((4, 4), np.float32), 4, 5)
    with pytest.raises(ValueError):
        ops.quantize_fp8(np.zeros(4), format="e3m4")
    # moe_layer: mismatched expert weights are refused before any pointer is handed over
    xm = b16.from_float32(np.zeros((4, 8)))
    lg = np.zeros((4, 2), np.float32)
    wg = b16.from_float32(np.zeros((2, 8, 16)))
    wd = b16.from_float32(np.zeros((2, 16, 8)))
    with pytest.raises(ValueError):
        ops.moe_layer(xm, None, wg, b16.from_float32(np.zeros((2, 8, 12))), wd, top_k=1, router_logits=lg)
    with pytest.raises(ValueError):
        ops.moe_layer(xm, None, b16.from_float32(np.zeros((2, 6, 16))), b16.from_float32(np.zeros((2, 6, 16))), wd,
                      top_k=1, router_logits=lg)
    with pytest.raises(ValueError):
        ops.moe_layer(xm, None, wg, wg, b16.from_float32(np.zeros((3, 16, 8))), top_k=1, router_logits=lg)
    with pytest.raises(ValueError):
        ops.moe_layer(xm, None, wg, wg, b16.from_float32(np.zeros((2, 12, 8))), top_k=1, router_logits=lg)
    with pytest.raises(ValueError):
        ops.moe_layer(xm, None, wg, wg, wd, top_k=3, router_logits=lg)


def test_gather_block_rejects_activations_past_the_buffer_range():
    """The gather form of the expert block reaches a token row through a buffer load
    whose range is 2 GiB from the start of x; rows past it would read as zeros, so
    the launcher refuses such an activation (rc 1) before it touches the device."""
    lib = lane.load()
    fake = 0x1000                                   # never dereferenced: the checks come first
    K = 4096
    rows_over = (0x7fffffff - 16) // (K * 2) + 1    # first row count whose last byte leaves the range
    args = lambda T: (fake, fake, fake, fake, fake, fake, fake, fake, T, 64, K, 64, K, 2, None)
    assert lib.tessera_gfx950_moe_swiglu_block_gather_bf16_dev(*args(rows_over)) == 1
    assert lib.tessera_gfx950_moe_swiglu_block_gather_bf16_dev(*args(300_000)) == 1      # 2.4 GB: was accepted
    if not lane.available():
        # just inside the range the shape is accepted and the call goes on to the device probe
        assert lib.tessera_gfx950_moe_swiglu_block_gather_bf16_dev(*args(rows_over - 1)) == 2


def test_bf16_host_array():
    x = np.array([1.0, 1 + 2.0 ** -8, 1 + 3 * 2.0 ** -8, -2.5, 0.0], np.float32)
    b = b16.from_float32(x)
    assert isinstance(b, b16.BF16Array) and b.dtype == np.uint16
    assert list(b.to_float32()) == [1.0, 1.0, 1 + 2.0 ** -6, -2.5, 0.0]
    assert b16.is_bf16(b) and not b16.is_bf16(x)
    assert np.array_equal(b16.from_bits(np.asarray(b, np.uint16)), b)


def test_execution_rows_and_launch_protocol():
    assert set(ex.executor_table()) == set(ex.KNOWN_EXECUTORS) == {r.executor_id for r in ex.EXECUTION_ROWS.values()}
    row = ex.lookup("rocm_gfx950", "gfx950_gemm")
    assert row.execution_kind == "native_gpu" and row.executable and row.execution_mode == "hip_runtime"
    assert ex.lookup("rocm", "gfx950_gemm") is None
    # an artifact that is not stamped executable is never launched
    art = ex.make_artifact("tessera.matmul", ["a", "b"], ["a", "b"], "gfx950_gemm", executable=False)
    res = ex.launch(art, (np.zeros((4, 4), np.float16),) * 2)
    assert res["ok"] is False and res["runtime_status"] == "unimplemented"
    # executor errors become invalid_artifact, never an exception (runtime.py:31021-31041)
    art = ex.make_artifact("tessera.conv2d", ["a", "b"], ["a", "b"], "gfx950_gemm", executable=True)
    res = ex.launch(art, (np.zeros((4, 4), np.float16),) * 2)
    assert res["ok"] is False and res["runtime_status"] == "invalid_artifact" and "exactly one" in res["reason"]
    art = ex.make_artifact("tessera.matmul", ["a", "b"], ["a", "b"], "gfx950_gemm", executable=True)
    res = ex.launch(art, (np.zeros((4, 5), np.float16), np.zeros((4, 4), np.float16)))
    assert res["runtime_status"] == "invalid_artifact" and "matching K" in res["reason"]
    res = ex.launch(art, (np.zeros((4, 4), np.float16),))
    assert res["runtime_status"] == "invalid_artifact" and "missing value" in res["reason"]
    art = ex.make_artifact("tessera.moe_dispatch", ["x", "plan"], ["x", "plan"], "gfx950_moe_transport", executable=True)
    res = ex.launch(art, {"x": np.zeros((4, 4), np.float32)})
    assert res["runtime_status"] == "invalid_artifact" and "missing moe_dispatch argument 'plan'" in res["reason"]
    if not lane.available():
        art = ex.make_artifact("tessera.matmul", ["a", "b"], ["a", "b"], "gfx950_gemm")
        assert art.metadata["executable"] is False and art.metadata["execution_kind"] == "artifact_only"


def test_plan_lowering_validates_like_the_reference():
    class Plan:
        expert_ids = np.array([[0, 1], [1, 0]])
        weights = np.ones((2, 2), np.float32) / 2
        kept_mask = np.ones((2, 2), bool)
        sort_perm = np.array([0, 3, 1, 2])
        group_sizes = np.array([2, 2])
        num_tokens, top_k, capacity = 2, 2, None
    t = ex._plan_to_transport(Plan)
    assert list(t.token_of_slot) == [0, 1, 0, 1] and list(t.expert_of_slot) == [0, 0, 1, 1]
    assert list(t.group_offsets) == [0, 2, 4] and t.token_of_slot.dtype == np.int32
    Plan.sort_perm = np.array([0, 0, 1, 2])
    with pytest.raises(ValueError, match="duplicate"):
        ex._plan_to_transport(Plan)
    Plan.sort_perm = np.array([0, 3, 1, 7])
    with pytest.raises(ValueError, match="invalid slot"):
        ex._plan_to_transport(Plan)


def test_candidate_registry_semantics():
    names = [c.name for c in cand.candidates_for(cand.TARGET, cand.OP_MATMUL)]
    assert names == ["gfx950_mfma_gemm"]
    cand.register_all()                                           # idempotent
    assert [c.name for c in cand.candidates_for(cand.TARGET, cand.OP_MATMUL)] == names
    assert cand.candidates_for(cand.TARGET, cand.OP_GROUPED_GEMM)[0].tier == cand.Tier.HAND_TUNED

    class Fake(cand.Candidate):
        target, op = "fake", cand.OP_MATMUL

        def __init__(self, name, tier, err=0.0, tag="fake_kernel", ok=True):
            self.name, self.tier, self.err, self.tag, self.ok = name, tier, err, tag, ok

        def available(self):
            return self.ok

        def run(self, region, A, B, *a, **k):
            return region.reference(A, B) + self.err, self.tag

    for c in (Fake("slow_good", cand.Tier.SYNTHESIZED), Fake("lead_wrong", cand.Tier.HAND_TUNED, err=1.0),
              Fake("lead_declines", cand.Tier.HAND_TUNED, tag="reference"), Fake("lead_absent", cand.Tier.HAND_TUNED, ok=False),
              Fake("emitted_good", cand.Tier.EMITTED)):
        cand.register_candidate(c)
    region = cand.MatmulRegion("bfloat16")
    assert cand.arbitrate(region, cand.OP_MATMUL, "fake").name == "emitted_good"      # wrong/declining leads dropped
    assert cand.arbitrate(region, cand.OP_MATMUL, "fake", verify=False).name == "lead_wrong"
    assert cand.arbitrate(region, cand.OP_MATMUL, "fake", measure=lambda c: {"slow_good": 1.0}.get(c.name, 5.0)).name == "slow_good"
    with pytest.raises(cand.ArbiterError):
        cand.arbitrate(region, cand.OP_MATMUL, "fake", force="lead_absent")
    cand.reset_arbiter_dispatch_log()
    A, B = np.ones((32, 32), np.float32), np.ones((32, 16), np.float32)
    out, tag = cand.run_arbitrated(region, cand.OP_MATMUL, "fake", A, B)
    assert tag == "fake_kernel" and np.all(out == 32)
    assert cand.arbiter_dispatch_histogram()[("fake", cand.OP_MATMUL)] == {"won": 1, "degraded": 0, "no_candidate": 0}
    with pytest.raises(ValueError):
        cand.register_candidate(Fake("", cand.Tier.EMITTED))


def test_region_references():
    r = cand.MatmulRegion("bfloat16", transpose_b=True)
    A = np.array([[1 + 2.0 ** -10, 2.0]], np.float32)
    Bt = np.array([[1024.0, 1.0]], np.float32)                   # raw (N, K)
    assert r.reference(A, Bt)[0, 0] == 1026.0                    # operand rounded to bf16 first
    att = cand.AttentionRegion(scale=1.0, causal=True)
    Q = K = np.eye(4, 16, dtype=np.float32)
    V = np.arange(64, dtype=np.float32).reshape(4, 16)
    assert np.allclose(att.reference(Q, K, V)[0], V[0])          # row 0 sees only key 0


def test_tile_table():
    ops_ = tile_table.lower_tile_op(tile_table.TileOp("tile.matmul", {"dtype": "bf16"}, 3))
    assert [o.name for o in ops_] == ["tessera_rocm.mfma", "tessera_rocm.mfma_gemm"]
    assert ops_[0].attrs["shape"] == "m32n32k16" and ops_[1].attrs["symbol"] == "tessera_gfx950_gemm_bf16"
    assert tile_table.lower_tile_op(tile_table.TileOp("tile.mma", {"dtype": "int8"}))[0].attrs["shape"] == "m32n32k32"
    fa = tile_table.lower_tile_op(tile_table.TileOp("tessera_attn.online_softmax", {"source": "tessera.flash_attn", "causal": True}))
    assert fa[0].name == "tessera_rocm.mfma_flash_attn" and fa[0].attrs["runtime_lane"] == "gfx950_flash_attn"
    gg = tile_table.lower_tile_op(tile_table.TileOp("tile.matmul", {"source": "tessera.grouped_gemm"}))
    assert gg[0].attrs["argument_layout"] == "device_offsets[E+1]" and gg[0].attrs["dispatches"] == 1
    assert tile_table.lower_tile_op(tile_table.TileOp("tile.kv_cache"))[0].name == "tessera.target.diagnostic"
    lanes = set(ex.executor_table())
    declared = set(_header_symbols())
    for e in tile_table.KERNEL_TABLE:
        assert e.runtime_lane in lanes
        assert set(e.symbols) <= declared


def test_gemm_schedule_query_needs_no_device():
    """The schedule descriptor reads the launcher's own tile / split-K decision."""
    from tessera_amd.schedule import select_gfx950_gemm_schedule as sel
    big = sel(8192, 8192, 8192, dtype="bf16")
    assert big.workgroup_tile == (256, 256, 64) and big.macro_tile == (8, 8) and big.split_k == 1
    assert big.instruction_tile == (32, 32, 16) and big.target_ir_attrs()["schedule_arch"] == "gfx950"
    dec = sel(4, 8192, 8192, dtype="bf16")                              # a few rows: the streaming kernel
    assert dec.workgroup_tile == (32, 64, 32) and dec.split_k == 2 and dec.waves_per_cu == 8
    assert sel(4, 32768, 8192).split_k == 1                             # enough column strips to fill the chip
    mid = sel(64, 8192, 8192, dtype="bf16")
    assert mid.workgroup_tile[:2] == (64, 64) and mid.split_k > 1 and 8192 % (mid.split_k * 64) == 0
    assert sel(128, 8192, 8192).workgroup_tile[:2] == (128, 128)
    assert sel(128, 256, 64, batch=4).split_k == 1                      # batched products never split K
    q = sel(4096, 8192, 8192, dtype="int8")
    assert q.workgroup_tile == (256, 256, 128) and q.instruction_tile == (32, 32, 32)
    assert sel(4096, 8192, 8192, dtype="fp8_e4m3").instruction_tile == (32, 32, 64)
    assert big.cache_key() != dec.cache_key()
    import pytest
    with pytest.raises(ValueError):
        sel(0, 8, 8)
    with pytest.raises(ValueError):
        sel(8, 8, 8, arch="gfx1151")
    with pytest.raises(ValueError):
        sel(8, 8, 8, dtype="f64")
