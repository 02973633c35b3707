"""No-GPU checks: the C-ABI library loads and exports every symbol the header
declares; shape validation happens before the device is touched; the host-side
mirrors of the reference's plugin interfaces behave as the reference's do."""
import ctypes
import re
from pathlib import Path

import numpy as np
import pytest

import standin_host as host
from tessera_amd import bf16 as b16
from tessera_amd import candidates as cand
from tessera_amd import executors as ex
from tessera_amd import install as inst
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
    ms = ctypes.c_double(0)
    assert lib.tessera_gfx950_flash_attn_bf16_bench(1, 4, 2, 64, 64, 24, 1, 3, ctypes.byref(ms)) == 1    # head dim
    assert lib.tessera_gfx950_flash_attn_bf16_bench(1, 4, 2, 64, 64, 128, 1, 0, ctypes.byref(ms)) == 1   # no launches
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
    api = host.CandidateHost()
    made = cand.register(api)
    assert made and not any(c.available() for c in made)
    assert api.arbitrate(host.MatmulRegion(), api.OP_MATMUL, cand.TARGET) is None
    with pytest.raises(host.ArbiterError):
        api.run(host.MatmulRegion(), api.OP_MATMUL, cand.TARGET, np.zeros((32, 32)), np.zeros((32, 16)))


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
    # the reference's positional parameters (Q, K, V, scale, causal, cache, dropout_p, ...) are accepted
    with pytest.raises(ValueError):
        ops.flash_attn(q, q, q, None, False, None, 1.5)                            # dropout_p out of range
    with pytest.raises(NotImplementedError):
        ops.flash_attn(q, q, q, dropout_p=0.1)
    with pytest.raises(NotImplementedError):
        ops.flash_attn(q, kv_state=object())
    with pytest.raises(ValueError):
        ops.flash_attn(q)
    k = np.zeros((1, 3, 8, 16), np.float16)
    with pytest.raises(ValueError):
        ops.gqa_attention(q, k, k)                                                 # 4 % 3
    with pytest.raises(ValueError):
        ops.gqa_attention(q, k, k, 4, 3)                                           # the reference's own check
    k2 = np.zeros((1, 2, 8, 16), np.float16)
    with pytest.raises(ValueError):
        ops.gqa_attention(q, k2, k2, 8, 2)                                         # 2 heads x 4 != 4 heads
    with pytest.raises(ValueError):
        ops.mqa_attention(q, k2, k2)                                               # MQA wants one K/V head
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


def test_candidates_derive_from_the_injected_host_api():
    """The plugin owns no registry and no base class: its candidates subclass the
    Candidate of whichever host API it is given and go through that host's
    register functions (the reference's backends do the same at import,
    compiler/emit/rocm_hip.py:809-818)."""
    api = host.CandidateHost()
    made = cand.register(api)
    assert [c.name for c in made] == ["gfx950_mfma_gemm", "gfx950_flash_attn", "gfx950_grouped_gemm",
                                      "gfx950_mfma_fused_gemm", "gfx950_mfma_gated_gemm"]
    assert all(isinstance(c, api.Candidate) and c.tier == api.Tier.HAND_TUNED and c.target == cand.TARGET
               for c in made)
    by_op = {c.op: c for c in made}
    assert set(by_op) == {api.OP_MATMUL, api.OP_ATTENTION, cand.OP_GROUPED_GEMM, api.OP_FUSED_REGION,
                          api.OP_GATED_MATMUL}
    assert [c.name for c in api.candidates_for(cand.TARGET, api.OP_MATMUL)] == ["gfx950_mfma_gemm"]
    cand.register(api)                                            # again: replaced by name, not duplicated
    assert [c.name for c in api.candidates_for(cand.TARGET, api.OP_MATMUL)] == ["gfx950_mfma_gemm"]
    # a second host gets classes of its own base
    other = host.CandidateHost()

    class OtherBase(host.Candidate):
        pass
    other.Candidate = OtherBase
    assert all(isinstance(c, OtherBase) for c in cand.build_candidates(other))
    # region filters read attributes only
    gemm, attn, fused, gated = by_op[api.OP_MATMUL], by_op[api.OP_ATTENTION], by_op[api.OP_FUSED_REGION], \
        by_op[api.OP_GATED_MATMUL]
    assert gemm.applies_to(host.MatmulRegion("float16")) and not gemm.applies_to(host.MatmulRegion("float32"))
    assert gemm.mma_prefer_shape == (32, 32, 16) and gemm.mma_arch == "gfx950"
    assert attn.applies_to(host.AttentionRegion(storage_dtype="bf16"))
    assert fused.applies_to(host.FusedRegion(("bias", "gelu"))) and not fused.applies_to(host.FusedRegion(("relu", "bias")))
    assert fused.mma_dtype(host.FusedRegion((), storage_dtype="bf16")) == "bf16"
    assert gated.applies_to(host.GatedMatmulRegion("sigmoid"))
    assert by_op[cand.OP_GROUPED_GEMM].applies_to(cand.GroupedGemmRegion((1, 2))) and \
        not by_op[cand.OP_GROUPED_GEMM].applies_to(cand.GroupedGemmRegion((1, 2), "float16"))


def test_install_registers_into_the_objects_it_is_given():
    """One call plugs candidates, execution-matrix rows and executor functions into the
    host's own objects (emit/candidate.py:81-87,206-236; execution_matrix.py:103,
    2495-2537; runtime.py:30515), and the host's launch then reaches the lane."""
    api, matrix = host.CandidateHost(), host.MatrixHost()
    runtime = host.RuntimeHost(matrix)
    report = inst.install(api, matrix, runtime)
    assert len(report["candidates"]) == 5 and len(report["rows"]) == 5 and len(report["executors"]) == 5
    row = matrix._MATRIX[("rocm_gfx950", "gfx950_flash_attn_bwd")]
    assert isinstance(row, matrix.ExecutionRow) and row.direction == "backward" and row.op_family == "flash_attn"
    assert row.executable and row.execution_kind == "native_gpu" and row.execution_mode == "hip_runtime"
    assert ("cpu", "jit_cpu_numpy") in matrix._MATRIX                      # the host's own rows are untouched
    assert set(report["executors"]) <= set(matrix.KNOWN_EXECUTORS)
    table = runtime._executor_table()
    assert "jit_cpu_numpy" in table and table["gfx950_gemm"] is ex.execute_gfx950_gemm
    assert {r.executor_id for k, r in matrix._MATRIX.items() if k[0] == "rocm_gfx950"} == set(report["executors"])
    inst.install(api, matrix, runtime)                                     # idempotent: wrapped once
    assert runtime._executor_table()["gfx950_gemm"] is ex.execute_gfx950_gemm
    plain: dict = {}
    inst.install(executor_table=plain)
    assert set(plain) == set(report["executors"])
    with pytest.raises(TypeError):
        inst.install(executor_table=object())
    # the host's launch resolves the lane's executor and reports its errors in its envelope
    art = ex.make_artifact("tessera.matmul", ["a", "b"], ["a", "b"], "gfx950_gemm", executable=True)
    res = runtime.launch(art, (np.zeros((4, 5), np.float16), np.zeros((4, 4), np.float16)))
    assert res["runtime_status"] == "invalid_artifact" and "matching K" in res["reason"]


def test_grouped_gemm_region_definition():
    r = cand.GroupedGemmRegion((1, 0, 2))
    x = np.array([[1.0, 2.0], [1.0, 0.0], [0.0, 1 + 2.0 ** -10]], np.float32)
    w = np.stack([np.eye(2), 7 * np.eye(2), np.array([[1.0, 2.0], [3.0, 4.0]])]).astype(np.float32)
    want = np.array([[1.0, 2.0], [1.0, 2.0], [3.0, 4.0]], np.float32)     # last row: operand rounded to bf16 first
    assert np.array_equal(r.reference(x, w), want)


def test_tile_table():
    ops_ = tile_table.lower_tile_op(tile_table.TileOp("tile.matmul", {"dtype": "bf16"}, 3))
    assert [o.name for o in ops_] == ["tessera_rocm.mfma", "tessera_rocm.mfma_gemm"]
    assert ops_[0].attrs["shape"] == "m16n16k32" and ops_[0].attrs["instr"] == "v_mfma_f32_16x16x32_bf16"
    assert ops_[1].attrs["symbol"] == "tessera_gfx950_gemm_bf16" and ops_[1].attrs["block_m"] == 256
    assert tile_table.lower_tile_op(tile_table.TileOp("tile.mma", {"dtype": "int8"}))[0].attrs["shape"] == "m32n32k32"
    fa = tile_table.lower_tile_op(tile_table.TileOp("tessera_attn.online_softmax", {"source": "tessera.flash_attn", "causal": True}))
    assert fa[0].name == "tessera_rocm.mfma_flash_attn" and fa[0].attrs["runtime_lane"] == "gfx950_flash_attn"
    gg = tile_table.lower_tile_op(tile_table.TileOp("tile.matmul", {"source": "tessera.grouped_gemm"}))
    assert gg[0].attrs["argument_layout"] == "device_offsets[E+1]" and gg[0].attrs["dispatches"] == 1
    assert gg[0].attrs["shape"] == "m16n16k32" and fa[0].attrs["shape"] == "m32n32k16"
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
    assert big.workgroup_tile == (256, 256, 64) and big.macro_tile == (16, 16) and big.split_k == 1
    assert big.instruction_tile == (16, 16, 32) and big.target_ir_attrs()["schedule_arch"] == "gfx950"
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
    # 8-bit: fewer tiles take the 128-row tile, up to 64 rows the streaming kernel (K split over ~256 workgroups)
    assert sel(1024, 8192, 8192, dtype="int8").workgroup_tile == (128, 256, 128)
    assert sel(2048, 2048, 2048, dtype="int8").workgroup_tile[0] == 128
    qd = sel(1, 8192, 8192, dtype="int8")
    assert qd.workgroup_tile == (32, 128, 64) and qd.split_k == 4 and qd.waves_per_cu == 8 and "wave-private" in qd.lds_layout
    assert sel(64, 8192, 8192, dtype="fp8_e4m3").workgroup_tile == (64, 128, 64)
    assert sel(64, 8192, 1000, dtype="int8").workgroup_tile[2] == 128           # K off the slice grid: the tile kernel
    assert big.cache_key() != dec.cache_key()
    import pytest
    with pytest.raises(ValueError):
        sel(0, 8, 8)
    with pytest.raises(ValueError):
        sel(8, 8, 8, arch="gfx1151")
    with pytest.raises(ValueError):
        sel(8, 8, 8, dtype="f64")


def test_typed_descriptor_hook_validates_before_the_device():
    """The native-launcher hook refuses what its descriptor does not cover with RuntimeError,
    before any device call (nothing here needs a GPU)."""
    from tessera_amd import native_launcher as nl
    runtime = host.NativeLauncherHost()
    assert inst.install(native_launchers=runtime)["native_launcher"] == nl.TARGET
    assert runtime.hooks[nl.TARGET][0] == ("shared_object",)
    inst.install(native_launchers=runtime)                                 # replace=True: no duplicate error
    bind = lambda *names: tuple(host.Binding(n, i) for i, n in enumerate(names))
    A = np.zeros((4, 8), np.float16)
    B = np.zeros((8, 6), np.float16)
    O = np.zeros((4, 6), np.float32)
    image = host.Image(nl.TARGET, "shared_object")
    cases = [
        (host.Descriptor("tessera.rocm.softmax.x_o_rows_k.f32.v1", "tessera_gfx950_gemm_f16", bind("A", "B", "O")),
         {"M": 4, "N": 6, "K": 8}, "unsupported"),
        (host.Descriptor(nl.MATMUL_F16_F32_ABI, "tessera_gfx950_gemm_bf16", bind("A", "B", "O")),
         {"M": 4, "N": 6, "K": 8}, "cannot launch"),
        (host.Descriptor(nl.MATMUL_F16_F32_ABI, "tessera_gfx950_gemm_f16", bind("A", "B")),
         {"M": 4, "N": 6, "K": 8}, "requires 3 buffers"),
        (host.Descriptor(nl.MATMUL_F16_F32_ABI, "tessera_gfx950_gemm_f16", bind("A", "B", "O")),
         {"M": 4, "N": 6, "K": 7}, "disagree"),
        (host.Descriptor(nl.MATMUL_BF16_F32_ABI, "tessera_gfx950_gemm_bf16", bind("A", "B", "O")),
         {"M": 4, "N": 6, "K": 8}, "disagree"),                            # f16 arrays under a bf16 ABI
    ]
    for desc, scalars, needle in cases:
        res = runtime.launch_descriptor(image, desc, {"A": A, "B": B, "O": O}, scalars)
        assert not res["ok"] and res["runtime_status"] == "device_error" and needle in res["reason"], (needle, res)
    x = np.zeros((3, 4), np.float32)
    res = runtime.launch_descriptor(
        image, host.Descriptor(nl.MOE_DISPATCH_F32_ABI, "tessera_gfx950_moe_dispatch", bind("X", "T", "O")),
        {"X": x, "T": np.array([0, 3], np.int32), "O": np.zeros((2, 4), np.float32)}, {"T": 3, "S": 2, "H": 4})
    assert not res["ok"] and "disagree" in res["reason"]                   # token id 3 is out of range
    assert set(nl.supported_abis()) >= {nl.MATMUL_F16_F32_ABI, nl.ATTN_BF16_ABI, nl.MOE_DISPATCH_F32_ABI}


class _LaunchParams(ctypes.Structure):
    """tsrGpuLaunchParams (src/runtime/include/tessera/tsr_types.h:83-89)."""
    _fields_ = [("buffers", ctypes.POINTER(ctypes.c_void_p)), ("num_buffers", ctypes.c_size_t),
                ("dims", ctypes.POINTER(ctypes.c_int64)), ("num_dims", ctypes.c_size_t)]


def launch_params(arrays, dims):
    bufs = (ctypes.c_void_p * len(arrays))(*[a.ctypes.data if a is not None else None for a in arrays])
    d = (ctypes.c_int64 * len(dims))(*dims)
    keep = (bufs, d, arrays)
    return _LaunchParams(bufs, len(arrays), d, len(dims)), keep


def test_c_level_launcher_answers_like_the_runtime_expects():
    """The tsrGpuLauncherFn entry point: TsrStatus codes (tsr_status.h:7-14) for everything
    that is decided before a device is touched."""
    SUCCESS, INVALID, NOT_FOUND, DEVICE_ERROR = 0, 1, 2, 7
    lib = lane.load()
    fn = lib.tessera_gfx950_gpu_launcher
    a = np.zeros((4, 8), np.uint16)
    b = np.zeros((8, 4), np.uint16)
    d = np.zeros((4, 4), np.float32)
    ok, keep = launch_params([a, b, d], [4, 4, 8])
    assert fn(b"apple_gpu", b"tessera_gfx950_gemm_bf16", ctypes.byref(ok), None) == NOT_FOUND
    assert fn(b"rocm_gfx1151", b"tessera_gfx950_gemm_bf16", ctypes.byref(ok), None) == NOT_FOUND
    assert fn(b"rocm", b"tessera_rocm_gemm_f32", ctypes.byref(ok), None) == NOT_FOUND            # a name it does not bridge
    assert fn(b"rocm", b"tessera_gfx950_gemm_bf16", None, None) == INVALID
    assert fn(None, b"tessera_gfx950_gemm_bf16", ctypes.byref(ok), None) == INVALID
    two, keep2 = launch_params([a, b], [4, 4, 8])
    assert fn(b"rocm", b"tessera_gfx950_gemm_bf16", ctypes.byref(two), None) == INVALID          # buffer count
    four, keep4 = launch_params([a, b, d], [4, 4, 8, 1])
    assert fn(b"rocm", b"tessera_gfx950_gemm_bf16", ctypes.byref(four), None) == INVALID         # dim count
    assert fn(b"rocm", b"tessera_gfx950_batched_gemm_bf16", ctypes.byref(ok), None) == INVALID   # wants {batch,M,N,K}
    null, keepn = launch_params([a, None, d], [4, 4, 8])
    assert fn(b"rocm_gfx950", b"tessera_gfx950_gemm_bf16", ctypes.byref(null), None) == INVALID
    zero, keepz = launch_params([a, b, d], [0, 4, 8])
    assert fn(b"rocm_gfx950", b"tessera_gfx950_gemm_bf16", ctypes.byref(zero), None) == INVALID  # rc 1 of the entry point
    huge, keeph = launch_params([a, b, d], [4, 4, 1 << 40])
    assert fn(b"rocm_gfx950", b"tessera_gfx950_gemm_bf16", ctypes.byref(huge), None) == INVALID  # does not fit a C int
    attn, keepa = launch_params([a, a, a, d], [1, 1, 4, 4, 0, 1])
    assert fn(b"rocm", b"tessera_gfx950_flash_attn_bf16", ctypes.byref(attn), None) == INVALID
    if not lane.available():
        assert fn(b"rocm", b"tessera_gfx950_gemm_bf16", ctypes.byref(ok), None) == DEVICE_ERROR  # no gfx950 here
    else:
        assert fn(b"rocm", b"tessera_gfx950_gemm_bf16", ctypes.byref(ok), None) == SUCCESS



def test_expert_capacity_follows_the_reference_order():
    """capacity = ceil(cf * (T / E)) (distributed/moe.py:79-92).  (cf * T) / E rounds
    differently on about 0.04 % of triples; the known one is cf=1.1, T=540, E=3 -> 199."""
    import math
    from fractions import Fraction

    import tessera_oracle as orc
    from tessera_amd import ops
    assert ops.expert_capacity(1.1, 540, 3) == 199 == orc.compute_capacity(1.1, 540, 3)
    assert int(math.ceil(1.1 * 540 / 3)) == 198          # the other order, for the record
    differ = 0
    for cf in (1.0, 1.05, 1.1, 1.25, 1.3, 1.7, 2.0, 2.2):
        for T in range(1, 700, 7):
            for E in (1, 3, 6, 7, 8, 12, 48, 64):
                got = ops.expert_capacity(cf, T, E)
                assert got == orc.compute_capacity(cf, T, E)
                # never below the exact rational value's ceiling minus the float slack of one slot
                exact = math.ceil(Fraction(cf) * Fraction(T, E))
                assert abs(got - exact) <= 1
                differ += got != int(math.ceil(cf * T / E))
    assert differ > 0
