"""Tile-IR op → gfx950 kernel table.

The reference lowers Tile IR to Target IR per backend in ``_lower_rocm_op``
(``python/tessera/compiler/target_ir.py:1321-1439``): ``tile.matmul`` /
``tile.mma`` become a ``tessera_rocm.mfma`` shape marker plus the concrete
``tessera_rocm.wmma_gemm`` directive (16x16x16, RDNA), ``tessera.grouped_gemm``
becomes ``tessera_rocm.grouped_gemm`` with ``argument_layout =
"device_offsets[E+1]"``, and ``tessera.flash_attn`` / ``tessera_attn.*`` get an
"unsupported" diagnostic (``:1407-1413``).  This module is the ``rocm_gfx950``
branch of that table: the same ``TargetOp`` shape, real CDNA4 MFMA instruction
shapes, a flash-attention lowering instead of the diagnostic, and for every
directive the C-ABI symbol and executor lane that realise it.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Optional

ARCH = "gfx950"
TARGET = "rocm_gfx950"

#: Tile ops of the attention dialect the reference recognises (``tile_ir.py:32-38``).
ATTN_OPS = frozenset({
    "tessera_attn.scaled_dot_product",
    "tessera_attn.online_softmax",
    "tessera_attn.lse_save",
    "tessera_attn.attend_v",
})


@dataclass
class TileOp:
    """The slice of ``tile_ir.TileOp`` the lowering reads."""
    op_name: str
    attrs: dict = field(default_factory=dict)
    ordinal: int = 0


@dataclass
class TargetOp:
    """Same fields as ``target_ir.TargetOp``: an op name and its attribute dict."""
    name: str
    attrs: dict


@dataclass(frozen=True)
class KernelEntry:
    """One row of the op → kernel table."""
    source_op: str              # Graph-IR op the Tile op came from
    tile_ops: tuple             # Tile-IR op names that select this row
    directive: str              # Target-IR op emitted
    mfma_shape: str             # matrix-core instruction shape
    mfma_instr: str
    dtypes: tuple
    symbols: tuple              # C-ABI entry points
    runtime_lane: str           # executor_id in the execution matrix
    workgroup_tile: str
    lds_bytes: int


#: MFMA instruction of the 256 x 256 workgroup tile per storage dtype on gfx950 (the 16-bit
#: tiles run the 16-wide form, which spends less power per FLOP; their smaller tiles and the
#: attention kernels run m32n32k16; the f8f6f4 form is the full-rate fp8 path).
MFMA_BY_DTYPE = {
    "f16": ("m16n16k32", "v_mfma_f32_16x16x32_f16"),
    "bf16": ("m16n16k32", "v_mfma_f32_16x16x32_bf16"),
    "int8": ("m32n32k32", "v_mfma_i32_32x32x32_i8"),
    "fp8_e4m3": ("m32n32k64", "v_mfma_f32_32x32x64_f8f6f4"),
}

KERNEL_TABLE: tuple = (
    KernelEntry("tessera.matmul", ("tile.matmul", "tile.mma"), "tessera_rocm.mfma_gemm", "m16n16k32",
                "v_mfma_f32_16x16x32_{f16,bf16} (256x256 tiles); v_mfma_f32_32x32x16_{f16,bf16} (smaller tiles)", ("f16", "bf16"),
                ("tessera_gfx950_gemm_f16", "tessera_gfx950_gemm_bf16", "tessera_gfx950_gemm_f16_f16",
                 "tessera_gfx950_gemm_bf16_bf16", "tessera_gfx950_batched_gemm_f16",
                 "tessera_gfx950_batched_gemm_bf16"),
                "gfx950_gemm", "256x256x64, 2x2 waves of 128x128", 135168),
    KernelEntry("tessera.matmul", ("tile.matmul", "tile.mma"), "tessera_rocm.mfma_gemm", "m32n32k32",
                "v_mfma_i32_32x32x32_i8", ("int8",),
                ("tessera_gfx950_gemm_i8_i32", "tessera_gfx950_gemm_w8a8_f32"),
                "gfx950_gemm", "256x256x128, 2x2 waves of 128x128", 135168),
    KernelEntry("tessera.fused_epilogue", ("tile.matmul", "tile.mma"), "tessera_rocm.mfma_gemm", "m16n16k32",
                "v_mfma_f32_16x16x32_{f16,bf16} (256x256 tiles); v_mfma_f32_32x32x16_{f16,bf16} (smaller tiles)", ("f16", "bf16"),
                ("tessera_gfx950_gemm_bias_act_f16", "tessera_gfx950_gemm_bias_act_bf16",
                 "tessera_gfx950_gated_gemm_f16", "tessera_gfx950_gated_gemm_bf16"),
                "gfx950_gemm", "256x256x64, bias + activation (or gate * up) in the epilogue", 135168),
    KernelEntry("tessera.fp8_gemm", ("tile.matmul", "tile.mma"), "tessera_rocm.mfma_gemm", "m32n32k64",
                "v_mfma_f32_32x32x64_f8f6f4", ("fp8_e4m3",),
                ("tessera_gfx950_gemm_e4m3_bf16", "tessera_gfx950_gemm_e4m3_f32"),
                "gfx950_quant_gemm", "256x256x128, 2x2 waves of 128x128", 135168),
    KernelEntry("tessera.flash_attn", tuple(sorted(ATTN_OPS)), "tessera_rocm.mfma_flash_attn", "m32n32k16",
                "v_mfma_f32_32x32x16_{f16,bf16}", ("f16", "bf16"),
                ("tessera_gfx950_flash_attn_f16", "tessera_gfx950_flash_attn_bf16",
                 "tessera_gfx950_flash_attn_gqa_f16", "tessera_gfx950_flash_attn_gqa_bf16"),
                "gfx950_flash_attn", "256 q rows x 64 keys, 8 waves of 32 rows", 65536),
    KernelEntry("tessera.flash_attn_bwd", ("tessera_attn.backward",), "tessera_rocm.mfma_flash_attn_bwd", "m32n32k16",
                "v_mfma_f32_32x32x16_{f16,bf16}", ("f16", "bf16"),
                ("tessera_gfx950_flash_attn_bwd_f16", "tessera_gfx950_flash_attn_bwd_bf16"),
                "gfx950_flash_attn_bwd", "dQ: 256 q rows x 64 keys; dK/dV: 128 keys x 64 q rows", 66560),
    KernelEntry("tessera.grouped_gemm", ("tile.matmul", "tile.mma"), "tessera_rocm.grouped_gemm", "m16n16k32",
                "v_mfma_f32_16x16x32_bf16", ("bf16",),
                ("tessera_gfx950_grouped_gemm_bf16", "tessera_gfx950_grouped_gemm_bf16_f32",
                 "tessera_gfx950_moe_swiglu_block_bf16"),
                "gfx950_moe_transport", "256x256x64 per (expert, row tile), one launch", 135168),
)


def entries_for(source_op: str, dtype: Optional[str] = None) -> list:
    return [e for e in KERNEL_TABLE if e.source_op == source_op and (dtype is None or dtype in e.dtypes)]


def _norm_dtype(raw: Any) -> str:
    d = str(raw or "f16")
    return {"float16": "f16", "fp16": "f16", "bfloat16": "bf16", "i8": "int8", "e4m3": "fp8_e4m3",
            "fp8": "fp8_e4m3"}.get(d, d)


def lower_tile_op(op: TileOp, *, arch: str = ARCH) -> list:
    """Tile op → Target ops for ``rocm_gfx950`` (the counterpart of
    ``_lower_rocm_op``).  Unknown ops get the reference's diagnostic form."""
    if op.op_name in {"tile.debug_artifact", "tile.debug_barrier"}:
        return []
    source = str(op.attrs.get("source", ""))
    base = {"ordinal": op.ordinal, "target": TARGET, "source": source or op.op_name}
    if source == "tessera.grouped_gemm":
        return [TargetOp("tessera_rocm.grouped_gemm", {
            **base, "name": "grouped_gemm", "arch": arch, "status": "device_verified_abi",
            "runtime_lane": "gfx950_moe_transport", "argument_layout": "device_offsets[E+1]", "dispatches": 1,
            "shape": "m16n16k32", "symbol": "tessera_gfx950_grouped_gemm_bf16"})]
    if source == "tessera.flash_attn" or op.op_name in ATTN_OPS:
        dtype = _norm_dtype(op.attrs.get("dtype", "bf16"))
        if dtype not in ("f16", "bf16"):
            dtype = "bf16"
        return [TargetOp("tessera_rocm.mfma_flash_attn", {
            **base, "name": "flash_attn_fwd", "arch": arch, "status": "device_verified_abi",
            "runtime_lane": "gfx950_flash_attn", "shape": "m32n32k16", "dtype": dtype, "accum": "f32",
            "tile_q": 256, "tile_kv": 64, "causal": bool(op.attrs.get("causal", False)),
            "gqa": True, "lse": True, "symbol": f"tessera_gfx950_flash_attn_gqa_{dtype}"})]
    if op.op_name in {"tile.matmul", "tile.mma"}:
        dtype = _norm_dtype(op.attrs.get("dtype", "f16"))
        if dtype not in MFMA_BY_DTYPE:
            dtype = "f16"
        shape, instr = MFMA_BY_DTYPE[dtype]
        symbol = {"f16": "tessera_gfx950_gemm_f16", "bf16": "tessera_gfx950_gemm_bf16",
                  "int8": "tessera_gfx950_gemm_i8_i32", "fp8_e4m3": "tessera_gfx950_gemm_e4m3_bf16"}[dtype]
        lane = "gfx950_quant_gemm" if dtype == "fp8_e4m3" else "gfx950_gemm"
        return [
            TargetOp("tessera_rocm.mfma", {**base, "arch": arch, "shape": shape, "instr": instr,
                                           "accum": "i32" if dtype == "int8" else "f32"}),
            TargetOp("tessera_rocm.mfma_gemm", {
                **base, "name": "gemm", "arch": arch, "dtype": dtype, "shape": shape,
                "block_m": 256, "block_n": 256, "block_k_bytes": 128, "waves": "2x2",
                "lds_layout": "A xor-swizzled 16B chunks; B natural + transposing ds_read",
                "schedule_pipeline_stages": 2, "runtime_lane": lane, "symbol": symbol,
                "status": "device_verified_abi"}),
        ]
    return [TargetOp("tessera.target.diagnostic", {
        **base, "severity": "unsupported",
        "reason": f"{op.op_name} has no kernel on the gfx950 dense-op lane"})]
