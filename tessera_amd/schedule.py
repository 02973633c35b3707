"""GEMM schedule descriptor for the gfx950 lane.

The counterpart of ``python/tessera/compiler/rocm_schedule.py``:
``select_gfx950_gemm_schedule(m, n, k, dtype=...)`` returns a descriptor with the
fields of ``ROCmScheduleDescriptor`` (``:40-92``) — instruction tile, macro tile in
instruction tiles, waves per CU, pipeline stages, LDS layout, ownership, register
estimate, raster order — serialisable into the same Target-IR attributes
(``target_ir_attrs``).  The tile and K-split choice is not restated here: it is read
from the library (``tessera_gfx950_gemm_schedule``, a host-only query), so the
descriptor always describes what the launcher will actually run.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Any

from . import lane as _lane

_DTYPES = {
    "f16": ("f16", 2), "float16": ("f16", 2), "fp16": ("f16", 2),
    "bf16": ("bf16", 2), "bfloat16": ("bf16", 2),
    "int8": ("int8", 1), "i8": ("int8", 1),
    "fp8_e4m3": ("fp8_e4m3", 1), "e4m3": ("fp8_e4m3", 1), "fp8": ("fp8_e4m3", 1),
}
_INSTRUCTION_TILE = {"f16": (32, 32, 16), "bf16": (32, 32, 16), "int8": (32, 32, 32), "fp8_e4m3": (32, 32, 64)}
# accumulators + operand fragments + staging of one wave, from the assembler's report
_VGPRS = {(256, 256): 508, (128, 256): 360, (128, 128): 170, (64, 64): 96, (32, 64): 137}


@dataclass(frozen=True)
class Gfx950ScheduleDescriptor:
    arch: str
    dtype: str
    instruction_tile: tuple
    macro_tile: tuple                 # in instruction tiles, as the reference's (mt, nt)
    workgroup_tile: tuple             # (BM, BN, BK) in elements
    waves_per_cu: int
    pipeline_stages: int
    lds_layout: str
    ownership: str
    vgpr_estimate: int
    split_k: int
    source: str
    raster_order: str = "xcd_banded"
    raster_group: int = 4
    rest_tiles: int = 0               # tiles beyond the last full round of 256 workgroups that are ...
    rest_split_k: int = 1             # ... split along K into this many parts (1: none are)

    @property
    def mt(self) -> int:
        return self.macro_tile[0]

    @property
    def nt(self) -> int:
        return self.macro_tile[1]

    def target_ir_attrs(self) -> dict:
        return {
            "mt": self.mt, "nt": self.nt,
            "schedule_arch": self.arch,
            "schedule_pipeline_stages": self.pipeline_stages,
            "schedule_lds_layout": self.lds_layout,
            "schedule_ownership": self.ownership,
            "schedule_vgpr_estimate": self.vgpr_estimate,
            "schedule_source": self.source,
            "schedule_raster_order": self.raster_order,
            "schedule_raster_group": self.raster_group,
            "schedule_split_k": self.split_k,
            "schedule_rest_tiles": self.rest_tiles,
            "schedule_rest_split_k": self.rest_split_k,
        }

    def cache_key(self) -> tuple:
        return tuple(self.target_ir_attrs().values()) + (self.dtype, self.instruction_tile)


def select_gfx950_gemm_schedule(m: int, n: int, k: int, *, dtype: str = "bf16", batch: int = 1,
                                arch: str = "gfx950") -> Gfx950ScheduleDescriptor:
    """The schedule the library runs for an aligned ``m x n x k`` product."""
    if min(m, n, k, batch) < 1:
        raise ValueError(f"GEMM dimensions must be positive, got {(m, n, k)} x {batch}")
    if arch.lower().replace("_", "") != "gfx950":
        raise ValueError(f"unsupported schedule arch {arch!r}: this lane is gfx950 only")
    if dtype not in _DTYPES:
        raise ValueError(f"unsupported GEMM dtype {dtype!r}")
    name, nbytes = _DTYPES[dtype]
    tm, tn, tk, sk = (ctypes.c_int(0) for _ in range(4))
    _lane.check(_lane.load().tessera_gfx950_gemm_schedule(
        int(m), int(n), int(k), int(batch), nbytes, ctypes.byref(tm), ctypes.byref(tn), ctypes.byref(tk),
        ctypes.byref(sk)), "gemm_schedule")
    rest_tiles, rest_split = ctypes.c_int(0), ctypes.c_int(1)
    if nbytes == 2:
        _lane.check(_lane.load().tessera_gfx950_gemm_rest_split(
            int(m), int(n), int(k), int(batch), ctypes.byref(rest_tiles), ctypes.byref(rest_split)), "gemm_rest_split")
    inst = _INSTRUCTION_TILE[name]
    if name in ("f16", "bf16") and max(tm.value, tn.value) == 256:
        inst = (16, 16, 32)       # the 256-wide tiles run v_mfma_f32_16x16x32 (less power per FLOP)
    # the few-row streaming kernels: 32 x 64 strips (16-bit), 32 or 64 x 128 strips (8-bit)
    streaming = tm.value == 32 or (nbytes == 1 and tn.value == 128)
    return Gfx950ScheduleDescriptor(
        arch="gfx950", dtype=name, instruction_tile=inst,
        macro_tile=(max(1, tm.value // inst[0]), tn.value // inst[1]),
        workgroup_tile=(tm.value, tn.value, tk.value),
        waves_per_cu=8 if tm.value == 32 else 4, pipeline_stages=2,
        lds_layout=("A from global in operand order; B wave-private [k][n] slices + transposing ds_read"
                    if streaming else "A xor-swizzled 16B chunks; B natural [k][n] + transposing ds_read"),
        ownership="wave", vgpr_estimate=_VGPRS.get((tm.value, tn.value), 508), split_k=sk.value,
        source="tessera_gfx950_gemm_schedule (the launcher's own decision)",
        rest_tiles=rest_tiles.value, rest_split_k=rest_split.value)


__all__ = ["Gfx950ScheduleDescriptor", "select_gfx950_gemm_schedule"]
