"""The oracle against the committed vectors of the reference's compiled x86 kernels
(tests/golden/ref_vectors.npz, written by tests/golden/make_ref_vectors.py)."""
from pathlib import Path

import numpy as np
import pytest

import tessera_oracle as orc

GOLD = np.load(Path(__file__).parent / "golden" / "ref_vectors.npz")


def test_gemm_bf16_golden():
    a, b = orc.bf16_bits_to_f32(GOLD["gemm_bf16_a"]), orc.bf16_bits_to_f32(GOLD["gemm_bf16_b"])
    got = orc.gemm_f32(a.reshape(GOLD["gemm_bf16_a"].shape), b.reshape(GOLD["gemm_bf16_b"].shape))
    assert orc.max_rel_err(got, GOLD["gemm_bf16_d"]) <= 1e-6      # f32 summation order only


def test_gemm_int8_golden():
    a = GOLD["gemm_i8_a"].astype(np.int8)                       # values 0..127: u8 == s8
    assert np.array_equal(orc.gemm_i8_i32(a, GOLD["gemm_i8_b"]), GOLD["gemm_i8_c"])


@pytest.mark.parametrize("tag", ["fa_causal_gqa", "fa_causal_offset", "fa_full", "fa_window_causal",
                                 "fa_window_centered", "fa_softcap"])
def test_flash_attn_golden(tag):
    q, k, v = GOLD[f"{tag}_q"], GOLD[f"{tag}_k"], GOLD[f"{tag}_v"]
    o, lse = orc.flash_attn_dense(q, k, v, causal=bool(GOLD[f"{tag}_causal"]), window=int(GOLD[f"{tag}_window"]),
                                  softcap=float(GOLD[f"{tag}_softcap"]))
    assert orc.max_rel_err(o, GOLD[f"{tag}_o"]) <= 1e-5
    assert np.max(np.abs(lse - GOLD[f"{tag}_lse"])) <= 1e-5


def test_fpquant_golden():
    assert np.array_equal(orc.fpquant_grid(GOLD["fpq_x"]), GOLD["fpq_y"])


FP_GRID_TAGS = ("e5m2", "e2m3", "e3m2", "e2m1", "e2m1_floor0")


@pytest.mark.parametrize("tag", FP_GRID_TAGS)
def test_fpquant_other_grids_golden(tag):
    """e5m2, both fp6 grids and E2M1 (free exponent and the NVFP4 floor) against the
    reference's compiled kernel: every grid point, every tie, subnormals, saturation, NaN."""
    mx, mant, min_exp = GOLD[f"fpq_{tag}_fmt"]
    got = orc.fpquant_grid(GOLD[f"fpq_{tag}_x"], float(mx), int(mant), int(min_exp))
    assert np.array_equal(got, GOLD[f"fpq_{tag}_y"], equal_nan=True)
