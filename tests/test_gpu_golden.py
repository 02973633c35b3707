"""HIP kernels (through the C ABI) against the committed vectors of the reference's
compiled x86 kernels (tests/golden/ref_vectors.npz).  Tolerances: 2e-3 normwise
for 16-bit-operand float work, exact for integers and e4m3 grid values."""
from pathlib import Path

import numpy as np
import pytest

from tessera_amd import bf16 as b16
from tessera_amd import ops
import tessera_oracle as orc

pytestmark = pytest.mark.gpu
GOLD = np.load(Path(__file__).parent / "golden" / "ref_vectors.npz")


def test_gemm_bf16_golden(lane):
    d = ops.gemm(b16.from_bits(GOLD["gemm_bf16_a"]), b16.from_bits(GOLD["gemm_bf16_b"]), out="f32")
    assert orc.max_rel_err(d, GOLD["gemm_bf16_d"]) <= 2e-3


def test_gemm_int8_golden(lane):
    c = ops.gemm_i8(GOLD["gemm_i8_a"].astype(np.int8), GOLD["gemm_i8_b"])
    assert np.array_equal(c, GOLD["gemm_i8_c"])


@pytest.mark.parametrize("tag", ["fa_causal_gqa", "fa_causal_offset", "fa_full", "fa_window_causal",
                                 "fa_window_centered", "fa_softcap"])
def test_flash_attn_golden(lane, tag):
    q, k, v = (b16.from_float32(GOLD[f"{tag}_{n}"]) for n in "qkv")   # already bf16-representable
    o, lse = ops.gqa_attention(q, k, v, causal=bool(GOLD[f"{tag}_causal"]), return_lse=True, out="f32",
                               window=int(GOLD[f"{tag}_window"]), logit_softcap=float(GOLD[f"{tag}_softcap"]))
    assert orc.max_rel_err(o, GOLD[f"{tag}_o"]) <= 2e-3
    assert np.max(np.abs(lse - GOLD[f"{tag}_lse"])) <= 2e-3


def test_e4m3_grid_golden(lane):
    codes, scale = ops.quantize_fp8_codes(GOLD["fpq_x"], scale=1.0)
    got = ops.e4m3_table()[codes]
    assert scale == np.float32(1.0)
    assert np.array_equal(got, GOLD["fpq_y"])
