#!/usr/bin/env python3
"""Write ``ref_vectors.npz``: small input/output vectors from the reference's own
compiled x86 kernels (``oracle/_ref/libtessera_x86_ref.so``, built from the
reference sources by ``oracle/Makefile``).  The reference's tests keep no stored
vectors (they recompute numpy from a seed), so these are the committed fixtures
the oracle and the HIP kernels are checked against where the reference sources
are not present.  Run in the build container: ``python3 tests/golden/make_ref_vectors.py``.
"""
from __future__ import annotations

import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT / "oracle"))
import c_oracle as co            # noqa: E402
import tessera_oracle as orc     # noqa: E402


def main() -> int:
    if co.ref() is None:
        print("compiled reference twins unavailable (needs /root/reference and an AVX-512 host)", file=sys.stderr)
        return 1
    rng = np.random.default_rng(20240611)
    out = {}
    # bf16 GEMM twin: tessera_x86_reference_gemm_bf16 (avx512_gemm_bf16.cpp:13-26)
    a = orc.f32_to_bf16_bits(rng.standard_normal((24, 40), dtype=np.float32) / np.sqrt(40))
    b = orc.f32_to_bf16_bits(rng.standard_normal((40, 56), dtype=np.float32) / np.sqrt(40))
    out["gemm_bf16_a"], out["gemm_bf16_b"] = a, b
    out["gemm_bf16_d"] = co.ref_gemm_bf16(a, b)
    # integer GEMM twin: tessera_x86_reference_gemm_u8s8_s32 (avx512_vnni_gemm_int8.cpp:5-18)
    au = rng.integers(0, 128, (16, 64)).astype(np.uint8)
    bs = rng.integers(-127, 128, (64, 48)).astype(np.int8)
    out["gemm_i8_a"], out["gemm_i8_b"] = au, bs
    out["gemm_i8_c"] = co.ref_gemm_u8s8(au, bs)
    # flash attention with LSE and GQA: tessera_x86_flash_attn_ext_lse_f32
    # (avx512_flash_attn_f32.cpp:379-422); causal with Sk > Sq (bottom-right aligned)
    for tag, (B, Hq, Hkv, Sq, Sk, D, causal, window, cap) in {
        "fa_causal_gqa": (2, 4, 2, 48, 48, 32, True, 0, 0.0),
        "fa_causal_offset": (1, 2, 1, 20, 52, 16, True, 0, 0.0),
        "fa_full": (1, 3, 3, 33, 40, 64, False, 0, 0.0),
        "fa_window_causal": (1, 2, 1, 70, 90, 32, True, 24, 0.0),      # sliding window, Sk > Sq
        "fa_window_centered": (1, 2, 2, 50, 50, 16, False, 14, 0.0),    # non-causal band
        "fa_softcap": (1, 2, 2, 40, 40, 64, True, 0, 4.0),               # logit soft cap
    }.items():
        q = rng.standard_normal((B, Hq, Sq, D), dtype=np.float32)
        k = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32)
        v = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32)
        q, k, v = (orc.bf16_bits_to_f32(orc.f32_to_bf16_bits(t)).reshape(t.shape) for t in (q, k, v))
        o, lse = co.ref_flash_attn_lse(q, k, v, 1.0 / np.sqrt(D), causal, window, cap)
        out[f"{tag}_q"], out[f"{tag}_k"], out[f"{tag}_v"] = q, k, v
        out[f"{tag}_o"], out[f"{tag}_lse"] = o, lse
        out[f"{tag}_causal"] = np.array(int(causal))
        out[f"{tag}_window"] = np.array(int(window))
        out[f"{tag}_softcap"] = np.array(float(cap))
    # fp8 grid: scalar_fpquant(v, 448, 3, -6) (avx512_fpquant_f32.cpp:28-41)
    x = np.concatenate([
        rng.standard_normal(512).astype(np.float32) * 4,
        np.array([0.0, -0.0, 448.0, 449.0, 1e9, -1e9, 2.0 ** -9, 2.0 ** -10, 1.5 * 2.0 ** -9, 0.0135, 17.0, 18.0, 19.0,
                  -2.5 * 2.0 ** -9, 3.5 * 2.0 ** -9], np.float32),
    ])
    out["fpq_x"], out["fpq_y"] = x, co.ref_fpquant(x)
    # the same kernel on the other grids of its format table (runtime.py:16939-16946):
    # e5m2, the two fp6 grids and e2m1, each over magnitudes from far below the smallest
    # step to beyond saturation, every grid point, every midpoint between neighbours (the
    # ties), NaN and both zeros; plus E2M1 with the exponent floor at 0, the NVFP4 code grid
    for tag, (mx, mant, min_exp) in {"e5m2": (57344.0, 2, -14), "e2m3": (7.5, 3, -126), "e3m2": (28.0, 2, -126),
                                     "e2m1": (6.0, 1, -126), "e2m1_floor0": (6.0, 1, 0)}.items():
        lo = max(min_exp, -20)
        pts = [np.ldexp(1.0 + m / 2.0 ** mant, e) for e in range(lo - 2, int(np.log2(mx)) + 1) for m in range(2 ** mant)]
        pts = np.array(sorted(p for p in pts if p <= mx), np.float64)
        mids = (pts[1:] + pts[:-1]) / 2
        mag = np.exp(rng.uniform(np.log(2.0 ** (lo - 6)), np.log(mx * 4), 768))
        vals = np.concatenate([pts, mids, np.nextafter(mids.astype(np.float32), np.float32(0)),
                               np.nextafter(mids.astype(np.float32), np.float32(np.inf)), mag,
                               [0.0, -0.0, np.nan, mx, mx * 1.01, 1e30, np.ldexp(1.0, lo - 3), 1e-40, 2.0 ** -126]])
        xs = (vals * rng.choice([-1.0, 1.0], vals.size)).astype(np.float32)
        out[f"fpq_{tag}_x"], out[f"fpq_{tag}_y"] = xs, co.ref_fpquant(xs, mx, mant, min_exp)
        out[f"fpq_{tag}_fmt"] = np.array([mx, mant, min_exp], np.float64)
    np.savez_compressed(Path(__file__).with_name("ref_vectors.npz"), **out)
    print("wrote", len(out), "arrays")
    return 0


if __name__ == "__main__":
    sys.exit(main())
