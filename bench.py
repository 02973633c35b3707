#!/usr/bin/env python3
"""Headline benchmark of the gfx950 dense-op lane on one MI355X.

A "step" is one pass of the hot path over one batch of synthetic input: one
``D = A . B`` with A, B bf16 8192 x 8192 (entries N(0,1)/sqrt(K), seeded), f32
accumulate, bf16 output — the configuration the headline metric is quoted on.  Inputs are resident in
HBM before the timed region; the timed region is K launches through the C ABI's
device-pointer entry point, bracketed by a device synchronise on both sides.

One JSON line is printed.  ``roofline`` prices the GEMM kernel against the
MI355X dense bf16 MFMA peak from its average launch duration, measured with HIP
events on the launch stream over the same timed region.  ``cpu_baseline`` times
the oracle's numpy restatement of the reference's CPU path on this host's cores.
``also`` carries the same measurement for the other kernels of the path
(flash-attention forward, fp8 / int8 GEMM, decode-shaped GEMM, the MoE layer), each
with its own parity figure against the oracle on a sample and the oracle's CPU time
on that sample; they are reported, not part of ``value``.

``roofline`` also carries the rate a register-only MFMA loop reaches on this board
on operands distributed like the workload's and on constant ones, with the clock
and power sampled under each: the matrix-pipe ceiling the board grants at its power
limit, measured in the same run.

``--only NAME`` runs one workload alone and ``--profile`` makes the clock ramp before
every timed region use a different kernel instantiation (the f32-output GEMM): a
profiler run of ``--only-headline --profile --warmup 0`` (or ``--only NAME --profile
--warmup 0``) then has one per-kernel row per workload that holds exactly the timed
launches.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

PEAK_BF16_TFLOPS = 2500.0      # MI355X dense bf16/f16 MFMA
PEAK_FP8_TFLOPS = 5000.0
PEAK_INT8_TOPS = 5000.0
PEAK_HBM_GBS = 8000.0
PEAK_CLOCK_MHZ = 2400.0         # shader clock the MFMA peaks are quoted at
# HBM-side bytes one launch of the headline kernel moves: FETCH_SIZE + WRITE_SIZE per
# dispatch from two counter runs of this script, each scaled by the same counter's
# reading for the 1 GiB copy kernel (profiles/bench_all_kernels_hbm_bytes.txt).  A
# profiler figure carried into the line, not something this run measures.
TRAFFIC_BYTES_GEMM_BF16_8192 = 1.7454e9


RAMP_SECONDS = 0.1
_RAMP = {"foreign": False}


def _ramp(lane, launch):
    """Bring the clocks up before a timed region.

    After the host-side data preparation the GPU has idled and its clocks ramp back
    up over the first tens of milliseconds of load (measured: the first 25 launches
    of the headline GEMM run 3-70 % slower than the steady state).  The ramp keeps the
    timed kernel itself running, untimed, for RAMP_SECONDS, which also settles the clock
    at the level the board grants THAT kernel.  Under ``--profile`` the ramp is a kernel
    of its own instead — the f32-output 4096^3 GEMM, an instantiation no timed workload
    uses — so that a profiler's per-kernel row of the timed kernel holds timed launches
    only (for kernels that draw less power than a GEMM the first timed launches then still
    run at the GEMM's lower clock: such rows read a few percent slow)."""
    if not _RAMP["foreign"]:
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < _RAMP.get("seconds", RAMP_SECONDS):
            for _ in range(4):
                launch()
            lane.synchronize()
        return
    if "bufs" not in _RAMP:
        n = 4096
        a = lane.DeviceBuffer.from_host(np.full((n, n), 0x3C3C, np.uint16))
        b = lane.DeviceBuffer.from_host(np.full((n, n), 0x3C3C, np.uint16))
        _RAMP["bufs"] = (a, b, lane.DeviceBuffer(n * n * 4), n)
    a, b, d, n = _RAMP["bufs"]
    fn = lane.load().tessera_gfx950_gemm_bf16_dev
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < _RAMP.get("seconds", RAMP_SECONDS):
        for _ in range(8):
            lane.check(fn(a.ptr, b.ptr, d.ptr, n, n, n, None), "ramp")
        lane.synchronize()


def _timed(lane, launch, steps, warmup):
    """(wall ms/step, event ms/step) for `steps` launches after the clock ramp and
    `warmup` untimed launches; the timed region is exactly `steps` launches."""
    _ramp(lane, launch)
    for _ in range(warmup):
        launch()
    lane.synchronize()
    timer = lane.DeviceTimer()
    t0 = time.perf_counter()
    timer.start()
    for _ in range(steps):
        launch()
    timer.stop()
    lane.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    ev = timer.elapsed_ms() / steps
    timer.close()
    return wall, ev


def _oracle():
    sys.path.insert(0, str(ROOT / "oracle"))
    import tessera_oracle as orc
    return orc


def _blas_threads():
    threads = os.cpu_count() or 1
    try:
        from threadpoolctl import threadpool_info
        blas = [p for p in threadpool_info() if p.get("user_api") == "blas"]
        if blas:
            threads = int(blas[0]["num_threads"])
    except Exception:
        pass
    return threads


def _bf16(x):
    from tessera_amd import bf16
    return np.ascontiguousarray(np.asarray(bf16.from_float32(x), np.uint16))


def bench_gemm(lane, M, N, K, steps, warmup, seed=0):
    rng = np.random.default_rng(seed)
    A = (rng.standard_normal((M, K), dtype=np.float32) / np.sqrt(K)).astype(np.float32)
    B = (rng.standard_normal((K, N), dtype=np.float32) / np.sqrt(K)).astype(np.float32)
    a, b = _bf16(A), _bf16(B)
    da, db = lane.DeviceBuffer.from_host(a), lane.DeviceBuffer.from_host(b)
    dd = lane.DeviceBuffer(M * N * 2)
    fn = lane.load().tessera_gfx950_gemm_bf16_bf16_dev

    def launch():
        lane.check(fn(da.ptr, db.ptr, dd.ptr, M, N, K, None), "gemm_bf16")

    wall, ev = _timed(lane, launch, steps, warmup)
    out = dd.download((M, N), np.uint16)
    for buf in (da, db, dd):
        buf.close()
    return wall, ev, (A, B, a, b, out)


def calibrate_copy(lane, reps=3, nbytes=1 << 30):
    """Launch the library's plain copy kernel on `nbytes` (reads nbytes, writes
    nbytes): the known-size kernel the FETCH_SIZE / WRITE_SIZE counters of a
    profiled run are scaled by."""
    src, dst = lane.DeviceBuffer(nbytes), lane.DeviceBuffer(nbytes)
    src.zero()
    fn = lane.load().tessera_gfx950_memcpy_d2d_dev
    _, ev = _timed(lane, lambda: lane.check(fn(dst.ptr, src.ptr, nbytes, None), "copy"), reps, 1)
    src.close()
    dst.close()
    return {"bytes_each_way": nbytes, "ms": ev, "gbs": 2.0 * nbytes / ev / 1e6}


def bench_attention(lane, steps, warmup, check=True):
    B, Hq, Hkv, S, D = 4, 32, 8, 4096, 128
    rng = np.random.default_rng(1)
    q = _bf16(rng.standard_normal((B, Hq, S, D), dtype=np.float32))
    k = _bf16(rng.standard_normal((B, Hkv, S, D), dtype=np.float32))
    v = _bf16(rng.standard_normal((B, Hkv, S, D), dtype=np.float32))
    dq, dk, dv = (lane.DeviceBuffer.from_host(x) for x in (q, k, v))
    do = lane.DeviceBuffer(q.size * 2)
    dl = lane.DeviceBuffer(B * Hq * S * 4)
    fn = lane.load().tessera_gfx950_flash_attn_gqa_bf16_dev
    scale = 1.0 / np.sqrt(D)

    def launch():
        lane.check(fn(dq.ptr, dk.ptr, dv.ptr, do.ptr, dl.ptr, B, Hq, Hkv, S, S, D, scale, 1, 1, None), "flash_attn")

    wall, ev = _timed(lane, launch, steps, warmup)
    flop = 4.0 * B * Hq * (S * (S + 1) / 2) * D          # the reference's causal FLOP model
    out = {"workload": "flash_attn_fwd_bf16_causal_B4_Hq32_Hkv8_S4096_D128", "ms": ev,
           "tflops": flop / ev / 1e9, "frac_mfma_peak": flop / ev / 1e9 / PEAK_BF16_TFLOPS}
    if check:
        # parity and CPU time on a sample of (batch, head) pairs: the oracle's blockwise
        # restatement of the reference's attention, f32 O and LSE of the same launch shape
        orc = _oracle()
        o32 = lane.DeviceBuffer(q.size * 4)
        lane.check(fn(dq.ptr, dk.ptr, dv.ptr, o32.ptr, dl.ptr, B, Hq, Hkv, S, S, D, scale, 1, 0, None), "flash_attn")
        lane.synchronize()
        got_o = o32.download((B, Hq, S, D), np.float32)
        got_l = dl.download((B, Hq, S), np.float32)
        o32.close()
        heads = [(0, 0), (3, 31)]
        f32 = lambda bits: (bits.astype(np.uint32) << 16).view(np.float32)
        t0 = time.perf_counter()
        ro, rl = orc.flash_attn_blockwise(f32(q), f32(k), f32(v), scale=scale, causal=True, heads=heads)
        dt = time.perf_counter() - t0
        o_err = max(orc.max_rel_err(got_o[b, h], ro[b, h]) for b, h in heads)
        l_err = max(float(np.max(np.abs(got_l[b, h] - rl[b, h]))) for b, h in heads)
        out["parity"] = {"o_max_rel": o_err, "lse_max_abs": l_err, "bound": 2e-3,
                         "sample": f"{len(heads)} of {B * Hq} (batch, head) pairs, all 4096 rows each"}
        sample_flop = flop * len(heads) / (B * Hq)
        out["cpu_baseline"] = {"value": sample_flop / dt / 1e12, "unit": "TFLOP/s", "cores": _blas_threads(),
                               "kind": "port", "sample": f"{len(heads)} (batch, head) pairs blockwise in numpy f32, "
                                                         f"{dt:.2f} s; the full workload is {B * Hq // len(heads)}x that"}
    for buf in (dq, dk, dv, do, dl):
        buf.close()
    return out


def bench_attention_decode(lane, steps, warmup, check=True):
    """One query row per head against a long key range (a decode step with a KV cache): bound by
    reading K and V once, 537 MB here (more than the memory-side cache holds).  The rows of a GQA
    group share one MFMA tile and the key range is split over the chip (the decode kernel)."""
    B, Hq, Hkv, Sk, D = 64, 32, 8, 2048, 128
    rng = np.random.default_rng(2)
    q = _bf16(rng.standard_normal((B, Hq, 1, D), dtype=np.float32))
    # eight distinct batches of K / V, repeated: the bytes streamed are what matters for the timing
    k8 = _bf16(rng.standard_normal((8, Hkv, Sk, D), dtype=np.float32))
    v8 = _bf16(rng.standard_normal((8, Hkv, Sk, D), dtype=np.float32))
    k, v = np.tile(k8, (B // 8, 1, 1, 1)), np.tile(v8, (B // 8, 1, 1, 1))
    dq, dk, dv = (lane.DeviceBuffer.from_host(x) for x in (q, k, v))
    do = lane.DeviceBuffer(q.size * 4)
    dl = lane.DeviceBuffer(B * Hq * 4)
    fn = lane.load().tessera_gfx950_flash_attn_gqa_bf16_dev
    scale = 1.0 / np.sqrt(D)

    def launch():
        lane.check(fn(dq.ptr, dk.ptr, dv.ptr, do.ptr, dl.ptr, B, Hq, Hkv, 1, Sk, D, scale, 0, 0, None), "flash_attn")

    wall, ev = _timed(lane, launch, max(steps, 50), warmup)
    nbytes = 2 * k.size * 2 + q.size * 2 + q.size * 4
    out = {"workload": f"flash_attn_decode_bf16_B{B}_Hq{Hq}_Hkv{Hkv}_Sq1_Sk{Sk}_D{D}", "ms": ev,
           "gbs": nbytes / ev / 1e6, "frac_hbm_peak": nbytes / ev / 1e6 / PEAK_HBM_GBS}
    if check:
        orc = _oracle()
        lane.synchronize()
        got_o = do.download((B, Hq, 1, D), np.float32)
        got_l = dl.download((B, Hq, 1), np.float32)
        f32 = lambda bits: (bits.astype(np.uint32) << 16).view(np.float32)
        sample = [0, 9, 63]
        ro, rl = orc.flash_attn_dense(f32(q[sample]), f32(k[sample]), f32(v[sample]), scale=scale, causal=False)
        out["parity"] = {"o_max_rel": orc.max_rel_err(got_o[sample], ro),
                         "lse_max_abs": float(np.max(np.abs(got_l[sample] - rl))), "bound": 2e-3,
                         "sample": f"{len(sample)} of {B} batches, all heads, dense f64 oracle"}
    for buf in (dq, dk, dv, do, dl):
        buf.close()
    return out


def bench_attention_bwd(lane, steps, warmup):
    """Backward of the same attention configuration with the forward's O and LSE
    saved (dQ, dK, dV kernels + the Delta pass), and with the forward recomputed."""
    B, Hq, Hkv, S, D = 4, 32, 8, 4096, 128
    rng = np.random.default_rng(5)
    q, do = (_bf16(rng.standard_normal((B, Hq, S, D), dtype=np.float32)) for _ in range(2))
    k, v = (_bf16(rng.standard_normal((B, Hkv, S, D), dtype=np.float32)) for _ in range(2))
    dq, dk, dv, ddo = (lane.DeviceBuffer.from_host(x) for x in (q, k, v, do))
    o32, lse = lane.DeviceBuffer(q.size * 4), lane.DeviceBuffer(B * Hq * S * 4)
    gq, gk, gv = lane.DeviceBuffer(q.size * 4), lane.DeviceBuffer(k.size * 4), lane.DeviceBuffer(k.size * 4)
    lib = lane.load()
    scale = 1.0 / np.sqrt(D)
    lane.check(lib.tessera_gfx950_flash_attn_gqa_bf16_dev(dq.ptr, dk.ptr, dv.ptr, o32.ptr, lse.ptr, B, Hq, Hkv, S, S,
                                                          D, scale, 1, 0, None), "flash_attn")
    fn = lib.tessera_gfx950_flash_attn_bwd_bf16_dev
    saved = lambda: lane.check(fn(ddo.ptr, dq.ptr, dk.ptr, dv.ptr, o32.ptr, lse.ptr, gq.ptr, gk.ptr, gv.ptr,
                                  B, Hq, Hkv, S, S, D, scale, 1, None), "flash_attn_bwd")
    recomp = lambda: lane.check(fn(ddo.ptr, dq.ptr, dk.ptr, dv.ptr, None, None, gq.ptr, gk.ptr, gv.ptr,
                                   B, Hq, Hkv, S, S, D, scale, 1, None), "flash_attn_bwd")
    _, ev = _timed(lane, saved, steps, warmup)
    _, ev_re = _timed(lane, recomp, steps, warmup)
    for buf in (dq, dk, dv, ddo, o32, lse, gq, gk, gv):
        buf.close()
    flop = 2.5 * 4.0 * B * Hq * (S * (S + 1) / 2) * D        # five S x S x D products against the forward's two
    return {"workload": "flash_attn_bwd_bf16_causal_B4_Hq32_Hkv8_S4096_D128", "ms": ev, "ms_with_forward_recompute": ev_re,
            "tflops": flop / ev / 1e9, "frac_mfma_peak": flop / ev / 1e9 / PEAK_BF16_TFLOPS}


def bench_quant(lane, steps, warmup, check=True):
    """Config 5: M=4096, N=K=8192, operands quantised from N(0,1) data by the lane's own
    quantisers — (a) e4m3 codes with per-tensor scales, bf16 out; (b) int8 with per-row
    activation and per-column weight scales (W8A8), int32 accumulate, f32 out."""
    import ctypes
    M, N, K = 4096, 8192, 8192
    rng = np.random.default_rng(2)
    X = rng.standard_normal((M, K), dtype=np.float32)
    W = rng.standard_normal((K, N), dtype=np.float32)
    lib = lane.load()
    out = {}
    xf, wf = lane.DeviceBuffer.from_host(X), lane.DeviceBuffer.from_host(W)
    xq, wq = lane.DeviceBuffer(M * K), lane.DeviceBuffer(K * N)
    rs, cs = lane.DeviceBuffer(M * 4), lane.DeviceBuffer(N * 4)
    dd = lane.DeviceBuffer(M * N * 4)
    ops = 2.0 * M * N * K
    sample = np.sort(rng.choice(M, 64, replace=False))
    orc = _oracle() if check else None

    # ---- (b) int8 W8A8 -----------------------------------------------------------------
    q_rows = lambda: lane.check(lib.tessera_gfx950_quantize_i8_f32_dev(xf.ptr, M, K, 1, xq.ptr, rs.ptr, None), "quantize_i8")
    lane.check(lib.tessera_gfx950_quantize_i8_f32_dev(wf.ptr, K, N, 0, wq.ptr, cs.ptr, None), "quantize_i8")
    _, ev = _timed(lane, q_rows, steps, warmup)
    qbytes = 5.0 * M * K + 4.0 * M
    out["quantize_int8_rows_4096x8192"] = {"ms": ev, "gbs": qbytes / ev / 1e6, "frac_hbm_peak": qbytes / ev / 1e6 / PEAK_HBM_GBS}
    _, ev = _timed(lane, lambda: lane.check(lib.tessera_gfx950_gemm_i8_i32_dev(xq.ptr, wq.ptr, dd.ptr, M, N, K, None),
                                            "gemm_i8"), steps, warmup)
    out["gemm_int8_4096x8192x8192"] = {"workload": "int8 codes of N(0,1) data (per-row / per-column absmax), int32 out",
                                       "ms": ev, "tops": ops / ev / 1e9, "frac_mfma_peak": ops / ev / 1e9 / PEAK_INT8_TOPS}
    _, ev = _timed(lane, lambda: lane.check(lib.tessera_gfx950_gemm_w8a8_f32_dev(xq.ptr, wq.ptr, rs.ptr, cs.ptr, dd.ptr,
                                                                                 None, M, N, K, None), "gemm_w8a8"),
                   steps, warmup)
    w8 = {"workload": "W8A8: the same codes, f32(acc) * row_scale * col_scale, f32 out", "ms": ev,
          "tops": ops / ev / 1e9, "frac_mfma_peak": ops / ev / 1e9 / PEAK_INT8_TOPS}
    if check:
        acc = lane.DeviceBuffer(M * N * 4)
        lane.check(lib.tessera_gfx950_gemm_w8a8_f32_dev(xq.ptr, wq.ptr, rs.ptr, cs.ptr, dd.ptr, acc.ptr, M, N, K, None),
                   "gemm_w8a8")
        lane.synchronize()
        got_y = dd.download((M, N), np.float32)[sample]
        got_acc = acc.download((M, N), np.int32)[sample]
        acc.close()
        t0 = time.perf_counter()
        ry, racc, rxq, ras, rwq, rws = orc.w8a8_matmul(X[sample], W)
        dt = time.perf_counter() - t0
        codes_ok = bool(np.array_equal(xq.download((M, K), np.int8)[sample], rxq) and
                        np.array_equal(wq.download((K, N), np.int8), rwq))
        w8["parity"] = {"int32_accumulators_bit_exact": bool(np.array_equal(got_acc, racc)),
                        "codes_and_scales_bit_exact": codes_ok and bool(
                            np.array_equal(rs.download((M,), np.float32)[sample], ras.reshape(-1)) and
                            np.array_equal(cs.download((N,), np.float32), rws)),
                        "y_max_rel": orc.max_rel_err(got_y, ry), "sample": "64 of 4096 rows, all 8192 columns"}
        w8["cpu_baseline"] = {"value": 2.0 * len(sample) * N * K / dt / 1e12, "unit": "TOP/s", "cores": _blas_threads(),
                              "kind": "port", "sample": f"quantise + exact integer product of 64 rows in numpy, {dt:.2f} s "
                                                        "(includes quantising the whole 8192 x 8192 weight); "
                                                        "the full workload has 64x the rows"}
    out["gemm_w8a8_scaled_4096x8192x8192"] = w8
    # quantised decode: a few rows of int8 activations against the same 8192 x 8192 int8 weight, launches cycling
    # over four copies of it so that the 67 MB do not sit in the memory-side cache (HBM-bound: one pass over B)
    wcopies = [wq] + [lane.DeviceBuffer(K * N) for _ in range(3)]
    for c in wcopies[1:]:
        lane.check(lib.tessera_gfx950_memcpy_d2d_dev(c.ptr, wq.ptr, K * N, None), "copy")
    lane.synchronize()
    for Md in (1, 16, 32):
        turn = [0]
        def dec():
            turn[0] += 1
            lane.check(lib.tessera_gfx950_gemm_w8a8_f32_dev(xq.ptr, wcopies[turn[0] & 3].ptr, rs.ptr, cs.ptr, dd.ptr, None,
                                                            Md, N, K, None), "gemm_w8a8")
        # (a short run — the counter passes of the profiles use --steps 3 — stays short)
        _, ev = _timed(lane, dec, max(steps, 50) if steps >= 10 else steps, warmup)
        dbytes = 1.0 * K * N + Md * K + 4.0 * Md * N
        out[f"gemm_w8a8_decode_M{Md}_8192x8192"] = {"ms": ev, "gbs": dbytes / ev / 1e6,
                                                    "frac_hbm_peak": dbytes / ev / 1e6 / PEAK_HBM_GBS, "weights_cycled": 4}
    for c in wcopies[1:]:
        c.close()
    # the int8 matrix pipes' own rate on such codes, no memory access: the ceiling of both rows above
    c8 = mfma_ceiling(lane, _OPTS["ceiling_seconds"], "int8")
    out["mfma_ceiling_int8"] = c8
    for key in ("gemm_int8_4096x8192x8192", "gemm_w8a8_scaled_4096x8192x8192"):
        out[key].update(_ceiling_fields(c8, out[key]["tops"]))

    # ---- (a) fp8 e4m3, per-tensor scales ---------------------------------------------------
    sx, sw = lane.DeviceBuffer(4), lane.DeviceBuffer(4)
    q_e4 = lambda: lane.check(lib.tessera_gfx950_quantize_e4m3_f32_dev(xf.ptr, M * K, 0.0, xq.ptr, sx.ptr, None), "quantize_e4m3")
    lane.check(lib.tessera_gfx950_quantize_e4m3_f32_dev(wf.ptr, K * N, 0.0, wq.ptr, sw.ptr, None), "quantize_e4m3")
    _, ev = _timed(lane, q_e4, steps, warmup)
    ebytes = 9.0 * M * K
    out["quantize_e4m3_tensor_4096x8192"] = {"ms": ev, "gbs": ebytes / ev / 1e6, "frac_hbm_peak": ebytes / ev / 1e6 / PEAK_HBM_GBS}
    # the per-tensor float-grid kernel (e5m2 here): absmax pass, then read f32 / write the dequantised f32
    _, ev = _timed(lane, lambda: lane.check(lib.tessera_gfx950_fake_quantize_fp_f32_dev(
        xf.ptr, M * K, ctypes.c_float(57344.0), 2, -14, ctypes.c_float(0.0), dd.ptr, None, None, None), "quantize_fp"),
        steps, warmup)
    gbytes = 12.0 * M * K
    out["fake_quantize_e5m2_tensor_4096x8192"] = {"ms": ev, "gbs": gbytes / ev / 1e6,
                                                  "frac_hbm_peak": gbytes / ev / 1e6 / PEAK_HBM_GBS}
    lane.synchronize()
    scale_a = float(sx.download((1,), np.float32)[0])
    scale_b = float(sw.download((1,), np.float32)[0])
    _, ev = _timed(lane, lambda: lane.check(
        lib.tessera_gfx950_gemm_e4m3_bf16_dev(xq.ptr, wq.ptr, ctypes.c_float(scale_a), ctypes.c_float(scale_b), dd.ptr,
                                              M, N, K, None), "gemm_e4m3"), steps, warmup)
    f8 = {"workload": "e4m3 codes of N(0,1) data, per-tensor scales amax/448, bf16 out", "ms": ev,
          "tflops": ops / ev / 1e9, "frac_mfma_peak": ops / ev / 1e9 / PEAK_FP8_TFLOPS}
    if check:
        lane.check(lib.tessera_gfx950_gemm_e4m3_f32_dev(xq.ptr, wq.ptr, ctypes.c_float(scale_a), ctypes.c_float(scale_b),
                                                        dd.ptr, M, N, K, None), "gemm_e4m3")
        lane.synchronize()
        got = dd.download((M, N), np.float32)[sample]
        a_codes = xq.download((M, K), np.uint8)[sample]
        b_codes = wq.download((K, N), np.uint8)
        t0 = time.perf_counter()
        ra, _, rsa = orc.quantize_fp8_e4m3(X)            # the scale is per tensor: the whole activation
        rb, _, rsb = orc.quantize_fp8_e4m3(W)
        ref_q = orc.gemm_e4m3(ra[sample], rb, rsa, rsb)
        dt = time.perf_counter() - t0
        ref_full = X[sample].astype(np.float64) @ W.astype(np.float64)
        tbl = orc.e4m3_decode_table()                     # (-0 and +0 are two codes of one value)
        f8["parity"] = {"codes_equal_as_values": bool(np.array_equal(tbl[a_codes], tbl[ra[sample]]) and
                                                      np.array_equal(tbl[b_codes], tbl[rb])),
                        "scales_equal": bool(np.float32(scale_a) == rsa and np.float32(scale_b) == rsb),
                        "max_rel_vs_product_of_dequantised_operands": orc.max_rel_err(got, ref_q),
                        "max_rel_vs_unquantised_f64_product": orc.max_rel_err(got, ref_full),
                        "bounds": {"dequantised": 2e-3, "unquantised": 5e-2},
                        "sample": "64 of 4096 rows, all 8192 columns"}
        f8["cpu_baseline"] = {"value": 2.0 * len(sample) * N * K / dt / 1e12, "unit": "TFLOP/s", "cores": _blas_threads(),
                              "kind": "port", "sample": f"quantise both tensors + f64 product of 64 dequantised rows in "
                                                        f"numpy, {dt:.2f} s; the full workload has 64x the rows"}
    # the same product on e5m2 codes (the matrix instruction's second fp8 operand format)
    lane.check(lib.tessera_gfx950_quantize_e5m2_f32_dev(xf.ptr, M * K, 0.0, xq.ptr, sx.ptr, None), "quantize_e5m2")
    lane.check(lib.tessera_gfx950_quantize_e5m2_f32_dev(wf.ptr, K * N, 0.0, wq.ptr, sw.ptr, None), "quantize_e5m2")
    lane.synchronize()
    s5a, s5b = float(sx.download((1,), np.float32)[0]), float(sw.download((1,), np.float32)[0])
    _, ev = _timed(lane, lambda: lane.check(
        lib.tessera_gfx950_gemm_e5m2_bf16_dev(xq.ptr, wq.ptr, ctypes.c_float(s5a), ctypes.c_float(s5b), dd.ptr,
                                              M, N, K, None), "gemm_e5m2"), steps, warmup)
    out["gemm_fp8_e5m2_4096x8192x8192"] = {"workload": "e5m2 codes of N(0,1) data, per-tensor scales amax/57344, bf16 out",
                                           "ms": ev, "tflops": ops / ev / 1e9,
                                           "frac_mfma_peak": ops / ev / 1e9 / PEAK_FP8_TFLOPS}
    cf = mfma_ceiling(lane, _OPTS["ceiling_seconds"], "fp8")
    out["mfma_ceiling_fp8"] = cf
    f8.update(_ceiling_fields(cf, f8["tflops"]))
    out["gemm_fp8_e4m3_4096x8192x8192"] = f8
    for buf in (xf, wf, xq, wq, rs, cs, dd, sx, sw):
        buf.close()
    return out


def bench_gemm_constant_operands(lane, steps):
    """The headline product on constant operands (every element 0x3c3c = 0.0114), timed by
    the library's own loop.  Same kernel, same launches: the only difference from the
    headline figure is that the operands do not toggle, so the matrix cores draw less
    power and the part holds a higher clock.  The gap between the two numbers is the
    power limit, not the kernel's schedule."""
    import ctypes
    ms = ctypes.c_double(0.0)
    M = N = K = 8192
    lane.check(lane.load().tessera_gfx950_gemm_bf16_bench(M, N, K, max(steps, 20), ctypes.byref(ms)), "gemm_bench")
    tf = 2.0 * M * N * K / ms.value / 1e9
    return {"ms": ms.value, "tflops": tf, "frac_mfma_peak": tf / PEAK_BF16_TFLOPS,
            "note": "constant operands: not the metric, shows the power limit on random data"}


def bench_batched_small(lane, steps, warmup):
    """The reference README's step(): A[4,128,64] f16 x W[4,64,256] f16 -> f32, one
    strided-batched launch.  Launch-latency bound: microseconds per launch and the
    rate of its 720,896 algorithmic bytes."""
    Bt, M, K, N = 4, 128, 64, 256
    rng = np.random.default_rng(0)
    a = (rng.standard_normal((Bt, M, K)) / 8).astype(np.float16)
    w = (rng.standard_normal((Bt, K, N)) / 8).astype(np.float16)
    da, dw = lane.DeviceBuffer.from_host(a), lane.DeviceBuffer.from_host(w)
    dd = lane.DeviceBuffer(Bt * M * N * 4)
    fn = lane.load().tessera_gfx950_batched_gemm_f16_dev

    def launch():
        lane.check(fn(da.ptr, dw.ptr, dd.ptr, Bt, M, N, K, None), "batched_gemm_f16")

    wall, ev = _timed(lane, launch, max(steps, 200), warmup)
    got = dd.download((Bt, M, N), np.float32)
    ref = np.matmul(a.astype(np.float32), w.astype(np.float32))
    for buf in (da, dw, dd):
        buf.close()
    nbytes = a.nbytes + w.nbytes + got.nbytes
    return {"workload": "batched_gemm_f16_4x128x64x256_f32out", "us": ev * 1e3, "us_wall": wall * 1e3,
            "gbs": nbytes / ev / 1e6, "gflops": 2.0 * Bt * M * N * K / ev / 1e6,
            "max_rel_vs_f32": float(np.max(np.abs(got - ref)) / np.max(np.abs(ref)))}


def bench_decode(lane, steps, warmup):
    """Decode-shaped products (M rows against an 8192 x 8192 weight).  The launches
    cycle over four weight matrices inside the library's own timing loop: one matrix
    (134 MB) would stay in the 256 MB memory-side cache and not be read from HBM."""
    import ctypes
    N = K = 8192
    out = {}
    fn = lane.load().tessera_gfx950_gemm_bf16_bench_rotating
    ms = ctypes.c_double(0.0)
    for M in (1, 16, 128):
        lane.check(fn(M, N, K, max(steps, 50), 4, ctypes.byref(ms)), "gemm_bench")
        ev = ms.value
        nbytes = K * N * 2 + M * K * 2 + M * N * 2
        out[f"gemm_bf16_decode_M{M}_8192x8192"] = {"ms": ev, "gbs": nbytes / ev / 1e6,
                                                   "frac_hbm_peak": nbytes / ev / 1e6 / PEAK_HBM_GBS,
                                                   "weights_cycled": 4}
    return out


def _expert_weights(E, rows, cols, seed):
    """E expert matrices ~ N(0, 0.02) in bf16: one seeded block per matrix, re-used for
    every expert with its own row rotation and sign pattern (drawing 1.1e9 normals for
    the three weight tensors would take longer than everything else in this script)."""
    r = np.random.default_rng(seed)
    base = _bf16(0.02 * r.standard_normal((rows, cols), dtype=np.float32))
    flip = (r.integers(0, 2, (rows, cols), dtype=np.uint16) << 15).astype(np.uint16)
    w = np.empty((E, rows, cols), np.uint16)
    for e in range(E):
        w[e] = np.roll(base, 17 * e + 3, axis=0) ^ np.roll(flip, 5 * e + 1, axis=1)
    return w


def bench_moe(lane, steps, warmup, check=True):
    """Config 4: the whole layer through its device-resident entry point (routing ->
    expert block reading x through the dispatch map -> combine, one stream, no host hop),
    with the router logits given; the stages are also timed on their own."""
    import ctypes
    T, H, F, E, k = 8192, 4096, 1408, 64, 8
    rng = np.random.default_rng(4)
    S = T * k
    logits = rng.standard_normal((T, E), dtype=np.float32)
    lib = lane.load()
    dlog = lane.DeviceBuffer.from_host(logits)
    dtos, deos, dcw = lane.DeviceBuffer(S * 4), lane.DeviceBuffer(S * 4), lane.DeviceBuffer(S * 4)
    dgs, dgo, dn = lane.DeviceBuffer(E * 4), lane.DeviceBuffer((E + 1) * 4), lane.DeviceBuffer(4)
    x = _bf16(rng.standard_normal((T, H), dtype=np.float32))
    dx = lane.DeviceBuffer.from_host(x)
    wg, wu, wd = _expert_weights(E, H, F, 11), _expert_weights(E, H, F, 12), _expert_weights(E, F, H, 13)
    dwg, dwu, dwd = (lane.DeviceBuffer.from_host(w) for w in (wg, wu, wd))
    wr = _bf16(rng.standard_normal((H, E), dtype=np.float32) / np.sqrt(H))
    dwr = lane.DeviceBuffer.from_host(wr)
    need = ctypes.c_size_t(0)
    lane.check(lib.tessera_gfx950_moe_layer_workspace_bytes(T, H, F, H, E, k, ctypes.byref(need)), "workspace")
    dws = lane.DeviceBuffer(need.value)
    dout = lane.DeviceBuffer(T * H * 4)

    def layer(router):
        return lambda: lane.check(lib.tessera_gfx950_moe_layer_bf16_dev(
            dx.ptr, dwr.ptr if router else None, None if router else dlog.ptr, dwg.ptr, dwu.ptr, dwd.ptr, dout.ptr,
            dws.ptr, need.value, T, H, F, H, E, k, 1, 0, dtos.ptr, deos.ptr, dcw.ptr, dgs.ptr, dgo.ptr, dn.ptr, None),
            "moe_layer")

    _, ev_layer = _timed(lane, layer(False), steps, warmup)
    got = dout.download((T, H), np.float32)
    plan = [b.download(shape, dt) for b, shape, dt in ((dtos, (S,), np.int32), (deos, (S,), np.int32),
                                                       (dcw, (S,), np.float32), (dgs, (E,), np.int32),
                                                       (dgo, (E + 1,), np.int32))]
    _, ev_layer_r = _timed(lane, layer(True), steps, warmup)
    # the stages on their own (the routing of the timed layer is still in the plan buffers:
    # re-run it from the given logits first)
    route = lambda: lane.check(lib.tessera_gfx950_moe_route_f32_dev(
        dlog.ptr, T, E, k, 1, 0, dtos.ptr, deos.ptr, dcw.ptr, dgs.ptr, dgo.ptr, dn.ptr, None), "route")
    _, ev_route = _timed(lane, route, steps, warmup)
    dh, dy = lane.DeviceBuffer(S * F * 2), lane.DeviceBuffer(S * H * 2)
    ffn_g = lambda: lane.check(lib.tessera_gfx950_moe_swiglu_block_gather_bf16_dev(
        dx.ptr, dtos.ptr, dwg.ptr, dwu.ptr, dwd.ptr, dgo.ptr, dy.ptr, dh.ptr, T, S, H, F, H, E, None), "swiglu_gather")
    _, ev_ffn_g = _timed(lane, ffn_g, steps, warmup)
    comb = lambda: lane.check(lib.tessera_gfx950_moe_combine_bf16_dev(dy.ptr, dtos.ptr, dcw.ptr, dout.ptr, T, S, H, None),
                              "combine")
    _, ev_comb = _timed(lane, comb, steps, warmup)
    flop = 6.0 * S * H * F
    out = {"workload": "moe_T8192_H4096_E64_top8_F1408_bf16 (router logits given)",
           "layer_ms": ev_layer, "layer_with_router_gemm_ms": ev_layer_r,
           "route_ms": ev_route, "dispatch_fused_expert_ffn_ms": ev_ffn_g, "combine_ms": ev_comb,
           "layer_tflops": flop / ev_layer / 1e9, "frac_mfma_peak": flop / ev_layer / 1e9 / PEAK_BF16_TFLOPS,
           "expert_ffn_tflops": flop / ev_ffn_g / 1e9, "expert_ffn_frac_mfma_peak": flop / ev_ffn_g / 1e9 / PEAK_BF16_TFLOPS,
           "note": "frac_mfma_peak prices the expert FFN's 6 S H F FLOP against the time of the WHOLE layer "
                   "(routing and combine included)"}
    if check:
        orc = _oracle()
        f32 = lambda bits: (bits.astype(np.uint32) << 16).view(np.float32)
        r = orc.route_tokens(logits, E, k)
        desc = orc.plan_dispatch(r.assignment, r.weights, E)
        idx_ok = bool(np.array_equal(plan[0], desc.token_of_slot) and np.array_equal(plan[1], desc.expert_of_slot) and
                      np.array_equal(plan[3], desc.group_sizes) and np.array_equal(plan[4], desc.group_offsets))
        tokens = np.sort(rng.choice(T, 16, replace=False))
        slots = np.flatnonzero(np.isin(desc.token_of_slot, tokens))
        tok_of = desc.token_of_slot[slots].astype(np.int64)
        exp_of = desc.expert_of_slot[slots].astype(np.int64)
        xs = f32(x)[tok_of]
        t0 = time.perf_counter()
        y = np.zeros((slots.size, H), np.float32)
        for e in np.unique(exp_of):
            rows = np.flatnonzero(exp_of == e)
            y[rows] = orc.moe_swiglu_block(xs[rows], f32(wg[e:e + 1]), f32(wu[e:e + 1]), f32(wd[e:e + 1]), [rows.size])
        dt = time.perf_counter() - t0
        ref = np.zeros((T, H), np.float64)
        np.add.at(ref, tok_of, y.astype(np.float64) * desc.combine_weights[slots][:, None].astype(np.float64))
        out["parity"] = {"indices_bit_exact": idx_ok, "combine_weights_max_abs": float(np.max(np.abs(plan[2] - desc.combine_weights))),
                         "out_max_rel": orc.max_rel_err(got[tokens], ref[tokens]), "bound": 2e-3 + 2.0 ** -8,
                         "sample": "all 65,536 slot indices; layer output of 16 of 8192 tokens (128 slots)"}
        out["cpu_baseline"] = {"value": 6.0 * slots.size * H * F / dt / 1e12, "unit": "TFLOP/s", "cores": _blas_threads(),
                               "kind": "port", "sample": f"expert FFN of 128 of 65,536 slots in numpy (one small product "
                                                         f"per expert touched), {dt:.2f} s"}
    for buf in (dlog, dtos, deos, dcw, dgs, dgo, dn, dx, dwg, dwu, dwd, dwr, dws, dh, dy, dout):
        buf.close()
    return out


def mfma_ceiling(lane, seconds=2.0, kind="bf16"):
    """The rate a register-only loop of independent matrix instructions reaches on this board
    (tessera_gfx950_mfma_probe_dev: no memory access inside the loop; 16x16x32 bf16 -- the
    instruction of the 256 x 256 GEMM tile --, 32x32x16 bf16 ("bf16_32x32x16": attention and the
    MoE block), 32x32x32 int8 or 32x32x64 fp8), on operands distributed like the workload's and on constant ones,
    with the shader clock and socket power sampled while it runs.  The matrix pipes draw more
    power on toggling operands, the board holds its power limit by lowering the clock, and the
    published peak assumes PEAK_CLOCK_MHZ: the random-operand figure is the ceiling a GEMM on
    such data is up against on this board.  bf16: N(0,1)/sqrt(8192) values; int8 and fp8: the
    codes the lane's own quantisers give N(0,1) data (per-row absmax / per-tensor amax)."""
    import ctypes
    lib = lane.load()
    rng = np.random.default_rng(7)
    nbytes = 16 * 8 * 64 * 16                               # the probe's fragment buffer
    code = {"bf16": 3, "bf16_32x32x16": 0, "int8": 1, "fp8": 2}[kind]
    sink = lane.DeviceBuffer(1024 * 256 * 4)
    ops = ctypes.c_double(0.0)
    rounds = 300 if kind == "bf16" else 600 if kind == "bf16_32x32x16" else 300
    if kind.startswith("bf16"):
        random_frags = lane.DeviceBuffer.from_host(_bf16(rng.standard_normal(nbytes // 2, dtype=np.float32) / np.sqrt(8192.0)))
        constant = np.full(nbytes // 2, 0x3C3C, np.uint16)
    else:
        xf = lane.DeviceBuffer.from_host(rng.standard_normal(nbytes, dtype=np.float32))
        random_frags, scales = lane.DeviceBuffer(nbytes), lane.DeviceBuffer(16 * 4)
        if kind == "int8":
            lane.check(lib.tessera_gfx950_quantize_i8_f32_dev(xf.ptr, 16, nbytes // 16, 1, random_frags.ptr, scales.ptr, None),
                       "quantize_i8")
            constant = np.full(nbytes, 1, np.int8)
        else:
            lane.check(lib.tessera_gfx950_quantize_e4m3_f32_dev(xf.ptr, nbytes, 0.0, random_frags.ptr, scales.ptr, None),
                       "quantize_e4m3")
            constant = np.full(nbytes, 0x38, np.uint8)       # 1.0 in e4m3
        lane.synchronize()
        xf.close()
        scales.close()
    out = {}
    for tag, frags in (("random", random_frags), ("constant", lane.DeviceBuffer.from_host(constant))):
        launch = lambda: lane.check(lib.tessera_gfx950_mfma_probe_dev(code, frags.ptr, rounds, sink.ptr,
                                                                      ctypes.byref(ops), None), "mfma_probe")
        _, ev = _timed(lane, launch, 20, 5)
        r = {"tflops": ops.value / ev / 1e9, "ms": ev}
        if seconds > 0:
            held = _sustained(lane, launch, seconds)
            if "ms" in held:
                r.update({"tflops_sustained": ops.value / held["ms"] / 1e9, "gfx_clock_mhz": held["gfx_clock_mhz"],
                          "socket_power_w": held["socket_power_w"]})
        out[tag] = r
        frags.close()
    sink.close()
    return out


def _ceiling_fields(ceil, rate):
    """What a roofline entry says about the measured matrix-pipe ceiling."""
    rnd, cst = ceil["random"], ceil["constant"]
    top = rnd.get("tflops_sustained", rnd["tflops"])
    return {"ceiling_random_tflops": top, "ceiling_constant_tflops": cst.get("tflops_sustained", cst["tflops"]),
            "ceiling_random_clock_mhz": rnd.get("gfx_clock_mhz"), "ceiling_random_power_w": rnd.get("socket_power_w"),
            "ceiling_constant_clock_mhz": cst.get("gfx_clock_mhz"), "ceiling_constant_power_w": cst.get("socket_power_w"),
            "frac_of_random_ceiling": rate / top}


_OPTS = {"ceiling_seconds": 1.5}      # 0: time the ceiling probes without sampling clock and power


_VENDOR_SNIPPET = r"""
import json, time, torch
M = N = K = 8192
g = torch.Generator(device="cpu").manual_seed(0)
a = (torch.randn(M, K, generator=g) / K ** 0.5).to(torch.bfloat16).cuda()
b = (torch.randn(K, N, generator=g) / K ** 0.5).to(torch.bfloat16).cuda()
for _ in range(150):
    c = torch.mm(a, b)
torch.cuda.synchronize()
e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
e0.record()
for _ in range(50):
    c = torch.mm(a, b)
e1.record()
torch.cuda.synchronize()
ms = e0.elapsed_time(e1) / 50
print(json.dumps({"ms": ms, "tflops": 2.0 * M * N * K / ms / 1e9, "library": "torch.mm bf16 (hipBLASLt / rocBLAS), row-major A and B",
                  "torch": torch.__version__}))
"""


def _run_child(cmd, timeout_s):
    """Run `cmd` in a process group of its own, wait for it, and make sure nothing it started
    outlives this call (the group is ended and reaped whichever way the child finished)."""
    import signal
    import subprocess
    p = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, start_new_session=True)
    try:
        out, err = p.communicate(timeout=timeout_s)
    except subprocess.TimeoutExpired:
        out, err = "", f"timed out after {timeout_s} s"
    finally:
        try:
            os.killpg(p.pid, signal.SIGKILL)          # the group this call created, by its exact id
        except (ProcessLookupError, PermissionError):
            pass
        p.wait()
    return p.returncode, out, err


def vendor_gemm_same_box(timeout_s=240):
    """The vendor library's GEMM of the same shape, layout and data distribution on the
    same box, in a child process (PyTorch is not part of this package): a yardstick for
    what a production kernel reaches under the same power limit.  Any failure is reported,
    not raised."""
    try:
        rc, out, err = _run_child([sys.executable, "-c", _VENDOR_SNIPPET], timeout_s)
        line = [l for l in out.splitlines() if l.startswith("{")]
        if rc != 0 or not line:
            return {"error": (err or out).strip().splitlines()[-1:] or ["no output"]}
        d = json.loads(line[-1])
        d["frac_mfma_peak"] = d["tflops"] / PEAK_BF16_TFLOPS
        return d
    except (OSError, ValueError) as exc:
        return {"error": str(exc)}


def _smi_sample():
    """(mean shader clock over the XCDs in MHz, socket power in W) from amd-smi, or None."""
    try:
        _, out, _ = _run_child(["/opt/rocm/bin/amd-smi", "metric", "-p", "-c", "--json"], 20)
        j = json.loads(out)
        g = j[0] if isinstance(j, list) else j["gpu_data"][0]
        clk = [v["clk"]["value"] for k, v in g["clock"].items() if k.startswith("gfx_")]
        return float(np.mean(clk)), float(g["power"]["socket_power"]["value"])
    except (OSError, ValueError, KeyError, IndexError, TypeError):
        return None


def _sustained(lane, fn, seconds):
    """Launch `fn` back to back on a second thread for 1 s + `seconds` and sample clock and
    power over the last `seconds`: ms per launch, mean clock, mean power."""
    import threading
    stop, count = [False], [0]

    def loop():
        while not stop[0]:
            for _ in range(20):
                fn()
            lane.synchronize()
            count[0] += 20
    th = threading.Thread(target=loop)
    th.start()
    time.sleep(1.0)                                           # clocks settle
    n0, t0, seen = count[0], time.perf_counter(), []
    while time.perf_counter() - t0 < seconds:
        got = _smi_sample()
        if got:
            seen.append(got)
        else:
            time.sleep(0.1)
    n1, t1 = count[0], time.perf_counter()
    stop[0] = True
    th.join()
    if not seen:
        return {"error": "amd-smi gave no reading"}
    return {"ms": (t1 - t0) / max(n1 - n0, 1) * 1e3, "gfx_clock_mhz": float(np.mean([c for c, _ in seen])),
            "socket_power_w": float(np.mean([w for _, w in seen])), "samples": len(seen)}


def clock_and_power_trace(lane, seconds=4.0):
    """Shader clock (mean over the XCDs) and socket power, sampled with amd-smi while
    each kernel runs back to back on a second thread, on random and on constant
    operands.  Shows which figures are set by the board's power limit rather than by
    the kernel's schedule: the MFMA peak is quoted at 2400 MHz, and a launch that runs
    at 1700 MHz cannot pass 71 % of it whatever its instruction stream."""
    import ctypes

    def measure(fn):
        return _sustained(lane, fn, seconds)

    lib = lane.load()
    rng = np.random.default_rng(1)

    def operand(shape, constant):
        if constant:
            return lane.DeviceBuffer.from_host(np.full(shape, 0x3C3C, np.uint16))
        return lane.DeviceBuffer.from_host(_bf16(rng.standard_normal(shape, dtype=np.float32)))

    out = {"idle": dict(zip(("gfx_clock_mhz", "socket_power_w"), _smi_sample() or (None, None)))}
    M = N = K = 8192
    B, Hq, Hkv, S, D = 4, 32, 8, 4096, 128
    scale = ctypes.c_float(1.0 / np.sqrt(D))
    for constant in (False, True):
        tag = "constant" if constant else "random"
        a, b, c = operand((M, K), constant), operand((K, N), constant), lane.DeviceBuffer(M * N * 2)
        r = measure(lambda: lib.tessera_gfx950_gemm_bf16_bf16_dev(a.ptr, b.ptr, c.ptr, M, N, K, None))
        r["tflops"] = 2.0 * M * N * K / r["ms"] / 1e9 if "ms" in r else None
        out[f"gemm_bf16_8192_{tag}"] = r
        del a, b, c
        q, do = operand((B, Hq, S, D), constant), operand((B, Hq, S, D), constant)
        k, v = operand((B, Hkv, S, D), constant), operand((B, Hkv, S, D), constant)
        o32, lse = lane.DeviceBuffer(B * Hq * S * D * 4), lane.DeviceBuffer(B * Hq * S * 4)
        r = measure(lambda: lib.tessera_gfx950_flash_attn_gqa_bf16_dev(q.ptr, k.ptr, v.ptr, o32.ptr, lse.ptr, B, Hq,
                                                                      Hkv, S, S, D, scale, 1, 0, None))
        fwd_flop = 4.0 * B * Hq * (S * (S + 1) / 2) * D
        r["tflops"] = fwd_flop / r["ms"] / 1e9 if "ms" in r else None
        out[f"flash_attn_fwd_{tag}"] = r
        gq, gk, gv = (lane.DeviceBuffer(n * 4) for n in (B * Hq * S * D, B * Hkv * S * D, B * Hkv * S * D))
        r = measure(lambda: lib.tessera_gfx950_flash_attn_bwd_bf16_dev(do.ptr, q.ptr, k.ptr, v.ptr, o32.ptr, lse.ptr,
                                                                      gq.ptr, gk.ptr, gv.ptr, B, Hq, Hkv, S, S, D,
                                                                      scale, 1, None))
        r["tflops"] = 2.5 * fwd_flop / r["ms"] / 1e9 if "ms" in r else None
        out[f"flash_attn_bwd_{tag}"] = r
        del q, do, k, v, o32, lse, gq, gk, gv
    return out


def operand_residency_trace(lane, seconds=2.0):
    """What the operand traffic of the headline GEMM costs at the board's power limit.

    The same 256 x 256 tile kernel runs the same number of MFMAs (2 * 8192^3 FLOP per
    launch) on problems whose operands do or do not have to come through the fabric:
    one 8192^3 product; 64 products of 2048^3 on 64 distinct operand pairs; the same 64
    products all reading ONE operand pair (stride 0: 16 MB, resident in the memory-side
    cache and largely in the L2s); and likewise 512 products of 1024^3 (4 MB shared).
    Shared against distinct operands at equal K-loop length is the cost of the traffic:
    TFLOP/s, and the clock and power the board settles at."""
    lib = lane.load()
    rng = np.random.default_rng(0)
    fn = lib.tessera_gfx950_batched_gemm_strided_bf16_dev
    rows = []
    for tag, batch, n, shared in (("1 x 8192^3", 1, 8192, False), ("64 x 2048^3, distinct operands", 64, 2048, False),
                                  ("64 x 2048^3, one shared operand pair (16 MB)", 64, 2048, True),
                                  ("512 x 1024^3, distinct operands", 512, 1024, False),
                                  ("512 x 1024^3, one shared operand pair (4 MB)", 512, 1024, True)):
        cnt = 1 if shared else batch
        a = _bf16(rng.standard_normal((cnt, n, n), dtype=np.float32) / np.sqrt(n))
        b = _bf16(rng.standard_normal((cnt, n, n), dtype=np.float32) / np.sqrt(n))
        da, db, dd = lane.DeviceBuffer.from_host(a), lane.DeviceBuffer.from_host(b), lane.DeviceBuffer(batch * n * n * 2)
        st = 0 if shared else n * n
        launch = lambda: lane.check(fn(da.ptr, db.ptr, dd.ptr, batch, n, n, n, st, st, n * n, 1, None), "strided gemm")
        _, ev = _timed(lane, launch, 20, 5)
        held = _sustained(lane, launch, seconds)
        flop = 2.0 * batch * n ** 3
        rows.append({"case": tag, "ms": ev, "tflops": flop / ev / 1e9,
                     "tflops_sustained": flop / held["ms"] / 1e9 if "ms" in held else None,
                     "gfx_clock_mhz": held.get("gfx_clock_mhz"), "socket_power_w": held.get("socket_power_w")})
        for buf in (da, db, dd):
            buf.close()
    return rows


def gemm_f32_accumulators(lane, a_bits, b_bits, M, N, K):
    """A . B through the f32-output entry point (the accumulators before any storage rounding)."""
    lib = lane.load()
    da, db, dd = lane.DeviceBuffer.from_host(a_bits), lane.DeviceBuffer.from_host(b_bits), lane.DeviceBuffer(M * N * 4)
    lane.check(lib.tessera_gfx950_gemm_bf16_dev(da.ptr, db.ptr, dd.ptr, M, N, K, None), "gemm f32")
    lane.synchronize()
    acc = dd.download((M, N), np.float32)
    for buf in (da, db, dd):
        buf.close()
    return acc


def cpu_baseline(A, B):
    """The reference's CPU path for this config is ``np.matmul`` on f32-promoted
    operands; the oracle restates it.  Timed once on the full workload."""
    orc = _oracle()
    threads = _blas_threads()
    orc.gemm_f32(A[:256], B[:, :256])                         # warm the BLAS pool
    t0 = time.perf_counter()
    ref = orc.gemm_f32(A, B)
    dt = time.perf_counter() - t0
    M, K = A.shape
    N = B.shape[1]
    return ref, {"value": 2.0 * M * N * K / dt / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
                 "sample": f"full {M}x{N}x{K} product once, numpy f32 matmul of the bf16-rounded operands, {dt:.2f} s"}


ALSO = ("flash_attn", "flash_attn_decode", "flash_attn_bwd", "quant", "gemm_constant", "batched", "decode", "moe",
        "mfma_ceiling", "vendor_gemm")


def run_also(lane, name, steps, warmup, check):
    """One of the `also` workloads -> dict of result entries."""
    if name == "flash_attn":
        return {"flash_attn": bench_attention(lane, steps, warmup, check)}
    if name == "flash_attn_decode":
        return {"flash_attn_decode": bench_attention_decode(lane, steps, warmup, check)}
    if name == "flash_attn_bwd":
        return {"flash_attn_bwd": bench_attention_bwd(lane, steps, warmup)}
    if name == "quant":
        return bench_quant(lane, steps, warmup, check)
    if name == "gemm_constant":
        return {"gemm_bf16_8192_constant_operands": bench_gemm_constant_operands(lane, steps)}
    if name == "batched":
        return {"batched_gemm_readme_step": bench_batched_small(lane, steps, warmup)}
    if name == "decode":
        return bench_decode(lane, steps, warmup)
    if name == "moe":
        return {"moe": bench_moe(lane, steps, warmup, check)}
    if name == "vendor_gemm":
        return {"vendor_gemm_same_box": vendor_gemm_same_box()}
    raise ValueError(name)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip every CPU baseline / parity leg")
    ap.add_argument("--only-headline", action="store_true", help="skip the `also` measurements")
    ap.add_argument("--only", choices=ALSO, help="run this one `also` workload alone and print its entry "
                                                 "(for a profiler run with one clean row per workload)")
    ap.add_argument("--profile", action="store_true",
                    help="ramp the clocks with a kernel no workload times (clean per-kernel rows under a profiler)")
    ap.add_argument("--ramp-seconds", type=float, default=RAMP_SECONDS,
                    help="length of the untimed clock ramp before every timed region (a counter pass of a profiler "
                         "records every launch: a shorter ramp keeps its output small)")
    ap.add_argument("--no-vendor", action="store_true", help="skip the vendor-library GEMM leg (a PyTorch child process)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch a 1 GiB copy kernel (counter calibration for profiled runs)")
    ap.add_argument("--no-clock", action="store_true",
                    help="skip the clock / power readings (headline kernel and MFMA ceiling probe)")
    ap.add_argument("--residency", action="store_true",
                    help="instead of the bench line: the headline kernel on streamed against cache-resident operands")
    ap.add_argument("--clocks", action="store_true",
                    help="instead of the bench line: shader clock and socket power under each kernel")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one MI355X; this build has no multi-GPU path (--gpus must be 1)", file=sys.stderr)
        return 2
    from tessera_amd import lane
    lane.load()
    if not lane.available():
        print("gfx950 lane unavailable: no MI355X or library not built", file=sys.stderr)
        return 3

    _RAMP["foreign"] = bool(args.profile)
    _RAMP["seconds"] = max(0.0, float(args.ramp_seconds))
    if args.no_clock or args.profile:
        _OPTS["ceiling_seconds"] = 0.0
    if args.clocks:
        print(json.dumps(clock_and_power_trace(lane), indent=1))
        return 0
    if args.residency:
        print(json.dumps(operand_residency_trace(lane), indent=1))
        return 0
    if args.only:
        if args.only == "mfma_ceiling":
            print(json.dumps({"mfma_ceiling": {k: mfma_ceiling(lane, 0.0 if args.no_clock else 2.0, k)
                                                for k in ("bf16", "bf16_32x32x16", "int8", "fp8")}}))
        else:
            print(json.dumps(run_also(lane, args.only, args.steps, args.warmup, not args.no_cpu)))
        return 0
    copy_cal = calibrate_copy(lane) if args.calibrate_copy else None
    M = N = K = 8192
    wall, ev, (A, B, a, b, out) = bench_gemm(lane, M, N, K, args.steps, args.warmup)
    flop = 2.0 * M * N * K
    result = {
        "metric": "TFLOP/s and % MFMA peak: bf16 GEMM 8192^3 + causal flash-attn fwd, 1 MI355X",
        "value": flop / wall / 1e9, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic (seeded N(0,1)/sqrt(K) operands, resident in HBM)",
        "config": {"workload": "gemm_bf16_8192x8192x8192_f32acc_bf16out", "M": M, "N": N, "K": K,
                   "device": lane.device_name()},
        "roofline": {"bound": "mfma", "achieved": flop / ev / 1e9, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": flop / ev / 1e9 / PEAK_BF16_TFLOPS, "traffic": TRAFFIC_BYTES_GEMM_BF16_8192,
                     "traffic_source": "profiles/bench_all_kernels_hbm_bytes.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of an "
                                       "earlier run, scaled by the copy kernel's readings; not measured by this run)",
                     "kernel": "gemm16_kernel<BF16,256,256,2,2,STORE16,mfma 16x16x32>", "avg_launch_ms": ev},
    }
    if copy_cal:
        result["copy_calibration"] = copy_cal
    if not args.no_clock:
        # what the matrix pipes deliver on this board with no memory access at all, on operands
        # like the workload's and on constant ones, clock and power sampled under each
        ceil = mfma_ceiling(lane)
        result["mfma_ceiling"] = ceil
        result["roofline"].update(_ceiling_fields(ceil, flop / ev / 1e9))
        # the same launches kept up for 2 s: what clock the board grants this kernel on this
        # data (the peak is quoted at PEAK_CLOCK_MHZ), and the busy fraction at that clock
        lib = lane.load()
        da, db, dd = lane.DeviceBuffer.from_host(a), lane.DeviceBuffer.from_host(b), lane.DeviceBuffer(M * N * 2)
        held = _sustained(lane, lambda: lib.tessera_gfx950_gemm_bf16_bf16_dev(da.ptr, db.ptr, dd.ptr, M, N, K, None),
                          2.0)
        for buf in (da, db, dd):
            buf.close()
        if "ms" in held:
            tf = flop / held["ms"] / 1e9
            held.update({"tflops_sustained": tf, "peak_clock_mhz": PEAK_CLOCK_MHZ,
                         "frac_of_peak_at_measured_clock":
                             tf / (PEAK_BF16_TFLOPS * held["gfx_clock_mhz"] / PEAK_CLOCK_MHZ)})
        result["clock_under_load"] = held
    if not args.no_cpu:
        ref, result["cpu_baseline"] = cpu_baseline(A, B)
        got = (out.astype(np.uint32) << 16).view(np.float32)
        err = float(np.max(np.abs(got - ref)) / np.max(np.abs(ref)))
        result["parity_max_rel_vs_cpu"] = err                 # includes the bf16 store (<= 2^-8)
        # The same product with the f32 epilogue: the kernel's own error, without the store's
        # rounding, and whether the stored output is exactly the RNE of those accumulators.
        acc = gemm_f32_accumulators(lane, a, b, M, N, K)
        result["parity_f32_accumulators_max_rel_vs_cpu"] = float(np.max(np.abs(acc - ref)) / np.max(np.abs(ref)))
        result["stored_output_is_rne_of_accumulators"] = bool(np.array_equal(_bf16(acc), out))
        result["parity_bounds"] = {"f32_accumulators": 2e-3, "bf16_stored": 2e-3 + 2.0 ** -8}
        if result["parity_f32_accumulators_max_rel_vs_cpu"] > 2e-3 or err > 2e-3 + 2.0 ** -8:
            print("bench: parity bound exceeded", file=sys.stderr)
            print(json.dumps(result))
            return 4
        del acc
    del A, B, a, b, out
    if not args.only_headline:
        also = {}
        s_, w_ = max(3, args.steps // 2), max(2, args.warmup // 2)
        for name in ALSO:
            if name == "mfma_ceiling" or (name == "vendor_gemm" and args.no_vendor):
                continue
            also.update(run_also(lane, name, s_, w_, not args.no_cpu))
        result["also"] = also
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
