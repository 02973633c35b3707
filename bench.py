#!/usr/bin/env python3
"""Headline benchmark of the gfx950 dense-op lane on one MI355X.

A "step" is one pass of the hot path over one batch of synthetic input: one
``D = A . B`` with A, B bf16 8192 x 8192 (entries N(0,1)/sqrt(K), seeded), f32
accumulate, bf16 output — BASELINE.json's configs[1].  Inputs are resident in
HBM before the timed region; the timed region is K launches through the C ABI's
device-pointer entry point, bracketed by a device synchronise on both sides.

One JSON line is printed.  ``roofline`` prices the GEMM kernel against the
MI355X dense bf16 MFMA peak from its average launch duration, measured with HIP
events on the launch stream over the same timed region.  ``cpu_baseline`` times
the oracle's numpy restatement of the reference's CPU path on this host's cores.
``also`` carries the same measurement for the other kernels of the path
(flash-attention forward, fp8 / int8 GEMM, decode-shaped GEMM, the MoE expert
block); they are reported, not part of ``value``.
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
# reading for the 1 GiB copy kernel (profiles/bench_all_kernels_hbm_bytes.txt).
TRAFFIC_BYTES_GEMM_BF16_8192 = 1.7497e9


RAMP_SECONDS = 0.1


def _timed(lane, launch, steps, warmup):
    """(wall ms/step, event ms/step) for `steps` launches after `warmup`.

    After the host-side data preparation the GPU has idled and its clocks ramp back
    up over the first tens of milliseconds of load (measured: the first 25 launches
    of the headline GEMM run 3-70 % slower than the steady state).  The untimed
    warm-up therefore first keeps the kernel running for RAMP_SECONDS, then does the
    `warmup` steps; the timed region is exactly `steps` launches."""
    t_ramp = time.perf_counter()
    while time.perf_counter() - t_ramp < RAMP_SECONDS:
        for _ in range(4):
            launch()
        lane.synchronize()
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


def bench_attention(lane, steps, warmup):
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
    for buf in (dq, dk, dv, do, dl):
        buf.close()
    flop = 4.0 * B * Hq * (S * (S + 1) / 2) * D          # the reference's causal FLOP model
    return {"workload": "flash_attn_fwd_bf16_causal_B4_Hq32_Hkv8_S4096_D128", "ms": ev,
            "tflops": flop / ev / 1e9, "frac_mfma_peak": flop / ev / 1e9 / PEAK_BF16_TFLOPS}


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


def bench_quant(lane, steps, warmup):
    M, N, K = 4096, 8192, 8192
    rng = np.random.default_rng(2)
    out = {}
    a8 = rng.integers(-127, 128, (M, K)).astype(np.int8)
    b8 = rng.integers(-127, 128, (K, N)).astype(np.int8)
    da, db = lane.DeviceBuffer.from_host(a8), lane.DeviceBuffer.from_host(b8)
    dd = lane.DeviceBuffer(M * N * 4)
    lib = lane.load()
    _, ev = _timed(lane, lambda: lane.check(lib.tessera_gfx950_gemm_i8_i32_dev(da.ptr, db.ptr, dd.ptr, M, N, K, None),
                                            "gemm_i8"), steps, warmup)
    ops = 2.0 * M * N * K
    out["gemm_int8_4096x8192x8192"] = {"ms": ev, "tops": ops / ev / 1e9, "frac_mfma_peak": ops / ev / 1e9 / PEAK_INT8_TOPS}
    # W8A8 with scales: f32(acc) * row_scale[m] * col_scale[n], f32 out, no accumulator copy
    rs = lane.DeviceBuffer.from_host(rng.uniform(0.5, 1.5, M).astype(np.float32) / 127.0)
    cs = lane.DeviceBuffer.from_host(rng.uniform(0.5, 1.5, N).astype(np.float32) / 127.0)
    _, ev = _timed(lane, lambda: lane.check(lib.tessera_gfx950_gemm_w8a8_f32_dev(da.ptr, db.ptr, rs.ptr, cs.ptr, dd.ptr,
                                                                                 None, M, N, K, None), "gemm_w8a8"),
                   steps, warmup)
    out["gemm_w8a8_scaled_4096x8192x8192"] = {"ms": ev, "tops": ops / ev / 1e9,
                                              "frac_mfma_peak": ops / ev / 1e9 / PEAK_INT8_TOPS}
    # per-row int8 quantiser of the f32 activation (reads 4 M K bytes, writes M K + 4 M)
    xf = lane.DeviceBuffer.from_host(rng.standard_normal((M, K), dtype=np.float32))
    xq, xs = lane.DeviceBuffer(M * K), lane.DeviceBuffer(M * 4)
    _, ev = _timed(lane, lambda: lane.check(lib.tessera_gfx950_quantize_i8_f32_dev(xf.ptr, M, K, 1, xq.ptr, xs.ptr, None),
                                            "quantize_i8"), steps, warmup)
    qbytes = 5.0 * M * K + 4.0 * M
    out["quantize_int8_rows_4096x8192"] = {"ms": ev, "gbs": qbytes / ev / 1e6, "frac_hbm_peak": qbytes / ev / 1e6 / PEAK_HBM_GBS}
    # per-tensor e4m3 quantiser with a dynamic scale: absmax pass + quantising pass
    # (reads 8 M K bytes, writes M K)
    _, ev = _timed(lane, lambda: lane.check(lib.tessera_gfx950_quantize_e4m3_f32_dev(xf.ptr, M * K, 0.0, xq.ptr, xs.ptr,
                                                                                     None), "quantize_e4m3"),
                   steps, warmup)
    ebytes = 9.0 * M * K
    out["quantize_e4m3_tensor_4096x8192"] = {"ms": ev, "gbs": ebytes / ev / 1e6, "frac_hbm_peak": ebytes / ev / 1e6 / PEAK_HBM_GBS}
    for buf in (rs, cs, xf, xq, xs):
        buf.close()
    # e4m3 codes with |value| <= 15 (no NaN codes)
    af = ((a8.view(np.uint8) & 0x80) | np.minimum(a8.view(np.uint8) & 0x7F, 0x47)).astype(np.uint8)
    bf = ((b8.view(np.uint8) & 0x80) | np.minimum(b8.view(np.uint8) & 0x7F, 0x47)).astype(np.uint8)
    da.upload(af)
    db.upload(bf)
    _, ev = _timed(lane, lambda: lane.check(
        lib.tessera_gfx950_gemm_e4m3_bf16_dev(da.ptr, db.ptr, 1.0, 1.0, dd.ptr, M, N, K, None), "gemm_e4m3"), steps, warmup)
    out["gemm_fp8_e4m3_4096x8192x8192"] = {"ms": ev, "tflops": ops / ev / 1e9,
                                           "frac_mfma_peak": ops / ev / 1e9 / PEAK_FP8_TFLOPS}
    for buf in (da, db, dd):
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


def bench_moe(lane, steps, warmup):
    T, H, F, E, k = 8192, 4096, 1408, 64, 8
    rng = np.random.default_rng(4)
    S = T * k
    logits = rng.standard_normal((T, E), dtype=np.float32)
    lib = lane.load()
    dlog = lane.DeviceBuffer.from_host(logits)
    dtos, deos, dcw = lane.DeviceBuffer(S * 4), lane.DeviceBuffer(S * 4), lane.DeviceBuffer(S * 4)
    dgs, dgo, dn = lane.DeviceBuffer(E * 4), lane.DeviceBuffer((E + 1) * 4), lane.DeviceBuffer(4)
    route = lambda: lane.check(lib.tessera_gfx950_moe_route_f32_dev(
        dlog.ptr, T, E, k, 1, 0, dtos.ptr, deos.ptr, dcw.ptr, dgs.ptr, dgo.ptr, dn.ptr, None), "route")
    _, ev_route = _timed(lane, route, steps, warmup)
    x = _bf16(rng.standard_normal((T, H), dtype=np.float32))
    dx = lane.DeviceBuffer.from_host(x)
    dxp = lane.DeviceBuffer(S * H * 2)
    disp = lambda: lane.check(lib.tessera_gfx950_moe_dispatch_dev(dx.ptr, dtos.ptr, dxp.ptr, T, S, H, 2, None), "dispatch")
    _, ev_disp = _timed(lane, disp, steps, warmup)
    w = lambda shape: _bf16(0.02 * rng.standard_normal(shape, dtype=np.float32))
    dwg, dwu = lane.DeviceBuffer.from_host(w((E, H, F))), lane.DeviceBuffer.from_host(w((E, H, F)))
    dwd = lane.DeviceBuffer.from_host(w((E, F, H)))
    dh, dy = lane.DeviceBuffer(S * F * 2), lane.DeviceBuffer(S * H * 2)
    ffn = lambda: lane.check(lib.tessera_gfx950_moe_swiglu_block_bf16_dev(
        dxp.ptr, dwg.ptr, dwu.ptr, dwd.ptr, dgo.ptr, dy.ptr, dh.ptr, S, H, F, H, E, None), "swiglu")
    _, ev_ffn = _timed(lane, ffn, steps, warmup)
    # the same block reading x through the dispatch map (no dispatch pass, no x_perm)
    ffn_g = lambda: lane.check(lib.tessera_gfx950_moe_swiglu_block_gather_bf16_dev(
        dx.ptr, dtos.ptr, dwg.ptr, dwu.ptr, dwd.ptr, dgo.ptr, dy.ptr, dh.ptr, T, S, H, F, H, E, None), "swiglu_gather")
    _, ev_ffn_g = _timed(lane, ffn_g, steps, warmup)
    dout = lane.DeviceBuffer(T * H * 4)
    comb = lambda: lane.check(lib.tessera_gfx950_moe_combine_bf16_dev(dy.ptr, dtos.ptr, dcw.ptr, dout.ptr, T, S, H, None),
                              "combine")
    _, ev_comb = _timed(lane, comb, steps, warmup)
    for buf in (dlog, dtos, deos, dcw, dgs, dgo, dn, dx, dxp, dwg, dwu, dwd, dh, dy, dout):
        buf.close()
    flop = 6.0 * S * H * F
    return {"workload": "moe_T8192_H4096_E64_top8_F1408_bf16", "route_ms": ev_route, "dispatch_ms": ev_disp,
            "expert_ffn_ms": ev_ffn, "dispatch_fused_expert_ffn_ms": ev_ffn_g, "combine_ms": ev_comb,
            "layer_ms": ev_route + ev_ffn_g + ev_comb, "expert_ffn_tflops": flop / ev_ffn / 1e9,
            "frac_mfma_peak": flop / ev_ffn / 1e9 / PEAK_BF16_TFLOPS,
            "dispatch_gbs": 2.0 * S * H * 2 / ev_disp / 1e6}


def _smi_sample():
    """(mean shader clock over the XCDs in MHz, socket power in W) from amd-smi, or None."""
    import subprocess
    try:
        r = subprocess.run(["/opt/rocm/bin/amd-smi", "metric", "-p", "-c", "--json"], capture_output=True, text=True,
                           timeout=20)
        j = json.loads(r.stdout)
        g = j[0] if isinstance(j, list) else j["gpu_data"][0]
        clk = [v["clk"]["value"] for k, v in g["clock"].items() if k.startswith("gfx_")]
        return float(np.mean(clk)), float(g["power"]["socket_power"]["value"])
    except (OSError, ValueError, KeyError, IndexError, TypeError, subprocess.SubprocessError):
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


def cpu_baseline(A, B):
    """The reference's CPU path for this config is ``np.matmul`` on f32-promoted
    operands; the oracle restates it.  Timed once on the full workload."""
    sys.path.insert(0, str(ROOT / "oracle"))
    import tessera_oracle as orc
    threads = os.cpu_count() or 1
    try:
        from threadpoolctl import threadpool_info
        blas = [p for p in threadpool_info() if p.get("user_api") == "blas"]
        if blas:
            threads = int(blas[0]["num_threads"])
    except Exception:
        pass
    orc.gemm_f32(A[:256], B[:, :256])                         # warm the BLAS pool
    t0 = time.perf_counter()
    ref = orc.gemm_f32(A, B)
    dt = time.perf_counter() - t0
    M, K = A.shape
    N = B.shape[1]
    return ref, {"value": 2.0 * M * N * K / dt / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
                 "sample": f"full {M}x{N}x{K} product once, numpy f32 matmul of the bf16-rounded operands, {dt:.2f} s"}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only-headline", action="store_true", help="skip the `also` measurements")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch a 1 GiB copy kernel (counter calibration for profiled runs)")
    ap.add_argument("--no-clock", action="store_true", help="skip the 3 s clock / power reading of the headline kernel")
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

    if args.clocks:
        print(json.dumps(clock_and_power_trace(lane), indent=1))
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
                     "kernel": "gemm16_kernel<BF16,256,256,2,2,STORE16>", "avg_launch_ms": ev},
    }
    if copy_cal:
        result["copy_calibration"] = copy_cal
    if not args.no_clock:
        # the same launches kept up for 3 s: what clock the board grants this kernel on this
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
    if not args.only_headline:
        also = {}
        s, w = max(3, args.steps // 2), max(2, args.warmup // 2)
        also["flash_attn"] = bench_attention(lane, s, w)
        also["flash_attn_bwd"] = bench_attention_bwd(lane, s, w)
        also.update(bench_quant(lane, s, w))
        also["gemm_bf16_8192_constant_operands"] = bench_gemm_constant_operands(lane, s)
        also["batched_gemm_readme_step"] = bench_batched_small(lane, s, w)
        also.update(bench_decode(lane, s, w))
        also["moe"] = bench_moe(lane, s, w)
        result["also"] = also
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
