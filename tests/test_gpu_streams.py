"""The `_dev` entry points on caller-owned HIP streams, from several host threads.

Every `_dev` entry point takes a `hipStream_t`, enqueues and returns; the kernels that need
scratch memory take it from a workspace the library keeps per (device, stream).  The other GPU
tests pass the null stream.  Here the streams are the caller's (created through the HIP
runtime, default priority), two host threads drive one stream each at the same time (ctypes
drops the GIL during a call), and every result must equal, bit for bit, what the same call
gives on the null stream: a workspace shared between streams, or a launch that ignored its
stream argument, shows up as a mismatch.
"""
import ctypes
import threading

import numpy as np
import pytest

from tessera_amd import bf16 as b16

pytestmark = pytest.mark.gpu


class _Hip:
    """The three runtime calls a caller needs to own a stream."""

    def __init__(self):
        self.lib = ctypes.CDLL("libamdhip64.so", mode=ctypes.RTLD_LOCAL)
        self.lib.hipStreamCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.lib.hipStreamSynchronize.argtypes = [ctypes.c_void_p]
        self.lib.hipStreamDestroy.argtypes = [ctypes.c_void_p]

    def stream(self):
        s = ctypes.c_void_p()
        assert self.lib.hipStreamCreate(ctypes.byref(s)) == 0
        return s

    def sync(self, s):
        assert self.lib.hipStreamSynchronize(s) == 0

    def destroy(self, s):
        assert self.lib.hipStreamDestroy(s) == 0


@pytest.fixture(scope="module")
def hip():
    return _Hip()


def _splitk_case(lane, seed, M=16, N=1024, K=4096):
    """A decode-shaped product: the K-split form, whose partials live in the stream's workspace."""
    rng = np.random.default_rng(seed)
    a = b16.from_float32(rng.standard_normal((M, K)).astype(np.float32) * 0.5)
    b = b16.from_float32(rng.standard_normal((K, N)).astype(np.float32) * 0.5)
    da = lane.DeviceBuffer.from_host(np.asarray(a, np.uint16))
    db = lane.DeviceBuffer.from_host(np.asarray(b, np.uint16))
    dd = lane.DeviceBuffer(M * N * 4)
    return da, db, dd, (M, N, K)


def _route_case(lane, seed, T=700, E=64, k=8):
    rng = np.random.default_rng(seed)
    lg = rng.standard_normal((T, E)).astype(np.float32)
    S = T * k
    bufs = dict(lg=lane.DeviceBuffer.from_host(lg), tos=lane.DeviceBuffer(S * 4), eos=lane.DeviceBuffer(S * 4),
                cw=lane.DeviceBuffer(S * 4), gs=lane.DeviceBuffer(E * 4), go=lane.DeviceBuffer((E + 1) * 4),
                n=lane.DeviceBuffer(4))
    return bufs, (T, E, k)


def _gemm(lane, case, stream):
    da, db, dd, (M, N, K) = case
    dd.zero()
    lane.check(lane.load().tessera_gfx950_gemm_bf16_dev(da.ptr, db.ptr, dd.ptr, M, N, K, stream), "gemm")


def _route(lane, case, stream):
    b, (T, E, k) = case
    for name in ("tos", "eos", "cw", "gs", "go", "n"):
        b[name].zero()
    lane.check(lane.load().tessera_gfx950_moe_route_f32_dev(b["lg"].ptr, T, E, k, 1, 0, b["tos"].ptr, b["eos"].ptr,
                                                            b["cw"].ptr, b["gs"].ptr, b["go"].ptr, b["n"].ptr, stream),
               "route")


def _read_gemm(case):
    _, _, dd, (M, N, _) = case
    return dd.download((M, N), np.float32)


def _read_route(case):
    b, (T, E, k) = case
    S = T * k
    return [b["tos"].download((S,), np.int32), b["eos"].download((S,), np.int32), b["cw"].download((S,), np.float32),
            b["gs"].download((E,), np.int32), b["go"].download((E + 1,), np.int32)]


def test_caller_streams_give_the_null_stream_results(lane, hip):
    assert lane.load().tessera_gfx950_probe() == 0
    g, r = _splitk_case(lane, 1), _route_case(lane, 2)
    _gemm(lane, g, None)
    _route(lane, r, None)
    lane.synchronize()
    want_g, want_r = _read_gemm(g), _read_route(r)
    s = hip.stream()
    try:
        for _ in range(3):
            _gemm(lane, g, s)
            _route(lane, r, s)
            hip.sync(s)
            assert np.array_equal(_read_gemm(g), want_g)
            for got, want in zip(_read_route(r), want_r):
                assert np.array_equal(got, want)
    finally:
        hip.destroy(s)


def test_two_threads_two_streams_at_once(lane, hip):
    """Each thread owns a stream, its own operands and outputs, and alternates the K-split
    product and the routing 40 times; the other thread does the same with different data at the
    same time.  Every round must reproduce the thread's null-stream reference."""
    cases = []
    for t in range(2):
        g, r = _splitk_case(lane, 10 + t, M=16 + 16 * t), _route_case(lane, 20 + t, T=500 + 300 * t)
        _gemm(lane, g, None)
        _route(lane, r, None)
        lane.synchronize()
        cases.append((g, r, _read_gemm(g), _read_route(r)))
    streams = [hip.stream(), hip.stream()]
    errors = []

    def work(i):
        g, r, want_g, want_r = cases[i]
        try:
            for round_ in range(40):
                _gemm(lane, g, streams[i])
                _route(lane, r, streams[i])
                hip.sync(streams[i])
                if not np.array_equal(_read_gemm(g), want_g):
                    errors.append((i, round_, "gemm"))
                for got, want in zip(_read_route(r), want_r):
                    if not np.array_equal(got, want):
                        errors.append((i, round_, "route"))
        except Exception as exc:                          # noqa: BLE001 - reported by the main thread
            errors.append((i, "raised", repr(exc)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    try:
        for th in threads:
            th.start()
        for th in threads:
            th.join(timeout=100)
        assert not any(th.is_alive() for th in threads), "a stream thread did not finish"
        assert not errors, errors[:5]
    finally:
        for s in streams:
            hip.sync(s)
            hip.destroy(s)


def test_stream_release_frees_and_a_later_call_reallocates(lane, hip):
    """`tessera_gfx950_stream_release` waits for the stream and frees its workspace; the next
    call on the stream sizes a new one and gives the same result.  Releasing a stream that has
    no workspace is not an error."""
    lib = lane.load()
    g = _splitk_case(lane, 61)
    _gemm(lane, g, None)
    lane.synchronize()
    want = _read_gemm(g)
    s = hip.stream()
    try:
        assert lib.tessera_gfx950_stream_release(s) == 0           # nothing kept yet
        for _ in range(2):
            _gemm(lane, g, s)
            assert lib.tessera_gfx950_stream_release(s) == 0       # synchronises, then frees
            assert np.array_equal(_read_gemm(g), want)
    finally:
        hip.destroy(s)


def test_host_pointer_entry_points_from_two_threads(lane):
    """The host-pointer ABI is re-entrant like the reference's (which allocates per call): two
    host threads inside `tessera_gfx950_gemm_bf16` (a K-split shape, partials in scratch memory)
    and `tessera_gfx950_moe_route_f32` (routing lists in scratch memory) at the same time must
    each get what the call gives when it runs alone."""
    lib = lane.load()

    def make(seed, M, T):
        rng = np.random.default_rng(seed)
        N, K, E, k = 1024, 4096, 64, 8
        a = np.ascontiguousarray(np.asarray(b16.from_float32(rng.standard_normal((M, K)).astype(np.float32) * 0.5),
                                            np.uint16))
        b = np.ascontiguousarray(np.asarray(b16.from_float32(rng.standard_normal((K, N)).astype(np.float32) * 0.5),
                                            np.uint16))
        lg = rng.standard_normal((T, E)).astype(np.float32)
        return dict(a=a, b=b, lg=lg, M=M, N=N, K=K, T=T, E=E, k=k)

    def run(c):
        d = np.zeros((c["M"], c["N"]), np.float32)
        assert lib.tessera_gfx950_gemm_bf16(c["a"].ctypes.data, c["b"].ctypes.data, d.ctypes.data, c["M"], c["N"],
                                            c["K"]) == 0
        S = c["T"] * c["k"]
        tos, eos = np.zeros(S, np.int32), np.zeros(S, np.int32)
        cw = np.zeros(S, np.float32)
        gs, go, n = np.zeros(c["E"], np.int32), np.zeros(c["E"] + 1, np.int32), np.zeros(1, np.int32)
        assert lib.tessera_gfx950_moe_route_f32(c["lg"].ctypes.data, c["T"], c["E"], c["k"], 1, 0, tos.ctypes.data,
                                                eos.ctypes.data, cw.ctypes.data, gs.ctypes.data, go.ctypes.data,
                                                n.ctypes.data) == 0
        return [d, tos, eos, cw, gs, go, n]

    cases = [make(51, 16, 500), make(52, 32, 800)]
    want = [run(c) for c in cases]
    errors = []

    def work(i):
        try:
            for round_ in range(25):
                for idx, (got, ref) in enumerate(zip(run(cases[i]), want[i])):
                    if not np.array_equal(got, ref):
                        errors.append((i, round_, idx))
        except Exception as exc:                          # noqa: BLE001 - reported by the main thread
            errors.append((i, "raised", repr(exc)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
    assert not any(th.is_alive() for th in threads), "a host-pointer thread did not finish"
    assert not errors, errors[:5]


def test_dev_entry_points_under_stream_capture(lane, hip):
    """The `_dev` calls record into a HIP graph (they clear their counters with a fill kernel,
    not a memset node, and take scratch from a workspace that already has its size after one
    eager call).  The graph is replayed several times with eager work and synchronisations in
    between; every replay must reproduce the eager results bit for bit."""
    L = hip.lib
    L.hipStreamBeginCapture.argtypes = [ctypes.c_void_p, ctypes.c_int]
    L.hipStreamEndCapture.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p)]
    L.hipGraphInstantiate.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p, ctypes.c_void_p,
                                      ctypes.c_void_p, ctypes.c_size_t]
    L.hipGraphLaunch.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
    L.hipGraphExecDestroy.argtypes = [ctypes.c_void_p]
    L.hipGraphDestroy.argtypes = [ctypes.c_void_p]
    lib = lane.load()
    g, r = _splitk_case(lane, 31), _route_case(lane, 32)
    da, db, dd, (M, N, K) = g
    rb, (T, E, k) = r
    # attention operands
    rng = np.random.default_rng(33)
    B, Hq, Hkv, Sq, Sk, D = 1, 4, 2, 200, 264, 128
    q, kk, v = (lane.DeviceBuffer.from_host(np.asarray(b16.from_float32(
        rng.standard_normal(shape).astype(np.float32)), np.uint16)) for shape in
        ((B, Hq, Sq, D), (B, Hkv, Sk, D), (B, Hkv, Sk, D)))
    o, lse = lane.DeviceBuffer(B * Hq * Sq * D * 4), lane.DeviceBuffer(B * Hq * Sq * 4)
    # a whole MoE layer with its router product (caller-provided workspace)
    mT, mH, mF, mE, mk = 300, 256, 384, 8, 2
    bits = lambda a: np.asarray(b16.from_float32(a.astype(np.float32)), np.uint16)
    mx = lane.DeviceBuffer.from_host(bits(rng.standard_normal((mT, mH))))
    mwr = lane.DeviceBuffer.from_host(bits(rng.standard_normal((mH, mE)) / 16))
    mwg, mwu = (lane.DeviceBuffer.from_host(bits(rng.standard_normal((mE, mH, mF)) / 16)) for _ in range(2))
    mwd = lane.DeviceBuffer.from_host(bits(rng.standard_normal((mE, mF, mH)) / 20))
    need = ctypes.c_size_t(0)
    lane.check(lib.tessera_gfx950_moe_layer_workspace_bytes(mT, mH, mF, mH, mE, mk, ctypes.byref(need)), "workspace")
    mws, mout = lane.DeviceBuffer(need.value), lane.DeviceBuffer(mT * mH * 4)
    mS = mT * mk
    mplan = [lane.DeviceBuffer(mS * 4), lane.DeviceBuffer(mS * 4), lane.DeviceBuffer(mS * 4), lane.DeviceBuffer(mE * 4),
             lane.DeviceBuffer((mE + 1) * 4), lane.DeviceBuffer(4)]

    def enqueue(s):
        lane.check(lib.tessera_gfx950_moe_layer_bf16_dev(
            mx.ptr, mwr.ptr, None, mwg.ptr, mwu.ptr, mwd.ptr, mout.ptr, mws.ptr, need.value, mT, mH, mF, mH, mE, mk, 1, 0,
            *(b.ptr for b in mplan), s), "moe_layer")
        lane.check(lib.tessera_gfx950_gemm_bf16_dev(da.ptr, db.ptr, dd.ptr, M, N, K, s), "gemm")
        lane.check(lib.tessera_gfx950_moe_route_f32_dev(rb["lg"].ptr, T, E, k, 1, 0, rb["tos"].ptr, rb["eos"].ptr,
                                                        rb["cw"].ptr, rb["gs"].ptr, rb["go"].ptr, rb["n"].ptr, s), "route")
        lane.check(lib.tessera_gfx950_flash_attn_gqa_bf16_dev(q.ptr, kk.ptr, v.ptr, o.ptr, lse.ptr, B, Hq, Hkv, Sq, Sk, D,
                                                              ctypes.c_float(D ** -0.5), 1, 0, s), "flash_attn")

    def read():
        return [_read_gemm(g)] + _read_route(r) + [o.download((B, Hq, Sq, D), np.float32),
                                                  lse.download((B, Hq, Sq), np.float32),
                                                  mout.download((mT, mH), np.float32),
                                                  mplan[0].download((mS,), np.int32)]

    def clear():
        for buf in (dd, o, lse, rb["tos"], rb["eos"], rb["cw"], rb["gs"], rb["go"], rb["n"], mout, mws, *mplan):
            buf.zero()

    s = hip.stream()
    graph, exe = ctypes.c_void_p(), ctypes.c_void_p()
    try:
        enqueue(s)                                   # eager: sizes the stream's workspace, gives the reference
        hip.sync(s)
        want = read()
        assert L.hipStreamBeginCapture(s, 0) == 0
        enqueue(s)
        assert L.hipStreamEndCapture(s, ctypes.byref(graph)) == 0 and graph.value
        assert L.hipGraphInstantiate(ctypes.byref(exe), graph, None, None, 0) == 0
        for replay in range(4):
            clear()
            # the program's own eager work between replays, on the same and on the null stream
            _gemm(lane, _splitk_case(lane, 40 + replay, M=8), s)
            hip.sync(s)
            lane.synchronize()
            clear()
            assert L.hipGraphLaunch(exe, s) == 0
            hip.sync(s)
            for idx, (got, ref) in enumerate(zip(read(), want)):
                assert np.array_equal(got, ref, equal_nan=True), (replay, idx)
    finally:
        if exe.value:
            L.hipGraphExecDestroy(exe)
        if graph.value:
            L.hipGraphDestroy(graph)
        hip.sync(s)
        hip.destroy(s)


def test_layer_with_logits_given_captures_on_a_fresh_stream(lane, hip):
    """The whole-layer entry with the router logits given takes every temporary from the caller's
    workspace: it records into a capture on a stream that has run nothing eagerly (no workspace of the
    library's to size), and the replays equal the eager result of another stream bit for bit."""
    L = hip.lib
    L.hipStreamBeginCapture.argtypes = [ctypes.c_void_p, ctypes.c_int]
    L.hipStreamEndCapture.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p)]
    L.hipGraphInstantiate.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p, ctypes.c_void_p,
                                      ctypes.c_void_p, ctypes.c_size_t]
    L.hipGraphLaunch.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
    L.hipGraphExecDestroy.argtypes = [ctypes.c_void_p]
    L.hipGraphDestroy.argtypes = [ctypes.c_void_p]
    lib = lane.load()
    assert lib.tessera_gfx950_probe() == 0                     # the device is initialised before any capture
    rng = np.random.default_rng(71)
    T, H, F, E, k = 260, 128, 192, 8, 2
    bits = lambda a: np.asarray(b16.from_float32(a.astype(np.float32)), np.uint16)
    x = lane.DeviceBuffer.from_host(bits(rng.standard_normal((T, H))))
    lg = lane.DeviceBuffer.from_host(rng.standard_normal((T, E)).astype(np.float32))
    wg, wu = (lane.DeviceBuffer.from_host(bits(rng.standard_normal((E, H, F)) / 12)) for _ in range(2))
    wd = lane.DeviceBuffer.from_host(bits(rng.standard_normal((E, F, H)) / 14))
    need = ctypes.c_size_t(0)
    lane.check(lib.tessera_gfx950_moe_layer_workspace_bytes(T, H, F, H, E, k, ctypes.byref(need)), "workspace")
    ws, out = lane.DeviceBuffer(need.value), lane.DeviceBuffer(T * H * 4)
    S = T * k
    plan = [lane.DeviceBuffer(S * 4), lane.DeviceBuffer(S * 4), lane.DeviceBuffer(S * 4), lane.DeviceBuffer(E * 4),
            lane.DeviceBuffer((E + 1) * 4), lane.DeviceBuffer(4)]

    def enqueue(s):
        lane.check(lib.tessera_gfx950_moe_layer_bf16_dev(
            x.ptr, None, lg.ptr, wg.ptr, wu.ptr, wd.ptr, out.ptr, ws.ptr, need.value, T, H, F, H, E, k, 1, 0,
            *(b.ptr for b in plan), s), "moe_layer")

    eager, fresh = hip.stream(), hip.stream()
    graph, exe = ctypes.c_void_p(), ctypes.c_void_p()
    try:
        enqueue(eager)
        hip.sync(eager)
        want = out.download((T, H), np.float32)
        assert np.isfinite(want).all() and np.abs(want).max() > 0
        assert L.hipStreamBeginCapture(fresh, 0) == 0
        enqueue(fresh)
        assert L.hipStreamEndCapture(fresh, ctypes.byref(graph)) == 0 and graph.value
        assert L.hipGraphInstantiate(ctypes.byref(exe), graph, None, None, 0) == 0
        for replay in range(3):
            for buf in (out, ws, *plan):
                buf.zero()
            assert L.hipGraphLaunch(exe, fresh) == 0
            hip.sync(fresh)
            assert np.array_equal(out.download((T, H), np.float32), want), replay
    finally:
        if exe.value:
            L.hipGraphExecDestroy(exe)
        if graph.value:
            L.hipGraphDestroy(graph)
        for s in (eager, fresh):
            hip.sync(s)
            hip.destroy(s)
        for b in (x, lg, wg, wu, wd, ws, out, *plan):
            b.close()
