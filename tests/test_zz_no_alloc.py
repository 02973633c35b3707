"""The routing entry point that allocates nothing
(``tessera_gfx950_moe_route_f32_noalloc_dev``) against the workspace-backed
``tessera_gfx950_moe_route_f32_dev``, through the C ABI: the five arrays of the
transport descriptor and the slot count, bit for bit, on two calls in a row, the
second on a smaller input (the fixed scratch keeps the first call's contents).
Collected last so that a failure here hides no other test."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _route(lane, entry, logits, k, normalize, capacity):
    """Run one routing entry point on device buffers and fetch every output."""
    lib = lane.load()
    T, E = logits.shape
    S = T * k
    d_scores = lane.DeviceBuffer.from_host(logits)
    bufs = {name: lane.DeviceBuffer(n * 4) for name, n in
            (("tos", S), ("eos", S), ("cw", S), ("gs", E), ("go", E + 1), ("n", 1))}
    for b in bufs.values():
        b.zero()
    rc = getattr(lib, entry)(d_scores.ptr, T, E, k, int(normalize), capacity, bufs["tos"].ptr, bufs["eos"].ptr,
                             bufs["cw"].ptr, bufs["gs"].ptr, bufs["go"].ptr, bufs["n"].ptr, None)
    lane.check(rc, entry)
    lane.synchronize()
    n = int(bufs["n"].download((1,), np.int32)[0])
    out = (n, bufs["tos"].download((S,), np.int32)[:n], bufs["eos"].download((S,), np.int32)[:n],
           bufs["cw"].download((S,), np.float32)[:n], bufs["gs"].download((E,), np.int32),
           bufs["go"].download((E + 1,), np.int32))
    for b in list(bufs.values()) + [d_scores]:
        b.close()
    return out


def _same(a, b):
    assert a[0] == b[0]
    for x, y in zip(a[1:], b[1:]):
        assert x.dtype == y.dtype and np.array_equal(x.view(np.uint32), y.view(np.uint32))


def test_noalloc_route_matches_workspace_route_on_two_calls_in_a_row(lane):
    rng = np.random.default_rng(2024)
    big = rng.standard_normal((8192, 64)).astype(np.float32)        # the headline MoE routing shape
    small = rng.standard_normal((777, 24)).astype(np.float32)       # ragged, fewer experts, capacity drops
    first = _route(lane, "tessera_gfx950_moe_route_f32_noalloc_dev", big, 8, True, 0)
    second = _route(lane, "tessera_gfx950_moe_route_f32_noalloc_dev", small, 3, False, 90)
    _same(first, _route(lane, "tessera_gfx950_moe_route_f32_dev", big, 8, True, 0))
    _same(second, _route(lane, "tessera_gfx950_moe_route_f32_dev", small, 3, False, 90))
    assert first[0] == 8192 * 8 and second[0] < 777 * 3            # the second call dropped slots
    # and once more in the other order, larger after smaller
    _same(_route(lane, "tessera_gfx950_moe_route_f32_noalloc_dev", big, 8, True, 0), first)


def test_noalloc_route_rejects_sizes_beyond_its_scratch(lane):
    lib = lane.load()
    fake = 0x1000                                                   # never dereferenced: rejected first
    T, E, k = 1 << 20, 64, 8                                        # 8 Mi slots: 64 MiB of ids and weights
    rc = lib.tessera_gfx950_moe_route_f32_noalloc_dev(fake, T, E, k, 1, 0, fake, fake, fake, fake, fake, None, None)
    assert rc == lane.BAD_SHAPE


def test_noalloc_route_on_a_caller_stream_and_under_graph_capture(lane):
    """The entry point on a caller-owned stream, then recorded into a HIP graph and replayed
    three times with eager work in between: every result equals the eager null-stream one bit
    for bit.  (The scratch array's address was looked up when the library first touched the
    device, so nothing inside the capture is more than kernel launches.)"""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so", mode=ctypes.RTLD_LOCAL)
    hip.hipStreamCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
    hip.hipStreamSynchronize.argtypes = [ctypes.c_void_p]
    hip.hipStreamDestroy.argtypes = [ctypes.c_void_p]
    hip.hipStreamBeginCapture.argtypes = [ctypes.c_void_p, ctypes.c_int]
    hip.hipStreamEndCapture.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p)]
    hip.hipGraphInstantiate.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p, ctypes.c_void_p,
                                        ctypes.c_void_p, ctypes.c_size_t]
    hip.hipGraphLaunch.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
    hip.hipGraphExecDestroy.argtypes = [ctypes.c_void_p]
    hip.hipGraphDestroy.argtypes = [ctypes.c_void_p]
    lib = lane.load()
    assert lib.tessera_gfx950_probe() == 0
    rng = np.random.default_rng(77)
    logits = rng.standard_normal((1500, 32)).astype(np.float32)
    T, E, k = 1500, 32, 4
    S = T * k
    want = _route(lane, "tessera_gfx950_moe_route_f32_dev", logits, k, True, 0)
    d_scores = lane.DeviceBuffer.from_host(logits)
    bufs = {name: lane.DeviceBuffer(n * 4) for name, n in
            (("tos", S), ("eos", S), ("cw", S), ("gs", E), ("go", E + 1), ("n", 1))}

    def enqueue(stream):
        lane.check(lib.tessera_gfx950_moe_route_f32_noalloc_dev(
            d_scores.ptr, T, E, k, 1, 0, bufs["tos"].ptr, bufs["eos"].ptr, bufs["cw"].ptr, bufs["gs"].ptr,
            bufs["go"].ptr, bufs["n"].ptr, stream), "noalloc route")

    def read():
        n = int(bufs["n"].download((1,), np.int32)[0])
        return (n, bufs["tos"].download((S,), np.int32)[:n], bufs["eos"].download((S,), np.int32)[:n],
                bufs["cw"].download((S,), np.float32)[:n], bufs["gs"].download((E,), np.int32),
                bufs["go"].download((E + 1,), np.int32))

    def clear():
        for b in bufs.values():
            b.zero()

    s = ctypes.c_void_p()
    assert hip.hipStreamCreate(ctypes.byref(s)) == 0
    graph, exe = ctypes.c_void_p(), ctypes.c_void_p()
    try:
        clear()
        enqueue(s)
        assert hip.hipStreamSynchronize(s) == 0
        _same(read(), want)
        assert hip.hipStreamBeginCapture(s, 0) == 0
        enqueue(s)
        assert hip.hipStreamEndCapture(s, ctypes.byref(graph)) == 0 and graph.value
        assert hip.hipGraphInstantiate(ctypes.byref(exe), graph, None, None, 0) == 0
        other = rng.standard_normal((300, 16)).astype(np.float32)
        for _ in range(3):
            # eager work through the same scratch between replays
            _route(lane, "tessera_gfx950_moe_route_f32_noalloc_dev", other, 2, False, 0)
            clear()
            lane.synchronize()
            assert hip.hipGraphLaunch(exe, s) == 0
            assert hip.hipStreamSynchronize(s) == 0
            _same(read(), want)
    finally:
        if exe.value:
            hip.hipGraphExecDestroy(exe)
        if graph.value:
            hip.hipGraphDestroy(graph)
        hip.hipStreamSynchronize(s)
        hip.hipStreamDestroy(s)
        for b in list(bufs.values()) + [d_scores]:
            b.close()
