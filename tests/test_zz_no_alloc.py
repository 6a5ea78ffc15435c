"""om_mi355x_DynamicQuantizeLinearNoAlloc, the entry point that allocates
nothing: its results must equal om_mi355x_DynamicQuantizeLinear's bit for bit,
call after call on the one scratch array each GPU holds (the second and later
calls with smaller inputs than the one before), and it must refuse what it
cannot do without allocating."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _both(rt, x):
    dx = rt.DeviceArray.from_numpy(x)
    want = rt.DynamicQuantizeLinear(dx)
    out = (rt.DeviceArray(x.shape, np.uint8), rt.DeviceArray((), np.float32),
           rt.DeviceArray((), np.uint8))
    got = rt.DynamicQuantizeLinearNoAlloc(dx, out)
    rt.synchronize()
    res = [(g.numpy(), w.numpy()) for g, w in zip(got, want)]
    for a in (dx,) + tuple(want) + tuple(out):
        a.free()
    return res


# largest first: two launches (beyond what the one-launch kernel holds in
# registers), then the one-launch kernel with 16, 4 and 1 float4 per thread
# and fewer blocks than CUs, then the single-block kernel, a ragged size and
# an empty tensor
SHAPES = [(5000, 4099), (4096, 3072), (4096, 768), (16, 4096), (257, 1031), (100,), (7,), (0,)]


def test_matches_the_allocating_entry_point_on_calls_in_a_row(rt, oracle):
    rt.synchronize()  # the calling thread's stream exists from here on
    rng = np.random.default_rng(20250)
    for shape in SHAPES:
        x = rng.normal(0.0, 1.5, shape).astype(np.float32)
        (y, yw), (s, sw), (z, zw) = _both(rt, x)
        assert np.array_equal(y, yw), shape
        assert s.view(np.uint32) == sw.view(np.uint32), shape
        assert z == zw, shape
        # and both equal the oracle's restatement of the reference
        oy, os_, oz = oracle.dynamic_quantize_linear(x)
        assert np.array_equal(y, oy) and np.float32(s) == os_ and int(z) == int(oz), shape


def test_same_input_twice_then_smaller(rt):
    rt.synchronize()
    rng = np.random.default_rng(7)
    big = rng.normal(0.0, 3.0, (4096, 768)).astype(np.float32)
    small = (big[:64, :640] * np.float32(0.25)).copy()
    for x in (big, big, small, small):
        (y, yw), (s, sw), (z, zw) = _both(rt, x)
        assert np.array_equal(y, yw) and s.view(np.uint32) == sw.view(np.uint32) and z == zw


def test_refuses_host_tensors_and_oversized_inputs(rt):
    rt.synchronize()
    x = np.zeros((4, 4), np.float32)
    dx = rt.DeviceArray.from_numpy(x)
    dy, ds, dz = rt.DeviceArray(x.shape, np.uint8), rt.DeviceArray((), np.float32), rt.DeviceArray((), np.uint8)
    with pytest.raises(rt.RuntimeError_, match="GPU memory"):
        rt.DynamicQuantizeLinearNoAlloc(dx, (np.empty(x.shape, np.uint8), ds, dz))
    with pytest.raises(rt.RuntimeError_, match="GPU memory"):
        rt.DynamicQuantizeLinearNoAlloc(x, (dy, ds, dz))

    # tensor headers claiming 2^31 + 4 elements over small buffers: the size
    # check must refuse them before anything is launched
    big_x = rt.DeviceArray.__new__(rt.DeviceArray)
    big_x.shape, big_x.dtype, big_x.ptr = ((1 << 31) + 4,), np.dtype(np.float32), dx.ptr
    big_x.owner = dx
    big_y = rt.DeviceArray.__new__(rt.DeviceArray)
    big_y.shape, big_y.dtype, big_y.ptr = ((1 << 31) + 4,), np.dtype(np.uint8), dy.ptr
    big_y.owner = dy
    with pytest.raises(rt.RuntimeError_, match="limit"):
        rt.DynamicQuantizeLinearNoAlloc(big_x, (big_y, ds, dz))
    rt.synchronize()


def test_refuses_a_thread_without_a_stream(rt):
    import threading
    x = np.ones((8, 8), np.float32)
    dx = rt.DeviceArray.from_numpy(x)
    out = (rt.DeviceArray(x.shape, np.uint8), rt.DeviceArray((), np.float32), rt.DeviceArray((), np.uint8))
    seen = []

    def fresh_thread():
        try:
            rt.DynamicQuantizeLinearNoAlloc(dx, out)
            seen.append("no error")
        except rt.RuntimeError_ as e:
            seen.append(str(e))

    t = threading.Thread(target=fresh_thread)
    t.start()
    t.join()
    assert len(seen) == 1 and "no stream yet" in seen[0], seen


def test_allocates_no_gpu_memory(rt):
    """Free GPU memory as the driver reports it is the same before and after a
    run of calls of every size class (the allocating entry point's pool would
    grow by the temporaries of the largest one)."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    free_b, total_b = ctypes.c_size_t(), ctypes.c_size_t()

    def free_bytes():
        assert hip.hipMemGetInfo(ctypes.byref(free_b), ctypes.byref(total_b)) == 0
        return free_b.value

    rt.synchronize()
    rng = np.random.default_rng(3)
    cases = []
    for shape in ((4096, 3072), (4096, 768), (257, 1031), (7,)):
        x = rng.normal(0.0, 1.0, shape).astype(np.float32)
        cases.append((rt.DeviceArray.from_numpy(x),
                      (rt.DeviceArray(shape, np.uint8), rt.DeviceArray((), np.float32), rt.DeviceArray((), np.uint8))))
    rt.synchronize()
    before = free_bytes()
    for _ in range(3):
        for dx, out in cases:
            rt.DynamicQuantizeLinearNoAlloc(dx, out)
    rt.synchronize()
    assert free_bytes() == before
    for dx, out in cases:
        dx.free()
        for o in out:
            o.free()
