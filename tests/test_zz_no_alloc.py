"""ghip_forward_noalloc (the entry point that allocates nothing) against ghip_net_forward_resident,
the existing entry point it is a variant of: same kernels, so the outputs must agree bit for bit.
Two calls in a row share the GPU's fixed scratch array, the second with a smaller input."""
import ctypes as C

import numpy as np
import pytest

import pyglades as pg

pytestmark = pytest.mark.gpu


_hip = None


def hip():
    """The HIP runtime the library itself is linked against (loading it by its soname returns the
    copy already in the process): device memory for the caller's side of the test."""
    global _hip
    if _hip is None:
        pg.load()
        _hip = C.CDLL("libamdhip64.so.7")
        _hip.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        _hip.hipFree.argtypes = [C.c_void_p]
        _hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        _hip.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
        _hip.hipStreamCreate.argtypes = [C.POINTER(C.c_void_p)]
        _hip.hipStreamSynchronize.argtypes = [C.c_void_p]
        _hip.hipStreamDestroy.argtypes = [C.c_void_p]
    return _hip


def free_device_bytes():
    free, total = C.c_size_t(), C.c_size_t()
    assert hip().hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


class DeviceArray:
    """A float32 array in device memory that the test owns."""

    def __init__(self, host=None, shape=None, fill=None):
        if host is None:
            host = np.full(shape, fill, np.float32)
        host = np.ascontiguousarray(host, np.float32)
        self.shape, self.nbytes = host.shape, max(host.nbytes, 16)
        self.ptr = C.c_void_p()
        assert hip().hipMalloc(C.byref(self.ptr), self.nbytes) == 0
        assert hip().hipMemcpy(self.ptr, host.ctypes.data, host.nbytes, 1) == 0  # host to device

    def numpy(self):
        out = np.empty(self.shape, np.float32)
        assert hip().hipDeviceSynchronize() == 0
        assert hip().hipMemcpy(out.ctypes.data, self.ptr, out.nbytes, 2) == 0  # device to host
        return out

    def free(self):
        assert hip().hipFree(self.ptr) == 0


def _reference_forward(spec, sizes, Ws, bs, X):
    """The existing path: a handle, the table resident, ghip_net_forward_resident into caller memory."""
    net = pg.Net(spec)
    for l in range(len(Ws)):
        net.set_params(l, Ws[l], bs[l])
    net.set_dataset(X, np.zeros((X.shape[0], sizes[-1]), np.float32))
    out = DeviceArray(shape=(X.shape[0], sizes[-1]), fill=np.nan)
    pg._check(net.lib.ghip_net_forward_resident(net.h, 0, X.shape[0], out.ptr))
    net.sync()
    res = out.numpy()
    out.free()
    net.close()
    return res


def _noalloc_forward(spec, sizes, Ws, bs, X):
    lib = pg.load()
    dW = [DeviceArray(w) for w in Ws]
    db = [DeviceArray(b) for b in bs]
    dX = DeviceArray(X)
    out = DeviceArray(shape=(X.shape[0], sizes[-1]), fill=np.nan)
    nl = len(Ws)
    pw = (C.c_void_p * nl)(*[t.ptr.value for t in dW])
    pb = (C.c_void_p * nl)(*[t.ptr.value for t in db])
    pg._check(lib.ghip_forward_noalloc(C.byref(spec), pw, pb, dX.ptr, X.shape[0], out.ptr, None))
    res = out.numpy()
    for t in dW + db + [dX, out]:
        t.free()
    return res


def _case(rng, sizes, acts, batch):
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l])) / np.sqrt(sizes[l])).astype(np.float32) for l in range(len(sizes) - 1)]
    bs = [(0.1 * rng.standard_normal(sizes[l + 1])).astype(np.float32) for l in range(len(sizes) - 1)]
    X = rng.standard_normal((batch, sizes[0])).astype(np.float32)
    spec = pg.make_spec(sizes, acts, cost=pg.CLASSIFICATION, mode=pg.MODE_CANONICAL, dtype=pg.F32)
    return spec, Ws, bs, X


def test_noalloc_forward_equals_the_resident_forward_on_two_calls_in_a_row():
    pg._check(pg.load().ghip_init(0))
    rng = np.random.default_rng(11)
    # first call: three hidden layers (both halves of the scratch are written), GEMM output layer + softmax
    sizes1, acts1 = [96, 320, 200, 136, 40], [pg.RELU, pg.TANH, pg.SIGMOID, pg.SOFTMAX]
    spec1, W1, b1, X1 = _case(rng, sizes1, acts1, 700)
    got1 = _noalloc_forward(spec1, sizes1, W1, b1, X1)
    # second call, smaller in batch and in width: whatever the first left in the scratch must not show
    sizes2, acts2 = [40, 64, 24, 3], [pg.TANH, pg.RELU, pg.SIGMOID]
    spec2, W2, b2, X2 = _case(rng, sizes2, acts2, 37)
    got2 = _noalloc_forward(spec2, sizes2, W2, b2, X2)
    want1 = _reference_forward(spec1, sizes1, W1, b1, X1)
    want2 = _reference_forward(spec2, sizes2, W2, b2, X2)
    assert got1.tobytes() == want1.tobytes()
    assert got2.tobytes() == want2.tobytes()
    assert np.isfinite(got1).all() and np.isfinite(got2).all()


def test_noalloc_forward_refuses_what_its_scratch_cannot_hold():
    lib = pg.load()
    pg._check(lib.ghip_init(0))
    sizes = [8, 4096, 2]
    spec = pg.make_spec(sizes, [pg.RELU, pg.LINEAR], mode=pg.MODE_CANONICAL, dtype=pg.F32)
    t = DeviceArray(shape=(16,), fill=0.0)
    p2 = (C.c_void_p * 2)(t.ptr.value, t.ptr.value)
    # 2048 rows x 4096 units is over the limit of 4 Mi activations per layer: refused before any launch
    rc = lib.ghip_forward_noalloc(C.byref(spec), p2, p2, t.ptr, 2048, t.ptr, None)
    assert rc == -1 and b"scratch" in lib.ghip_last_error()
    exact = pg.make_spec(sizes, [pg.RELU, pg.LINEAR], mode=pg.MODE_EXACT)
    rc = lib.ghip_forward_noalloc(C.byref(exact), p2, p2, t.ptr, 4, t.ptr, None)
    assert rc == -1
    t.free()


def test_noalloc_forward_allocates_nothing_and_takes_a_stream():
    """What the entry point is for: between two readings of the device's free memory, with the caller's buffers
    already in place and one warm-up call behind (the first call on a device resolves the scratch array's
    address and may load code), calls on a stream of the caller's change the free memory by nothing; the result
    on that stream is the null stream's bit for bit; a pointer off the 16-byte grid is refused."""
    lib = pg.load()
    pg._check(lib.ghip_init(0))
    rng = np.random.default_rng(12)
    sizes, acts = [64, 256, 128, 10], [pg.RELU, pg.TANH, pg.SOFTMAX]
    spec, Ws, bs, X = _case(rng, sizes, acts, 300)
    dW = [DeviceArray(w) for w in Ws]
    db = [DeviceArray(b) for b in bs]
    dX = DeviceArray(X)
    out0 = DeviceArray(shape=(300, 10), fill=np.nan)
    out1 = DeviceArray(shape=(300, 10), fill=np.nan)
    pw = (C.c_void_p * 3)(*[t.ptr.value for t in dW])
    pb = (C.c_void_p * 3)(*[t.ptr.value for t in db])
    stream = C.c_void_p()
    assert hip().hipStreamCreate(C.byref(stream)) == 0
    pg._check(lib.ghip_forward_noalloc(C.byref(spec), pw, pb, dX.ptr, 300, out0.ptr, None))      # warm-up, null stream
    pg._check(lib.ghip_forward_noalloc(C.byref(spec), pw, pb, dX.ptr, 300, out1.ptr, stream))   # warm-up of the stream
    assert hip().hipStreamSynchronize(stream) == 0 and hip().hipDeviceSynchronize() == 0
    before = free_device_bytes()
    for _ in range(5):
        pg._check(lib.ghip_forward_noalloc(C.byref(spec), pw, pb, dX.ptr, 300, out1.ptr, stream))
    assert hip().hipStreamSynchronize(stream) == 0
    after = free_device_bytes()
    assert after == before, (before, after)
    assert out1.numpy().tobytes() == out0.numpy().tobytes()
    # a pointer off the 16-byte grid
    rc = lib.ghip_forward_noalloc(C.byref(spec), pw, pb, C.c_void_p(dX.ptr.value + 4), 299, out1.ptr, stream)
    assert rc == -1 and b"aligned" in lib.ghip_last_error()
    assert hip().hipStreamDestroy(stream) == 0
    for t in dW + db + [dX, out0, out1]:
        t.free()
