"""tq_linear_forward_static: the forward entry point that allocates nothing (its matrix-core workspaces
live in a fixed array inside the library), through the C-ABI, against tq_linear_forward on the same
inputs: same kernels, so the same bits.  Two calls in a row share the array, the second with a smaller
input; a layer whose workspace exceeds the array is refused with a clear error."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tq():
    import __graft_entry__ as entry
    pkg = entry.load_package()
    pkg.lib()
    return pkg


class _Hip:
    def __init__(self):
        import os
        path = "/opt/rocm/lib/libamdhip64.so"
        self.rt = ctypes.CDLL(path if os.path.exists(path) else "libamdhip64.so")
        self.rt.hipMalloc.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t]
        self.rt.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
        self.rt.hipMemset.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t]
        self.rt.hipFree.argtypes = [ctypes.c_void_p]

    def upload(self, a):
        a = np.ascontiguousarray(a)
        p = ctypes.c_void_p()
        assert self.rt.hipMalloc(ctypes.byref(p), max(a.nbytes, 4)) == 0
        assert self.rt.hipMemcpy(p, a.ctypes.data_as(ctypes.c_void_p), a.nbytes, 1) == 0
        return p

    def alloc(self, nbytes):
        p = ctypes.c_void_p()
        assert self.rt.hipMalloc(ctypes.byref(p), nbytes) == 0
        assert self.rt.hipMemset(p, 0xFF, nbytes) == 0
        return p

    def download(self, p, shape, dtype):
        out = np.empty(shape, dtype)
        assert self.rt.hipDeviceSynchronize() == 0
        assert self.rt.hipMemcpy(out.ctypes.data_as(ctypes.c_void_p), p, out.nbytes, 2) == 0
        return out

    def free(self, *ptrs):
        for p in ptrs:
            self.rt.hipFree(p)

    def free_bytes(self):
        """Free device memory as the runtime reports it: any hipMalloc / hipFree in between changes it."""
        free, total = ctypes.c_size_t(), ctypes.c_size_t()
        assert self.rt.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
        return free.value


def _make(o, out, inf, bs, mode, seed=7):
    w = (np.random.default_rng(seed).standard_normal((out, inf)) * 0.05).astype(np.float32)
    cb = o.generate_codebook(4)
    if mode == "shared":
        qw = o.quantize_weight(w, cb, cb, 4, 4, bs, True)
    elif mode == "dual":
        qw = o.quantize_weight(w, cb, cb, 4, 4, bs, False)
    else:
        qw = o.quantize_weight(w, cb, cb, 4, 0, bs, False)
    return qw, cb


def _rel(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b.astype(np.float64)) / np.linalg.norm(b.astype(np.float64)))


# (out, in, block, first batch, second and smaller batch): small-batch kernels with the rotation inside
# (blocks <= 512) and behind the separate rotation kernel (block 1024), and the prefill kernels
CASES = [(300, 1024, 256, 8, 3), (513, 2048, 1024, 15, 2), (257, 1536, 512, 100, 20), (64, 512, 512, 300, 40),
         (1000, 5120, 512, 9, 1),
         (16500, 512, 256, 300, 100)]     # enough tiles for the panel kernel: three row blocks per wave, then one (two wave groups)


@pytest.mark.parametrize("mode", ["shared", "dual", "primary_only"])
@pytest.mark.parametrize("out,inf,bs,batch_a,batch_b", CASES)
def test_static_forward_equals_forward_two_calls_in_a_row(tq, oracle, mode, out, inf, bs, batch_a, batch_b):
    hip = _Hip()
    o = oracle
    qw, cb = _make(o, out, inf, bs, mode)
    layer = tq.TurboQuantLinear(inf, out, qw, cb, cb, bs)
    w_ref = o.dequantize_weight_cpu(qw, cb, cb, bs)
    bufs = []
    for k, batch in enumerate((batch_a, batch_b)):                       # second call: smaller input, same scratch
        xbits = o.f32_to_bf16_bits(np.random.default_rng(50 + k).standard_normal((batch, inf)).astype(np.float32))
        x_dev = hip.upload(xbits)
        y_ref_dev, y_dev = hip.alloc(batch * out * 4), hip.alloc(batch * out * 4)
        layer.forward_device(x_dev, tq.BF16, batch, y_ref_dev, tq.F32)
        want = hip.download(y_ref_dev, (batch, out), np.float32)
        free_before = hip.free_bytes()
        layer.forward_static_device(x_dev, tq.BF16, batch, y_dev, tq.F32)
        assert hip.rt.hipDeviceSynchronize() == 0
        assert hip.free_bytes() == free_before, "the static entry point allocated or freed device memory"
        got = hip.download(y_dev, (batch, out), np.float32)
        assert np.array_equal(got, want), f"call {k}, batch {batch}"      # same kernels: bit-exact
        ref = o.matmul_xwT(o.bf16_bits_to_f32(xbits), w_ref, acc_double=True)
        assert _rel(got, ref) < 1e-3                                      # and right, against the CPU oracle
        bufs += [x_dev, y_ref_dev, y_dev]
    hip.free(*bufs)
    layer.close()


def test_static_forward_two_plane_five_bit_layer(tq, oracle):
    """A 5-bit primary with its own residual rotation: at two or more rows the static entry point also
    keeps the fp32 results of the two planes in the array."""
    hip = _Hip()
    o = oracle
    out, inf, bs = 200, 2048, 512
    w = (np.random.default_rng(3).standard_normal((out, inf)) * 0.05).astype(np.float32)
    cbp, cbr = o.generate_codebook(5), o.generate_codebook(4)
    qw = o.quantize_weight(w, cbp, cbr, 5, 4, bs, False)
    layer = tq.TurboQuantLinear(inf, out, qw, cbp, cbr, bs)
    assert layer.mode() == "dual_5bit"
    w_ref = o.dequantize_weight_cpu(qw, cbp, cbr, bs)
    bufs = []
    for k, (batch, ydt, ynp) in enumerate(((40, tq.F32, np.float32), (6, tq.BF16, np.uint16), (1, tq.F32, np.float32))):
        xbits = o.f32_to_bf16_bits(np.random.default_rng(60 + k).standard_normal((batch, inf)).astype(np.float32))
        x_dev = hip.upload(xbits)
        nb = batch * out * np.dtype(ynp).itemsize
        y_ref_dev, y_dev = hip.alloc(nb), hip.alloc(nb)
        layer.forward_device(x_dev, tq.BF16, batch, y_ref_dev, ydt)
        want = hip.download(y_ref_dev, (batch, out), ynp)
        layer.forward_static_device(x_dev, tq.BF16, batch, y_dev, ydt)
        got = hip.download(y_dev, (batch, out), ynp)
        assert np.array_equal(got, want), f"call {k}, batch {batch}"
        gf = got if ydt == tq.F32 else o.bf16_bits_to_f32(got)
        ref = o.matmul_xwT(o.bf16_bits_to_f32(xbits), w_ref, acc_double=True)
        assert _rel(gf, ref) < (5e-3 if ydt == tq.BF16 else 1e-3)      # (a bf16 output adds its own rounding)
        bufs += [x_dev, y_ref_dev, y_dev]
    hip.free(*bufs)
    layer.close()


def test_static_forward_cuts_k_into_fewer_ranges_when_the_array_is_short(tq, oracle):
    """1536 x 16384 at 500 tokens: 2 x 6 output tiles, so the allocating entry point cuts K into 16 ranges
    (16 MiB of tile images + 16 x 2.9 MiB of fp32 products); the static array holds the images and five ranges.
    Same result up to the order of the fp32 sums, and right against the CPU oracle."""
    hip = _Hip()
    o = oracle
    out, inf, bs, batch = 1536, 16384, 512, 500
    qw, cb = _make(o, out, inf, bs, "shared")
    layer = tq.TurboQuantLinear(inf, out, qw, cb, cb, bs)
    o.set_threads(8)
    w_ref = o.dequantize_weight_cpu(qw, cb, cb, bs)
    xbits = o.f32_to_bf16_bits(np.random.default_rng(70).standard_normal((batch, inf)).astype(np.float32))
    ref = o.matmul_xwT(o.bf16_bits_to_f32(xbits), w_ref, acc_double=True)
    o.set_threads(1)
    x_dev = hip.upload(xbits)
    y_ref_dev, y_dev = hip.alloc(batch * out * 4), hip.alloc(batch * out * 4)
    layer.forward_device(x_dev, tq.BF16, batch, y_ref_dev, tq.F32)
    want = hip.download(y_ref_dev, (batch, out), np.float32)
    for _ in range(2):
        free_before = hip.free_bytes()
        layer.forward_static_device(x_dev, tq.BF16, batch, y_dev, tq.F32)
        assert hip.rt.hipDeviceSynchronize() == 0
        assert hip.free_bytes() == free_before, "the static entry point allocated or freed device memory"
        got = hip.download(y_dev, (batch, out), np.float32)
        assert _rel(got, want) < 1e-5
        assert _rel(got, ref) < 1e-3
        assert hip.rt.hipMemset(y_dev, 0xFF, batch * out * 4) == 0             # the second call starts from NaNs again
    assert _rel(want, ref) < 1e-3
    hip.free(x_dev, y_ref_dev, y_dev)
    layer.close()


def test_static_forward_refuses_a_workspace_beyond_the_array(tq, oracle):
    hip = _Hip()
    o = oracle
    # 512 rows of 16384 columns at 1100 tokens: 5 tile images of 256 x 16384 bf16 = 40 MiB > 32 MiB
    out, inf, bs = 32, 16384, 512
    qw, cb = _make(o, out, inf, bs, "shared")
    layer = tq.TurboQuantLinear(inf, out, qw, cb, cb, bs)
    batch = 1100
    x_dev = hip.upload(np.zeros((batch, inf), np.uint16))
    y_dev = hip.alloc(batch * out * 4)
    with pytest.raises(RuntimeError, match="more than the static"):
        layer.forward_static_device(x_dev, tq.BF16, batch, y_dev, tq.F32)
    layer.forward_static_device(x_dev, tq.BF16, 512, y_dev, tq.F32)       # 16 MiB: accepted
    assert np.array_equal(hip.download(y_dev, (512, out), np.float32), np.zeros((512, out), np.float32))
    with pytest.raises(RuntimeError):
        layer.forward_static_device(None, tq.BF16, 4, y_dev, tq.F32)
    hip.free(x_dev, y_dev)
    layer.close()
