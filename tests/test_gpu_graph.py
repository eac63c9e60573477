"""Forward calls under HIP graph capture, through the C-ABI.  After tq_linear_reserve no forward call of up
to that many rows allocates, so the batch-1, small-batch and prefill paths can be captured and replayed; a
call that would have to grow a workspace while its stream is being captured is refused and leaves the
capture usable; a workspace that is outgrown later stays valid for the graphs that hold its address.
Every replay is compared with the eager result of the same call (same kernels: the same bits), with eager
work and synchronisations between the replays.  The HIP runtime is driven through ctypes, like the other
tests of the C-ABI: one runtime in the process, the one the library itself is linked against."""
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
        rt = self.rt = ctypes.CDLL(path if os.path.exists(path) else "libamdhip64.so")
        vp, vpp = ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p)
        rt.hipMalloc.argtypes = [vpp, ctypes.c_size_t]
        rt.hipMemcpy.argtypes = [vp, vp, ctypes.c_size_t, ctypes.c_int]
        rt.hipMemset.argtypes = [vp, ctypes.c_int, ctypes.c_size_t]
        rt.hipFree.argtypes = [vp]
        rt.hipStreamCreate.argtypes = [vpp]
        rt.hipStreamDestroy.argtypes = [vp]
        rt.hipStreamSynchronize.argtypes = [vp]
        rt.hipStreamBeginCapture.argtypes = [vp, ctypes.c_int]
        rt.hipStreamEndCapture.argtypes = [vp, vpp]
        rt.hipGraphInstantiate.argtypes = [vpp, vp, vp, vp, ctypes.c_size_t]
        rt.hipGraphLaunch.argtypes = [vp, vp]
        rt.hipGraphExecDestroy.argtypes = [vp]
        rt.hipGraphDestroy.argtypes = [vp]
        self.stream = ctypes.c_void_p()
        assert rt.hipStreamCreate(ctypes.byref(self.stream)) == 0
        self.owned = []

    def upload(self, a):
        a = np.ascontiguousarray(a)
        p = ctypes.c_void_p()
        assert self.rt.hipMalloc(ctypes.byref(p), max(a.nbytes, 4)) == 0
        assert self.rt.hipMemcpy(p, a.ctypes.data_as(ctypes.c_void_p), a.nbytes, 1) == 0
        self.owned.append(p)
        return p

    def alloc(self, nbytes):
        p = ctypes.c_void_p()
        assert self.rt.hipMalloc(ctypes.byref(p), nbytes) == 0
        self.owned.append(p)
        self.fill(p, nbytes)
        return p

    def fill(self, p, nbytes, byte=0xFF):                      # 0xFF bytes: fp32 NaN, never equal to a result
        assert self.rt.hipDeviceSynchronize() == 0
        assert self.rt.hipMemset(p, byte, nbytes) == 0
        assert self.rt.hipDeviceSynchronize() == 0

    def download(self, p, shape, dtype=np.float32):
        out = np.empty(shape, dtype)
        assert self.rt.hipDeviceSynchronize() == 0
        assert self.rt.hipMemcpy(out.ctypes.data_as(ctypes.c_void_p), p, out.nbytes, 2) == 0
        return out

    def begin_capture(self):
        assert self.rt.hipStreamBeginCapture(self.stream, 0) == 0          # hipStreamCaptureModeGlobal

    def end_capture(self):
        graph, ex = ctypes.c_void_p(), ctypes.c_void_p()
        assert self.rt.hipStreamEndCapture(self.stream, ctypes.byref(graph)) == 0
        assert self.rt.hipGraphInstantiate(ctypes.byref(ex), graph, None, None, 0) == 0
        return graph, ex

    def replay(self, ex):
        assert self.rt.hipGraphLaunch(ex, self.stream) == 0
        assert self.rt.hipStreamSynchronize(self.stream) == 0

    def drop(self, graph_and_exec):
        self.rt.hipGraphExecDestroy(graph_and_exec[1])
        self.rt.hipGraphDestroy(graph_and_exec[0])

    def close(self):
        assert self.rt.hipDeviceSynchronize() == 0
        for p in self.owned:
            self.rt.hipFree(p)
        self.rt.hipStreamDestroy(self.stream)


def _layer(tq, o, out, inf, bs, mode, seed=11):
    w = (np.random.default_rng(seed).standard_normal((out, inf)) * 0.05).astype(np.float32)
    cb = o.generate_codebook(4)
    if mode == "dual_5bit":                                    # byte primary plane + nibble residual plane
        cb5 = o.generate_codebook(5)
        qw = o.quantize_weight(w, cb5, cb, 5, 4, bs, False)
        return tq.TurboQuantLinear(inf, out, qw, cb5, cb, bs), qw, (cb5, cb)
    if mode == "shared":
        qw = o.quantize_weight(w, cb, cb, 4, 4, bs, True)
    elif mode == "dual":
        qw = o.quantize_weight(w, cb, cb, 4, 4, bs, False)
    else:
        qw = o.quantize_weight(w, cb, cb, 4, 0, bs, False)
    return tq.TurboQuantLinear(inf, out, qw, cb, cb, bs), qw, cb


def _rel(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b.astype(np.float64)) / np.linalg.norm(b.astype(np.float64)))


def _bits(o, rng, batch, inf):
    return o.f32_to_bf16_bits(rng.standard_normal((batch, inf)).astype(np.float32))


BATCHES = (1, 4, 15, 24, 40)      # batch-1 kernel, small-batch kernels (one and two sets of rows), prefill kernel


# (a layer with tiles for more than half the CUs: the panel kernel with one, two, three row blocks per wave, whole panels)
PANEL_BATCHES = (40, 130, 300, 600)


@pytest.mark.parametrize("mode,out,inf,bs,BATCHES", [("shared", 640, 2048, 512, BATCHES), ("dual", 640, 2048, 512, BATCHES),
                                                     ("primary_only", 640, 2048, 512, BATCHES), ("dual_5bit", 640, 2048, 512, BATCHES),
                                                     ("shared", 16500, 512, 256, PANEL_BATCHES), ("dual", 16500, 512, 256, PANEL_BATCHES)])
def test_reserved_layer_is_captured_and_replayed(tq, oracle, mode, out, inf, bs, BATCHES):
    o, hip = oracle, _Hip()
    layer, qw, cb = _layer(tq, o, out, inf, bs, mode)
    layer.reserve(max(BATCHES))
    rng = np.random.default_rng(5)
    xbits = {b: _bits(o, rng, b, inf) for b in BATCHES}
    xs = {b: hip.upload(xbits[b]) for b in BATCHES}
    eager = {b: hip.alloc(b * out * 4) for b in BATCHES}
    replayed = {b: hip.alloc(b * out * 4) for b in BATCHES}
    for b in BATCHES:
        layer.forward_device(xs[b], tq.BF16, b, eager[b], tq.F32, hip.stream)
    want = {b: hip.download(eager[b], (b, out)) for b in BATCHES}
    # the eager results are right (CPU oracle), so bit-equality below is equality with a checked result
    cbs = cb if isinstance(cb, tuple) else (cb, cb)
    w_ref = o.dequantize_weight_cpu(qw, cbs[0], cbs[1], bs)
    for b in BATCHES:
        ref = o.matmul_xwT(o.bf16_bits_to_f32(xbits[b]), w_ref, acc_double=True)
        assert _rel(want[b], ref) < 1e-3
    hip.begin_capture()
    for b in BATCHES:
        layer.forward_device(xs[b], tq.BF16, b, replayed[b], tq.F32, hip.stream)
    graph = hip.end_capture()
    for turn in range(4):
        for b in BATCHES:
            hip.fill(replayed[b], b * out * 4)                 # eager work between the replays
        other = BATCHES[turn % len(BATCHES)]
        layer.forward_device(xs[other], tq.BF16, other, eager[other], tq.F32, None)
        hip.replay(graph[1])
        for b in BATCHES:
            assert np.array_equal(hip.download(replayed[b], (b, out)), want[b]), f"replay {turn}, batch {b}"
    hip.drop(graph)
    layer.close()
    hip.close()


@pytest.mark.parametrize("dual,out,inf,bs,batches", [(False, 12300, 8192, 512, (3, 8, 11)),     # rows rotated in the kernel; two sets of rows, rotated by a kernel of their own
                                                     (False, 4700, 14336, 256, (4,)),        # images that do not fit LDS
                                                     (True, 19701, 5120, 512, (2, 4))])      # nibble planes: two rotations
def test_whole_row_kernel_with_rotated_rows_is_captured_and_replayed(tq, oracle, dual, out, inf, bs, batches):
    """The kernel for two to twelve rows where a kernel of its own rotates the rows into the layer's workspace: after
    tq_linear_reserve both launches of a call are captured, and every replay gives the bits of the eager call (a
    sample of whose rows is checked against the oracle)."""
    o, hip = oracle, _Hip()
    rng = np.random.default_rng(out)
    cb = o.generate_codebook(4)
    pp = rng.integers(0, 256, size=(out, inf // 2)).astype(np.uint8)
    pr = rng.integers(0, 256, size=(out, inf // 2)).astype(np.uint8)
    norms = (rng.random(out) + 0.5).astype(np.float32)
    qw = o.QuantizedWeight(pp, pr, norms, np.array([rng.integers(1, 2 ** 32), rng.integers(1, 2 ** 32) if dual else 0, bs], np.uint32))
    layer = tq.TurboQuantLinear(inf, out, qw, cb, cb, bs)
    layer.reserve(max(batches))
    xbits = {b: _bits(o, rng, b, inf) for b in batches}
    xs = {b: hip.upload(xbits[b]) for b in batches}
    eager = {b: hip.alloc(b * out * 4) for b in batches}
    replayed = {b: hip.alloc(b * out * 4) for b in batches}
    for b in batches:
        layer.forward_device(xs[b], tq.BF16, b, eager[b], tq.F32, hip.stream)
    want = {b: hip.download(eager[b], (b, out)) for b in batches}
    rows = np.unique(np.concatenate([np.arange(5), np.arange(out - 5, out), np.arange(0, out, 173)]))
    sub = o.QuantizedWeight(pp[rows], pr[rows], norms[rows], qw.seeds)
    w_ref = o.dequantize_weight_cpu(sub, cb, cb, bs)
    for b in batches:
        assert _rel(want[b][:, rows], o.matmul_xwT(o.bf16_bits_to_f32(xbits[b]), w_ref, acc_double=True)) < 1e-3
    hip.begin_capture()
    for b in batches:
        layer.forward_device(xs[b], tq.BF16, b, replayed[b], tq.F32, hip.stream)
    graph = hip.end_capture()
    for turn in range(3):
        for b in batches:
            hip.fill(replayed[b], b * out * 4)                 # eager work between the replays
        other = batches[turn % len(batches)]
        layer.forward_device(xs[other], tq.BF16, other, eager[other], tq.F32, None)
        hip.replay(graph[1])
        for b in batches:
            assert np.array_equal(hip.download(replayed[b], (b, out)), want[b]), f"replay {turn}, batch {b}"
    hip.drop(graph)
    layer.close()
    hip.close()


def test_growth_is_refused_while_capturing_and_capture_survives(tq, oracle):
    o, hip = oracle, _Hip()
    out, inf, bs = 320, 1024, 512
    layer, qw, cb = _layer(tq, o, out, inf, bs, "shared")     # no reserve
    L = tq.lib()
    rng = np.random.default_rng(6)
    x1, x9, x15, x64 = (hip.upload(_bits(o, rng, b, inf)) for b in (1, 9, 15, 64))
    y1, y1g = hip.alloc(out * 4), hip.alloc(out * 4)
    y9, y9g = hip.alloc(9 * out * 4), hip.alloc(9 * out * 4)
    y15, y64 = hip.alloc(15 * out * 4), hip.alloc(64 * out * 4)
    layer.forward_device(x1, tq.BF16, 1, y1, tq.F32, hip.stream)
    want1 = hip.download(y1, (1, out))
    hip.fill(y9g, 9 * out * 4, 0)
    hip.begin_capture()
    # nine rows go through per-chunk partial products in a workspace the layer does not have yet
    rc = L.tq_linear_forward(layer._h, x9, tq.BF16, 9, y9g, tq.F32, hip.stream)
    message = tq.last_error()
    layer.forward_device(x1, tq.BF16, 1, y1g, tq.F32, hip.stream)      # one row needs no workspace: captured
    graph = hip.end_capture()
    assert rc != 0 and "tq_linear_reserve" in message
    hip.replay(graph[1])
    assert np.array_equal(hip.download(y1g, (1, out)), want1)
    assert not hip.download(y9g, (9, out)).any()               # the refused call launched nothing
    # outside a capture the same call allocates and runs; afterwards it can be captured
    layer.forward_device(x9, tq.BF16, 9, y9, tq.F32, None)
    want9 = hip.download(y9, (9, out))
    hip.begin_capture()
    layer.forward_device(x9, tq.BF16, 9, y9g, tq.F32, hip.stream)
    graph9 = hip.end_capture()
    # larger batches outgrow the workspaces graph9 holds; the old ones must stay valid for graph9
    layer.forward_device(x15, tq.BF16, 15, y15, tq.F32, None)
    layer.forward_device(x64, tq.BF16, 64, y64, tq.F32, None)
    for _ in range(3):
        hip.fill(y9g, 9 * out * 4)
        hip.replay(graph9[1])
        assert np.array_equal(hip.download(y9g, (9, out)), want9)
    hip.drop(graph)
    hip.drop(graph9)
    layer.close()
    hip.close()


def test_reserve_error_conventions(tq, oracle):
    L = tq.lib()
    assert L.tq_linear_reserve(None, 8) != 0
    layer, _, _ = _layer(tq, oracle, 64, 512, 512, "shared")
    assert L.tq_linear_reserve(layer._h, 0) != 0
    assert L.tq_linear_reserve(layer._h, -3) != 0
    assert L.tq_linear_reserve(layer._h, 1) == 0
    assert L.tq_linear_reserve(layer._h, 300) == 0
    assert L.tq_linear_reserve(layer._h, 8) == 0               # never shrinks
    layer.close()
