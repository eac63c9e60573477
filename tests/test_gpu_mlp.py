"""Gated MLP block (tq_mlp_*) and the 5-bit primary layers on the fused kernels, against the
CPU oracle: dequantise each layer, fp32 matmul, SiLU gate in fp32 between the linears."""
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
    """Device buffers through the HIP runtime the library itself is linked against (ctypes, no torch:
    another copy of the runtime in the process, such as the one torch bundles, does not see the
    device this library initialised)."""

    def __init__(self):
        import ctypes
        import os
        self.c = ctypes
        path = "/opt/rocm/lib/libamdhip64.so"
        self.rt = ctypes.CDLL(path if os.path.exists(path) else "libamdhip64.so")
        self.rt.hipMalloc.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t]
        self.rt.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
        self.rt.hipFree.argtypes = [ctypes.c_void_p]

    def upload(self, a):
        a = np.ascontiguousarray(a)
        p = self.c.c_void_p()
        assert self.rt.hipMalloc(self.c.byref(p), max(a.nbytes, 4)) == 0
        assert self.rt.hipMemcpy(p, a.ctypes.data_as(self.c.c_void_p), a.nbytes, 1) == 0
        return p

    def alloc(self, nbytes):
        p = self.c.c_void_p()
        assert self.rt.hipMalloc(self.c.byref(p), nbytes) == 0
        return p

    def download(self, p, shape, dtype):
        out = np.empty(shape, dtype)
        assert self.rt.hipDeviceSynchronize() == 0
        assert self.rt.hipMemcpy(out.ctypes.data_as(self.c.c_void_p), p, out.nbytes, 2) == 0
        return out

    def free(self, *ptrs):
        for p in ptrs:
            self.rt.hipFree(p)


def _rel(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b.astype(np.float64)) / np.linalg.norm(b.astype(np.float64)))


def _layer(tq, o, out_f, in_f, bs, shared, seed, scale=0.05, fit=True):
    w = (np.random.default_rng(seed).standard_normal((out_f, in_f)) * scale).astype(np.float32)
    if fit and out_f * in_f <= 1 << 21:
        cbp, cbr = o.fit_layer_codebooks(w, bs)
    else:                                    # the CPU fit takes seconds per million weights
        cbp = cbr = o.generate_codebook(4)
    qw = o.quantize_weight(w, cbp, cbr, 4, 4, bs, shared)
    return tq.TurboQuantLinear(in_f, out_f, qw, cbp, cbr, bs), o.dequantize_weight_cpu(qw, cbp, cbr, bs)


def _silu(g):
    g = g.astype(np.float32)
    return g / (np.float32(1.0) + np.exp(-g))


@pytest.mark.parametrize("shared", [True, False])
@pytest.mark.parametrize("hidden,inter,bs,batch,x_dt", [(512, 1536, 256, 1, "bf16"), (512, 1536, 256, 4, "bf16"),
                                                         (256, 640, 128, 3, "f32"), (512, 1024, 512, 40, "bf16"),
                                                         # wide rows at batch 1: gated store with a cross-wave sum
                                                         # (hidden 4096) and with rows served in pairs (hidden 5120; the 3072-wide down projection)
                                                         (5120, 1024, 512, 1, "bf16"), (4096, 3072, 512, 1, "f32"),
                                                         # intermediate rows wider than 16384 columns at batch 1: gate and up in
                                                         # one launch, silu(gate) * up formed where the row is rotated
                                                         (3072, 16896, 512, 1, "bf16"), (2560, 16896, 256, 1, "f32")])
def test_mlp_block_matches_oracle(tq, oracle, shared, hidden, inter, bs, batch, x_dt):
    hip = _Hip()
    o = oracle
    gate, wg = _layer(tq, o, inter, hidden, bs, shared, 1)
    up, wu = _layer(tq, o, inter, hidden, bs, shared, 2)
    down, wd = _layer(tq, o, hidden, inter, bs, shared, 3)
    mlp = tq.TurboQuantMLP(gate, up, down, max_batch=batch)

    x32 = np.random.default_rng(batch).standard_normal((batch, hidden)).astype(np.float32)
    if x_dt == "bf16":
        xbits = o.f32_to_bf16_bits(x32)
        x_ref = o.bf16_bits_to_f32(xbits)
        x_dev = hip.upload(xbits)
        code = tq.BF16
    else:
        x_ref = x32
        x_dev = hip.upload(x32)
        code = tq.F32
    y_dev = hip.alloc(batch * hidden * 4)
    for _ in range(2):                                   # the block reuses its intermediates
        mlp.forward_device(x_dev, code, batch, y_dev, tq.F32)
        y = hip.download(y_dev, (batch, hidden), np.float32)

    act = _silu(o.matmul_xwT(x_ref, wg, acc_double=True)) * o.matmul_xwT(x_ref, wu, acc_double=True)
    want = o.matmul_xwT(act.astype(np.float32), wd, acc_double=True)
    # the activation between the linears stays fp32 at every batch; from two rows on the linears keep fp16
    # weights and rotated activations (3e-4 each)
    assert _rel(y, want) < 1e-3
    with pytest.raises(RuntimeError):
        mlp.forward_device(x_dev, code, batch + 1, y_dev, tq.F32)
    mlp.close()
    hip.free(x_dev, y_dev)
    for l in (gate, up, down):
        l.close()


@pytest.mark.parametrize("batch,x_dt", [(1, "bf16"), (1, "f32"), (5, "bf16"), (3, "f32"), (24, "bf16")])
def test_mlp_block_of_five_bit_two_plane_layers(tq, oracle, batch, x_dt):
    """The block over layers in the default output format of `tq-convert --bits 5` (5-bit primary, 4-bit residual
    with its own rotation): one row on the generic kernels with the gate folded into the store, more rows with
    each plane through the tuned kernels."""
    hip = _Hip()
    o = oracle
    hidden, inter, bs = 512, 1536, 256
    cb5, cb4 = o.generate_codebook(5), o.generate_codebook(4)
    layers, refs = [], []
    for k, (out_f, in_f) in enumerate(((inter, hidden), (inter, hidden), (hidden, inter))):
        w = (np.random.default_rng(30 + k).standard_normal((out_f, in_f)) * 0.05).astype(np.float32)
        qw = o.quantize_weight(w, cb5, cb4, 5, 4, bs, False)
        layers.append(tq.TurboQuantLinear(in_f, out_f, qw, cb5, cb4, bs))
        assert layers[-1].mode() == "dual_5bit"
        refs.append(o.dequantize_weight_cpu(qw, cb5, cb4, bs))
    mlp = tq.TurboQuantMLP(layers[0], layers[1], layers[2], max_batch=batch)
    x32 = np.random.default_rng(batch).standard_normal((batch, hidden)).astype(np.float32)
    if x_dt == "bf16":
        xbits = o.f32_to_bf16_bits(x32)
        x_ref, x_dev, code = o.bf16_bits_to_f32(xbits), hip.upload(xbits), tq.BF16
    else:
        x_ref, x_dev, code = x32, hip.upload(x32), tq.F32
    y_dev = hip.alloc(batch * hidden * 4)
    for _ in range(2):
        mlp.forward_device(x_dev, code, batch, y_dev, tq.F32)
        y = hip.download(y_dev, (batch, hidden), np.float32)
    act = _silu(o.matmul_xwT(x_ref, refs[0], acc_double=True)) * o.matmul_xwT(x_ref, refs[1], acc_double=True)
    want = o.matmul_xwT(act.astype(np.float32), refs[2], acc_double=True)
    assert _rel(y, want) < 1e-3
    mlp.close()
    hip.free(x_dev, y_dev)
    for l in layers:
        l.close()


def test_mlp_create_rejects_mismatched_layers(tq, oracle):
    a, _ = _layer(tq, oracle, 256, 128, 128, True, 1)
    b, _ = _layer(tq, oracle, 128, 128, 128, True, 2)
    with pytest.raises(ValueError):
        tq.TurboQuantMLP(a, b, a)
    for l in (a, b):
        l.close()


@pytest.mark.parametrize("rbits,shared", [(3, True), (0, True)])
@pytest.mark.parametrize("out_f,in_f,bs,batch", [(96, 512, 256, 1), (64, 2048, 512, 3), (80, 512, 128, 32)])
def test_five_bit_primary_fused_forward(tq, oracle, rbits, shared, out_f, in_f, bs, batch):
    """5-bit primary + 3-bit shared-rotation residual (and 5-bit alone) run on the fused kernels
    through a one-byte-per-weight plane; the dequantised weight stays bit-exact."""
    o = oracle
    w = (np.random.default_rng(5).standard_normal((out_f, in_f)) * 0.03).astype(np.float32)
    cbp, cbr = o.generate_codebook(5), o.generate_codebook(rbits if rbits else 3)
    qw = o.quantize_weight(w, cbp, cbr, 5, rbits, bs, shared)
    w_ref = o.dequantize_weight_cpu(qw, cbp, cbr, bs)
    layer = tq.TurboQuantLinear(in_f, out_f, qw, cbp, cbr, bs)
    assert layer.mode() == ("shared_5bit" if rbits else "primary_only_5bit")
    assert np.array_equal(layer.dequantize(), w_ref)
    x = np.random.default_rng(batch).standard_normal((batch, in_f)).astype(np.float32)
    y = layer.forward(x)
    assert _rel(y, o.matmul_xwT(x, w_ref, acc_double=True)) < 1e-3
    xb = o.f32_to_bf16_bits(x)
    yb = layer.forward(xb, tq.BF16, tq.F32)
    assert _rel(yb, o.matmul_xwT(o.bf16_bits_to_f32(xb), w_ref, acc_double=True)) < 1e-3
    layer.close()


@pytest.mark.parametrize("rbits,shared", [(3, False), (4, False), (4, True), (0, False)],
                         ids=["5+3dual", "5+4dual", "5+4shared", "5+0_long_residual_codebook"])
@pytest.mark.parametrize("out_f,in_f,bs,batch", [(16, 128, 64, 1), (96, 512, 256, 3), (70, 2048, 512, 1),
                                                 (33, 5120, 512, 2), (24, 1024, 1024, 20), (200, 5120, 512, 6),
                                                 (96, 2048, 512, 40), (50, 1024, 1024, 2), (300, 3584, 512, 15),
                                                 (12, 48, 16, 3)])
def test_five_bit_two_plane_forward(tq, oracle, rbits, shared, out_f, in_f, bs, batch):
    """5-bit primary with its own residual rotation, or with a 4-bit residual (what `--bits 5` of the
    converter writes by default): byte primary plane + nibble residual plane, two rotations, the case of
    metal/turboquant_dequant_mm.metal:240-248, 277-292.  One row runs both planes in one generic pass; two
    or more rows run each plane through the tuned kernels as a layer of its own and add the results."""
    o = oracle
    w = (np.random.default_rng(5 + out_f).standard_normal((out_f, in_f)) * 0.03).astype(np.float32)
    cbp = o.generate_codebook(5)
    cbr = o.generate_codebook(rbits) if rbits else o.generate_codebook(4)   # 16 residual centroids nobody reads
    qw = o.quantize_weight(w, cbp, cbr, 5, rbits, bs, shared)
    w_ref = o.dequantize_weight_cpu(qw, cbp, cbr, bs)
    layer = tq.TurboQuantLinear(in_f, out_f, qw, cbp, cbr, bs)
    assert layer.mode() == ("primary_only_5bit" if rbits == 0 else "shared_5bit" if shared else "dual_5bit")
    assert np.array_equal(layer.dequantize(), w_ref)
    x = np.random.default_rng(batch).standard_normal((batch, in_f)).astype(np.float32)
    y = layer.forward(x)
    assert y.shape == (batch, out_f)
    assert _rel(y, o.matmul_xwT(x, w_ref, acc_double=True)) < 1e-3
    xb = o.f32_to_bf16_bits(x)
    yb = layer.forward(xb, tq.BF16, tq.F32)
    assert _rel(yb, o.matmul_xwT(o.bf16_bits_to_f32(xb), w_ref, acc_double=True)) < 1e-3
    y16 = o.bf16_bits_to_f32(layer.forward(x.astype(np.float16), tq.F16, tq.BF16))
    assert _rel(y16, o.matmul_xwT(x.astype(np.float16).astype(np.float32), w_ref, acc_double=True)) < 5e-3
    layer.close()


@pytest.mark.parametrize("shared", [True, False])
@pytest.mark.parametrize("outs,in_f,bs,x_dt", [((640, 128, 131), 5120, 512, "bf16"),     # q, k, v: rows served in pairs
                                                 ((1100, 1000), 4096, 512, "f32"),         # gate, up: two slabs
                                                 ((300, 40, 7), 3072, 256, "f16"),
                                                 ((700, 300), 8192, 512, "bf16"),          # four slabs (dual: old tables)
                                                 ((9000, 7001), 4096, 512, "bf16"),        # many rows per stream (dual: groups of four rows)
                                                 ((257, 255), 2048, 512, "bf16"),          # one slab: shared rotation runs them one by one
                                                 ((96, 64), 18944, 512, "bf16")])          # too wide to share a launch
def test_forward_group_equals_single_forwards(tq, oracle, shared, outs, in_f, bs, x_dt):
    """tq_linear_forward_group: two or three layers on the same activation row.  Bit-identical to one
    tq_linear_forward per layer whether the layers share a launch or not, and within the fp32 tolerance
    of the oracle."""
    hip = _Hip()
    layers, dense = [], []
    for j, out_f in enumerate(outs):
        layer, w = _layer(tq, oracle, out_f, in_f, bs, shared, seed=50 + j)
        layers.append(layer); dense.append(w)
    x32 = np.random.default_rng(9).standard_normal((1, in_f)).astype(np.float32)
    if x_dt == "bf16":
        xbits = oracle.f32_to_bf16_bits(x32); xin = oracle.bf16_bits_to_f32(xbits); xarg, xcode = xbits, tq.BF16
    elif x_dt == "f16":
        xarg = x32.astype(np.float16); xin = xarg.astype(np.float32); xcode = tq.F16
    else:
        xarg, xin, xcode = x32, x32, tq.F32
    dx = hip.upload(xarg)
    ys_group = [hip.alloc(o * 4) for o in outs]
    ys_single = [hip.alloc(o * 4) for o in outs]
    for _ in range(2):                                   # twice: nothing stale between calls
        tq.forward_group_device(layers, dx, xcode, 1, ys_group, tq.F32)
    for layer, yp in zip(layers, ys_single):
        layer.forward_device(dx, xcode, 1, yp, tq.F32)
    for j, o in enumerate(outs):
        yg = hip.download(ys_group[j], (1, o), np.float32)
        y1 = hip.download(ys_single[j], (1, o), np.float32)
        assert np.array_equal(yg, y1)
        assert _rel(yg, xin @ dense[j].T) < 1e-3
    hip.free(dx, *ys_group, *ys_single)
    for layer in layers:
        layer.close()


def test_forward_group_rejects_bad_arguments(tq, oracle):
    layer, _ = _layer(tq, oracle, 64, 512, 256, True, seed=3)
    other, _ = _layer(tq, oracle, 64, 1024, 256, True, seed=4)
    hip = _Hip()
    dx = hip.upload(np.zeros((1, 1024), np.float32)); dy = hip.alloc(64 * 4)
    with pytest.raises(RuntimeError):
        tq.forward_group_device([layer, other], dx, tq.F32, 1, [dy, dy], tq.F32)   # different in_features
    with pytest.raises(RuntimeError):
        tq.forward_group_device([layer] * 4, dx, tq.F32, 1, [dy] * 4, tq.F32)      # more than three layers
    with pytest.raises(RuntimeError):
        tq.forward_group_device([other], dx, tq.F32, 0, [dy], tq.F32)              # no rows
    hip.free(dx, dy)
    layer.close(); other.close()


@pytest.mark.parametrize("shared", [True, False])
@pytest.mark.parametrize("batch", [2, 5, 8, 15, 16, 27, 32])
@pytest.mark.parametrize("outs,in_f,bs", [((640, 128, 131), 5120, 512), ((1100, 1000), 4096, 256), ((50, 33), 1024, 512),
                                          ((40, 24), 2048, 1024)])
def test_forward_group_small_batches(tq, oracle, shared, batch, outs, in_f, bs):
    """tq_linear_forward_group with 2..15 rows of bf16 activations: shared-rotation layers with blocks of
    at most 512 columns share the matrix-core kernel and its reduction, everything else (dual rotation,
    larger blocks) is run layer by layer.  Bit-identical to separate calls either way; bf16 tolerance
    against the dense product."""
    hip = _Hip()
    layers, dense = [], []
    for j, out_f in enumerate(outs):
        layer, w = _layer(tq, oracle, out_f, in_f, bs, shared, seed=70 + j)
        layers.append(layer); dense.append(w)
    xbits = oracle.f32_to_bf16_bits(np.random.default_rng(batch).standard_normal((batch, in_f)).astype(np.float32))
    xin = oracle.bf16_bits_to_f32(xbits)
    dx = hip.upload(xbits)
    ys_group = [hip.alloc(batch * o * 4) for o in outs]
    ys_single = [hip.alloc(batch * o * 4) for o in outs]
    for _ in range(2):
        tq.forward_group_device(layers, dx, tq.BF16, batch, ys_group, tq.F32)
    for layer, yp in zip(layers, ys_single):
        layer.forward_device(dx, tq.BF16, batch, yp, tq.F32)
    for j, o in enumerate(outs):
        yg = hip.download(ys_group[j], (batch, o), np.float32)
        y1 = hip.download(ys_single[j], (batch, o), np.float32)
        assert np.array_equal(yg, y1)
        assert _rel(yg, xin @ dense[j].T) < 1e-3
    hip.free(dx, *ys_group, *ys_single)
    for layer in layers:
        layer.close()


@pytest.mark.parametrize("outs,in_f,bs,batch,dual", [((9900, 9850), 10240, 512, 8, False),     # two sets of four rows: 96 MB and more per layer
                                                     ((4700, 4800, 4690), 14336, 256, 4, False),   # images that do not fit LDS
                                                     ((19701, 19800), 5120, 512, 3, True),         # nibble planes: two rotations per layer
                                                     ((12300, 12400), 8192, 256, 6, True),
                                                     ((12300, 12500), 8192, 512, 10, False)])      # three sets of four rows
def test_forward_group_rows_rotated_by_a_kernel_of_their_own(tq, oracle, outs, in_f, bs, batch, dual):
    """tq_linear_forward_group where the kernel for two to twelve rows takes rows that come rotated: one rotation launch
    writes every layer's rotation (each layer has a seed of its own) into its part of the first layer's workspace.
    Bit-identical to separate calls, twice in a row; a sample of the rows against the dense product."""
    hip = _Hip()
    cb = oracle.generate_codebook(4)
    layers, qws = [], []
    for j, o in enumerate(outs):
        rng = np.random.default_rng(900 + j)
        pp = rng.integers(0, 256, size=(o, in_f // 2)).astype(np.uint8)
        pr = rng.integers(0, 256, size=(o, in_f // 2)).astype(np.uint8)
        norms = (rng.random(o) + 0.5).astype(np.float32)
        qw = oracle.QuantizedWeight(pp, pr, norms, np.array([rng.integers(1, 2 ** 32), rng.integers(1, 2 ** 32) if dual else 0, bs], np.uint32))
        qws.append(qw)
        layers.append(tq.TurboQuantLinear(in_f, o, qw, cb, cb, bs))
    xbits = oracle.f32_to_bf16_bits(np.random.default_rng(batch).standard_normal((batch, in_f)).astype(np.float32))
    xin = oracle.bf16_bits_to_f32(xbits)
    dx = hip.upload(xbits)
    ys_group = [hip.alloc(batch * o * 4) for o in outs]
    ys_single = [hip.alloc(batch * o * 4) for o in outs]
    for _ in range(2):
        tq.forward_group_device(layers, dx, tq.BF16, batch, ys_group, tq.F32)
    for layer, yp in zip(layers, ys_single):
        layer.forward_device(dx, tq.BF16, batch, yp, tq.F32)
    for j, o in enumerate(outs):
        yg = hip.download(ys_group[j], (batch, o), np.float32)
        y1 = hip.download(ys_single[j], (batch, o), np.float32)
        assert np.isfinite(yg).all() and np.array_equal(yg, y1)
        rows = np.unique(np.concatenate([np.arange(5), np.arange(o - 5, o), np.arange(0, o, 211)]))
        sub = oracle.QuantizedWeight(qws[j].packed_primary[rows], qws[j].packed_residual[rows], qws[j].norms[rows], qws[j].seeds)
        assert _rel(yg[:, rows], xin @ oracle.dequantize_weight_cpu(sub, cb, cb, bs).T) < 1e-3
    hip.free(dx, *ys_group, *ys_single)
    for layer in layers:
        layer.close()


def _random_groups(n, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(n):
        inf = int(rng.choice([512, 1024, 2048, 2560, 3072, 4096, 5120, 6144, 8192, 12288, 17408]))
        bs = int(rng.choice([b for b in (128, 256, 512, 1024) if inf % b == 0]))
        k = int(rng.integers(1, 4))
        outs = tuple(int(rng.integers(1, max(2, min(1500, (2 << 20) // inf)))) for _ in range(k))
        cases.append((outs, inf, bs, bool(rng.integers(0, 2)), int(rng.choice([1, 1, 2, 4, 9, 15, 20]))))
    return cases


@pytest.mark.parametrize("outs,in_f,bs,shared,batch", _random_groups(40, 77))
def test_forward_group_random_configurations(tq, oracle, outs, in_f, bs, shared, batch):
    """tq_linear_forward_group on random layer sets and batch sizes: whichever way the call is served
    (shared launches or layer by layer), every output equals the one of a separate tq_linear_forward."""
    hip = _Hip()
    layers = [_layer(tq, oracle, o, in_f, bs, shared, seed=200 + j, fit=False)[0] for j, o in enumerate(outs)]
    xbits = oracle.f32_to_bf16_bits(np.random.default_rng(batch + in_f).standard_normal((batch, in_f)).astype(np.float32))
    dx = hip.upload(xbits)
    ys_group = [hip.alloc(batch * o * 4) for o in outs]
    ys_single = [hip.alloc(batch * o * 4) for o in outs]
    tq.forward_group_device(layers, dx, tq.BF16, batch, ys_group, tq.F32)
    for layer, yp in zip(layers, ys_single):
        layer.forward_device(dx, tq.BF16, batch, yp, tq.F32)
    for j, o in enumerate(outs):
        yg = hip.download(ys_group[j], (batch, o), np.float32)
        y1 = hip.download(ys_single[j], (batch, o), np.float32)
        assert np.isfinite(yg).all() and np.array_equal(yg, y1)
    hip.free(dx, *ys_group, *ys_single)
    for layer in layers:
        layer.close()
