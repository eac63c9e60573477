"""Parity at the full sizes of the benchmark configurations (4096 x 4096, the 151936 x 2048
lm_head, the 18944 x 3584 / 3584 x 18944 MLP block, the 27648 x 5120 up-projection at 512 and 2048
tokens, the 5120 x 27648 down projection at 4 and 8 rows and at 40, 512 and 2048 tokens).

A whole-matrix fp32 reference product is too slow for the CPU oracle at these sizes, so each case
is checked three ways:
  * the dequantised weight of the whole layer is compared bit for bit with the oracle's
    (one pass over the packed bytes: seconds with the oracle's OpenMP loop);
  * a random sample of output rows is recomputed by the oracle from the packed bytes of just
    those rows (rows are independent: own norm, own packed bytes) and compared with the same
    rows of the fused forward, within the tolerance of the activation type;
  * size-independent properties: scaling the input by 2 scales the fp32 output exactly
    (every operation of the path is linear and a factor 2 is exact in binary floating
    point), and a row of a batch equals the same vector sent alone.
Weights follow the benchmark recipe (N(0, sigma^2) with 1% Student-t(3) tails) and are quantized
by this library's GPU quantizer.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tq():
    import __graft_entry__ as entry
    pkg = entry.load_package()
    pkg.lib()
    return pkg


def _rel(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b.astype(np.float64)) / np.linalg.norm(b.astype(np.float64)))


def _weights(out_f, in_f, sigma, seed):
    rng = np.random.default_rng(seed)
    w = rng.standard_normal((out_f, in_f), dtype=np.float32) * np.float32(sigma)
    n_tail = out_f * in_f // 100
    idx = rng.integers(0, out_f * in_f, n_tail)
    t = rng.standard_t(3, n_tail).astype(np.float32) * np.float32(sigma)
    w.reshape(-1)[idx] = t
    return w


def _rows_subset(o, qw, rows):
    return o.QuantizedWeight(np.ascontiguousarray(qw.packed_primary[rows]), np.ascontiguousarray(qw.packed_residual[rows]),
                             np.ascontiguousarray(qw.norms[rows]), qw.seeds)


@pytest.mark.parametrize("shared", [True, False])
def test_bench_linear_shape_4096x4096_fp32(tq, oracle, shared):
    o = oracle
    out_f = in_f = 4096
    bs = 512
    cb = o.generate_codebook(4)
    w = _weights(out_f, in_f, 0.02, 11)
    qw = tq.quantize_weight(w, cb, cb, 4, 4, bs, shared)
    layer = tq.TurboQuantLinear(in_f, out_f, qw, cb, cb, bs)
    assert layer.mode() == ("shared_lut" if shared else "dual")

    o.set_threads(8)
    w_ref = o.dequantize_weight_cpu(qw, cb, cb, bs)
    o.set_threads(1)
    assert np.array_equal(layer.dequantize(), w_ref)                     # whole layer, bit-exact
    assert _rel(w_ref, w) < 0.15                                         # and it is the weight that went in (reference bound)

    x = np.random.default_rng(3).standard_normal((1, in_f)).astype(np.float32)
    y = layer.forward(x)
    want = o.matmul_xwT(x, w_ref, acc_double=True)                       # 16.8 M products: fine at this size
    assert _rel(y, want) < 1e-3
    assert np.array_equal(layer.forward(2.0 * x), 2.0 * y)               # exact linearity in a factor 2
    xb = np.concatenate([x, -x, 0.5 * x], axis=0)
    yb = layer.forward(xb)
    # (three rows take the small-batch kernel, fp16 operands: each row within the forward tolerance of the
    # one-row result, and the rows related exactly as their inputs are)
    assert _rel(yb[0:1], y) < 1e-3 and _rel(yb, np.concatenate([want, -want, 0.5 * want])) < 1e-3
    assert _rel(yb[1:2], -yb[0:1]) < 1e-6 and _rel(yb[2:3], 0.5 * yb[0:1]) < 1e-6
    layer.close()


def test_lm_head_151936x2048_bf16_activations(tq, oracle):
    o = oracle
    out_f, in_f, bs = 151936, 2048, 512
    w = _weights(out_f, in_f, 0.02, 21)
    cbp, cbr = tq.fit_layer_codebooks(w, bs)                             # per-layer Lloyd-Max, on the GPU
    qw = tq.quantize_weight(w, cbp, cbr, 4, 4, bs, True)
    del w
    layer = tq.TurboQuantLinear(in_f, out_f, qw, cbp, cbr, bs)

    o.set_threads(8)
    w_ref = o.dequantize_weight_cpu(qw, o.Codebook(cbp.centroids, 4), o.Codebook(cbr.centroids, 4), bs)
    o.set_threads(1)
    got = layer.dequantize()
    assert np.array_equal(got, w_ref)                                    # 311 M weights, bit-exact
    del got

    xbits = o.f32_to_bf16_bits(np.random.default_rng(5).standard_normal((1, in_f)).astype(np.float32))
    x = o.bf16_bits_to_f32(xbits)
    y = layer.forward(xbits, tq.BF16, tq.F32)
    assert y.shape == (1, out_f)
    rows = np.sort(np.random.default_rng(9).choice(out_f, 4096, replace=False))
    want = o.matmul_xwT(x, w_ref[rows], acc_double=True)
    assert _rel(y[:, rows], want) < 1e-3                                 # bf16 inputs are exact values; fp32 path
    # every logit, against the fp32 product of the bit-exact dequantised weight (numpy, float64 accumulate)
    full = (w_ref.astype(np.float64) @ x[0].astype(np.float64)).astype(np.float32)
    assert _rel(y[0], full) < 1e-3
    assert np.array_equal(layer.forward(o.f32_to_bf16_bits(2.0 * x), tq.BF16, tq.F32), 2.0 * y)
    layer.close()


def test_up_projection_27648x5120_prefill_512_tokens(tq, oracle):
    o = oracle
    out_f, in_f, bs, m = 27648, 5120, 512, 512
    cb = o.generate_codebook(4)
    w = _weights(out_f, in_f, 0.01, 31)
    qw = tq.quantize_weight(w, cb, cb, 4, 4, bs, True)
    del w
    layer = tq.TurboQuantLinear(in_f, out_f, qw, cb, cb, bs)
    xbits = o.f32_to_bf16_bits(np.random.default_rng(7).standard_normal((m, in_f)).astype(np.float32))
    x = o.bf16_bits_to_f32(xbits)
    y = o.bf16_bits_to_f32(layer.forward(xbits, tq.BF16, tq.BF16))       # M x 27648 bf16
    assert y.shape == (m, out_f)

    rows = np.sort(np.random.default_rng(13).choice(out_f, 256, replace=False))
    w_rows = o.dequantize_weight_cpu(_rows_subset(o, qw, rows), cb, cb, bs)
    want = o.matmul_xwT(x, w_rows, acc_double=True)                      # [512, 256]
    assert _rel(y[:, rows], want) < 5e-3                                 # fp16 tiles (3e-4) + bf16 rounding of the outputs (2^-9)
    # the batch-1 kernel (fp32 weights, fp32 accumulate) on three of the tokens
    for tkn in (0, 255, 511):
        y1 = layer.forward(xbits[tkn:tkn + 1], tq.BF16, tq.F32)
        assert _rel(y[tkn:tkn + 1], y1) < 5e-3
        assert _rel(y1[:, rows], want[tkn:tkn + 1]) < 1e-3
    layer.close()


class _Hip:
    """Device buffers through the HIP runtime the library is linked against (ctypes)."""

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


def _silu(g):
    g = g.astype(np.float32)
    return g / (np.float32(1.0) + np.exp(-g))


def _full_layer(tq, o, out_f, in_f, bs, sigma, seed, shared, per_layer=True):
    """Benchmark-recipe layer at full size: (layer, bit-exact checked fp32 weight of the oracle, qw, codebooks)."""
    w = _weights(out_f, in_f, sigma, seed)
    if per_layer:
        cbp, cbr = tq.fit_layer_codebooks(w, bs)
    else:
        cbp = cbr = tq.generate_codebook(4)
    qw = tq.quantize_weight(w, cbp, cbr, 4, 4, bs, shared)
    del w
    layer = tq.TurboQuantLinear(in_f, out_f, qw, cbp, cbr, bs)
    ocp, ocr = o.Codebook(cbp.centroids, 4), o.Codebook(cbr.centroids, 4)
    o.set_threads(8)
    w_ref = o.dequantize_weight_cpu(qw, ocp, ocr, bs)
    o.set_threads(1)
    got = layer.dequantize()
    assert np.array_equal(got, w_ref)                                    # whole layer, bit-exact
    return layer, w_ref, qw, ocp, ocr


@pytest.mark.parametrize("shared", [True, False], ids=["shared_rotation", "dual_rotation"])
def test_mlp_block_18944x3584_bf16_batch1(tq, oracle, shared):
    """The 7B-shaped decode MLP block: gate, up 18944 x 3584 and down 3584 x 18944, per-layer
    codebooks, bf16 activations, one row, SiLU gate in fp32 between the linears."""
    o = oracle
    hip = _Hip()
    hidden, inter, bs = 3584, 18944, 512
    gate, wg, qg, gcp, gcr = _full_layer(tq, o, inter, hidden, bs, 0.015, 41, shared)
    up, wu, qu, ucp, ucr = _full_layer(tq, o, inter, hidden, bs, 0.015, 42, shared)
    down, wd, qd, dcp, dcr = _full_layer(tq, o, hidden, inter, bs, 0.015, 43, shared)
    assert gate.mode() == ("shared_lut" if shared else "dual")

    xbits = o.f32_to_bf16_bits(np.random.default_rng(44).standard_normal((1, hidden)).astype(np.float32))
    x = o.bf16_bits_to_f32(xbits)
    # each linear on its own: sampled rows recomputed by the oracle from those rows' packed bytes, and every
    # output against the float64 product with the bit-exact dequantised weight
    rs = np.random.default_rng(45)
    yg = gate.forward(xbits, tq.BF16, tq.F32)
    yu = up.forward(xbits, tq.BF16, tq.F32)
    for y, w_ref, qw, cp, cr in ((yg, wg, qg, gcp, gcr), (yu, wu, qu, ucp, ucr)):
        rows = np.sort(rs.choice(inter, 512, replace=False))
        want = o.matmul_xwT(x, o.dequantize_weight_cpu(_rows_subset(o, qw, rows), cp, cr, bs), acc_double=True)
        assert _rel(y[:, rows], want) < 1e-3
        assert _rel(y[0], (w_ref.astype(np.float64) @ x[0].astype(np.float64)).astype(np.float32)) < 1e-3
    act = (_silu(yg) * yu).astype(np.float32)
    yd = down.forward(act, tq.F32, tq.F32)
    rows = np.sort(rs.choice(hidden, 512, replace=False))
    want = o.matmul_xwT(act, o.dequantize_weight_cpu(_rows_subset(o, qd, rows), dcp, dcr, bs), acc_double=True)
    assert _rel(yd[:, rows], want) < 1e-3

    # gate and up in one launch (width 3584): the same bits as two calls
    x_dev = hip.upload(xbits)
    g_dev, u_dev = hip.alloc(inter * 4), hip.alloc(inter * 4)
    tq.forward_group_device([gate, up], x_dev, tq.BF16, 1, [g_dev, u_dev], tq.F32)
    assert np.array_equal(hip.download(g_dev, (1, inter), np.float32), yg)
    assert np.array_equal(hip.download(u_dev, (1, inter), np.float32), yu)

    # the block
    mlp = tq.TurboQuantMLP(gate, up, down, max_batch=1)
    y_dev = hip.alloc(hidden * 4)
    for _ in range(2):
        mlp.forward_device(x_dev, tq.BF16, 1, y_dev, tq.F32)
        y = hip.download(y_dev, (1, hidden), np.float32)
    g64 = wg.astype(np.float64) @ x[0].astype(np.float64)
    u64 = wu.astype(np.float64) @ x[0].astype(np.float64)
    act64 = _silu(g64.astype(np.float32)) * u64.astype(np.float32)
    want = (wd.astype(np.float64) @ act64.astype(np.float64)).astype(np.float32)
    assert _rel(y[0], want) < 1e-3
    assert _rel(y[0, rows], o.matmul_xwT(act64[None, :].astype(np.float32),
                                         o.dequantize_weight_cpu(_rows_subset(o, qd, rows), dcp, dcr, bs),
                                         acc_double=True)[0]) < 1e-3
    mlp.close()
    hip.free(x_dev, g_dev, u_dev, y_dev)
    for l in (gate, up, down):
        l.close()


def test_up_projection_27648x5120_prefill_2048_tokens(tq, oracle):
    """2048 tokens: 8 x 108 tiles of 256 x 256 (3.4 rounds of the 256 CUs), the XCD-aware tile order."""
    o = oracle
    out_f, in_f, bs, m = 27648, 5120, 512, 2048
    cb = o.generate_codebook(4)
    w = _weights(out_f, in_f, 0.01, 31)
    qw = tq.quantize_weight(w, cb, cb, 4, 4, bs, True)
    del w
    layer = tq.TurboQuantLinear(in_f, out_f, qw, cb, cb, bs)
    xbits = o.f32_to_bf16_bits(np.random.default_rng(17).standard_normal((m, in_f)).astype(np.float32))
    x = o.bf16_bits_to_f32(xbits)
    y = o.bf16_bits_to_f32(layer.forward(xbits, tq.BF16, tq.BF16))       # 2048 x 27648 bf16
    assert y.shape == (m, out_f)
    assert np.isfinite(y).all()
    # sampled rows of the weight (every N tile is hit: 4 rows in each of the 108), all tokens
    rs = np.random.default_rng(19)
    rows = np.sort(np.concatenate([t * 256 + rs.choice(256, 4, replace=False) for t in range(out_f // 256)]))
    w_rows = o.dequantize_weight_cpu(_rows_subset(o, qw, rows), cb, cb, bs)
    o.set_threads(8)
    want = o.matmul_xwT(x, w_rows, acc_double=True)                      # [2048, 432]
    o.set_threads(1)
    assert _rel(y[:, rows], want) < 5e-3
    for t in range(m // 256):                                            # no M tile is off
        sl = slice(t * 256, (t + 1) * 256)
        assert _rel(y[sl][:, rows], want[sl]) < 5e-3
    for n0 in range(0, len(rows), 4):                                    # nor an N tile
        assert _rel(y[:, rows[n0:n0 + 4]], want[:, n0:n0 + 4]) < 5e-3
    # the same tokens at 512 give the same bits (a row's result does not depend on the batch it came in)
    y512 = o.bf16_bits_to_f32(layer.forward(xbits[1024:1536], tq.BF16, tq.BF16))
    assert np.array_equal(y512, y[1024:1536])
    layer.close()


@pytest.mark.parametrize("shared", [True, False], ids=["shared_rotation", "dual_rotation"])
@pytest.mark.parametrize("batch", [4, 8])
def test_down_projection_5120x27648_small_batch(tq, oracle, batch, shared):
    """32B-shaped down projection, 54 chunks of 512 columns, 4 and 8 rows of bf16 activations: the
    small-batch matrix-core path (fp16 weights and rotated activations, fp32 accumulation): 1e-3 with fp32
    outputs, 5e-3 where the outputs are rounded to bf16."""
    o = oracle
    out_f, in_f, bs = 5120, 27648, 512
    layer, w_ref, qw, cp, cr = _full_layer(tq, o, out_f, in_f, bs, 0.01, 51, shared)
    xbits = o.f32_to_bf16_bits(np.random.default_rng(52 + batch).standard_normal((batch, in_f)).astype(np.float32))
    x = o.bf16_bits_to_f32(xbits)
    y = layer.forward(xbits, tq.BF16, tq.F32)
    assert y.shape == (batch, out_f)
    want = (x.astype(np.float64) @ w_ref.astype(np.float64).T).astype(np.float32)
    assert _rel(y, want) < 1e-3
    for b in range(batch):
        assert _rel(y[b], want[b]) < 1e-3
    rows = np.sort(np.random.default_rng(53).choice(out_f, 256, replace=False))
    want_rows = o.matmul_xwT(x, o.dequantize_weight_cpu(_rows_subset(o, qw, rows), cp, cr, bs), acc_double=True)
    assert _rel(y[:, rows], want_rows) < 1e-3
    yb = o.bf16_bits_to_f32(layer.forward(xbits, tq.BF16, tq.BF16))
    assert _rel(yb, want) < 5e-3
    y1 = layer.forward(xbits[batch - 1:batch], tq.BF16, tq.F32)          # exact fp32 batch-1 kernel
    assert _rel(y1[0], want[batch - 1]) < 1e-3
    assert _rel(y[batch - 1:batch], y1) < 1e-3
    layer.close()


@pytest.mark.parametrize("shared", [True, False], ids=["shared_rotation", "dual_rotation"])
def test_down_projection_5120x27648_prefill_few_output_tiles(tq, oracle, shared):
    """32B-shaped down projection at 512 and 40 tokens: 2 x 20 (1 x 20) output tiles for 256 CUs, so K is cut
    into 6 (12) ranges of 144 (72) steps whose fp32 products a second kernel adds.  All tokens against
    sampled rows of the oracle's weight, every output tile hit; 2048 tokens (160 tiles, one range) on a
    token slice for comparison."""
    o = oracle
    out_f, in_f, bs = 5120, 27648, 512
    layer, w_ref, qw, cp, cr = _full_layer(tq, o, out_f, in_f, bs, 0.01, 61, shared)
    rs = np.random.default_rng(62)
    rows = np.sort(np.concatenate([t * 256 + rs.choice(256, 6, replace=False) for t in range(out_f // 256)]))
    w_rows = np.ascontiguousarray(w_ref[rows])
    del w_ref
    xbits = o.f32_to_bf16_bits(rs.standard_normal((2048, in_f)).astype(np.float32))
    x = o.bf16_bits_to_f32(xbits)
    o.set_threads(8)
    want = o.matmul_xwT(x, w_rows, acc_double=True)                      # [2048, 120]
    o.set_threads(1)
    for m in (512, 40, 2048):
        y = layer.forward(xbits[:m], tq.BF16, tq.F32)
        assert y.shape == (m, out_f) and np.isfinite(y).all()
        assert _rel(y[:, rows], want[:m]) < 1e-3
        for n0 in range(0, len(rows), 6):                                # no output tile is off
            assert _rel(y[:, rows[n0:n0 + 6]], want[:m, n0:n0 + 6]) < 1e-3
        for t0 in range(0, m, 256):                                      # nor a token tile
            assert _rel(y[t0:t0 + 256][:, rows], want[t0:min(t0 + 256, m)]) < 1e-3
    yb = o.bf16_bits_to_f32(layer.forward(xbits[:512], tq.BF16, tq.BF16))
    assert _rel(yb[:, rows], want[:512]) < 5e-3
    layer.close()


@pytest.mark.parametrize("shared", [True, False], ids=["shared_rotation", "dual_rotation"])
def test_decoder_layer_projections_32b_batch_1_4_8(tq, oracle, shared):
    """The 32B-shaped decoder layer as the benchmark launches it: q + k + v (5120 + 1024 + 1024 rows) and
    gate + up (2 x 27648 rows) through tq_linear_forward_group, o alone, at 1, 4 and 8 rows of bf16
    activations.  The host-computed row partition of a shared launch depends on every layer's row count, so
    the full row counts are what is run: sampled rows of every layer against the oracle (recomputed from the
    packed bytes of just those rows), first and last rows included, the grouped results equal bit for bit to
    one call per layer, and q, o, k, v alone as well."""
    o = oracle
    hip = _Hip()
    hidden, kv, inter, bs = 5120, 1024, 27648, 512
    cb = o.generate_codebook(4)
    shapes = {"q": hidden, "k": kv, "v": kv, "o": hidden, "gate": inter, "up": inter}
    layers, qws = {}, {}
    for i, (name, rows) in enumerate(shapes.items()):
        w = _weights(rows, hidden, 0.01, 70 + i)
        qws[name] = tq.quantize_weight(w, cb, cb, 4, 4, bs, shared)
        del w
        layers[name] = tq.TurboQuantLinear(hidden, rows, qws[name], cb, cb, bs)
        assert layers[name].mode() == ("shared_lut" if shared else "dual")
    rs = np.random.default_rng(77)
    samples, w_rows = {}, {}
    o.set_threads(8)
    for name, rows in shapes.items():
        pick = np.unique(np.concatenate([[0, 1, rows - 2, rows - 1], rs.choice(rows, 300, replace=False)]))
        samples[name] = pick
        w_rows[name] = o.dequantize_weight_cpu(_rows_subset(o, qws[name], pick), cb, cb, bs)
    o.set_threads(1)
    xbits = o.f32_to_bf16_bits(rs.standard_normal((8, hidden)).astype(np.float32))
    x = o.bf16_bits_to_f32(xbits)
    for batch in (1, 4, 8):
        x_dev = hip.upload(xbits[:batch])
        want = {name: o.matmul_xwT(x[:batch], w_rows[name], acc_double=True) for name in shapes}
        alone = {name: layers[name].forward(xbits[:batch], tq.BF16, tq.F32) for name in shapes}
        for name in shapes:                                              # every layer by itself
            assert alone[name].shape == (batch, shapes[name]) and np.isfinite(alone[name]).all()
            assert _rel(alone[name][:, samples[name]], want[name]) < 1e-3
            for b in range(batch):
                assert _rel(alone[name][b, samples[name]], want[name][b]) < 1e-3
        for group in (("q", "k", "v"), ("gate", "up")):                  # the shared launches of the benchmark
            outs = [hip.alloc(batch * shapes[n] * 4) for n in group]
            tq.forward_group_device([layers[n] for n in group], x_dev, tq.BF16, batch, outs, tq.F32)
            for n, ptr in zip(group, outs):
                y = hip.download(ptr, (batch, shapes[n]), np.float32)
                assert np.array_equal(y, alone[n])                       # same bits as one call per layer
                assert _rel(y[:, samples[n]], want[n]) < 1e-3
            hip.free(*outs)
        hip.free(x_dev)
    for l in layers.values():
        l.close()
