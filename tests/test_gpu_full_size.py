"""Parity at the full sizes of the benchmark configurations (4096 x 4096, the 151936 x 2048
lm_head, the 27648 x 5120 up-projection at 512 tokens).

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
    assert _rel(yb[0:1], y) < 1e-6 and _rel(yb[1:2], -y) < 1e-6 and _rel(yb[2:3], 0.5 * y) < 1e-6
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
    assert _rel(y[:, rows], want) < 7e-3                                 # bf16 tiles + bf16 rounding of the outputs
    # the batch-1 kernel (fp32 weights, fp32 accumulate) on three of the tokens
    for tkn in (0, 255, 511):
        y1 = layer.forward(xbits[tkn:tkn + 1], tq.BF16, tq.F32)
        assert _rel(y[tkn:tkn + 1], y1) < 7e-3
        assert _rel(y1[:, rows], want[tkn:tkn + 1]) < 1e-3
    layer.close()
