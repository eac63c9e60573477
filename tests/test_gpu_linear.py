"""GPU parity tests of the HIP TQ8 linear path against the CPU oracle, through the C-ABI
(ctypes).  Tolerances: rotation and dequantised weights bit-exact (the kernels keep the
reference's fp32 operation order); layer outputs within 1e-3 relative L2 for fp32
activations and 5e-3 for bf16/f16 activations."""
import numpy as np
import pytest

import __graft_entry__ as entry

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tq():
    return entry.load_package()


def _rel(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b.astype(np.float64)) / max(np.linalg.norm(b.astype(np.float64)), 1e-30))


# ---------------------------------------------------------------- rotation
@pytest.mark.parametrize("rows,cols,bs", [(1, 512, 512), (1, 384, 128), (4, 896, 128), (2, 4864, 256),
                                          (3, 256, 64), (2, 64, 32), (5, 2048, 512), (3, 5120, 512),
                                          (2, 4096, 1024), (2, 4096, 2048), (2, 96, 16), (3, 64, 2),
                                          (2, 27648, 512)])
def test_rotation_bit_exact(tq, oracle, rows, cols, bs):
    rng = np.random.default_rng(rows * 1000 + cols + bs)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    for seed in (42, 0xCAFEBABE):
        assert np.array_equal(tq.apply_wht_rotation(x, seed, bs), oracle.wht_forward(x, seed, bs))
        assert np.array_equal(tq.apply_inverse_wht_rotation(x, seed, bs), oracle.wht_inverse(x, seed, bs))
    rt = tq.apply_inverse_wht_rotation(tq.apply_wht_rotation(x, 42, bs), 42, bs)
    assert np.abs(rt - x).max() < 1e-4                      # tests/unit/test_rotation.cpp:17-34


def test_rotation_rejects_non_divisible(tq):
    with pytest.raises(ValueError):
        tq.apply_wht_rotation(np.zeros((1, 96), np.float32), 1, 64)


# ------------------------------------------------------------- dequantiser
MODES = {
    "shared": dict(pb=4, rb=4, shared=True),
    "dual": dict(pb=4, rb=4, shared=False),
    "primary_only": dict(pb=4, rb=0, shared=False),
    "shared_3bit_res": dict(pb=4, rb=3, shared=True),
    "5+3shared": dict(pb=5, rb=3, shared=True),
    "5+3dual": dict(pb=5, rb=3, shared=False),
    "5+0": dict(pb=5, rb=0, shared=False),
}
SHAPES = [(64, 128, 128), (32, 128, 128), (16, 512, 256), (24, 384, 128), (16, 256, 256), (16, 896, 128),
          (7, 2048, 512), (5, 4096, 512), (3, 5120, 512), (2, 18944, 512), (9, 64, 32), (4, 64, 16)]


def _make(oracle, out, inf, bs, mode, seed=42, fitted=False):
    m = MODES[mode]
    w = oracle.lcg_matrix(out, inf, seed) if out * inf <= 1 << 16 else \
        np.random.default_rng(seed).standard_normal((out, inf)).astype(np.float32) * 0.02
    cbp = oracle.generate_codebook(m["pb"])
    cbr = oracle.generate_codebook(m["rb"] if m["rb"] else 4)
    if fitted:
        cbp, cbr = oracle.fit_layer_codebooks(w, bs, m["pb"], m["rb"])
    qw = oracle.quantize_weight(w, cbp, cbr, m["pb"], m["rb"], bs, m["shared"])
    return qw, cbp, cbr


@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("out,inf,bs", SHAPES)
def test_dequantize_bit_exact(tq, oracle, mode, out, inf, bs):
    qw, cbp, cbr = _make(oracle, out, inf, bs, mode)
    got = tq.dequantize_weight_gpu(qw, cbp, cbr, bs)
    want = oracle.dequantize_weight_cpu(qw, cbp, cbr, bs)
    assert got.dtype == np.float32 and got.shape == (out, inf)
    assert np.array_equal(got, want)


def test_dequantize_fitted_codebooks_and_index_clamp(tq, oracle):
    qw, cbp, cbr = _make(oracle, 48, 1024, 512, "shared", fitted=True)
    assert np.array_equal(tq.dequantize_weight_gpu(qw, cbp, cbr, 512), oracle.dequantize_weight_cpu(qw, cbp, cbr, 512))
    # 3-bit codebooks with 4-bit index planes: dual path clamps, LUT path zero-fills (src/dequantizer.cpp:94,144-150)
    cb3 = oracle.generate_codebook(3)
    rng = np.random.default_rng(0)
    for seeds1 in (0, 1234):
        q = oracle.QuantizedWeight(rng.integers(0, 256, (8, 256), dtype=np.uint8), rng.integers(0, 256, (8, 256), dtype=np.uint8),
                                   rng.random(8, dtype=np.float32) + 0.5, np.array([99, seeds1, 128], np.uint32))
        assert np.array_equal(tq.dequantize_weight_gpu(q, cb3, cb3, 128), oracle.dequantize_weight_cpu(q, cb3, cb3, 128))


def test_oversized_primary_codebook_on_nibble_planes(tq, oracle):
    """32 primary centroids under 4-bit planes, shared rotation: the reference's table loop wraps the index
    at 8 bits (src/dequantizer.cpp:144-150), so odd residual indices select centroids 16..31.  Dequantised
    weights equal the oracle's bit for bit and every forward path uses the same table."""
    cb5, cb4 = oracle.generate_codebook(5), oracle.generate_codebook(4)
    rng = np.random.default_rng(4)
    out, inf, bs = 40, 1024, 256
    q = oracle.QuantizedWeight(rng.integers(0, 256, (out, inf // 2), dtype=np.uint8),
                               rng.integers(0, 256, (out, inf // 2), dtype=np.uint8),
                               rng.random(out, dtype=np.float32) + 0.5, np.array([99, 0, bs], np.uint32))
    want = oracle.dequantize_weight_cpu(q, cb5, cb4, bs)
    capped = oracle.dequantize_weight_cpu(q, oracle.Codebook(cb5.centroids[:16], 4), cb4, bs)
    assert not np.array_equal(want, capped)                              # the wrap matters on this input
    assert np.array_equal(tq.dequantize_weight_gpu(q, cb5, cb4, bs), want)
    layer = tq.TurboQuantLinear(inf, out, q, cb5, cb4, bs)
    for batch, xd in ((1, "f32"), (3, "f32"), (6, "bf16"), (40, "bf16")):
        x32 = rng.standard_normal((batch, inf)).astype(np.float32)
        if xd == "bf16":
            xbits = oracle.f32_to_bf16_bits(x32)
            y = layer.forward(xbits, tq.BF16, tq.F32)
            ref = oracle.matmul_xwT(oracle.bf16_bits_to_f32(xbits), want, acc_double=True)
        else:
            y = layer.forward(x32, tq.F32, tq.F32)
            ref = oracle.matmul_xwT(x32, want, acc_double=True)
        assert _rel(y, ref) < (1e-3 if xd == "f32" else 5e-3), (batch, xd)
    layer.close()


# ------------------------------------------------------------------ forward
@pytest.mark.parametrize("mode", ["shared", "dual", "primary_only", "shared_3bit_res"])
@pytest.mark.parametrize("out,inf,bs", [(64, 128, 128), (32, 128, 128), (16, 512, 256), (24, 384, 128), (16, 896, 128),
                                        (37, 2048, 512), (130, 4096, 512), (33, 5120, 512), (21, 3584, 512),
                                        (9, 18944, 512), (5, 27648, 512), (9, 64, 32), (6, 64, 16)])
@pytest.mark.parametrize("batch", [1, 2, 3, 4, 8])
def test_forward_fp32(tq, oracle, mode, out, inf, bs, batch):
    qw, cbp, cbr = _make(oracle, out, inf, bs, mode)
    x = np.random.default_rng(batch).standard_normal((batch, inf)).astype(np.float32)
    layer = tq.TurboQuantLinear(inf, out, qw, cbp, cbr, bs)
    assert layer.in_features() == inf and layer.out_features() == out
    y = layer.forward(x)
    layer.close()
    assert y.shape == (batch, out) and y.dtype == np.float32
    want = oracle.linear_forward(qw, cbp, cbr, bs, x)
    assert _rel(y, want) < 1e-3
    assert np.abs(y - want).max() < 0.15                     # the reference's own bound, test_linear.cpp:135


@pytest.mark.parametrize("mode", ["shared", "primary_only", "dual"])
@pytest.mark.parametrize("out,inf,bs", [(1000, 3072, 512), (777, 5120, 512), (5000, 5120, 128), (600, 6144, 512),
                                        (515, 7168, 256), (300, 8192, 512), (64, 9216, 512), (260, 15360, 512),
                                        (130, 16384, 512), (3, 5120, 512), (2049, 12288, 64)])
def test_forward_batch1_wide_rows(tq, oracle, mode, out, inf, bs):
    """One activation row on rows of 3 to 8 slabs (and, shared rotation, of an odd number of
    1024-column halves, which are served two rows at a time; dual rotation with the waves
    of a row split by plane): the one-workgroup-per-CU kernel.
    Row counts are chosen so that streams get ragged, empty and single-row ranges; fp32 and bf16
    activations; every output against the oracle within the fp32 tolerance."""
    qw, cbp, cbr = _make(oracle, out, inf, bs, mode)
    layer = tq.TurboQuantLinear(inf, out, qw, cbp, cbr, bs)
    x = np.random.default_rng(out + inf).standard_normal((1, inf)).astype(np.float32)
    want = oracle.linear_forward(qw, cbp, cbr, bs, x)
    y = layer.forward(x)
    assert y.shape == (1, out) and _rel(y, want) < 1e-3
    assert np.array_equal(layer.forward(2.0 * x), 2.0 * y)                 # exact linearity in a factor 2
    xbits = oracle.f32_to_bf16_bits(x)
    xb = oracle.bf16_bits_to_f32(xbits)
    yb = layer.forward(xbits, tq.BF16, tq.F32)
    assert _rel(yb, oracle.linear_forward(qw, cbp, cbr, bs, xb)) < 1e-3
    # three rows of fp32 activations: the small-batch kernels (fp16 operands on the matrix cores where the
    # width is a multiple of 512, else the fp32 kernels two rows at a time): each row agrees with the one-row
    # kernel to the forward tolerance, and the rows with each other as their inputs do (factors -1 and 0.5
    # are exact in fp16 and in fp32).
    x3 = np.concatenate([x, -x, 0.5 * x], axis=0)
    y3 = layer.forward(x3)
    assert _rel(y3[0:1], y) < 1e-3 and _rel(y3, oracle.linear_forward(qw, cbp, cbr, bs, x3)) < 1e-3
    assert _rel(y3[1:2], -y3[0:1]) < 1e-6 and _rel(y3[2:3], 0.5 * y3[0:1]) < 1e-6
    layer.close()


@pytest.mark.parametrize("mode", ["shared", "primary_only", "dual"])
@pytest.mark.parametrize("out,inf,bs", [(20001, 2048, 512), (16500, 1024, 256), (33003, 1536, 512), (4099, 2048, 128)])
def test_forward_batch1_one_slab_rows(tq, oracle, mode, out, inf, bs):
    """One activation row on rows of one slab (at most 2048 columns) with enough rows for groups of
    two rows per wave: shared rotation and primary only hand the row groups of a workgroup to its
    waves from a counter in LDS, dual rotation splits the waves by plane.  Row counts leave ragged
    last groups and workgroups of unequal ranges; fp32 and bf16 activations against the oracle."""
    qw, cbp, cbr = _make(oracle, out, inf, bs, mode)
    layer = tq.TurboQuantLinear(inf, out, qw, cbp, cbr, bs)
    x = np.random.default_rng(out + inf).standard_normal((1, inf)).astype(np.float32)
    want = oracle.linear_forward(qw, cbp, cbr, bs, x)
    y = layer.forward(x)
    assert y.shape == (1, out) and _rel(y, want) < 1e-3
    assert np.abs(y - want).max() < 1e-2 * np.abs(want).max()             # no row left out or taken twice
    assert np.array_equal(layer.forward(2.0 * x), 2.0 * y)
    assert np.array_equal(layer.forward(x), y)                             # same result on every call
    xbits = oracle.f32_to_bf16_bits(x)
    yb = layer.forward(xbits, tq.BF16, tq.F32)
    assert _rel(yb, oracle.linear_forward(qw, cbp, cbr, bs, oracle.bf16_bits_to_f32(xbits))) < 1e-3
    layer.close()


@pytest.mark.parametrize("mode", ["primary_only", "dual"])
def test_forward_batch1_centroids_outside_fp16_range(tq, oracle, mode):
    """Codebooks whose values do not fit fp16 (1e5 times the usual ones): the one-row kernel must not
    use its fp16 centroid pairs for such a layer.  Same packed indices, scaled codebooks: the output is
    the scaled output, finite, and within the fp32 tolerance of the oracle."""
    out, inf, bs = 300, 4096, 512
    qw, cbp, cbr = _make(oracle, out, inf, bs, mode)
    big_p = oracle.Codebook(cbp.centroids * np.float32(1e5), cbp.bits)
    big_r = oracle.Codebook(cbr.centroids * np.float32(1e5), cbr.bits)
    x = np.random.default_rng(3).standard_normal((1, inf)).astype(np.float32)
    layer = tq.TurboQuantLinear(inf, out, qw, big_p, big_r, bs)
    y = layer.forward(x)
    layer.close()
    want = oracle.linear_forward(qw, big_p, big_r, bs, x)
    assert np.isfinite(y).all() and _rel(y, want) < 1e-3


@pytest.mark.parametrize("mode", ["shared", "primary_only", "dual"])
@pytest.mark.parametrize("out,inf,bs", [(600, 27648, 512), (515, 18944, 256), (257, 17408, 512), (40, 20480, 2048)])
def test_forward_batch1_rows_beyond_16384_columns(tq, oracle, mode, out, inf, bs):
    """One activation row on rows of 9 to 14 slabs: the row is rotated once by a kernel of its own
    (blocks of at most 512 columns; larger blocks are rotated inside the product kernel) and every
    workgroup picks the result up.  fp32, bf16 and f16 activations, ragged row ranges, every output
    against the oracle within the fp32 tolerance; two calls in a row on one handle reuse the scratch."""
    qw, cbp, cbr = _make(oracle, out, inf, bs, mode)
    layer = tq.TurboQuantLinear(inf, out, qw, cbp, cbr, bs)
    x = np.random.default_rng(out + inf).standard_normal((1, inf)).astype(np.float32)
    want = oracle.linear_forward(qw, cbp, cbr, bs, x)
    y = layer.forward(x)
    assert y.shape == (1, out) and _rel(y, want) < 1e-3
    assert np.array_equal(layer.forward(2.0 * x), 2.0 * y)                 # exact linearity in a factor 2
    xbits = oracle.f32_to_bf16_bits(x)
    yb = layer.forward(xbits, tq.BF16, tq.F32)
    assert _rel(yb, oracle.linear_forward(qw, cbp, cbr, bs, oracle.bf16_bits_to_f32(xbits))) < 1e-3
    xh = x.astype(np.float16)
    yh = layer.forward(xh, tq.F16, tq.F32)
    assert _rel(yh, oracle.linear_forward(qw, cbp, cbr, bs, xh.astype(np.float32))) < 1e-3
    assert np.array_equal(layer.forward(x), y)                             # the scratch holds nothing stale
    x3 = np.concatenate([x, -x, 0.5 * x], axis=0)                          # three rows: the small-batch kernels
    y3 = layer.forward(x3)
    assert _rel(y3[0:1], y) < 1e-3 and _rel(y3, oracle.linear_forward(qw, cbp, cbr, bs, x3)) < 1e-3
    assert _rel(y3[1:2], -y3[0:1]) < 1e-6 and _rel(y3[2:3], 0.5 * y3[0:1]) < 1e-6
    layer.close()


@pytest.mark.parametrize("mode", ["shared", "dual", "primary_only"])
@pytest.mark.parametrize("xd", ["bf16", "f16"])
@pytest.mark.parametrize("yd", ["f32", "bf16", "f16"])
def test_forward_half_activations(tq, oracle, mode, xd, yd):
    out, inf, bs, batch = 96, 2048, 512, 3
    qw, cbp, cbr = _make(oracle, out, inf, bs, mode)
    x32 = np.random.default_rng(5).standard_normal((batch, inf)).astype(np.float32)
    if xd == "bf16":
        xbits = oracle.f32_to_bf16_bits(x32); xin = oracle.bf16_bits_to_f32(xbits); xarg, xcode = xbits, tq.BF16
    else:
        xarg = x32.astype(np.float16); xin = xarg.astype(np.float32); xcode = tq.F16
    ycode = {"f32": tq.F32, "bf16": tq.BF16, "f16": tq.F16}[yd]
    layer = tq.TurboQuantLinear(inf, out, qw, cbp, cbr, bs)
    y = layer.forward(xarg, xcode, ycode)
    layer.close()
    if yd == "bf16":
        y = oracle.bf16_bits_to_f32(y)
    y = y.astype(np.float32)
    want = oracle.linear_forward(qw, cbp, cbr, bs, xin)
    # three rows run on the matrix cores with fp16 weights and rotated activations (about 3e-4); a bf16
    # output adds its own rounding (2^-9 relative)
    assert _rel(y, want) < (5e-3 if yd == "bf16" else 1e-3)


def test_forward_fitted_codebooks_match_dequant_matmul(tq, oracle):
    qw, cbp, cbr = _make(oracle, 200, 2048, 512, "shared", fitted=True)
    x = np.random.default_rng(1).standard_normal((1, 2048)).astype(np.float32)
    y = tq.fused_dequant_matmul(qw, cbp, cbr, 512, x)
    assert _rel(y, oracle.linear_forward(qw, cbp, cbr, 512, x)) < 1e-3


def test_error_conventions(tq, oracle):
    L = tq.lib()
    assert L.tq_linear_in_features(None) == 0 and L.tq_linear_out_features(None) == 0
    L.tq_linear_free(None)                                   # no-op
    assert L.tq_linear_forward(None, None, 0, 1, None, 0, None) != 0
    qw, cbp, cbr = _make(oracle, 8, 128, 128, "shared")
    with pytest.raises(ValueError):
        tq.TurboQuantLinear(256, 8, qw, cbp, cbr, 128)       # shape mismatch
    with pytest.raises(ValueError):
        tq.TurboQuantLinear(128, 8, qw, cbp, cbr, 96)        # block size does not divide
    with pytest.raises(ValueError):
        tq.TurboQuantLinear(128, 8, qw, cbp, cbr, 4096)      # block wider than the row
    layer = tq.TurboQuantLinear(128, 8, qw, cbp, cbr, 128)
    with pytest.raises(RuntimeError):
        layer.forward_device(None, tq.F32, 1, None, tq.F32)
    layer.close()


# ------------------------------------------------------------------ prefill
@pytest.mark.parametrize("mode", ["shared", "dual", "primary_only"])
@pytest.mark.parametrize("out,inf,bs,batch", [(64, 128, 128, 16), (300, 512, 256, 37), (513, 2048, 512, 64),
                                              (256, 5120, 512, 300), (1000, 896 * 2, 128, 17),
                                              # K = 64, 192, 256, 384: 2, 6, 8, 12 steps of the 6-step pipeline
                                              (70, 64, 64, 16), (40, 192, 64, 20), (33, 256, 256, 300),
                                              (257, 384, 128, 513),
                                              # few output tiles: K is cut into ranges (5 of 32 steps; 34 + 34 + 32; 7 x 34 + 20)
                                              (256, 5120, 512, 40), (130, 3200, 128, 40), (90, 8256, 64, 130)])
def test_prefill_bf16_matches_dequant_matmul(tq, oracle, mode, out, inf, bs, batch):
    """batch >= 16 takes the MFMA path whatever the activation type (fp16 weight tiles, fp16 rotated
    activations, fp32 accumulation): 1e-3 relative L2 against dequantise + fp32 matmul, 5e-3 where the
    output itself is rounded to bf16."""
    qw, cbp, cbr = _make(oracle, out, inf, bs, mode)
    x32 = np.random.default_rng(batch).standard_normal((batch, inf)).astype(np.float32)
    xbits = oracle.f32_to_bf16_bits(x32)
    want = oracle.linear_forward(qw, cbp, cbr, bs, oracle.bf16_bits_to_f32(xbits))
    layer = tq.TurboQuantLinear(inf, out, qw, cbp, cbr, bs)
    y = layer.forward(xbits, tq.BF16, tq.F32)
    yb = oracle.bf16_bits_to_f32(layer.forward(xbits, tq.BF16, tq.BF16))
    y16 = layer.forward(x32.astype(np.float16), tq.F16, tq.F32)
    y32 = layer.forward(x32)
    layer.close()
    assert y.shape == (batch, out)
    assert _rel(y, want) < 1e-3
    assert _rel(yb, want) < 5e-3                      # includes the bf16 rounding of the outputs
    assert _rel(y16, oracle.linear_forward(qw, cbp, cbr, bs, x32.astype(np.float16).astype(np.float32))) < 1e-3
    assert _rel(y32, oracle.linear_forward(qw, cbp, cbr, bs, x32)) < 1e-3      # fp32 activations take the same path
    # every row of the batch must agree with the batch-1 kernel on the same row
    layer = tq.TurboQuantLinear(inf, out, qw, cbp, cbr, bs)
    y1 = layer.forward(xbits[3:4], tq.BF16, tq.F32)
    layer.close()
    assert _rel(y[3:4], y1) < 1e-3


# ------------------------------------------------------------------ prefill, 512-row activation panels
@pytest.mark.parametrize("mode", ["shared", "dual", "primary_only"])
@pytest.mark.parametrize("out,inf,bs,batch", [(16500, 256, 256, 257),      # one ragged panel, ragged last weight tile
                                              (16500, 512, 256, 33),       # one row block per wave, one token in wave 0's
                                              (16640, 256, 128, 128),      # one whole row block per wave
                                              (16500, 2048, 512, 100),     # ... and two wave groups that halve the row (widths that are multiples of 512)
                                              (16500, 512, 512, 129),      # two row blocks per wave
                                              (16640, 768, 256, 256),
                                              (16500, 256, 64, 300),       # three row blocks per wave
                                              (16640, 512, 128, 600),      # two panels, the second with 88 rows
                                              (33000, 768, 256, 1030),     # three panels
                                              (8300, 1024, 512, 1537)])    # four panels, 65 tiles each
def test_prefill_panel_kernel_matches_dequant_matmul(tq, oracle, mode, out, inf, bs, batch):
    """More than 32 rows on a layer with enough 512 x 128 output tiles for the chip and a width that is a
    multiple of 256 take tq_prefill_panel_kernel (activations as MFMA-operand images read straight from
    global memory, 128 x 128 accumulators per wave; up to 384 rows the kernel instances that multiply one,
    two or three of a wave's four row blocks): same tolerances as the other prefill kernel, every
    output dtype, and a row of the batch equal to its batch-1 result."""
    qw, cb = _packed_layer(oracle, out, inf, bs, mode, out + inf + batch)
    x32 = np.random.default_rng(batch).standard_normal((batch, inf)).astype(np.float32)
    xbits = oracle.f32_to_bf16_bits(x32)
    want = oracle.linear_forward(qw, cb, cb, bs, oracle.bf16_bits_to_f32(xbits))
    layer = tq.TurboQuantLinear(inf, out, qw, cb, cb, bs)
    y = layer.forward(xbits, tq.BF16, tq.F32)
    assert y.shape == (batch, out) and np.isfinite(y).all()
    assert _rel(y, want) < 1e-3
    for b in sorted({0, 31, 32, 127, 128, 255, 256, batch - 1} & set(range(batch))):      # no row leaks into another
        assert _rel(y[b:b + 1], want[b:b + 1]) < 1e-3
    for c in (0, 127, 128, out - 1):                         # nor a column
        assert _rel(y[:, c:c + 1], want[:, c:c + 1]) < 1e-3
    yb = oracle.bf16_bits_to_f32(layer.forward(xbits, tq.BF16, tq.BF16))
    assert _rel(yb, want) < 5e-3                             # includes the bf16 rounding of the outputs
    yh = layer.forward(xbits, tq.BF16, tq.F16).astype(np.float32)
    assert _rel(yh, want) < 1e-3
    y32 = layer.forward(x32)                                 # fp32 activations take the same path
    assert _rel(y32, oracle.linear_forward(qw, cb, cb, bs, x32)) < 1e-3
    y1 = layer.forward(xbits[batch - 1:batch], tq.BF16, tq.F32)
    assert _rel(y[batch - 1:batch], y1) < 1e-3
    layer.close()


@pytest.mark.parametrize("mode", ["shared", "dual", "primary_only"])
@pytest.mark.parametrize("out,inf,bs,batch,ydt", [(8448, 2048, 512, 2000, "f32"),    # 4 x 66 tiles: 8 left after one round of 256
                                                  (8400, 2304, 256, 1600, "bf16"),   # ragged last tile, 144 sub-steps in parts of 32 (the last one 16)
                                                  (16500, 2048, 128, 1025, "f16"),   # 3 x 129 tiles: 131 left after one round -> 1 part, whole
                                                  (33000, 2048, 256, 200, "bf16")])  # 258 tiles of two row blocks per wave, the last 2 cut
def test_prefill_panel_kernel_tail_tiles_in_k_ranges(tq, oracle, mode, out, inf, bs, batch, ydt):
    """Tiles left over after the last full round of the chip are cut into K ranges (dual rotation: one part per
    plane and range) where that is cheaper by the library's count of rounds; a second kernel adds their fp32 products:
    sampled rows of every panel against the oracle, in particular rows of the last panel, whose last tiles are
    the ones that are cut."""
    qw, cb = _packed_layer(oracle, out, inf, bs, mode, out + inf + batch)
    x32 = np.random.default_rng(batch).standard_normal((batch, inf)).astype(np.float32)
    xbits = oracle.f32_to_bf16_bits(x32)
    last = (batch - 1) // 512 * 512
    rows = sorted(r for r in {0, 511, 512, last - 1, last, last + 1, (last + batch) // 2, batch - 2, batch - 1} if r < batch)
    want = oracle.linear_forward(qw, cb, cb, bs, oracle.bf16_bits_to_f32(xbits[rows]))
    layer = tq.TurboQuantLinear(inf, out, qw, cb, cb, bs)
    code = {"f32": tq.F32, "bf16": tq.BF16, "f16": tq.F16}[ydt]
    y = layer.forward(xbits, tq.BF16, code)
    y = oracle.bf16_bits_to_f32(y) if ydt == "bf16" else y.astype(np.float32)
    assert y.shape == (batch, out) and np.isfinite(y).all()
    tol = 5e-3 if ydt == "bf16" else 1e-3
    assert _rel(y[rows], want) < tol
    for k, r in enumerate(rows):
        assert _rel(y[r:r + 1], want[k:k + 1]) < tol
    for c0 in range(0, out, 128):                            # every tile of weights, cut or whole
        assert _rel(y[rows][:, c0:c0 + 128], want[:, c0:c0 + 128]) < tol
    y1 = layer.forward(xbits[batch - 1:batch], tq.BF16, tq.F32)
    assert _rel(y[batch - 1:batch], y1) < tol
    layer.close()


@pytest.mark.parametrize("mode", ["shared", "dual", "primary_only"])
@pytest.mark.parametrize("out,inf,bs,batch,ydt", [(5100, 8192, 256, 2048, "f32"),   # 160 tiles, each in 3 ranges: two rounds of parts
                                                  (4400, 9216, 128, 2048, "f16"),   # 140 tiles, 576 sub-steps in 3 ranges, ragged last tile
                                                  (5000, 8192, 512, 1600, "bf16"),  # 160 tiles, the last panel 64 rows
                                                  (1280, 8192, 512, 100, "bf16"),   # 10 tiles of long rows, up to 128 tokens: 8 ranges each
                                                  (2000, 9216, 128, 40, "f32")])    # 16 tiles, ragged last one, one row block per wave
def test_prefill_panel_kernel_less_than_a_round_all_tiles_cut_along_k(tq, oracle, mode, out, inf, bs, batch, ydt):
    """Calls with fewer 512 x 128 tiles than the chip has CUs (more than half as many, or, up to 128 tokens of rows
    of 8192 columns and more, any number) and long rows: every tile is cut into K ranges (dual rotation: one part per plane and range, here two ranges) so that the parts
    fill the chip; more parts than CUs run in rounds, and the sum kernel adds them.  Sampled rows of every panel
    against the oracle."""
    qw, cb = _packed_layer(oracle, out, inf, bs, mode, out + inf + batch)
    x32 = np.random.default_rng(batch).standard_normal((batch, inf)).astype(np.float32)
    xbits = oracle.f32_to_bf16_bits(x32)
    last = (batch - 1) // 512 * 512
    rows = sorted(r for r in {0, 127, 128, 255, 256, 511, 512, last, (last + batch) // 2, batch - 1} if 0 <= r < batch)
    want = oracle.linear_forward(qw, cb, cb, bs, oracle.bf16_bits_to_f32(xbits[rows]))
    layer = tq.TurboQuantLinear(inf, out, qw, cb, cb, bs)
    code = {"f32": tq.F32, "bf16": tq.BF16, "f16": tq.F16}[ydt]
    y = layer.forward(xbits, tq.BF16, code)
    y = oracle.bf16_bits_to_f32(y) if ydt == "bf16" else y.astype(np.float32)
    assert y.shape == (batch, out) and np.isfinite(y).all()
    tol = 5e-3 if ydt == "bf16" else 1e-3
    assert _rel(y[rows], want) < tol
    for k, r in enumerate(rows):
        assert _rel(y[r:r + 1], want[k:k + 1]) < tol
    for c0 in range(0, out, 128):                            # every tile of weights
        assert _rel(y[rows][:, c0:c0 + 128], want[:, c0:c0 + 128]) < tol
    y1 = layer.forward(xbits[batch - 1:batch], tq.BF16, tq.F32)
    assert _rel(y[batch - 1:batch], y1) < tol
    y2 = layer.forward(xbits, tq.BF16, code)                 # the parts are added in a fixed order
    y2 = oracle.bf16_bits_to_f32(y2) if ydt == "bf16" else y2.astype(np.float32)
    assert np.array_equal(y, y2)
    layer.close()


# ------------------------------------------------------------------ small batches on the matrix cores
@pytest.mark.parametrize("mode", ["shared", "dual", "primary_only"])
@pytest.mark.parametrize("out,inf,bs,batch", [(64, 512, 512, 2), (300, 1024, 256, 5), (513, 2048, 512, 15),
                                              (1000, 5120, 512, 8), (16, 512, 64, 3), (47, 1536, 128, 9),
                                              # 17..32 rows: a second set of 16 batch rows on the same decoded weights
                                              (513, 2048, 512, 16), (300, 1024, 256, 17), (1000, 5120, 512, 32),
                                              (64, 512, 512, 25), (257, 2048, 1024, 31), (90, 1536, 512, 20),
                                              # widths that do not fill their last 512-column chunk (5.5, 2.625, 0.875,
                                              # 21.5, 1.75 and 0.375 chunks), the last two with two sets of rows
                                              (130, 2816, 256, 5), (77, 1344, 64, 3), (64, 448, 64, 9),
                                              (200, 11008, 256, 4), (90, 896, 128, 20), (33, 192, 64, 31)])
def test_small_batch_mfma_path_matches_oracle_and_batch1(tq, oracle, mode, out, inf, bs, batch):
    """2..32 rows on a layer whose width is a multiple of 64 (nibble planes: of 128) take the
    small-batch MFMA kernels (fp16 weights and rotated activations, fp32 accumulation over
    512-column chunks; for dual rotation one pass per plane, each with its own rotation):
    1e-3 relative L2 (5e-3 with a bf16 output), ragged row counts, every row equal to its batch-1 result."""
    qw, cbp, cbr = _make(oracle, out, inf, bs, mode)
    x32 = np.random.default_rng(100 + batch).standard_normal((batch, inf)).astype(np.float32)
    xbits = oracle.f32_to_bf16_bits(x32)
    want = oracle.linear_forward(qw, cbp, cbr, bs, oracle.bf16_bits_to_f32(xbits))
    layer = tq.TurboQuantLinear(inf, out, qw, cbp, cbr, bs)
    y = layer.forward(xbits, tq.BF16, tq.F32)
    assert y.shape == (batch, out)
    assert _rel(y, want) < 1e-3
    for b in range(batch):                                   # no row leaks into another
        assert _rel(y[b:b + 1], want[b:b + 1]) < 1e-3
    yb = oracle.bf16_bits_to_f32(layer.forward(xbits, tq.BF16, tq.BF16))
    assert _rel(yb, want) < 5e-3
    x16 = x32.astype(np.float16)
    y16 = layer.forward(x16, tq.F16, tq.F32)
    assert _rel(y16, oracle.linear_forward(qw, cbp, cbr, bs, x16.astype(np.float32))) < 1e-3
    y1 = layer.forward(xbits[batch - 1:batch], tq.BF16, tq.F32)      # exact fp32 batch-1 kernel
    assert _rel(y[batch - 1:batch], y1) < 1e-3
    # fp32 activations take the same kernels
    yf = layer.forward(x32)
    assert _rel(yf, oracle.linear_forward(qw, cbp, cbr, bs, x32)) < 1e-3
    layer.close()


# ------------------------------------------------------------------ two to twelve rows, whole weight rows per stream
@pytest.mark.parametrize("out,inf,bs,batch", [
    # the workgroups rotate the activation rows themselves: 2..7 segments of 256 columns per wave, one wave per row
    # quad (no cross-wave sum) or several
    (64, 256, 64, 2), (70, 1536, 512, 3), (64, 768, 256, 4), (66, 2048, 512, 2), (61, 1024, 64, 3),
    (64, 2560, 512, 4), (63, 1280, 256, 2), (65, 4352, 256, 3), (64, 3328, 256, 4), (67, 1792, 256, 2), (64, 4608, 512, 2),
    # fewer rows than a quad, ragged quads, widths that are not a multiple of a segment, many streams per workgroup
    (3, 1024, 64, 4), (1281, 5120, 512, 3), (6913, 5120, 512, 4), (130, 2816, 256, 4), (77, 1344, 64, 2),
    (3000, 2848, 32, 3), (16500, 2304, 256, 4),
    # four to six tiles of the rotation per wave
    (6000, 11520, 256, 2), (10000, 6400, 256, 4), (10000, 6656, 512, 4),
    # rows that come rotated from a kernel of their own: wider than 16384 columns (the layer's scratch row), or
    # images that do not fit LDS (a workspace)
    (4096, 17408, 512, 3), (3500, 24576, 512, 4), (2600, 27648, 512, 4), (2600, 32768, 512, 2), (5000, 14336, 512, 4),
    # five to eight rows: two sets of four on the same decoded weights, planes of 96 MB and more
    (19701, 5120, 512, 8), (12300, 8192, 256, 5), (6200, 16384, 512, 7), (66000, 1536, 512, 6), (49500, 2048, 128, 8),
    (197000, 512, 64, 6),
    # nine to twelve rows: three sets, two segments per wave, rows of eight waves and more
    (12300, 8192, 512, 9), (25000, 4096, 256, 12), (12400, 8192, 128, 11), (13200, 7680, 256, 10)])
def test_two_to_twelve_rows_whole_row_kernel(tq, oracle, out, inf, bs, batch):
    _whole_row_kernel_case(tq, oracle, "shared", out, inf, bs, batch)


@pytest.mark.parametrize("mode,out,inf,bs,batch", [
    # nibble planes of 96 MB and more: dual rotation (primary segments, then residual ones; two to four units of 512
    # columns per wave), five to eight rows where the row's units fill 14 waves and more, and primary only
    ("dual", 19701, 5120, 512, 4), ("dual", 12300, 8192, 256, 3), ("dual", 12300, 8192, 512, 7), ("dual", 33000, 3072, 128, 2),
    ("dual", 6200, 16384, 512, 4), ("dual", 25000, 4096, 512, 8), ("dual", 9000, 11264, 256, 3),
    ("primary_only", 39400, 5120, 512, 4), ("primary_only", 50000, 4096, 256, 6)])
def test_two_to_twelve_rows_whole_row_kernel_nibble_planes(tq, oracle, mode, out, inf, bs, batch):
    _whole_row_kernel_case(tq, oracle, mode, out, inf, bs, batch)


def _whole_row_kernel_case(tq, oracle, mode, out, inf, bs, batch):
    """2..12 rows (nibble planes: 2..8): the kernel that reads whole weight rows per stream (four weight rows by
    four activation rows per v_mfma_f32_4x4x4_16b_f16 block, fp16 weights and rotated activations, fp32 sums, the
    cross-wave sum inside the workgroup).  1e-3 relative L2 against the oracle for every activation type (5e-3 with a
    bf16 output), every activation row by itself, every row equal to its batch-1 result within the same bound, and
    the same bits on a second call.  Planes of more than 40 MB: a sample of the weight rows (the first and last
    quads, every 61st row) against the oracle, all of them for finiteness."""
    qw, cb = _packed_layer(oracle, out, inf, bs, mode, out + inf + batch)
    x32 = np.random.default_rng(batch + inf).standard_normal((batch, inf)).astype(np.float32)
    xbits = oracle.f32_to_bf16_bits(x32)
    rows = np.arange(out) if out * inf <= 40 << 20 else \
        np.unique(np.concatenate([np.arange(9), np.arange(out - 9, out), np.arange(0, out, 61)]))
    sub = oracle.QuantizedWeight(qw.packed_primary[rows], qw.packed_residual[rows], qw.norms[rows], qw.seeds)
    w = oracle.dequantize_weight_cpu(sub, cb, cb, bs)
    want = oracle.matmul_xwT(oracle.bf16_bits_to_f32(xbits), w, True)
    layer = tq.TurboQuantLinear(inf, out, qw, cb, cb, bs)
    y_all = layer.forward(xbits, tq.BF16, tq.F32)
    assert y_all.shape == (batch, out) and np.isfinite(y_all).all()
    y = y_all[:, rows]
    assert _rel(y, want) < 1e-3
    for b in range(batch):                                   # no activation row leaks into another
        assert _rel(y[b:b + 1], want[b:b + 1]) < 1e-3
    for c0 in range(0, len(rows), max(1, len(rows) // 7)):   # nor a weight row into another
        assert _rel(y[:, c0:c0 + 3], want[:, c0:c0 + 3]) < 2e-3
    assert np.array_equal(y_all, layer.forward(xbits, tq.BF16, tq.F32))
    yb = oracle.bf16_bits_to_f32(layer.forward(xbits, tq.BF16, tq.BF16))
    assert _rel(yb[:, rows], want) < 5e-3
    y1 = layer.forward(xbits[batch - 1:batch], tq.BF16, tq.F32)      # exact fp32 batch-1 kernel
    assert _rel(y_all[batch - 1:batch], y1) < 1e-3
    x16 = x32.astype(np.float16)
    assert _rel(layer.forward(x16, tq.F16, tq.F32)[:, rows], oracle.matmul_xwT(x16.astype(np.float32), w, True)) < 1e-3
    assert _rel(layer.forward(x32)[:, rows], oracle.matmul_xwT(x32, w, True)) < 1e-3
    layer.close()


@pytest.mark.parametrize("mode", ["shared", "dual"])
@pytest.mark.parametrize("batch", [2, 4, 16, 40, 64])
@pytest.mark.parametrize("scale", [1e-4, 1e3, 1e4])
def test_matrix_core_paths_hold_their_tolerance_over_the_fp16_range(tq, oracle, mode, batch, scale):
    """The matrix-core paths (2 rows and more) round the rotated activations, normalised by 1 / sqrt(block), to
    fp16.  Activations of 1e-4 .. 1e4 times a standard normal stay inside fp16's normal range after the rotation
    (a rotated value is bounded by the L2 norm of its block of the input), so the outputs keep 1e-3 against the
    oracle for fp32 and bf16 activations alike and agree with the exact fp32 batch-1 kernel on the same row.
    (Below about 1e-5 the rotated values become fp16 subnormals, beyond 65504 they saturate: the reference
    casts its input itself to f16, src/dequantizer.cpp:691, and has the same limits.)"""
    out, inf, bs = 300, 2048, 512
    qw, cbp, cbr = _make(oracle, out, inf, bs, mode)
    x32 = (np.random.default_rng(batch).standard_normal((batch, inf)) * scale).astype(np.float32)
    layer = tq.TurboQuantLinear(inf, out, qw, cbp, cbr, bs)
    want = oracle.linear_forward(qw, cbp, cbr, bs, x32)
    y = layer.forward(x32)
    assert np.isfinite(y).all() and _rel(y, want) < 1e-3
    for b in range(batch):
        assert _rel(y[b:b + 1], want[b:b + 1]) < 1e-3
    xbits = oracle.f32_to_bf16_bits(x32)
    yb = layer.forward(xbits, tq.BF16, tq.F32)
    assert _rel(yb, oracle.linear_forward(qw, cbp, cbr, bs, oracle.bf16_bits_to_f32(xbits))) < 1e-3
    y1 = layer.forward(x32[batch - 1:batch])                  # one row: the fp32 kernel
    assert _rel(y[batch - 1:batch], y1) < 1e-3
    layer.close()


def _random_cases(n, seed):
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < n:
        inf = int(rng.choice([64, 96, 128, 384, 512, 1024, 1536, 2048, 2560, 3072, 3584, 4096, 5120, 6144, 7168, 8192,
                              9216, 11264, 13312, 16384, 17408, 18944, 24576, 27648, 32768]))
        divisors = [b for b in (16, 32, 64, 128, 256, 512, 1024, 2048) if inf % b == 0]
        bs = int(rng.choice(divisors))
        out = int(rng.integers(1, max(2, min(3000, (6 << 20) // inf))))
        mode = str(rng.choice(["shared", "dual", "primary_only"]))
        batch = int(rng.choice([1, 1, 1, 2, 3, 5, 8, 15, 16, 17, 33]))
        xd = str(rng.choice(["f32", "bf16", "f16"]))
        cases.append((out, inf, bs, mode, batch, xd))
    return cases


@pytest.mark.parametrize("out,inf,bs,mode,batch,xd", _random_cases(160, 20240611))
def test_forward_random_configurations(tq, oracle, out, inf, bs, mode, batch, xd):
    """Whatever kernel a call is routed to (one-workgroup-per-CU, pre-rotated, narrow, small-batch or
    prefill): the output agrees with the oracle's dense product on the same quantised weights within
    1e-3, also where fp16 weights are used (2+ rows of 16-bit activations, 16+ rows of any type)."""
    qw, cbp, cbr = _make(oracle, out, inf, bs, mode, seed=out + inf)
    x32 = np.random.default_rng(out * 7 + batch).standard_normal((batch, inf)).astype(np.float32)
    if xd == "bf16":
        xarg = oracle.f32_to_bf16_bits(x32); xin = oracle.bf16_bits_to_f32(xarg); code = tq.BF16
    elif xd == "f16":
        xarg = x32.astype(np.float16); xin = xarg.astype(np.float32); code = tq.F16
    else:
        xarg, xin, code = x32, x32, tq.F32
    layer = tq.TurboQuantLinear(inf, out, qw, cbp, cbr, bs)
    y = layer.forward(xarg, code, tq.F32)
    layer.close()
    want = oracle.linear_forward(qw, cbp, cbr, bs, xin)
    assert y.shape == (batch, out) and np.isfinite(y).all()
    assert _rel(y, want) < 1e-3


# ------------------------------------------------------------------ every shape the reference accepts
def _packed_layer(o, out, inf, bs, mode, seed):
    """Random packed planes (no quantizer involved: the oracle's dequantiser defines the layer)."""
    rng = np.random.default_rng(seed)
    cb = o.generate_codebook(4)
    pp = rng.integers(0, 256, size=(out, inf // 2)).astype(np.uint8)
    pr = rng.integers(0, 256, size=(out, inf // 2)).astype(np.uint8)
    if mode == "primary_only":
        pr[:] = 0
    norms = (rng.random(out) + 0.5).astype(np.float32)
    seeds = np.array([rng.integers(1, 2 ** 32), 0 if mode == "shared" else rng.integers(1, 2 ** 32), bs], np.uint32)
    return o.QuantizedWeight(pp, pr, norms, seeds), cb


@pytest.mark.parametrize("mode", ["shared", "dual", "primary_only"])
@pytest.mark.parametrize("out,inf,bs", [(5, 48, 16), (9, 24, 8), (7, 6, 2), (3, 80, 16), (4, 36, 4), (6, 64, 1),
                                        (2, 10, 1), (5, 96, 32), (3, 34816, 512), (2, 53248, 512), (3, 36864, 2048)])
def test_shapes_beyond_the_tuned_kernels(tq, oracle, mode, out, inf, bs):
    """The reference only requires in % block_size == 0 (src/rotation.cpp:374,396): widths that are not a
    multiple of 32 (blocks of 1 to 16 columns) and rows wider than 32768 columns load, dequantise bit-exactly,
    rotate bit-exactly and run forward."""
    qw, cb = _packed_layer(oracle, out, inf, bs, mode, out * 1000 + inf + bs)
    w_ref = oracle.dequantize_weight_cpu(qw, cb, cb, bs)
    layer = tq.TurboQuantLinear(inf, out, qw, cb, cb, bs)
    assert np.array_equal(layer.dequantize(), w_ref)
    for batch in (1, 3):
        x = np.random.default_rng(batch).standard_normal((batch, inf)).astype(np.float32)
        y = layer.forward(x)
        assert y.shape == (batch, out)
        assert _rel(y, oracle.matmul_xwT(x, w_ref, acc_double=True)) < 1e-3
        xb = oracle.f32_to_bf16_bits(x)
        yb = layer.forward(xb, tq.BF16, tq.F32)
        assert _rel(yb, oracle.matmul_xwT(oracle.bf16_bits_to_f32(xb), w_ref, acc_double=True)) < 5e-3
    layer.close()
    x = np.random.default_rng(9).standard_normal((2, inf)).astype(np.float32)
    assert np.array_equal(tq.apply_wht_rotation(x, 77, bs), oracle.wht_forward(x, 77, bs))
    assert np.array_equal(tq.apply_inverse_wht_rotation(x, 77, bs), oracle.wht_inverse(x, 77, bs))


# ------------------------------------------------------------------ many rows of one slab
@pytest.mark.parametrize("mode", ["shared", "dual", "primary_only"])
@pytest.mark.parametrize("out,inf,bs", [(70001, 512, 512), (66000, 2048, 256), (131074, 1024, 128)])
def test_one_slab_layers_with_many_rows(tq, oracle, mode, out, inf, bs):
    """Rows of one slab (the waves of a CU take their row groups from a counter in LDS) on layers of 65536
    rows and more, odd row counts included: every output against the float64 product with the oracle's
    weight (no row missing, doubled or misplaced), and the same bits on every call."""
    qw, cb = _packed_layer(oracle, out, inf, bs, mode, out + inf)
    oracle.set_threads(8)
    w_ref = oracle.dequantize_weight_cpu(qw, cb, cb, bs)
    oracle.set_threads(1)
    layer = tq.TurboQuantLinear(inf, out, qw, cb, cb, bs)
    x = np.random.default_rng(1).standard_normal((1, inf)).astype(np.float32)
    want = (w_ref.astype(np.float64) @ x[0].astype(np.float64)).astype(np.float32)
    ys = [layer.forward(x) for _ in range(3)]
    assert _rel(ys[0][0], want) < 1e-3
    assert np.abs(ys[0][0] - want).max() < 1e-3 * np.abs(want).max()
    for y in ys[1:]:
        assert np.array_equal(y, ys[0])
    xb = oracle.f32_to_bf16_bits(x)
    yb = layer.forward(xb, tq.BF16, tq.F32)
    wantb = (w_ref.astype(np.float64) @ oracle.bf16_bits_to_f32(xb)[0].astype(np.float64)).astype(np.float32)
    assert _rel(yb[0], wantb) < 1e-3
    layer.close()
