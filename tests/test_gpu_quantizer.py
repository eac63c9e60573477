"""GPU quantizer (tq_quantize_weight, tq_fit_layer_codebooks) against the CPU oracle.  Every fp32 step
follows the reference's order, so packed planes, seeds and norms are expected bit-identical; the only
freedom is the order of the double-precision row sums (rounded once to float)."""
import numpy as np
import pytest

import __graft_entry__ as entry

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tq():
    return entry.load_package()


CONFIGS = [dict(pb=4, rb=4, shared=True), dict(pb=4, rb=4, shared=False), dict(pb=4, rb=0, shared=False),
           dict(pb=4, rb=3, shared=True), dict(pb=5, rb=3, shared=True), dict(pb=5, rb=3, shared=False),
           # no residual pass but shared_rotation set: seeds[1] stays the derived seed (src/quantizer.cpp:255-256)
           dict(pb=4, rb=0, shared=True)]


@pytest.mark.parametrize("cfg", CONFIGS, ids=["shared", "dual", "primary", "4+3", "5+3s", "5+3d", "primary-shared-flag"])
@pytest.mark.parametrize("out,inf,bs", [(64, 128, 128), (16, 512, 256), (24, 384, 128), (16, 896, 128),
                                        (33, 2048, 512), (7, 5120, 512), (9, 64, 32), (40, 4096, 1024)])
def test_quantize_weight_matches_oracle(tq, oracle, cfg, out, inf, bs):
    w = oracle.lcg_matrix(out, inf, 42) if out * inf <= 1 << 16 else \
        (np.random.default_rng(3).standard_normal((out, inf)) * 0.02).astype(np.float32)
    w[out // 2] *= 0.0 if out > 8 else 1.0                     # a zero row must not produce NaN
    ocp, ocr = oracle.generate_codebook(cfg["pb"]), oracle.generate_codebook(cfg["rb"] if cfg["rb"] else 4)
    want = oracle.quantize_weight(w, ocp, ocr, cfg["pb"], cfg["rb"], bs, cfg["shared"])
    cp, cr = tq.generate_codebook(cfg["pb"]), tq.generate_codebook(cfg["rb"] if cfg["rb"] else 4)
    assert np.array_equal(cp.centroids, ocp.centroids) and np.array_equal(cp.boundaries, ocp.boundaries)
    got = tq.quantize_weight(w, cp, cr, cfg["pb"], cfg["rb"], bs, cfg["shared"])
    assert np.array_equal(got.seeds, want.seeds)
    assert (got.seeds[1] == 0) == (cfg["shared"] and cfg["rb"] > 0)
    assert got.packed_primary.shape == want.packed_primary.shape
    assert np.array_equal(got.packed_primary, want.packed_primary)
    assert np.array_equal(got.packed_residual, want.packed_residual)
    assert np.isfinite(got.norms).all()
    assert np.array_equal(got.norms, want.norms)


@pytest.mark.parametrize("cfg", CONFIGS, ids=["shared", "dual", "primary", "4+3", "5+3s", "5+3d", "primary-shared-flag"])
@pytest.mark.parametrize("out,inf,bs", [(7, 100, 4), (5, 36, 4), (6, 64, 1), (9, 48, 16), (3, 10, 2), (4, 24, 8),
                                        (11, 4112, 16), (2, 6, 1)])
def test_quantize_weight_any_width_the_reference_takes(tq, oracle, cfg, out, inf, bs):
    """The reference quantises every width that is a multiple of its block (src/quantizer.cpp:41-79; the block
    rule of src/converter.cpp:228-240 gives a width of 100 blocks of 4 columns): widths that are not a multiple
    of 32 and blocks of one column run on the small-block kernel, bit-identical to the oracle like the rest, and
    the result loads and dequantises."""
    w = oracle.lcg_matrix(out, inf, 17)
    if out > 4:
        w[1] *= 0.0                                                # a zero row must not produce NaN
    ocp, ocr = oracle.generate_codebook(cfg["pb"]), oracle.generate_codebook(cfg["rb"] if cfg["rb"] else 4)
    want = oracle.quantize_weight(w, ocp, ocr, cfg["pb"], cfg["rb"], bs, cfg["shared"])
    cp, cr = tq.generate_codebook(cfg["pb"]), tq.generate_codebook(cfg["rb"] if cfg["rb"] else 4)
    got = tq.quantize_weight(w, cp, cr, cfg["pb"], cfg["rb"], bs, cfg["shared"])
    assert np.array_equal(got.seeds, want.seeds)
    assert np.array_equal(got.packed_primary, want.packed_primary)
    assert np.array_equal(got.packed_residual, want.packed_residual)
    assert np.isfinite(got.norms).all() and np.array_equal(got.norms, want.norms)
    assert np.array_equal(tq.dequantize_weight_gpu(got, cp, cr, bs), oracle.dequantize_weight_cpu(want, ocp, ocr, bs))


def test_fit_layer_codebooks_on_a_narrow_layer(tq, oracle):
    """The per-layer recipe on a width of 100 (blocks of 4 columns): same samples, same fit as the oracle."""
    rng = np.random.default_rng(2)
    w = (rng.standard_normal((64, 100)) * 0.02).astype(np.float32)
    want_p, want_r = oracle.fit_layer_codebooks(w, 4)
    got_p, got_r = tq.fit_layer_codebooks(w, 4)
    assert np.abs(got_p.centroids - want_p.centroids).max() < 1e-6
    assert np.abs(got_r.centroids - want_r.centroids).max() < 1e-6


def test_fit_layer_codebooks_matches_oracle(tq, oracle):
    rng = np.random.default_rng(1)
    w = (rng.standard_normal((96, 1024)) * 0.02).astype(np.float32)
    tails = rng.random(w.shape) < 0.01
    w[tails] = (0.02 * rng.standard_t(3, size=int(tails.sum()))).astype(np.float32)
    want_p, want_r = oracle.fit_layer_codebooks(w, 512)
    got_p, got_r = tq.fit_layer_codebooks(w, 512)
    # same binning, double sums in a different (fixed) order: equal to the last float bit or two
    assert np.abs(got_p.centroids - want_p.centroids).max() < 1e-6
    assert np.abs(got_r.centroids - want_r.centroids).max() < 1e-6
    qw = tq.quantize_weight(w, got_p, got_r, 4, 4, 512, True)
    W = tq.dequantize_weight_gpu(qw, got_p, got_r, 512)
    rel = np.sqrt(((W - w) ** 2).mean() / (w ** 2).mean())
    assert rel < 0.05


def test_quantizer_error_conventions(tq):
    with pytest.raises(ValueError):
        tq.generate_codebook(6)
    cb = tq.generate_codebook(4)
    with pytest.raises(ValueError):
        tq.quantize_weight(np.zeros((4, 96), np.float32), cb, cb, 4, 4, 64, True)      # 96 % 64 != 0
    assert tq.best_block_size(896) == 128 and tq.best_block_size(27648) == 512 and tq.best_block_size(4864) == 256
