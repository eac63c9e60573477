"""Pins the CPU oracle (oracle/tq_oracle.c) without running the reference:
closed forms, textbook routines (scipy Hadamard, numpy searchsorted, scipy normal
moments), published FNV-1a vectors, brute force in float64, and the property
thresholds the reference's own tests assert (tests/unit/test_rotation.cpp,
test_codebook.cpp, test_quantizer.cpp, test_lut_dequant.cpp)."""
import math

import numpy as np
import pytest
import scipy.linalg
import scipy.stats


# ---------------------------------------------------------------- sign hash
def _sign_bigint(seed, i):
    M = (1 << 32) - 1
    h = (seed * 2654435761 + i * 2246822519) & M
    h ^= h >> 16
    h = (h * 0x45D9F3B) & M
    h ^= h >> 16
    return 1.0 if (h & 1) else -1.0


def test_sign_hash_u32_wraparound_and_values(oracle):
    # arbitrary-precision evaluation masks explicitly where C wraps implicitly
    for seed in (0, 1, 42, 99, 0xCAFEBABE, 0xFFFFFFFF, 2166136261):
        for i in list(range(0, 70)) + [511, 1023, 65535]:
            assert oracle.sign(seed, i) == _sign_bigint(seed, i)
    s = oracle.make_signs(42, 512)
    assert set(np.unique(s)) == {-1.0, 1.0}
    assert 180 < (s > 0).sum() < 332          # roughly balanced
    assert not np.array_equal(s, oracle.make_signs(99, 512))


# -------------------------------------------------------------------- FWHT
@pytest.mark.parametrize("n", [2, 4, 32, 128, 512])
def test_fwht_is_sylvester_hadamard(oracle, n):
    rng = np.random.default_rng(n)
    v = rng.integers(-8, 9, size=n).astype(np.float32)      # exact in fp32
    H = scipy.linalg.hadamard(n).astype(np.float64)
    assert np.array_equal(oracle.fwht(v).astype(np.float64), H @ v.astype(np.float64))
    assert np.array_equal(oracle.fwht(oracle.fwht(v)), v * n)


@pytest.mark.parametrize("rows,cols,bs", [(1, 512, 512), (1, 384, 128), (4, 896, 128),
                                          (2, 4864, 256), (3, 256, 64), (2, 64, 32)])
def test_block_rotation_matches_dense_orthonormal_matrix(oracle, rows, cols, bs):
    rng = np.random.default_rng(7)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    seed = 42
    s = np.array([_sign_bigint(seed, j) for j in range(bs)])
    H = scipy.linalg.hadamard(bs).astype(np.float64)
    fwd = (H @ np.diag(s)) / math.sqrt(bs)       # sign first, then H, then 1/sqrt
    inv = (np.diag(s) @ H) / math.sqrt(bs)       # H first, then sign
    assert np.allclose(fwd @ fwd.T, np.eye(bs), atol=1e-12)
    assert np.allclose(inv, fwd.T)
    want_f = np.concatenate([x[:, b:b + bs].astype(np.float64) @ fwd.T for b in range(0, cols, bs)], axis=1)
    want_i = np.concatenate([x[:, b:b + bs].astype(np.float64) @ inv.T for b in range(0, cols, bs)], axis=1)
    rot = oracle.wht_forward(x, seed, bs)
    assert np.abs(rot - want_f).max() < 2e-5
    assert np.abs(oracle.wht_inverse(x, seed, bs) - want_i).max() < 2e-5
    # tests/unit/test_rotation.cpp:17-48: round trip < 1e-4, norm ratio 1 +- 1e-3
    assert np.abs(oracle.wht_inverse(rot, seed, bs) - x).max() < 1e-4
    assert abs(np.linalg.norm(rot) / np.linalg.norm(x) - 1) < 1e-3
    assert np.array_equal(rot, oracle.wht_forward(x, seed, bs))
    assert not np.array_equal(rot, oracle.wht_forward(x, 99, bs))


def test_rotation_rejects_non_divisible(oracle):
    with pytest.raises(ValueError):
        oracle.wht_forward(np.zeros((1, 100), np.float32), 1, 64)


# --------------------------------------------------------------- codebooks
def test_codebook_tables(oracle):
    cb1 = oracle.generate_codebook(1)
    assert abs(cb1.centroids[1] - math.sqrt(2 / math.pi)) < 1e-5      # test_codebook.cpp:8-16
    assert abs(cb1.centroids[0] + math.sqrt(2 / math.pi)) < 1e-5
    cb2 = oracle.generate_codebook(2)
    assert np.allclose(cb2.centroids, [-1.510232, -0.45278, 0.45278, 1.510232], atol=1e-5)
    for bits in (1, 2, 3, 4, 5):
        cb = oracle.generate_codebook(bits)
        assert len(cb.centroids) == 1 << bits and len(cb.boundaries) == (1 << bits) - 1
        assert np.all(np.diff(cb.centroids) > 0)
        assert np.array_equal(cb.centroids, -cb.centroids[::-1])       # bit-exact symmetry
        assert np.array_equal(cb.boundaries, (cb.centroids[:-1] + cb.centroids[1:]) * np.float32(0.5))
        assert oracle.validate_codebook(cb)
    with pytest.raises(ValueError):
        oracle.generate_codebook(6)
    with pytest.raises(ValueError):
        oracle.generate_codebook(0)


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5])
def test_codebook_is_lloyd_max_fixed_point_of_standard_normal(oracle, bits):
    # each centroid must be E[z | bin] for N(0,1) with midpoint boundaries
    cb = oracle.generate_codebook(bits)
    edges = np.concatenate([[-np.inf], cb.boundaries.astype(np.float64), [np.inf]])
    pdf, cdf = scipy.stats.norm.pdf, scipy.stats.norm.cdf
    cond_mean = (pdf(edges[:-1]) - pdf(edges[1:])) / (cdf(edges[1:]) - cdf(edges[:-1]))
    assert np.abs(cond_mean - cb.centroids).max() < 2e-3


def test_validate_codebook_rejects_bad(oracle):
    cb = oracle.generate_codebook(4)
    bad = oracle.Codebook(cb.centroids.copy(), 4, analytical=True)
    bad.centroids[3] = bad.centroids[5]           # unsorted
    assert not oracle.validate_codebook(bad)
    skew = oracle.Codebook(cb.centroids + np.float32(0.01), 4, analytical=True)
    assert not oracle.validate_codebook(skew)     # analytical must be symmetric
    skew.analytical = False
    assert oracle.validate_codebook(skew)
    # boundaries must be the midpoints to 1e-5 (src/codebook.cpp:337-340): 1e-4 off fails, 5e-6 off passes
    off = oracle.Codebook(cb.centroids.copy(), 4, analytical=True)
    off.boundaries = off.boundaries.copy()
    off.boundaries[7] += np.float32(1e-4)
    assert not oracle.validate_codebook(off)
    near = oracle.Codebook(cb.centroids.copy(), 4, analytical=True)
    near.boundaries = near.boundaries.copy()
    near.boundaries[3] = np.float32(near.boundaries[3] + np.float32(5e-6))
    assert abs(float(near.boundaries[3]) - float((cb.centroids[3] + cb.centroids[4]) * np.float32(0.5))) < 1e-5
    assert oracle.validate_codebook(near)
    short = oracle.Codebook(cb.centroids.copy(), 4, analytical=True)
    short.boundaries = short.boundaries[:-1].copy()            # one boundary missing
    assert not oracle.validate_codebook(short)


def test_quantize_is_lower_bound(oracle):
    cb = oracle.generate_codebook(4)
    rng = np.random.default_rng(3)
    v = np.concatenate([rng.standard_normal(5000).astype(np.float32) * 2, cb.boundaries, cb.centroids,
                        np.array([-100, 100, 0], np.float32)])
    idx = oracle.quantize(v, cb)
    want = np.minimum(np.searchsorted(cb.boundaries, v, side="left"), 15)
    assert np.array_equal(idx, want.astype(np.uint8))
    # a value equal to a boundary goes to the lower bin
    assert np.array_equal(oracle.quantize(cb.boundaries, cb), np.arange(15, dtype=np.uint8))
    # centroid round trip (test_codebook.cpp:62-82)
    assert np.array_equal(oracle.dequantize(oracle.quantize(cb.centroids, cb), cb), cb.centroids)
    # index clamp
    assert oracle.dequantize(np.array([200], np.uint8), cb)[0] == cb.centroids[15]


def test_nibble_packing_all_bytes(oracle):
    allb = np.arange(256, dtype=np.uint8)
    idx = oracle.unpack4(allb)
    assert np.array_equal(idx[0::2], allb & 0x0F)      # lo nibble = even column
    assert np.array_equal(idx[1::2], allb >> 4)        # hi nibble = odd column
    assert np.array_equal(oracle.pack4(idx), allb)
    assert oracle.pack4(np.array([0xB, 0xA], np.uint8))[0] == 0xAB


# ------------------------------------------------------------------- seed
def _fnv1a(data: bytes, basis=0x811C9DC5):
    h = basis
    for b in data:
        h ^= b
        h = (h * 16777619) & 0xFFFFFFFF
    return h


def test_derive_seed_is_fnv1a(oracle):
    # published FNV-1a/32 vectors pin the independent implementation
    assert _fnv1a(b"") == 0x811C9DC5
    assert _fnv1a(b"a") == 0xE40C292C
    assert _fnv1a(b"foobar") == 0xBF9CF968
    w = np.frombuffer(b"foob", dtype=np.float32)
    assert oracle.derive_seed(w, 0) == _fnv1a(b"foob")
    rng = np.random.default_rng(0)
    for n in (1, 7, 1024, 1025, 5000, 128 * 64):
        w = rng.standard_normal(n).astype(np.float32)
        raw = w.tobytes()
        stride = len(raw) // 4096 if len(raw) > 4096 else 1
        for salt in (0, 1):
            assert oracle.derive_seed(w, salt) == _fnv1a(raw[::stride], 0x811C9DC5 ^ salt)
    assert oracle.derive_seed(w, 0) != 0 and oracle.derive_seed(w, 0) != oracle.derive_seed(w, 1)


def test_block_size_rule(oracle):
    # src/converter.cpp:228-240
    for inf, want in [(4096, 512), (2048, 512), (3584, 512), (18944, 512), (5120, 512),
                      (27648, 512), (896, 128), (4864, 256), (384, 128), (100, 4), (7, 1)]:
        assert oracle.best_block_size(inf, 512) == want
    assert oracle.best_block_size(4096, 128) == 128


# ------------------------------------------------------------- Lloyd-Max
def test_lloyd_max_fixed_point_and_normal_fit(oracle):
    rng = np.random.default_rng(11)
    data = rng.standard_normal(200000).astype(np.float32)
    cb = oracle.generate_codebook_from_data(data, 4, 100)
    ref = oracle.generate_codebook(4)
    assert np.abs(cb.centroids - ref.centroids).max() < 0.3      # test_parallel_converter.cpp:331-343
    assert np.all(np.diff(cb.centroids) > 0)
    # one more Lloyd step moves nothing by more than what 100 iterations leave
    idx = np.minimum(np.searchsorted(cb.boundaries, data, side="left"), 15)
    means = np.array([data[idx == k].astype(np.float64).mean() for k in range(16)])
    assert np.abs(means - cb.centroids).max() < 5e-3
    # empty data -> analytical table (src/codebook.cpp:270-272)
    assert np.array_equal(oracle.generate_codebook_from_data(np.zeros(0, np.float32), 4).centroids, ref.centroids)
    # skewed data gives an asymmetric codebook; a bin that never receives data keeps
    # its starting centroid (src/codebook.cpp:124)
    sk = oracle.generate_codebook_from_data(np.abs(data), 3, 50)
    assert sk.centroids[0] == oracle.generate_codebook(3).centroids[0]
    assert not np.array_equal(sk.centroids, -sk.centroids[::-1])
    # first iteration by hand: bins from the analytic table, double means
    one = oracle.generate_codebook_from_data(data, 4, 1)
    idx0 = np.minimum(np.searchsorted(ref.boundaries, data, side="left"), 15)
    m0 = np.array([np.float32(data[idx0 == k].astype(np.float64).sum() / (idx0 == k).sum()) for k in range(16)])
    assert np.allclose(one.centroids, m0, rtol=0, atol=1e-7)


def test_lloyd_max_runs_to_the_reference_stopping_rule(oracle):
    """The whole fit by hand (src/codebook.cpp:99-143): bins by lower_bound on the midpoints of the current
    centroids, means from double sums rounded once to float, a bin without data keeps its centroid, and the
    loop ends after the first iteration in which no centroid moves by 1e-6 or more
    (kLloydMaxShiftThreshold, src/codebook.cpp:68,132).  The oracle must stop in exactly the same iteration
    and hold the same centroids; a looser threshold stops several iterations earlier on this data."""
    rng = np.random.default_rng(23)
    data = np.concatenate([rng.standard_normal(20000) * 0.7, rng.standard_normal(3333) * 2.5 + 0.4]).astype(np.float32)
    for bits in (2, 3, 4):
        n = 1 << bits
        c = oracle.generate_codebook(bits).centroids.copy()
        stops = {}                                             # threshold -> iteration at which it would stop
        done = None
        for it in range(1, 301):
            b = ((c[:-1] + c[1:]) * np.float32(0.5)).astype(np.float32)
            idx = np.minimum(np.searchsorted(b, data, side="left"), n - 1)
            shift = np.float32(0.0)
            for k in range(n):
                sel = data[idx == k]
                if sel.size:
                    nv = np.float32(sel.astype(np.float64).sum() / sel.size)
                    shift = max(shift, np.float32(abs(nv - c[k])))
                    c[k] = nv
            for thr in (1e-3, 1e-4, 1e-5):
                if shift < np.float32(thr) and thr not in stops:
                    stops[thr] = it
            if shift < np.float32(1e-6):
                done = it
                break
        assert done is not None and done < 300
        got = oracle.generate_codebook_from_data(data, bits, 300)
        assert got.iterations == done
        assert np.abs(got.centroids - c).max() <= 1e-7
        assert np.array_equal(got.boundaries, ((c[:-1] + c[1:]) * np.float32(0.5)).astype(np.float32))
        # the test has teeth: looser thresholds would have stopped earlier, with other centroids (1e-5 cannot be
        # told from 1e-6 on data of this size: the last shifts drop from about 1e-5 to exactly 0 in one step)
        assert stops[1e-3] < done and stops[1e-4] <= done
        if bits < 4:
            assert stops[1e-3] < stops[1e-4] < done
        early = oracle.generate_codebook_from_data(data, bits, stops[1e-3])
        assert np.abs(early.centroids - c).max() > 1e-5
        # the iteration cap is honoured as well
        assert oracle.generate_codebook_from_data(data, bits, 2).iterations == 2


def test_lloyd_max_thread_invariance(oracle):
    rng = np.random.default_rng(5)
    data = (rng.standard_normal(100000) * 1.3).astype(np.float32)
    a = oracle.generate_codebook_from_data(data, 4, 30).centroids
    oracle.set_threads(4)
    try:
        b = oracle.generate_codebook_from_data(data, 4, 30).centroids
    finally:
        oracle.set_threads(1)
    assert np.abs(a - b).max() < 1e-6


# ----------------------------------------------------------- dequantizer
def _dense_dequant(o, qw, cbp, cbr, bs):
    """Brute force in float64 with a dense Hadamard matrix:
    W = diag(norm) . blockdiag(diag(s) H / sqrt(bs)) . (centroids / sqrt(in))."""
    pp, pr = qw.packed_primary, qw.packed_residual
    out = pp.shape[0]
    five = pp.shape[1] == 2 * pr.shape[1]
    inf = pp.shape[1] if five else pp.shape[1] * 2
    if five:
        pidx = pp.astype(int)
    else:
        pidx = np.stack([pp & 15, pp >> 4], axis=-1).reshape(out, inf).astype(int)
    ridx = np.stack([pr & 15, pr >> 4], axis=-1).reshape(out, inf).astype(int)
    cP = cbp.centroids.astype(np.float64)
    cR = cbr.centroids.astype(np.float64)
    P = cP[np.minimum(pidx, len(cP) - 1)]
    R = cR[np.minimum(ridx, len(cR) - 1)]
    has_res = bool(pr.any())
    H = scipy.linalg.hadamard(bs).astype(np.float64)

    def inv(M, seed):
        s = np.array([_sign_bigint(int(seed), j) for j in range(bs)])
        T = (np.diag(s) @ H) / math.sqrt(bs)
        return np.concatenate([M[:, b:b + bs] @ T.T for b in range(0, inf, bs)], axis=1)

    if has_res and qw.seeds[1] == 0:
        Wn = inv((P + R) / math.sqrt(inf), qw.seeds[0])
    else:
        Wn = inv(P / math.sqrt(inf), qw.seeds[0])
        if has_res:
            Wn = Wn + inv(R / math.sqrt(inf), qw.seeds[1])
    return Wn * qw.norms.astype(np.float64)[:, None]


MODES = [dict(shared_rotation=True), dict(shared_rotation=False), dict(residual_bits=0),
         dict(primary_bits=5, residual_bits=3, shared_rotation=True),
         dict(primary_bits=5, residual_bits=3, shared_rotation=False)]


@pytest.mark.parametrize("mode", MODES, ids=["shared", "dual", "primary_only", "5+3shared", "5+3dual"])
@pytest.mark.parametrize("out,inf,bs", [(8, 128, 128), (16, 512, 256), (5, 384, 128), (4, 64, 32)])
def test_dequantize_matches_dense_float64(oracle, mode, out, inf, bs):
    w = oracle.lcg_matrix(out, inf, 42)
    pb, rb = mode.get("primary_bits", 4), mode.get("residual_bits", 4)
    cbp, cbr = oracle.generate_codebook(pb), oracle.generate_codebook(rb if rb else 4)
    qw = oracle.quantize_weight(w, cbp, cbr, pb, rb, bs, mode.get("shared_rotation", False))
    assert qw.packed_primary.shape == (out, inf if pb == 5 else inf // 2)
    assert qw.packed_residual.shape == (out, inf // 2)
    assert qw.norms.dtype == np.float32 and qw.seeds.dtype == np.uint32
    assert qw.seeds[2] == bs and qw.seeds[0] != 0
    if rb and mode.get("shared_rotation"):
        assert qw.seeds[1] == 0
    else:
        assert qw.seeds[1] != 0
    if rb == 0:
        assert not qw.packed_residual.any()
    W = oracle.dequantize_weight_cpu(qw, cbp, cbr, bs)
    assert W.dtype == np.float32 and W.shape == (out, inf)        # test_dequant_dtype.cpp:22-43
    want = _dense_dequant(oracle, qw, cbp, cbr, bs)
    assert np.abs(W - want).max() < 1e-5 * max(1.0, np.abs(want).max())
    rel = np.sqrt(((W - w) ** 2).mean() / (w ** 2).mean())
    # test_quantizer.cpp: rel-RMSE < 0.15 for 4-bit primaries, < 0.30 for 5+3 (:503-517)
    assert rel < (0.30 if pb == 5 else 0.15)
    ratio = np.linalg.norm(W, axis=1) / np.linalg.norm(w, axis=1)
    assert np.all((ratio > 0.95) & (ratio < 1.05))


def test_lut_convention_and_dual_reduces_to_primary_only(oracle):
    cbp, cbr = oracle.generate_codebook(4), oracle.generate_codebook(4)
    # lut[(r<<4)|p] = cP[p] + cR[r]: a one-row weight whose packed bytes enumerate all pairs
    inf = 512
    p = (np.arange(inf) % 16).astype(np.uint8)
    r = ((np.arange(inf) // 16) % 16).astype(np.uint8)
    pp, pr = oracle.pack4(p)[None, :], oracle.pack4(r)[None, :]
    qw = oracle.QuantizedWeight(pp, pr, np.ones(1, np.float32), np.array([77, 0, inf], np.uint32))
    W = oracle.dequantize_weight_cpu(qw, cbp, cbr, inf)
    comb = (cbp.centroids[p] + cbr.centroids[r]) * np.float32(1.0 / np.sqrt(np.float32(inf)))
    assert np.array_equal(W, oracle.wht_inverse(comb[None, :], 77, inf))
    # zero residual bytes: dual path == primary only, whatever seeds[1] is
    qa = oracle.QuantizedWeight(pp, np.zeros_like(pr), np.ones(1, np.float32), np.array([77, 5, inf], np.uint32))
    qb = oracle.QuantizedWeight(pp, np.zeros_like(pr), np.ones(1, np.float32), np.array([77, 0, inf], np.uint32))
    Wa, Wb = oracle.dequantize_weight_cpu(qa, cbp, cbr, inf), oracle.dequantize_weight_cpu(qb, cbp, cbr, inf)
    assert np.array_equal(Wa, Wb)
    prim = cbp.centroids[p] * np.float32(1.0 / np.sqrt(np.float32(inf)))
    assert np.array_equal(Wa, oracle.wht_inverse(prim[None, :], 77, inf))


def test_quantizer_properties_from_reference_tests(oracle):
    cbp, cbr = oracle.generate_codebook(4), oracle.generate_codebook(4)
    w = oracle.lcg_matrix(16, 896, 42)
    q1 = oracle.quantize_weight(w, cbp, cbr, 4, 4, 128, False)
    q2 = oracle.quantize_weight(w, cbp, cbr, 4, 4, 128, False)
    for a, b in zip((q1.packed_primary, q1.packed_residual, q1.norms, q1.seeds),
                    (q2.packed_primary, q2.packed_residual, q2.norms, q2.seeds)):
        assert a.tobytes() == b.tobytes()                          # determinism
    mse = {}
    for name, kw in dict(dual=dict(shared_rotation=False), shared=dict(shared_rotation=True),
                         prim=dict(residual_bits=0)).items():
        q = oracle.quantize_weight(w, cbp, cbr, 4, kw.get("residual_bits", 4), 128, kw.get("shared_rotation", False))
        mse[name] = ((oracle.dequantize_weight_cpu(q, cbp, cbr, 128) - w) ** 2).mean()
    assert mse["dual"] < mse["prim"] and mse["shared"] < mse["prim"]       # residual lowers MSE
    assert mse["shared"] < 1.5 * mse["dual"] and mse["dual"] < 1.5 * mse["shared"]
    # zero row -> no NaN
    wz = w.copy(); wz[3] = 0
    qz = oracle.quantize_weight(wz, cbp, cbr, 4, 4, 128, True)
    Wz = oracle.dequantize_weight_cpu(qz, cbp, cbr, 128)
    assert np.isfinite(Wz).all() and np.isfinite(qz.norms).all()
    assert np.abs(Wz[3]).max() < 1e-6


def test_stored_residual_seed(oracle):
    """seeds[1] is 0 only when both passes share the rotation AND there is a residual pass
    (src/quantizer.cpp:255-256): a primary-only layer quantised with shared_rotation set keeps its derived
    residual seed, which equals the one the dual-rotation call stores, and is never 0."""
    w = oracle.lcg_matrix(16, 256, 7)
    cb = oracle.generate_codebook(4)
    shared44 = oracle.quantize_weight(w, cb, cb, 4, 4, 128, True)
    dual44 = oracle.quantize_weight(w, cb, cb, 4, 4, 128, False)
    shared40 = oracle.quantize_weight(w, cb, cb, 4, 0, 128, True)
    dual40 = oracle.quantize_weight(w, cb, cb, 4, 0, 128, False)
    assert shared44.seeds[1] == 0 and dual44.seeds[1] != 0
    assert shared40.seeds[1] != 0 and shared40.seeds[1] == dual44.seeds[1] == dual40.seeds[1]
    assert shared44.seeds[0] == dual44.seeds[0] == shared40.seeds[0] != 0
    assert shared44.seeds[0] != dual44.seeds[1]                # two salts (src/quantizer.cpp:82-83)
    assert all(q.seeds[2] == 128 for q in (shared44, dual44, shared40, dual40))
    assert not shared40.packed_residual.any()                  # no residual pass: an all-zero plane
    assert np.array_equal(shared40.packed_primary, dual40.packed_primary)


def test_threads_do_not_change_results(oracle):
    cbp, cbr = oracle.generate_codebook(4), oracle.generate_codebook(4)
    w = oracle.lcg_matrix(32, 512, 9)
    a = oracle.quantize_weight(w, cbp, cbr, 4, 4, 256, False)
    Wa = oracle.dequantize_weight_cpu(a, cbp, cbr, 256)
    oracle.set_threads(4)
    try:
        b = oracle.quantize_weight(w, cbp, cbr, 4, 4, 256, False)
        Wb = oracle.dequantize_weight_cpu(b, cbp, cbr, 256)
    finally:
        oracle.set_threads(1)
    assert a.packed_primary.tobytes() == b.packed_primary.tobytes()
    assert a.packed_residual.tobytes() == b.packed_residual.tobytes()
    assert a.norms.tobytes() == b.norms.tobytes() and Wa.tobytes() == Wb.tobytes()


def test_linear_forward_is_x_times_wT(oracle):
    cbp, cbr = oracle.generate_codebook(4), oracle.generate_codebook(4)
    w = oracle.lcg_matrix(64, 128, 42)
    x = oracle.lcg_matrix(8, 128, 99)
    qw = oracle.quantize_weight(w, cbp, cbr, 4, 4, 128, False)
    W = oracle.dequantize_weight_cpu(qw, cbp, cbr, 128)
    want = x.astype(np.float64) @ W.astype(np.float64).T
    assert np.abs(oracle.linear_forward(qw, cbp, cbr, 128, x) - want).max() < 1e-5
    assert np.abs(oracle.matmul_xwT(x, W, acc_double=False) - want).max() < 1e-4
    # quantised layer still approximates the dense layer (test_linear.cpp:134-145 uses 0.15 abs)
    assert np.abs(want - x.astype(np.float64) @ w.astype(np.float64).T).max() < 0.15 * 8


def test_layer_codebook_recipe(oracle):
    rng = np.random.default_rng(1)
    w = (rng.standard_normal((64, 512)) * 0.02).astype(np.float32)
    cbp, cbr = oracle.fit_layer_codebooks(w, 512)
    g = oracle.generate_codebook(4)
    assert np.abs(cbp.centroids - g.centroids).max() < 0.3
    assert np.all(np.diff(cbp.centroids) > 0) and np.all(np.diff(cbr.centroids) > 0)
    # residuals against the global codebook are small, so the outermost residual bins
    # never receive data and keep the table value (src/codebook.cpp:124)
    assert cbr.centroids[0] == g.centroids[0] and cbr.centroids[15] == g.centroids[15]
    assert np.abs(cbr.centroids[6:10]).max() < 0.15
    # by hand: primary samples = rotated * sqrt(in) of the normalised rows
    wn = w / np.maximum(np.linalg.norm(w.astype(np.float64), axis=1)[:, None], 1e-10).astype(np.float32)
    sc = oracle.wht_forward(wn.astype(np.float32), oracle.derive_seed(w, 0), 512) * np.float32(np.sqrt(np.float32(512)))
    by_hand = oracle.generate_codebook_from_data(sc, 4, 100)
    assert np.abs(by_hand.centroids - cbp.centroids).max() < 1e-5


def test_layer_codebook_recipe_residual_leg_uses_global_primary(oracle):
    """src/converter.cpp:345-357: the residual codebook is fitted on
    scaled - global_cb[quantize(scaled, global_cb)], the *global analytic* primary codebook,
    not the per-layer one fitted a few lines earlier.  Heavy-tailed rows make the two differ."""
    rng = np.random.default_rng(11)
    w = (rng.standard_normal((48, 512)) * 0.02).astype(np.float32)
    tail = rng.random(w.shape) < 0.05
    w[tail] = (rng.standard_t(2, size=int(tail.sum())) * 0.08).astype(np.float32)
    bs = 128
    cbp, cbr = oracle.fit_layer_codebooks(w, bs)
    g = oracle.generate_codebook(4)
    # by hand, in numpy: normalise, rotate, scale, bin against the global codebook, subtract
    nrm = np.sqrt((w.astype(np.float64) ** 2).sum(axis=1)).astype(np.float32)
    wn = (w / np.maximum(nrm, np.float32(1e-10))[:, None]).astype(np.float32)
    sc = (oracle.wht_forward(wn, oracle.derive_seed(w, 0), bs) * np.float32(np.sqrt(np.float32(512)))).ravel()
    gb = ((g.centroids[:-1] + g.centroids[1:]) * np.float32(0.5)).astype(np.float32)
    idx_g = np.searchsorted(gb, sc, side="left")                     # lower_bound, src/codebook.cpp:284-302
    resid_g = (sc - g.centroids[idx_g]).astype(np.float32)
    want = oracle.generate_codebook_from_data(resid_g, 4, 100)
    assert np.abs(want.centroids - cbr.centroids).max() < 1e-6
    # the wrong reading (residuals against the fitted primary) lands elsewhere on this data,
    # so the check above does discriminate
    fb = ((cbp.centroids[:-1] + cbp.centroids[1:]) * np.float32(0.5)).astype(np.float32)
    idx_f = np.searchsorted(fb, sc, side="left")
    resid_f = (sc - cbp.centroids[idx_f]).astype(np.float32)
    wrong = oracle.generate_codebook_from_data(resid_f, 4, 100)
    assert np.abs(wrong.centroids - cbr.centroids).max() > 1e-3
    assert np.abs(cbp.centroids - g.centroids).max() > 1e-2          # fitted != global here


def _dense_from_values(vals, seed, bs, norms):
    """diag(norm) . blockdiag(diag(s) H / sqrt(bs)) . (vals / sqrt(in)) in float64."""
    out, inf = vals.shape
    s = np.array([_sign_bigint(int(seed), j) for j in range(bs)])
    T = (np.diag(s) @ scipy.linalg.hadamard(bs).astype(np.float64)) / math.sqrt(bs)
    M = vals.astype(np.float64) / math.sqrt(inf)
    Wn = np.concatenate([M[:, b:b + bs] @ T.T for b in range(0, inf, bs)], axis=1)
    return Wn * norms.astype(np.float64)[:, None]


def test_short_primary_codebook_zero_fill_shared_and_clamp_dual(oracle):
    """A 3-bit primary codebook (8 centroids) under 4-bit planes that hold indices up to 15.
    Shared rotation goes through the 256-entry table, whose entries with p >= n_primary are never
    written and stay 0: the residual centroid is dropped too (src/dequantizer.cpp:144-150).  The
    dual-rotation and primary-only paths clamp the index to the last centroid (:94,103)."""
    rng = np.random.default_rng(3)
    out, inf, bs = 6, 256, 64
    p = rng.integers(0, 16, size=(out, inf)).astype(np.uint8)
    r = rng.integers(0, 16, size=(out, inf)).astype(np.uint8)
    assert (p >= 8).any() and r.any()
    pp = oracle.pack4(p).reshape(out, inf // 2)
    pr = oracle.pack4(r).reshape(out, inf // 2)
    norms = (rng.random(out) + 0.5).astype(np.float32)
    cb3, cb4 = oracle.generate_codebook(3), oracle.generate_codebook(4)
    cP, cR = cb3.centroids.astype(np.float64), cb4.centroids.astype(np.float64)

    # shared rotation: zero-fill
    qs = oracle.QuantizedWeight(pp, pr, norms, np.array([1234, 0, bs], np.uint32))
    W = oracle.dequantize_weight_cpu(qs, cb3, cb4, bs)
    vals = np.where(p < 8, cP[np.minimum(p, 7)] + cR[r], 0.0)
    want = _dense_from_values(vals, 1234, bs, norms)
    assert np.abs(W - want).max() < 1e-5 * max(1.0, np.abs(want).max())
    clamp = _dense_from_values(cP[np.minimum(p, 7)] + cR[r], 1234, bs, norms)
    assert np.abs(W - clamp).max() > 1e-2                      # a clamping oracle would fail above

    # dual rotation: clamp, two inverse rotations
    qd = oracle.QuantizedWeight(pp, pr, norms, np.array([1234, 777, bs], np.uint32))
    W = oracle.dequantize_weight_cpu(qd, cb3, cb4, bs)
    want = _dense_from_values(cP[np.minimum(p, 7)], 1234, bs, norms) + _dense_from_values(cR[r], 777, bs, norms)
    assert np.abs(W - want).max() < 1e-5 * max(1.0, np.abs(want).max())
    zero = _dense_from_values(np.where(p < 8, cP[np.minimum(p, 7)], 0.0), 1234, bs, norms) + \
        _dense_from_values(cR[r], 777, bs, norms)
    assert np.abs(W - zero).max() > 1e-2

    # primary only (all residual bytes zero): clamp as well
    qp = oracle.QuantizedWeight(pp, np.zeros_like(pr), norms, np.array([1234, 777, bs], np.uint32))
    W = oracle.dequantize_weight_cpu(qp, cb3, cb4, bs)
    want = _dense_from_values(cP[np.minimum(p, 7)], 1234, bs, norms)
    assert np.abs(W - want).max() < 1e-5 * max(1.0, np.abs(want).max())

    # a short residual codebook under dual rotation clamps too (:229)
    qd2 = oracle.QuantizedWeight(pp, pr, norms, np.array([1234, 777, bs], np.uint32))
    W = oracle.dequantize_weight_cpu(qd2, cb4, cb3, bs)
    c4 = cb4.centroids.astype(np.float64)
    want = _dense_from_values(c4[p], 1234, bs, norms) + _dense_from_values(cP[np.minimum(r, 7)], 777, bs, norms)
    assert np.abs(W - want).max() < 1e-5 * max(1.0, np.abs(want).max())


def test_oversized_primary_codebook_on_nibble_planes_wraps_in_the_shared_table(oracle):
    """A 32-entry primary codebook under 4-bit planes with shared rotation.  The reference fills its
    256-entry table with `lut[uint8_t((r << 4) | p)]` for every p below the codebook size
    (src/dequantizer.cpp:144-150): for p >= 16 bit 4 of p lands in the residual half of the index, and
    since r ascends in the outer loop and p in the inner one, what remains is, in closed form,
    entry (r, p) = cP[p] + cR[r] for even r and cP[p + 16] + cR[r] for odd r."""
    rng = np.random.default_rng(8)
    out, inf, bs = 5, 128, 32
    p = rng.integers(0, 16, size=(out, inf)).astype(np.uint8)
    r = rng.integers(0, 16, size=(out, inf)).astype(np.uint8)
    pp = oracle.pack4(p).reshape(out, inf // 2)
    pr = oracle.pack4(r).reshape(out, inf // 2)
    norms = (rng.random(out) + 0.5).astype(np.float32)
    cb5, cb4 = oracle.generate_codebook(5), oracle.generate_codebook(4)
    cP, cR = cb5.centroids.astype(np.float64), cb4.centroids.astype(np.float64)
    assert len(cP) == 32
    qs = oracle.QuantizedWeight(pp, pr, norms, np.array([4321, 0, bs], np.uint32))
    W = oracle.dequantize_weight_cpu(qs, cb5, cb4, bs)
    vals = np.where(r % 2 == 1, cP[p.astype(int) + 16], cP[p]) + cR[r]
    want = _dense_from_values(vals, 4321, bs, norms)
    assert np.abs(W - want).max() < 1e-5 * max(1.0, np.abs(want).max())
    capped = _dense_from_values(cP[p] + cR[r], 4321, bs, norms)        # a table that stops at p < 16
    assert np.abs(W - capped).max() > 1e-2
