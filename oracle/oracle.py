"""TEST INFRASTRUCTURE - NOT PRODUCT CODE.

ctypes/numpy front end for ``libtq_oracle.so`` (the plain-C restatement of the
reference CPU path, see ``tq_oracle.h``).  Only tests, the smoke check and the
benchmark's CPU-baseline leg import this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libtq_oracle.so")
_lib = None

_u8p = C.POINTER(C.c_uint8)
_f32p = C.POINTER(C.c_float)
_u32p = C.POINTER(C.c_uint32)


def build():
    """Compile the oracle with gcc (used by the repository build step)."""
    subprocess.check_call(["make", "-C", _HERE, "-B", "libtq_oracle.so"],
                          stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        L.tqo_sign.restype = C.c_float
        L.tqo_sign.argtypes = [C.c_uint32, C.c_uint32]
        L.tqo_derive_seed.restype = C.c_uint32
        L.tqo_derive_seed.argtypes = [_f32p, C.c_size_t, C.c_uint32]
        L.tqo_best_block_size.restype = C.c_uint32
        L.tqo_best_block_size.argtypes = [C.c_int, C.c_uint32]
        L.tqo_wht_forward.argtypes = [_f32p, _f32p, C.c_int, C.c_int, C.c_uint32, C.c_uint32]
        L.tqo_wht_inverse.argtypes = [_f32p, _f32p, C.c_int, C.c_int, C.c_uint32, C.c_uint32]
        L.tqo_fwht_inplace.argtypes = [_f32p, C.c_int]
        L.tqo_codebook_analytic.argtypes = [C.c_int, _f32p, _f32p]
        L.tqo_boundaries.argtypes = [_f32p, C.c_int, _f32p]
        L.tqo_validate_codebook.argtypes = [_f32p, C.c_int, _f32p, C.c_int, C.c_int, C.c_int]
        L.tqo_quantize.argtypes = [_f32p, C.c_size_t, _f32p, C.c_int, _u8p]
        L.tqo_dequantize.argtypes = [_u8p, C.c_size_t, _f32p, C.c_int, _f32p]
        L.tqo_pack4.argtypes = [_u8p, C.c_size_t, _u8p]
        L.tqo_unpack4.argtypes = [_u8p, C.c_size_t, _u8p]
        L.tqo_lloyd_max.argtypes = [_f32p, C.c_size_t, C.c_int, C.c_int, _f32p, _f32p]
        L.tqo_fit_layer_codebooks.argtypes = [_f32p, C.c_int, C.c_int, C.c_uint32, C.c_int, C.c_int,
                                              _f32p, C.c_int, _f32p, _f32p]
        L.tqo_quantize_weight.argtypes = [_f32p, C.c_int, C.c_int, _f32p, C.c_int, _f32p, C.c_int,
                                          C.c_int, C.c_int, C.c_uint32, C.c_int,
                                          _u8p, _u8p, _f32p, _u32p]
        L.tqo_dequantize_weight.argtypes = [_u8p, C.c_int, _u8p, C.c_int, _f32p, _u32p, C.c_int,
                                            _f32p, C.c_int, _f32p, C.c_int, C.c_uint32, _f32p]
        L.tqo_matmul_xwT.argtypes = [_f32p, _f32p, C.c_int, C.c_int, C.c_int, _f32p, C.c_int]
        L.tqo_matmul_xwT.restype = None
        L.tqo_f32_to_bf16.restype = C.c_uint16
        L.tqo_f32_to_bf16.argtypes = [C.c_float]
        L.tqo_bf16_to_f32.restype = C.c_float
        L.tqo_bf16_to_f32.argtypes = [C.c_uint16]
        _lib = L
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a, t):
    return a.ctypes.data_as(t)


def set_threads(n):
    lib().tqo_set_threads(int(n))


def sign(seed, index):
    return float(lib().tqo_sign(seed & 0xFFFFFFFF, index & 0xFFFFFFFF))


def make_signs(seed, block_size):
    return np.array([sign(seed, i) for i in range(block_size)], dtype=np.float32)


def fwht(v):
    v = _f32(v).copy()
    lib().tqo_fwht_inplace(_p(v, _f32p), v.size)
    return v


def wht_forward(m, seed, block_size):
    m = _f32(m)
    out = np.empty_like(m)
    rc = lib().tqo_wht_forward(_p(m, _f32p), _p(out, _f32p), m.shape[0], m.shape[1], seed, block_size)
    if rc != 0:
        raise ValueError("in_features must be divisible by block_size")
    return out


def wht_inverse(m, seed, block_size):
    m = _f32(m)
    out = np.empty_like(m)
    rc = lib().tqo_wht_inverse(_p(m, _f32p), _p(out, _f32p), m.shape[0], m.shape[1], seed, block_size)
    if rc != 0:
        raise ValueError("in_features must be divisible by block_size")
    return out


class Codebook:
    """Mirror of the reference's Codebook struct (include/turboquant/codebook.h:24-29)."""

    def __init__(self, centroids, bits, analytical=False):
        self.centroids = _f32(centroids)
        self.bits = int(bits)
        self.analytical = analytical
        self.boundaries = np.empty(max(len(self.centroids) - 1, 0), dtype=np.float32)
        lib().tqo_boundaries(_p(self.centroids, _f32p), len(self.centroids), _p(self.boundaries, _f32p))


def generate_codebook(bits):
    c = np.empty(32, dtype=np.float32)
    n = lib().tqo_codebook_analytic(bits, _p(c, _f32p), None)
    if n < 0:
        raise ValueError("Unsupported bit width; must be 1-5")
    return Codebook(c[:n].copy(), bits, analytical=True)


def validate_codebook(cb):
    return bool(lib().tqo_validate_codebook(_p(cb.centroids, _f32p), len(cb.centroids),
                                            _p(cb.boundaries, _f32p), len(cb.boundaries),
                                            cb.bits, int(cb.analytical)))


def generate_codebook_from_data(data, bits, iterations=100):
    data = _f32(data).ravel()
    c = np.empty(32, dtype=np.float32)
    b = np.empty(32, dtype=np.float32)
    it = lib().tqo_lloyd_max(_p(data, _f32p), data.size, bits, iterations, _p(c, _f32p), _p(b, _f32p))
    if it < 0:
        raise ValueError("Unsupported bit width; must be 1-5")
    cb = Codebook(c[:1 << bits].copy(), bits, analytical=(data.size == 0))
    cb.iterations = it
    return cb


def quantize(values, cb):
    v = _f32(values).ravel()
    out = np.empty(v.size, dtype=np.uint8)
    lib().tqo_quantize(_p(v, _f32p), v.size, _p(cb.boundaries, _f32p), len(cb.centroids), _p(out, _u8p))
    return out


def dequantize(indices, cb):
    idx = np.ascontiguousarray(indices, dtype=np.uint8).ravel()
    out = np.empty(idx.size, dtype=np.float32)
    lib().tqo_dequantize(_p(idx, _u8p), idx.size, _p(cb.centroids, _f32p), len(cb.centroids), _p(out, _f32p))
    return out


def pack4(indices):
    idx = np.ascontiguousarray(indices, dtype=np.uint8).ravel()
    out = np.empty(idx.size // 2, dtype=np.uint8)
    lib().tqo_pack4(_p(idx, _u8p), idx.size, _p(out, _u8p))
    return out


def unpack4(packed):
    pk = np.ascontiguousarray(packed, dtype=np.uint8).ravel()
    out = np.empty(pk.size * 2, dtype=np.uint8)
    lib().tqo_unpack4(_p(pk, _u8p), pk.size, _p(out, _u8p))
    return out


def derive_seed(weight, salt):
    w = _f32(weight)
    return int(lib().tqo_derive_seed(_p(w, _f32p), w.size, salt))


def best_block_size(in_features, max_block_size=512):
    return int(lib().tqo_best_block_size(in_features, max_block_size))


class QuantizedWeight:
    """Mirror of the reference's QuantizedWeight (include/turboquant/quantizer.h:22-27)."""

    def __init__(self, packed_primary, packed_residual, norms, seeds):
        self.packed_primary = packed_primary
        self.packed_residual = packed_residual
        self.norms = norms
        self.seeds = seeds

    @property
    def out_features(self):
        return self.packed_primary.shape[0]

    @property
    def in_features(self):
        return self.packed_residual.shape[1] * 2


def quantize_weight(weight, cbp, cbr, primary_bits=4, residual_bits=4, block_size=512,
                    shared_rotation=False):
    w = _f32(weight)
    out, inf = w.shape
    pcols = inf // 2 if primary_bits <= 4 else inf
    pp = np.empty((out, pcols), dtype=np.uint8)
    pr = np.empty((out, inf // 2), dtype=np.uint8)
    norms = np.empty(out, dtype=np.float32)
    seeds = np.empty(3, dtype=np.uint32)
    rc = lib().tqo_quantize_weight(_p(w, _f32p), out, inf,
                                   _p(cbp.centroids, _f32p), len(cbp.centroids),
                                   _p(cbr.centroids, _f32p), len(cbr.centroids),
                                   primary_bits, residual_bits, block_size, int(shared_rotation),
                                   _p(pp, _u8p), _p(pr, _u8p), _p(norms, _f32p), _p(seeds, _u32p))
    if rc != 0:
        raise ValueError("quantize_weight: bad shape or block size")
    return QuantizedWeight(pp, pr, norms, seeds)


def dequantize_weight_cpu(qw, cbp, cbr, block_size):
    pp = np.ascontiguousarray(qw.packed_primary, dtype=np.uint8)
    pr = np.ascontiguousarray(qw.packed_residual, dtype=np.uint8)
    norms = _f32(qw.norms)
    seeds = np.ascontiguousarray(qw.seeds, dtype=np.uint32)
    out = pp.shape[0]
    inf = pp.shape[1] if pp.shape[1] == 2 * pr.shape[1] else pp.shape[1] * 2
    W = np.empty((out, inf), dtype=np.float32)
    rc = lib().tqo_dequantize_weight(_p(pp, _u8p), pp.shape[1], _p(pr, _u8p), pr.shape[1],
                                     _p(norms, _f32p), _p(seeds, _u32p), out,
                                     _p(cbp.centroids, _f32p), len(cbp.centroids),
                                     _p(cbr.centroids, _f32p), len(cbr.centroids),
                                     block_size, _p(W, _f32p))
    if rc != 0:
        raise ValueError("dequantize_weight_cpu: bad shape or block size")
    return W


def fit_layer_codebooks(weight, block_size, primary_bits=4, residual_bits=4, global_primary=None):
    w = _f32(weight)
    g = global_primary if global_primary is not None else generate_codebook(primary_bits)
    cp = np.empty(32, dtype=np.float32)
    cr = np.empty(32, dtype=np.float32)
    rc = lib().tqo_fit_layer_codebooks(_p(w, _f32p), w.shape[0], w.shape[1], block_size,
                                       primary_bits, residual_bits,
                                       _p(g.centroids, _f32p), len(g.centroids),
                                       _p(cp, _f32p), _p(cr, _f32p))
    if rc != 0:
        raise ValueError("fit_layer_codebooks failed")
    cbp = Codebook(cp[:1 << primary_bits].copy(), primary_bits)
    cbr = Codebook(cr[:1 << residual_bits].copy(), residual_bits) if residual_bits > 0 else generate_codebook(4)
    return cbp, cbr


def matmul_xwT(x, w, acc_double=False):
    x = _f32(x)
    w = _f32(w)
    y = np.empty((x.shape[0], w.shape[0]), dtype=np.float32)
    lib().tqo_matmul_xwT(_p(x, _f32p), _p(w, _f32p), x.shape[0], x.shape[1], w.shape[0],
                         _p(y, _f32p), int(acc_double))
    return y


def linear_forward(qw, cbp, cbr, block_size, x, acc_double=True):
    """Reference forward as the reference's tests define it: CPU dequantise then
    fp32 x.W^T (tests/integration/test_linear.cpp:102-107)."""
    return matmul_xwT(x, dequantize_weight_cpu(qw, cbp, cbr, block_size), acc_double)


def f32_to_bf16_bits(a):
    """Round-to-nearest-even bf16 bit patterns of an fp32 array."""
    u = _f32(a).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return r


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def lcg_matrix(rows, cols, seed):
    """The reference tests' input generator (tests/integration/test_linear.cpp:26-34):
    state = state*1103515245+12345 (u32); v = (state>>16)/32768 - 1."""
    n = rows * cols
    out = np.empty(n, dtype=np.float32)
    state = seed & 0xFFFFFFFF
    for i in range(n):
        state = (state * 1103515245 + 12345) & 0xFFFFFFFF
        out[i] = np.float32(np.float32(state >> 16) / np.float32(32768.0)) - np.float32(1.0)
    return out.reshape(rows, cols)
