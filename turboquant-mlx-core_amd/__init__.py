"""Python binding (ctypes) of libturboquant_amd.so, the gfx950 TQ8 linear path.

The names mirror the reference's C++ API for this path
(include/turboquant/linear.h:11-35, include/turboquant/dequantizer.h:11-39,
include/turboquant/quantizer.h:22-42).  Everything computes on the GPU through
the C-ABI in include/turboquant_c/tq_linear.h; there is no CPU fallback, and a
missing library is an ImportError-like RuntimeError, never a silent substitute.

The directory name is not a Python identifier; load it with
``importlib`` (see ``__graft_entry__.load_package``) under the module name
``turboquant_mlx_core_amd``.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libturboquant_amd.so")

F32, F16, BF16 = 0, 1, 2
MODE_NAMES = {0: "primary_only", 1: "shared_lut", 2: "dual", 3: "shared_5bit",
              4: "primary_only_5bit", 5: "dual_5bit"}

_u8p = C.POINTER(C.c_uint8)
_f32p = C.POINTER(C.c_float)
_u32p = C.POINTER(C.c_uint32)
_lib = None


def build():
    """Compile the HIP library in-tree (hipcc cross-compiles gfx950 without a GPU)."""
    subprocess.check_call(["make", "-C", _HERE, "-B", "-j8"], stdout=subprocess.DEVNULL,
                          stderr=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `make -C {_HERE}`; "
                               "there is no CPU fallback for the TQ8 linear path")
        L = C.CDLL(LIB_PATH)
        L.tq_last_error.restype = C.c_char_p
        L.tq_linear_create.restype = C.c_void_p
        L.tq_linear_create.argtypes = [C.c_int, C.c_int, _u8p, C.c_int, _u8p, C.c_int, _f32p, _u32p,
                                       _f32p, C.c_int, _f32p, C.c_int, C.c_uint32]
        L.tq_linear_create_from_device.restype = C.c_void_p
        L.tq_linear_create_from_device.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_int,
                                                   C.c_void_p, _u32p, _f32p, C.c_int, _f32p, C.c_int, C.c_uint32]
        for name in ("tq_linear_in_features", "tq_linear_out_features", "tq_linear_mode"):
            getattr(L, name).argtypes = [C.c_void_p]
        L.tq_linear_forward.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_void_p]
        L.tq_linear_forward_static.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_void_p]
        L.tq_linear_reserve.argtypes = [C.c_void_p, C.c_int]
        L.tq_linear_forward_host.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int]
        L.tq_linear_forward_group.argtypes = [C.POINTER(C.c_void_p), C.c_int, C.c_void_p, C.c_int, C.c_int,
                                              C.POINTER(C.c_void_p), C.c_int, C.c_void_p]
        L.tq_linear_dequantize.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        L.tq_linear_dequantize_host.argtypes = [C.c_void_p, _f32p]
        L.tq_linear_free.argtypes = [C.c_void_p]
        L.tq_linear_free.restype = None
        L.tq_wht_rotate.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_uint32, C.c_uint32, C.c_int, C.c_void_p]
        L.tq_wht_rotate_host.argtypes = [_f32p, _f32p, C.c_int, C.c_int, C.c_uint32, C.c_uint32, C.c_int]
        L.tq_generate_codebook.argtypes = [C.c_int, _f32p, _f32p]
        L.tq_best_block_size.restype = C.c_uint32
        L.tq_best_block_size.argtypes = [C.c_int, C.c_uint32]
        L.tq_quantize_weight.argtypes = [C.c_void_p, C.c_int, C.c_int, _f32p, C.c_int, _f32p, C.c_int, C.c_int, C.c_int,
                                         C.c_uint32, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, _u32p]
        L.tq_quantize_weight_host.argtypes = [_f32p, C.c_int, C.c_int, _f32p, C.c_int, _f32p, C.c_int, C.c_int, C.c_int,
                                              C.c_uint32, C.c_int, _u8p, _u8p, _f32p, _u32p]
        L.tq_fit_layer_codebooks.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_uint32, C.c_int, C.c_int, _f32p, C.c_int,
                                             C.c_int, _f32p, _f32p]
        L.tq_fit_layer_codebooks_host.argtypes = [_f32p, C.c_int, C.c_int, C.c_uint32, C.c_int, C.c_int, _f32p, C.c_int,
                                                  C.c_int, _f32p, _f32p]
        L.tq_mlp_create.restype = C.c_void_p
        L.tq_mlp_create.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
        L.tq_mlp_forward.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_void_p]
        L.tq_mlp_free.argtypes = [C.c_void_p]
        L.tq_mlp_free.restype = None
        _lib = L
    return _lib


def last_error():
    return lib().tq_last_error().decode()


def _p(a, t):
    return a.ctypes.data_as(t)


_NP_DTYPE = {F32: np.float32, F16: np.float16, BF16: np.uint16}


class TurboQuantLinear:
    """Mirror of turboquant::TurboQuantLinear (include/turboquant/linear.h:11-35).

    ``weights`` is any object with ``packed_primary``, ``packed_residual``, ``norms`` and
    ``seeds`` numpy arrays (the reference's QuantizedWeight); codebooks are objects with a
    ``centroids`` array.  bf16 arrays travel as uint16 bit patterns.
    """

    def __init__(self, in_features, out_features, weights, primary_codebook, residual_codebook, block_size):
        pp = np.ascontiguousarray(weights.packed_primary, dtype=np.uint8)
        pr = np.ascontiguousarray(weights.packed_residual, dtype=np.uint8)
        norms = np.ascontiguousarray(weights.norms, dtype=np.float32)
        seeds = np.ascontiguousarray(weights.seeds, dtype=np.uint32)
        cp = np.ascontiguousarray(primary_codebook.centroids, dtype=np.float32)
        cr = np.ascontiguousarray(residual_codebook.centroids, dtype=np.float32)
        if pp.ndim != 2 or pr.ndim != 2 or pp.shape[0] != out_features or pr.shape[0] != out_features:
            raise ValueError("packed tensors must be [out_features, cols]")
        # (the C call reads out_features norms and two seeds through raw pointers)
        if norms.size != out_features:
            raise ValueError("norms must hold out_features values")
        if seeds.size < 2:
            raise ValueError("seeds must hold {seed_primary, seed_residual[, block_size]}")
        if cp.size < 1 or cr.size < 1:
            raise ValueError("codebooks must not be empty")
        self._h = lib().tq_linear_create(in_features, out_features, _p(pp, _u8p), pp.shape[1], _p(pr, _u8p),
                                         pr.shape[1], _p(norms, _f32p), _p(seeds, _u32p), _p(cp, _f32p), len(cp),
                                         _p(cr, _f32p), len(cr), block_size)
        if not self._h:
            raise ValueError(last_error())

    def in_features(self):
        return lib().tq_linear_in_features(self._h)

    def out_features(self):
        return lib().tq_linear_out_features(self._h)

    def mode(self):
        return MODE_NAMES[lib().tq_linear_mode(self._h)]

    def forward(self, x, x_dtype=F32, y_dtype=F32):
        """x: numpy [batch, in] (float32, float16, or uint16 bf16 bits) -> numpy [batch, out]."""
        x = np.ascontiguousarray(x, dtype=_NP_DTYPE[x_dtype])
        if x.ndim != 2 or x.shape[1] != self.in_features():
            raise ValueError("input must be [batch, in_features]")
        y = np.empty((x.shape[0], self.out_features()), dtype=_NP_DTYPE[y_dtype])
        rc = lib().tq_linear_forward_host(self._h, x.ctypes.data, x_dtype, x.shape[0], y.ctypes.data, y_dtype)
        if rc != 0:
            raise RuntimeError(last_error())
        return y

    def forward_device(self, x_ptr, x_dtype, batch, y_ptr, y_dtype, stream=None):
        """Asynchronous forward on raw device pointers (e.g. torch ``data_ptr()``)."""
        rc = lib().tq_linear_forward(self._h, x_ptr, x_dtype, batch, y_ptr, y_dtype, stream)
        if rc != 0:
            raise RuntimeError(last_error())

    def forward_static_device(self, x_ptr, x_dtype, batch, y_ptr, y_dtype, stream=None):
        """forward_device without any allocation: workspaces in the library's fixed scratch array."""
        rc = lib().tq_linear_forward_static(self._h, x_ptr, x_dtype, batch, y_ptr, y_dtype, stream)
        if rc != 0:
            raise RuntimeError(last_error())

    def reserve(self, max_batch):
        """Size the workspaces now so that forward_device with up to max_batch rows never allocates."""
        if lib().tq_linear_reserve(self._h, max_batch) != 0:
            raise RuntimeError(last_error())

    def dequantize(self):
        """dequantize_weight_gpu: float32 [out, in]."""
        w = np.empty((self.out_features(), self.in_features()), dtype=np.float32)
        if lib().tq_linear_dequantize_host(self._h, _p(w, _f32p)) != 0:
            raise RuntimeError(last_error())
        return w

    def dequantize_device(self, w_ptr, stream=None):
        if lib().tq_linear_dequantize(self._h, w_ptr, stream) != 0:
            raise RuntimeError(last_error())

    def close(self):
        if getattr(self, "_h", None):
            lib().tq_linear_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class TurboQuantMLP:
    """Gated MLP block y = down(silu(gate(x)) * up(x)) over three TurboQuantLinear layers
    (tq_mlp_* in include/turboquant_c/tq_mlp.h).  Device pointers in, device pointers out;
    the layers must stay alive as long as the block."""

    def __init__(self, gate, up, down, max_batch=1):
        self._layers = (gate, up, down)
        self._h = lib().tq_mlp_create(gate._h, up._h, down._h, max_batch)
        if not self._h:
            raise ValueError(last_error())

    def forward_device(self, x_ptr, x_dtype, batch, y_ptr, y_dtype, stream=None):
        if lib().tq_mlp_forward(self._h, x_ptr, x_dtype, batch, y_ptr, y_dtype, stream) != 0:
            raise RuntimeError(last_error())

    def close(self):
        if getattr(self, "_h", None):
            lib().tq_mlp_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def forward_group_device(layers, x_ptr, x_dtype, batch, y_ptrs, y_dtype, stream=None):
    """One to three TurboQuantLinear layers applied to the same activations on raw device pointers
    (q, k, v or gate, up of a decoder layer): shared kernel launches where the layers allow it, the
    same results as one forward_device call per layer."""
    n = len(layers)
    hs = (C.c_void_p * n)(*[layer._h for layer in layers])
    ys = (C.c_void_p * n)(*y_ptrs)
    if lib().tq_linear_forward_group(hs, n, x_ptr, x_dtype, batch, ys, y_dtype, stream) != 0:
        raise RuntimeError(last_error())


def fused_dequant_matmul(qw, primary_codebook, residual_codebook, block_size, x, x_dtype=F32, y_dtype=F32):
    """Mirror of turboquant::fused_dequant_matmul (include/turboquant/dequantizer.h:33-39)."""
    out = qw.packed_primary.shape[0]
    inf = qw.packed_residual.shape[1] * 2
    layer = TurboQuantLinear(inf, out, qw, primary_codebook, residual_codebook, block_size)
    try:
        return layer.forward(x, x_dtype, y_dtype)
    finally:
        layer.close()


def dequantize_weight_gpu(qw, primary_codebook, residual_codebook, block_size):
    """Mirror of turboquant::dequantize_weight_gpu (include/turboquant/dequantizer.h:19-25)."""
    out = qw.packed_primary.shape[0]
    inf = qw.packed_residual.shape[1] * 2
    layer = TurboQuantLinear(inf, out, qw, primary_codebook, residual_codebook, block_size)
    try:
        return layer.dequantize()
    finally:
        layer.close()


def _rotate(matrix, seed, block_size, inverse):
    m = np.ascontiguousarray(matrix, dtype=np.float32)
    if m.ndim != 2:
        raise ValueError("matrix must be 2-D")
    out = np.empty_like(m)
    rc = lib().tq_wht_rotate_host(_p(m, _f32p), _p(out, _f32p), m.shape[0], m.shape[1], seed, block_size, inverse)
    if rc != 0:
        raise ValueError(last_error())
    return out


def apply_wht_rotation(matrix, seed, block_size):
    """Mirror of turboquant::apply_wht_rotation (include/turboquant/quantizer.h:31-35)."""
    return _rotate(matrix, seed, block_size, 0)


def apply_inverse_wht_rotation(matrix, seed, block_size):
    """Mirror of turboquant::apply_inverse_wht_rotation (include/turboquant/quantizer.h:37-42)."""
    return _rotate(matrix, seed, block_size, 1)


class Codebook:
    """Mirror of turboquant::Codebook (include/turboquant/codebook.h:24-29)."""

    def __init__(self, centroids, bits):
        self.centroids = np.ascontiguousarray(centroids, dtype=np.float32)
        self.bits = int(bits)
        self.boundaries = ((self.centroids[:-1] + self.centroids[1:]) * np.float32(0.5)).astype(np.float32)


def generate_codebook(bits):
    """Mirror of turboquant::generate_codebook (include/turboquant/codebook.h:33)."""
    c = np.empty(32, dtype=np.float32)
    n = lib().tq_generate_codebook(bits, _p(c, _f32p), None)
    if n < 0:
        raise ValueError(last_error())
    return Codebook(c[:n].copy(), bits)


class QuantizedWeight:
    """Mirror of turboquant::QuantizedWeight (include/turboquant/quantizer.h:22-27), numpy tensors."""

    def __init__(self, packed_primary, packed_residual, norms, seeds):
        self.packed_primary = packed_primary
        self.packed_residual = packed_residual
        self.norms = norms
        self.seeds = seeds


def quantize_weight(weight, primary_codebook, residual_codebook, primary_bits=4, residual_bits=4,
                    block_size=512, shared_rotation=False):
    """Mirror of turboquant::quantize_weight (include/turboquant/quantizer.h:54-60) on the GPU."""
    w = np.ascontiguousarray(weight, dtype=np.float32)
    if w.ndim != 2:
        raise ValueError("weight must be [out, in]")
    out, inf = w.shape
    pp = np.empty((out, inf // 2 if primary_bits <= 4 else inf), dtype=np.uint8)
    pr = np.empty((out, inf // 2), dtype=np.uint8)
    norms = np.empty(out, dtype=np.float32)
    seeds = np.empty(3, dtype=np.uint32)
    cp = np.ascontiguousarray(primary_codebook.centroids, dtype=np.float32)
    cr = np.ascontiguousarray(residual_codebook.centroids, dtype=np.float32)
    rc = lib().tq_quantize_weight_host(_p(w, _f32p), out, inf, _p(cp, _f32p), len(cp), _p(cr, _f32p), len(cr),
                                       primary_bits, residual_bits, block_size, int(shared_rotation),
                                       _p(pp, _u8p), _p(pr, _u8p), _p(norms, _f32p), _p(seeds, _u32p))
    if rc != 0:
        raise ValueError(last_error())
    return QuantizedWeight(pp, pr, norms, seeds)


def fit_layer_codebooks(weight, block_size, primary_bits=4, residual_bits=4, global_primary=None, iterations=100):
    """Per-layer codebooks as the reference's converter fits them (src/converter.cpp:291-372)."""
    w = np.ascontiguousarray(weight, dtype=np.float32)
    g = global_primary if global_primary is not None else generate_codebook(primary_bits)
    gc = np.ascontiguousarray(g.centroids, dtype=np.float32)
    cp = np.empty(32, dtype=np.float32)
    cr = np.empty(32, dtype=np.float32)
    rc = lib().tq_fit_layer_codebooks_host(_p(w, _f32p), w.shape[0], w.shape[1], block_size, primary_bits,
                                           residual_bits, _p(gc, _f32p), len(gc), iterations, _p(cp, _f32p), _p(cr, _f32p))
    if rc != 0:
        raise ValueError(last_error())
    cbp = Codebook(cp[:1 << primary_bits].copy(), primary_bits)
    cbr = Codebook(cr[:1 << residual_bits].copy(), residual_bits) if residual_bits > 0 else generate_codebook(4)
    return cbp, cbr


def best_block_size(in_features, max_block_size=512):
    """Block-size rule of the reference's converter (src/converter.cpp:228-240)."""
    return int(lib().tq_best_block_size(in_features, max_block_size))
