#ifndef TURBOQUANT_C_TQ_LINEAR_H
#define TURBOQUANT_C_TQ_LINEAR_H

/*
 * C-ABI for the TQ8 quantized-linear forward path on AMD gfx950.
 *
 * The reference exposes this path only through its C++ API
 * (include/turboquant/linear.h:11-35, include/turboquant/dequantizer.h:11-39,
 * include/turboquant/quantizer.h:22-60); its C header has no per-layer entry
 * (include/turboquant_c/turboquant_c.h:25-31 - tq_model_forward is a stub,
 * src/turboquant_c.cpp:71-77).  The functions below are what a cgo / Swift /
 * N-API / ctypes binding for that path binds: plain pointers and sizes only.
 *
 * Conventions (same as src/turboquant_c.cpp): nothing throws across this
 * boundary; constructors return NULL on failure, int functions return 0 on
 * success and non-zero on failure, every *_free(NULL) is a no-op, getters on
 * NULL return 0.  tq_last_error() gives the message of the calling thread's
 * last failure.
 *
 * Pointers named *_dev are device (HIP) pointers, *_host are host pointers.
 * `stream` is a hipStream_t passed as void* (NULL = the default stream);
 * calls with a stream argument are asynchronous on it.
 */

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tq_linear_s* tq_linear_t;

/* Element types accepted for activations and outputs.  The reference casts
 * activations to f16 and returns f16 (src/dequantizer.cpp:691,713-715). */
enum { TQ_DTYPE_F32 = 0, TQ_DTYPE_F16 = 1, TQ_DTYPE_BF16 = 2 };

/* Decode mode inferred from the tensors exactly as the reference does
 * (src/dequantizer.cpp:72-75,118-133,674-675). */
enum {
    TQ_MODE_PRIMARY_ONLY    = 0,  /* packed_residual all zero                       */
    TQ_MODE_SHARED_LUT      = 1,  /* seeds[1]==0, residual present, 4-bit primary   */
    TQ_MODE_DUAL            = 2,  /* seeds[1]!=0, residual present                  */
    TQ_MODE_SHARED_5BIT     = 3,  /* seeds[1]==0, residual present, 5-bit primary   */
    TQ_MODE_PRIMARY_ONLY_5BIT = 4,
    TQ_MODE_DUAL_5BIT       = 5
};

/** Message of the calling thread's last failed call ("" if none). */
const char* tq_last_error(void);

/**
 * Build a TQ8 linear layer from host tensors; replaces
 * TurboQuantLinear::TurboQuantLinear (include/turboquant/linear.h:13-19,
 * src/linear.cpp:6-18) together with struct QuantizedWeight
 * (include/turboquant/quantizer.h:22-27) and struct Codebook
 * (include/turboquant/codebook.h:24-29).
 *
 *   packed_primary  u8 [out_features, primary_cols]   primary_cols = in/2 (4-bit) or in (5-bit)
 *   packed_residual u8 [out_features, residual_cols]  residual_cols = in/2
 *   norms           f32 [out_features]
 *   seeds           u32 [3] = {seed_primary, seed_residual or 0, block_size}
 *   cb_primary      f32 [n_primary], cb_residual f32 [n_residual]
 *
 * The tensors are copied to the GPU once; the handle owns the copies.
 */
tq_linear_t tq_linear_create(int in_features, int out_features,
                             const uint8_t* packed_primary_host, int primary_cols,
                             const uint8_t* packed_residual_host, int residual_cols,
                             const float* norms_host, const uint32_t* seeds_host,
                             const float* cb_primary_host, int n_primary,
                             const float* cb_residual_host, int n_residual,
                             uint32_t block_size);

/** Same, from tensors already resident on the GPU (copied device to device). */
tq_linear_t tq_linear_create_from_device(int in_features, int out_features,
                             const uint8_t* packed_primary_dev, int primary_cols,
                             const uint8_t* packed_residual_dev, int residual_cols,
                             const float* norms_dev, const uint32_t* seeds_host,
                             const float* cb_primary_host, int n_primary,
                             const float* cb_residual_host, int n_residual,
                             uint32_t block_size);

/** TurboQuantLinear::in_features / out_features (include/turboquant/linear.h:24-25). */
int tq_linear_in_features(tq_linear_t layer);
int tq_linear_out_features(tq_linear_t layer);
/** One of TQ_MODE_*. */
int tq_linear_mode(tq_linear_t layer);

/**
 * y[batch, out] = x[batch, in] . W^T; replaces TurboQuantLinear::forward
 * (include/turboquant/linear.h:21-22, src/linear.cpp:20-26) and
 * fused_dequant_matmul (include/turboquant/dequantizer.h:33-39,
 * src/dequantizer.cpp:606-721).  Accumulation is fp32.  x and y are dense
 * row-major device buffers of the given element types.
 */
int tq_linear_forward(tq_linear_t layer, const void* x_dev, int x_dtype, int batch,
                      void* y_dev, int y_dtype, void* stream);

/**
 * Size the layer's workspaces for calls of up to max_batch rows now, so that no later
 * tq_linear_forward / tq_linear_forward_group call with at most that many rows allocates (the
 * matrix-core paths for 2 or more rows otherwise allocate on first use, which
 * synchronises the device and cannot be captured in a HIP graph; a call that would have to grow a
 * workspace while its stream is being captured fails instead).  The reference allocates its output
 * per call (src/dequantizer.cpp:516) and has no such entry.
 */
int tq_linear_reserve(tq_linear_t layer, int max_batch);

/**
 * tq_linear_forward for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same
 * kernels and the same results as tq_linear_forward, but the workspaces of the matrix-core paths
 * (2 or more rows: rotated activations and partial
 * products) live in a fixed array of TQ_STATIC_SCRATCH_BYTES inside the library instead of buffers the
 * handle allocates on first use; the call allocates and frees nothing.  It fails (non-zero,
 * tq_last_error says how many bytes were needed) when layer and batch need more than that.  (From 16
 * rows on, a layer with few output tiles cuts K into ranges whose fp32 products are added afterwards:
 * here into as many ranges as the array holds, so the last bits of a result can differ from
 * tq_linear_forward's by the order of those sums.)  Each GPU has one such array, shared
 * by every call on it and keeping the previous call's contents: calls that overlap on one GPU
 * (different streams or threads) race.  One row uses no part of the array (layers wider than 16384 columns,
 * widths that are not a multiple of 32 and 5-bit layers that keep two planes use the handle's own rotated row
 * at one row too: serialise calls per handle on those, as with tq_linear_forward).  The array's address on the
 * current device is looked up when a layer is created, so the first call does no runtime work either.
 */
#define TQ_STATIC_SCRATCH_BYTES (32u << 20)
int tq_linear_forward_static(tq_linear_t layer, const void* x_dev, int x_dtype, int batch,
                             void* y_dev, int y_dtype, void* stream);

/**
 * One to three layers applied to the SAME activations: y_devs[j][batch, out_j] = x[batch, in] . W_j^T,
 * e.g. the q, k, v or the gate, up projections of a decoder layer.  Layers of equal width and mode share
 * their kernel launches where the kernels allow it (batch 1: shared or dual rotation, blocks <= 512, more
 * than 2048 columns for shared rotation; 2..32 rows: blocks <= 512);
 * anything else is run one layer after the other.  Results are identical to n calls of tq_linear_forward.
 * No counterpart in the reference, whose forward is per layer (include/turboquant/linear.h:21-22).
 */
int tq_linear_forward_group(const tq_linear_t* layers, int n, const void* x_dev, int x_dtype, int batch,
                            void* const* y_devs, int y_dtype, void* stream);

/** Same with host buffers (copies in, runs, copies out, synchronises). */
int tq_linear_forward_host(tq_linear_t layer, const void* x_host, int x_dtype, int batch,
                           void* y_host, int y_dtype);

/**
 * Materialise the dequantised weight f32 [out, in]; replaces
 * dequantize_weight_gpu (include/turboquant/dequantizer.h:19-25,
 * src/dequantizer.cpp:347-451) and follows dequantize_weight_cpu
 * (src/dequantizer.cpp:52-256) operation by operation.
 */
int tq_linear_dequantize(tq_linear_t layer, float* w_dev, void* stream);
int tq_linear_dequantize_host(tq_linear_t layer, float* w_host);

/* Same dequantisation with the fp32 result rounded to nearest-even into w_dtype
 * (TQ_DTYPE_F32 / F16 / BF16): the cast src/turboquant_c_dequant.cpp:155-167 applies
 * before it writes a weight back to a safetensors file, fused into the kernel's store. */
int tq_linear_dequantize_as(tq_linear_t layer, void* w_dev, int w_dtype, void* stream);
int tq_linear_dequantize_as_host(tq_linear_t layer, void* w_host, int w_dtype);

/** Release the layer and its device buffers.  Safe to call with NULL. */
void tq_linear_free(tq_linear_t layer);

/**
 * Blockwise randomised Walsh-Hadamard rotation of f32 [rows, cols] on the GPU;
 * replaces apply_wht_rotation / apply_inverse_wht_rotation
 * (include/turboquant/quantizer.h:31-42, src/rotation.cpp:291-350,364-403).
 * inverse == 0: sign -> FWHT -> 1/sqrt(bs); inverse != 0: FWHT -> 1/sqrt(bs)*sign.
 * Fails (non-zero) when cols is not a multiple of block_size, where the
 * reference asserts (src/rotation.cpp:374,396).  in_dev may equal out_dev.
 */
int tq_wht_rotate(const float* in_dev, float* out_dev, int rows, int cols,
                  uint32_t seed, uint32_t block_size, int inverse, void* stream);
int tq_wht_rotate_host(const float* in_host, float* out_host, int rows, int cols,
                       uint32_t seed, uint32_t block_size, int inverse);

#ifdef __cplusplus
}
#endif

#endif /* TURBOQUANT_C_TQ_LINEAR_H */
