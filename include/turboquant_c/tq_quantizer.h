#ifndef TURBOQUANT_C_TQ_QUANTIZER_H
#define TURBOQUANT_C_TQ_QUANTIZER_H

/*
 * C-ABI for the offline TQ8 quantizer on AMD gfx950: the producer of the tensors
 * tq_linear_create consumes.  Same conventions as tq_linear.h (0 = success,
 * tq_last_error() for the message, nothing throws).  Weight matrices are device
 * (HIP) pointers; codebooks and seeds are small host arrays.
 */

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/**
 * Precomputed N(0,1) Lloyd-Max centroids for 1..5 bits and their midpoint
 * boundaries; replaces generate_codebook (include/turboquant/codebook.h:33,
 * src/codebook.cpp:16-57,72-85).  centroids[2^bits], boundaries[2^bits - 1]
 * (boundaries may be NULL).  Returns the centroid count, or -1 for an
 * unsupported width (the reference throws std::invalid_argument).
 */
int tq_generate_codebook(int bits, float* centroids_host, float* boundaries_host);

/**
 * Quantize one fp32 weight matrix [out, in] resident on the GPU; replaces
 * quantize_weight (include/turboquant/quantizer.h:54-60, src/quantizer.cpp:41-261)
 * with QuantizerConfig{primary_bits, residual_bits, block_size, shared_rotation}
 * (quantizer.h:11-19; norm correction is unconditional as in the reference).
 *
 *   packed_primary_dev  u8 [out, in/2] (primary_bits <= 4) or [out, in] (5 bits)
 *   packed_residual_dev u8 [out, in/2] (zero filled when residual_bits == 0)
 *   norms_dev           f32 [out]  corrected row norms
 *   seeds_host          u32 [3] = {seed_primary, shared ? 0 : seed_residual, block_size}
 *
 * Synchronous (returns after the GPU work has finished).
 */
int tq_quantize_weight(const float* weight_dev, int out_features, int in_features,
                       const float* cb_primary_host, int n_primary,
                       const float* cb_residual_host, int n_residual,
                       int primary_bits, int residual_bits, uint32_t block_size, int shared_rotation,
                       uint8_t* packed_primary_dev, uint8_t* packed_residual_dev,
                       float* norms_dev, uint32_t* seeds_host);

/** Same with host tensors (copies the weight to the GPU, quantizes, copies the results back). */
int tq_quantize_weight_host(const float* weight_host, int out_features, int in_features,
                            const float* cb_primary_host, int n_primary,
                            const float* cb_residual_host, int n_residual,
                            int primary_bits, int residual_bits, uint32_t block_size, int shared_rotation,
                            uint8_t* packed_primary_host, uint8_t* packed_residual_host,
                            float* norms_host, uint32_t* seeds_host);

/**
 * Per-layer codebooks as the reference's converter fits them
 * (src/converter.cpp:291-372 with generate_codebook_from_data_cpu,
 * src/codebook.cpp:99-143): the primary codebook on the rotated * sqrt(in)
 * samples of the normalised rows, the residual codebook on the residuals taken
 * against the GLOBAL primary codebook, both from the analytic start, at most
 * `iterations` Lloyd-Max steps (the reference uses 100), stop when no centroid
 * moves by 1e-6.  Outputs 2^bits centroids each (residual untouched when
 * residual_bits == 0).  Needs 4*out*in bytes of temporary device memory.
 */
int tq_fit_layer_codebooks(const float* weight_dev, int out_features, int in_features,
                           uint32_t block_size, int primary_bits, int residual_bits,
                           const float* global_primary_host, int n_global_primary, int iterations,
                           float* cb_primary_host_out, float* cb_residual_host_out);

/** Same with a host weight matrix. */
int tq_fit_layer_codebooks_host(const float* weight_host, int out_features, int in_features,
                                uint32_t block_size, int primary_bits, int residual_bits,
                                const float* global_primary_host, int n_global_primary, int iterations,
                                float* cb_primary_host_out, float* cb_residual_host_out);

/**
 * Largest power of two <= max_block_size that divides in_features
 * (src/converter.cpp:228-240).
 */
uint32_t tq_best_block_size(int in_features, uint32_t max_block_size);

/* generate_codebook_from_data (reference src/codebook.cpp:99-143,284-302 -- the CPU form, which the
 * converter's workers force): Lloyd-Max from the analytic initialisation, lower_bound bins,
 * double-precision bin sums, at most `iterations` rounds, stop below a 1e-6 shift.  The
 * assignment pass runs on the GPU.  n == 0 returns the analytic codebook.  Returns the number of
 * centroids written, -1 on error.  boundaries_out may be NULL. */
int tq_generate_codebook_from_data_host(const float* data_host, size_t n, int bits, int iterations,
                                        float* centroids_out, float* boundaries_out);

/* quantize / dequantize of reference src/codebook.cpp:284-321 as elementwise GPU maps over host
 * buffers: lower_bound over the n_centroids-1 boundaries, clamp to the last bin; index -> centroid
 * with the same clamp.  Return 0 on success. */
int tq_codebook_quantize_host(const float* values_host, size_t n, const float* boundaries_host, int n_centroids,
                              uint8_t* indices_host);
int tq_codebook_dequantize_host(const uint8_t* indices_host, size_t n, const float* centroids_host, int n_centroids,
                                float* values_host);

#ifdef __cplusplus
}
#endif

#endif /* TURBOQUANT_C_TQ_QUANTIZER_H */
