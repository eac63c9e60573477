/*
 * TEST INFRASTRUCTURE - NOT PRODUCT CODE.
 *
 * CPU restatement of the TurboQuant TQ8 quantize / dequantize / linear path,
 * written in plain C so the GPU kernels can be checked against it.  Only the
 * tests, the smoke check and the benchmark's CPU-baseline leg may link or call
 * anything declared here; the shipped library never does.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the reference checkout).  Where the reference leaves an operation's
 * summation order to its tensor runtime (row-norm `sum`, test-side `matmul`)
 * the header says "parity unpinned" and names the order used here.
 */
#ifndef TQ_ORACLE_H
#define TQ_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Number of worker threads for the row-parallel loops (1 = the reference's
 * serial loops).  Rows are independent, so results do not depend on it, except
 * tqo_lloyd_max whose double-precision bin sums are reduced per thread. */
void tqo_set_threads(int n);
int  tqo_get_threads(void);

/* src/rotation.cpp:32-42  make_signs: +-1 from a u32 hash of (seed, index in block). */
float tqo_sign(uint32_t seed, uint32_t index);
void  tqo_make_signs(uint32_t seed, uint32_t block_size, float* signs);

/* src/rotation.cpp:14-25  fwht_inplace: unnormalised natural-order butterfly. */
void tqo_fwht_inplace(float* data, int n);

/* src/rotation.cpp:291-319  apply_wht_rotation_cpu: sign -> FWHT -> *1/sqrt(bs).
 * Returns 0, or -1 when cols is not a multiple of block_size (the reference
 * asserts, src/rotation.cpp:374). */
int tqo_wht_forward(const float* in, float* out, int rows, int cols,
                    uint32_t seed, uint32_t block_size);
/* src/rotation.cpp:323-350  apply_inverse_wht_rotation_cpu: FWHT -> *(1/sqrt(bs)*sign). */
int tqo_wht_inverse(const float* in, float* out, int rows, int cols,
                    uint32_t seed, uint32_t block_size);

/* src/codebook.cpp:16-57,72-85  generate_codebook: literal N(0,1) Lloyd-Max
 * tables for 1..5 bits; boundaries are midpoints.  Returns the centroid count
 * (2^bits) or -1 for an unsupported width.  boundaries may be NULL. */
int tqo_codebook_analytic(int bits, float* centroids, float* boundaries);
/* src/codebook.cpp:49-57  midpoints (c[i]+c[i+1])*0.5f. */
void tqo_boundaries(const float* centroids, int n, float* boundaries);
/* src/codebook.cpp:322-353  validate_codebook (analytical != 0 adds the exact symmetry test). */
int tqo_validate_codebook(const float* centroids, int n_centroids,
                          const float* boundaries, int n_boundaries,
                          int bits, int analytical);

/* src/codebook.cpp:284-302  quantize: std::lower_bound over the boundaries,
 * i.e. index = number of boundaries strictly below v; a value equal to a
 * boundary goes to the lower bin. */
void tqo_quantize(const float* values, size_t n, const float* boundaries,
                  int n_centroids, uint8_t* indices);
/* src/codebook.cpp:304-320  dequantize with index clamp. */
void tqo_dequantize(const uint8_t* indices, size_t n, const float* centroids,
                    int n_centroids, float* out);

/* src/quantizer.cpp:33-39  pack_4bit: lo | hi<<4;  src/dequantizer.cpp:43-50  unpack_4bit. */
void tqo_pack4(const uint8_t* indices, size_t count, uint8_t* packed);
void tqo_unpack4(const uint8_t* packed, size_t packed_count, uint8_t* indices);

/* src/quantizer.cpp:12-28  derive_seed: FNV-1a over sampled bytes of the fp32 weight. */
uint32_t tqo_derive_seed(const float* weight, size_t n_floats, uint32_t salt);

/* src/codebook.cpp:99-143  generate_codebook_from_data_cpu.  Returns the
 * number of iterations executed.  centroids[2^bits], boundaries[2^bits-1]. */
int tqo_lloyd_max(const float* data, size_t n, int bits, int iterations,
                  float* centroids, float* boundaries);

/* src/converter.cpp:228-240  largest power of two <= max_block_size dividing in_features. */
uint32_t tqo_best_block_size(int in_features, uint32_t max_block_size);

/* src/converter.cpp:291-372  per-layer codebook recipe: primary fitted on the
 * rotated*sqrt(in) values, residual fitted on residuals taken against the
 * GLOBAL codebook (global_primary_*), both with 100 iterations. */
int tqo_fit_layer_codebooks(const float* weight, int out_features, int in_features,
                            uint32_t block_size, int primary_bits, int residual_bits,
                            const float* global_primary_centroids, int n_global_primary,
                            float* primary_centroids, float* residual_centroids);

/* src/quantizer.cpp:41-261  quantize_weight.
 *   packed_primary : [out, in/2] (primary_bits<=4) or [out, in] (5 bit)
 *   packed_residual: [out, in/2] (zero filled when residual_bits == 0)
 *   norms          : f32 [out]   corrected row norms
 *   seeds          : u32 [3]     {seed_primary, shared ? 0 : seed_residual, block_size}
 * Row norms: the reference uses its runtime's `sum` (order unspecified, parity
 * unpinned); here each row is accumulated in double and rounded to float. */
int tqo_quantize_weight(const float* weight, int out_features, int in_features,
                        const float* cbp_centroids, int n_cbp,
                        const float* cbr_centroids, int n_cbr,
                        int primary_bits, int residual_bits, uint32_t block_size,
                        int shared_rotation,
                        uint8_t* packed_primary, uint8_t* packed_residual,
                        float* norms, uint32_t* seeds);

/* src/dequantizer.cpp:52-256  dequantize_weight_cpu (paths A, B, C), with the
 * inverse WHT taken from src/rotation.cpp:323-350.  primary_cols is the second
 * dimension of packed_primary, residual_cols of packed_residual; the mode is
 * inferred exactly as the reference does (src/dequantizer.cpp:72-75,118-133).
 * out_weight: f32 [out, in]. */
int tqo_dequantize_weight(const uint8_t* packed_primary, int primary_cols,
                          const uint8_t* packed_residual, int residual_cols,
                          const float* norms, const uint32_t* seeds,
                          int out_features,
                          const float* cbp_centroids, int n_cbp,
                          const float* cbr_centroids, int n_cbr,
                          uint32_t block_size, float* out_weight);

/* tests/integration/test_linear.cpp:102-107  reference forward used by the
 * reference's own tests: y = x . W^T in fp32.  The reference's matmul order is
 * its runtime's (parity unpinned); here each output is a sequential fp32
 * accumulation over k when acc_double == 0, or double accumulation rounded
 * once when acc_double != 0. */
void tqo_matmul_xwT(const float* x, const float* w, int batch, int in_features,
                    int out_features, float* y, int acc_double);

/* bf16 <-> f32 helpers (round to nearest even), used to build test inputs. */
uint16_t tqo_f32_to_bf16(float f);
float    tqo_bf16_to_f32(uint16_t h);

#ifdef __cplusplus
}
#endif
#endif /* TQ_ORACLE_H */
