/*
 * TEST INFRASTRUCTURE - NOT PRODUCT CODE.  See tq_oracle.h.
 *
 * Plain-C restatement of the reference CPU path.  Floating point follows the
 * reference operation by operation in fp32 (build with -ffp-contract=off so
 * no multiply-add is fused).
 */
#include "tq_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static int g_threads = 1;

void tqo_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
int  tqo_get_threads(void) { return g_threads; }

/* ---- sign hash: src/rotation.cpp:32-42 --------------------------------- */

float tqo_sign(uint32_t seed, uint32_t index) {
    uint32_t h = seed * 2654435761u + index * 2246822519u;
    h ^= h >> 16;
    h *= 0x45d9f3bu;
    h ^= h >> 16;
    return (h & 1u) ? 1.0f : -1.0f;
}

void tqo_make_signs(uint32_t seed, uint32_t block_size, float* signs) {
    for (uint32_t i = 0; i < block_size; ++i) signs[i] = tqo_sign(seed, i);
}

/* ---- butterfly: src/rotation.cpp:14-25 --------------------------------- */

void tqo_fwht_inplace(float* data, int n) {
    for (int h = 1; h < n; h <<= 1) {
        for (int i = 0; i < n; i += h << 1) {
            for (int j = i; j < i + h; ++j) {
                float a = data[j];
                float b = data[j + h];
                data[j]     = a + b;
                data[j + h] = a - b;
            }
        }
    }
}

/* ---- block rotations: src/rotation.cpp:291-350 -------------------------- */

int tqo_wht_forward(const float* in, float* out, int rows, int cols,
                    uint32_t seed, uint32_t block_size) {
    const int bs = (int)block_size;
    if (bs <= 0 || cols % bs != 0) return -1;
    const int num_full = cols / bs;
    const float inv_sqrt = 1.0f / sqrtf((float)bs);
    float* signs = (float*)malloc(sizeof(float) * (size_t)bs);
    tqo_make_signs(seed, block_size, signs);
    if (out != in) memcpy(out, in, sizeof(float) * (size_t)rows * (size_t)cols);
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int r = 0; r < rows; ++r) {
        float* row = out + (size_t)r * (size_t)cols;
        for (int b = 0; b < num_full; ++b) {
            float* blk = row + (size_t)b * bs;
            for (int j = 0; j < bs; ++j) blk[j] *= signs[j];
            tqo_fwht_inplace(blk, bs);
            for (int j = 0; j < bs; ++j) blk[j] *= inv_sqrt;
        }
    }
    free(signs);
    return 0;
}

int tqo_wht_inverse(const float* in, float* out, int rows, int cols,
                    uint32_t seed, uint32_t block_size) {
    const int bs = (int)block_size;
    if (bs <= 0 || cols % bs != 0) return -1;
    const int num_full = cols / bs;
    const float inv_sqrt = 1.0f / sqrtf((float)bs);
    float* signs = (float*)malloc(sizeof(float) * (size_t)bs);
    tqo_make_signs(seed, block_size, signs);
    if (out != in) memcpy(out, in, sizeof(float) * (size_t)rows * (size_t)cols);
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int r = 0; r < rows; ++r) {
        float* row = out + (size_t)r * (size_t)cols;
        for (int b = 0; b < num_full; ++b) {
            float* blk = row + (size_t)b * bs;
            tqo_fwht_inplace(blk, bs);
            for (int j = 0; j < bs; ++j) blk[j] *= inv_sqrt * signs[j];
        }
    }
    free(signs);
    return 0;
}

/* ---- codebooks: src/codebook.cpp:16-85 ---------------------------------- */

static const float kC1[] = { -0.7978845608f, 0.7978845608f };
static const float kC2[] = { -1.510232f, -0.4527800f, 0.4527800f, 1.510232f };
static const float kC3[] = {
    -2.152176f, -1.344318f, -0.756130f, -0.245379f,
     0.245379f,  0.756130f,  1.344318f,  2.152176f };
static const float kC4[] = {
    -2.732590f, -2.069017f, -1.618046f, -1.256231f,
    -0.942340f, -0.656759f, -0.388048f, -0.128395f,
     0.128395f,  0.388048f,  0.656759f,  0.942340f,
     1.256231f,  1.618046f,  2.069017f,  2.732590f };
static const float kC5[] = {
    -3.255544f, -2.685239f, -2.311434f, -2.022174f,
    -1.780580f, -1.569614f, -1.379896f, -1.205655f,
    -1.043046f, -0.889350f, -0.742542f, -0.601049f,
    -0.463598f, -0.329119f, -0.196679f, -0.065429f,
     0.065429f,  0.196679f,  0.329119f,  0.463598f,
     0.601049f,  0.742542f,  0.889350f,  1.043046f,
     1.205655f,  1.379896f,  1.569614f,  1.780580f,
     2.022174f,  2.311434f,  2.685239f,  3.255544f };

void tqo_boundaries(const float* c, int n, float* b) {
    for (int i = 0; i + 1 < n; ++i) b[i] = (c[i] + c[i + 1]) * 0.5f;
}

int tqo_codebook_analytic(int bits, float* centroids, float* boundaries) {
    const float* src;
    switch (bits) {
        case 1: src = kC1; break;
        case 2: src = kC2; break;
        case 3: src = kC3; break;
        case 4: src = kC4; break;
        case 5: src = kC5; break;
        default: return -1;
    }
    const int n = 1 << bits;
    memcpy(centroids, src, sizeof(float) * (size_t)n);
    if (boundaries) tqo_boundaries(centroids, n, boundaries);
    return n;
}

int tqo_validate_codebook(const float* c, int n, const float* b, int nb,
                          int bits, int analytical) {
    if (n != (1 << bits)) return 0;
    for (int i = 1; i < n; ++i) if (c[i] <= c[i - 1]) return 0;
    if (nb != n - 1) return 0;
    for (int i = 0; i < nb; ++i) {
        float mid = (c[i] + c[i + 1]) * 0.5f;
        if (fabsf(b[i] - mid) > 1e-5f) return 0;
    }
    if (analytical) {
        for (int i = 0; i < n / 2; ++i) if (c[i] + c[n - 1 - i] != 0.0f) return 0;
    }
    return 1;
}

/* ---- scalar quantise / dequantise: src/codebook.cpp:284-320 ------------- */

/* std::lower_bound: first boundary that is not < v. */
static inline int lower_bound_idx(const float* b, int nb, float v) {
    int lo = 0, len = nb;
    while (len > 0) {
        int half = len >> 1;
        if (b[lo + half] < v) { lo += half + 1; len -= half + 1; }
        else len = half;
    }
    return lo;
}

void tqo_quantize(const float* values, size_t n, const float* boundaries,
                  int n_centroids, uint8_t* indices) {
    const int nb = n_centroids - 1;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (size_t i = 0; i < n; ++i) {
        int idx = lower_bound_idx(boundaries, nb, values[i]);
        if (idx >= n_centroids) idx = n_centroids - 1;
        indices[i] = (uint8_t)idx;
    }
}

void tqo_dequantize(const uint8_t* indices, size_t n, const float* centroids,
                    int n_centroids, float* out) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (size_t i = 0; i < n; ++i) {
        size_t idx = indices[i];
        if (idx >= (size_t)n_centroids) idx = (size_t)n_centroids - 1;
        out[i] = centroids[idx];
    }
}

/* ---- nibble packing: src/quantizer.cpp:33-39, src/dequantizer.cpp:43-50 - */

void tqo_pack4(const uint8_t* indices, size_t count, uint8_t* packed) {
    for (size_t i = 0; i + 1 < count; i += 2)
        packed[i / 2] = (uint8_t)((indices[i] & 0x0F) | ((indices[i + 1] & 0x0F) << 4));
}

void tqo_unpack4(const uint8_t* packed, size_t packed_count, uint8_t* indices) {
    for (size_t i = 0; i < packed_count; ++i) {
        indices[i * 2]     = packed[i] & 0x0F;
        indices[i * 2 + 1] = (packed[i] >> 4) & 0x0F;
    }
}

/* ---- content-derived seed: src/quantizer.cpp:12-28 ---------------------- */

uint32_t tqo_derive_seed(const float* weight, size_t n_floats, uint32_t salt) {
    uint32_t hash = 2166136261u ^ salt;
    const uint8_t* bytes = (const uint8_t*)weight;
    size_t byte_count = n_floats * sizeof(float);
    size_t stride = (byte_count > 4096) ? (byte_count / 4096) : 1;
    for (size_t i = 0; i < byte_count; i += stride) {
        hash ^= bytes[i];
        hash *= 16777619u;
    }
    return hash;
}

/* ---- Lloyd-Max fit: src/codebook.cpp:99-143 ----------------------------- */

int tqo_lloyd_max(const float* data, size_t n, int bits, int iterations,
                  float* centroids, float* boundaries) {
    const int nc = tqo_codebook_analytic(bits, centroids, boundaries);
    if (nc < 0) return -1;
    if (n == 0) return 0;               /* src/codebook.cpp:270-272 */
    const int nb = nc - 1;
    const int T = g_threads;
    double* tsum = (double*)malloc(sizeof(double) * (size_t)T * (size_t)nc);
    size_t* tcnt = (size_t*)malloc(sizeof(size_t) * (size_t)T * (size_t)nc);
    int done = 0;
    for (int iter = 0; iter < iterations; ++iter) {
        tqo_boundaries(centroids, nc, boundaries);
        memset(tsum, 0, sizeof(double) * (size_t)T * (size_t)nc);
        memset(tcnt, 0, sizeof(size_t) * (size_t)T * (size_t)nc);
#pragma omp parallel num_threads(T)
        {
            int t = 0, nt = 1;
#ifdef _OPENMP
            t = omp_get_thread_num();
            nt = omp_get_num_threads();
#endif
            size_t lo = n * (size_t)t / (size_t)nt, hi = n * (size_t)(t + 1) / (size_t)nt;
            double* s = tsum + (size_t)t * nc;
            size_t* c = tcnt + (size_t)t * nc;
            for (size_t i = lo; i < hi; ++i) {
                int idx = lower_bound_idx(boundaries, nb, data[i]);
                if (idx >= nc) idx = nc - 1;
                s[idx] += (double)data[i];
                c[idx]++;
            }
        }
        float max_shift = 0.0f;
        for (int k = 0; k < nc; ++k) {
            double bs = 0.0; size_t bc = 0;
            for (int t = 0; t < T; ++t) { bs += tsum[(size_t)t * nc + k]; bc += tcnt[(size_t)t * nc + k]; }
            if (bc > 0) {
                float nv = (float)(bs / (double)bc);
                float shift = fabsf(nv - centroids[k]);
                if (shift > max_shift) max_shift = shift;
                centroids[k] = nv;
            }
        }
        done = iter + 1;
        if (max_shift < 1e-6f) break;
    }
    tqo_boundaries(centroids, nc, boundaries);
    free(tsum); free(tcnt);
    return done;
}

/* ---- block-size rule: src/converter.cpp:228-240 ------------------------- */

uint32_t tqo_best_block_size(int in_features, uint32_t max_block_size) {
    uint32_t best = 1;
    for (int p = 1; p < 20; ++p) {
        uint32_t c = 1u << p;
        if (c > max_block_size) break;
        if (in_features % (int)c == 0) best = c;
    }
    return best;
}

/* ---- shared helpers for the quantizer ----------------------------------- */

/* rows normalised by max(norm, 1e-10): src/quantizer.cpp:56-66.  Row sum of
 * squares is accumulated in double and rounded to float (parity unpinned). */
static void normalise_rows(const float* w, int out, int in, float* wn, float* norms) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int r = 0; r < out; ++r) {
        const float* row = w + (size_t)r * in;
        double acc = 0.0;
        for (int j = 0; j < in; ++j) { float sq = row[j] * row[j]; acc += (double)sq; }
        float nrm = sqrtf((float)acc);
        if (norms) norms[r] = nrm;
        float safe = nrm > 1e-10f ? nrm : 1e-10f;
        float* o = wn + (size_t)r * in;
        for (int j = 0; j < in; ++j) o[j] = row[j] / safe;
    }
}

static void scale_inplace(float* v, size_t n, float s) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (size_t i = 0; i < n; ++i) v[i] *= s;
}

/* ---- per-layer codebooks: src/converter.cpp:291-372 --------------------- */

int tqo_fit_layer_codebooks(const float* weight, int out, int in,
                            uint32_t block_size, int primary_bits, int residual_bits,
                            const float* gcp, int n_gcp,
                            float* primary_centroids, float* residual_centroids) {
    const size_t total = (size_t)out * (size_t)in;
    const float scale_factor = sqrtf((float)in);
    float* scaled = (float*)malloc(sizeof(float) * total);
    if (!scaled) return -1;
    normalise_rows(weight, out, in, scaled, NULL);
    uint32_t seed_p = tqo_derive_seed(weight, total, 0u);
    if (tqo_wht_forward(scaled, scaled, out, in, seed_p, block_size) != 0) { free(scaled); return -1; }
    scale_inplace(scaled, total, scale_factor);

    float bnd[32];
    if (tqo_lloyd_max(scaled, total, primary_bits, 100, primary_centroids, bnd) < 0) { free(scaled); return -1; }

    if (residual_bits > 0) {
        float gb[32];
        tqo_boundaries(gcp, n_gcp, gb);
        uint8_t* idx = (uint8_t*)malloc(total);
        tqo_quantize(scaled, total, gb, n_gcp, idx);
#pragma omp parallel for num_threads(g_threads) schedule(static)
        for (size_t i = 0; i < total; ++i) {
            size_t k = idx[i]; if (k >= (size_t)n_gcp) k = (size_t)n_gcp - 1;
            scaled[i] = scaled[i] - gcp[k];
        }
        free(idx);
        if (tqo_lloyd_max(scaled, total, residual_bits, 100, residual_centroids, bnd) < 0) { free(scaled); return -1; }
    }
    free(scaled);
    return 0;
}

/* ---- quantize_weight: src/quantizer.cpp:41-261 -------------------------- */

int tqo_quantize_weight(const float* weight, int out, int in,
                        const float* cbp, int n_cbp,
                        const float* cbr, int n_cbr,
                        int primary_bits, int residual_bits, uint32_t block_size,
                        int shared_rotation,
                        uint8_t* packed_primary, uint8_t* packed_residual,
                        float* norms, uint32_t* seeds) {
    if (out <= 0 || in <= 0 || (in & 1)) return -1;
    if (block_size == 0 || in % (int)block_size != 0) return -1;
    const size_t total = (size_t)out * (size_t)in;
    const float scale_factor = sqrtf((float)in);
    const float inv_scale = 1.0f / scale_factor;

    float bp[32], br[32];
    tqo_boundaries(cbp, n_cbp, bp);
    tqo_boundaries(cbr, n_cbr, br);

    float* orig_norm = (float*)malloc(sizeof(float) * (size_t)out);
    float* scaled = (float*)malloc(sizeof(float) * total);
    float* work = (float*)malloc(sizeof(float) * total);
    uint8_t* idx_p = (uint8_t*)malloc(total);
    uint8_t* idx_r = (uint8_t*)malloc(total);
    if (!orig_norm || !scaled || !work || !idx_p || !idx_r) {
        free(orig_norm); free(scaled); free(work); free(idx_p); free(idx_r); return -1;
    }

    /* Step 1-2: norms, normalise, seeds (:56-70) */
    normalise_rows(weight, out, in, scaled, orig_norm);
    const uint32_t seed_p = tqo_derive_seed(weight, total, 0u);
    const uint32_t seed_r = tqo_derive_seed(weight, total, 1u);

    /* Step 3: rotate, scale, quantise, pack (:74-107) */
    tqo_wht_forward(scaled, scaled, out, in, seed_p, block_size);
    scale_inplace(scaled, total, scale_factor);
    tqo_quantize(scaled, total, bp, n_cbp, idx_p);
    if (primary_bits <= 4) tqo_pack4(idx_p, total, packed_primary);
    else memcpy(packed_primary, idx_p, total);

    /* Step 4: residual (:111-160) */
    memset(packed_residual, 0, total / 2);
    if (residual_bits > 0) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
        for (size_t i = 0; i < total; ++i) {
            size_t k = idx_p[i]; if (k >= (size_t)n_cbp) k = (size_t)n_cbp - 1;
            work[i] = scaled[i] - cbp[k];
        }
        if (!shared_rotation) {
            scale_inplace(work, total, inv_scale);
            tqo_wht_inverse(work, work, out, in, seed_p, block_size);
            tqo_wht_forward(work, work, out, in, seed_r, block_size);
            scale_inplace(work, total, scale_factor);
        }
        tqo_quantize(work, total, br, n_cbr, idx_r);
        tqo_pack4(idx_r, total, packed_residual);
    }

    /* Step 5: reconstruction in normalised space (:166-234) */
    float* recon = scaled;              /* `scaled` is dead from here on */
    if (residual_bits > 0 && shared_rotation) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
        for (size_t i = 0; i < total; ++i) {
            size_t k = idx_p[i]; if (k >= (size_t)n_cbp) k = (size_t)n_cbp - 1;
            size_t q = idx_r[i] & 0x0F; if (q >= (size_t)n_cbr) q = (size_t)n_cbr - 1;
            float combined = cbp[k] + cbr[q];
            recon[i] = combined * inv_scale;
        }
        tqo_wht_inverse(recon, recon, out, in, seed_p, block_size);
    } else {
#pragma omp parallel for num_threads(g_threads) schedule(static)
        for (size_t i = 0; i < total; ++i) {
            size_t k = idx_p[i]; if (k >= (size_t)n_cbp) k = (size_t)n_cbp - 1;
            recon[i] = cbp[k] * inv_scale;
        }
        tqo_wht_inverse(recon, recon, out, in, seed_p, block_size);
        if (residual_bits > 0) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
            for (size_t i = 0; i < total; ++i) {
                size_t q = idx_r[i] & 0x0F; if (q >= (size_t)n_cbr) q = (size_t)n_cbr - 1;
                work[i] = cbr[q] * inv_scale;
            }
            tqo_wht_inverse(work, work, out, in, seed_r, block_size);
#pragma omp parallel for num_threads(g_threads) schedule(static)
            for (size_t i = 0; i < total; ++i) recon[i] = recon[i] + work[i];
        }
    }

    /* corrected norms (:237-248); row sum in double, rounded (parity unpinned) */
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int r = 0; r < out; ++r) {
        const float* row = recon + (size_t)r * in;
        double acc = 0.0;
        for (int j = 0; j < in; ++j) { float sq = row[j] * row[j]; acc += (double)sq; }
        float rn = sqrtf((float)acc);
        float safe = rn > 1e-10f ? rn : 1e-10f;
        norms[r] = orig_norm[r] / safe;
    }

    seeds[0] = seed_p;
    seeds[1] = (shared_rotation && residual_bits > 0) ? 0u : seed_r;   /* :255-256 */
    seeds[2] = block_size;

    free(orig_norm); free(scaled); free(work); free(idx_p); free(idx_r);
    return 0;
}

/* ---- dequantize_weight_cpu: src/dequantizer.cpp:52-256 ------------------ */

int tqo_dequantize_weight(const uint8_t* pp, int primary_cols,
                          const uint8_t* pr, int residual_cols,
                          const float* norms, const uint32_t* seeds,
                          int out,
                          const float* cbp, int n_cbp,
                          const float* cbr, int n_cbr,
                          uint32_t block_size, float* W) {
    const int in_from_res = residual_cols * 2;
    const int primary_5bit = (primary_cols == in_from_res);          /* :72-75 */
    const int in = primary_5bit ? primary_cols : primary_cols * 2;
    if (out <= 0 || in <= 0 || block_size == 0 || in % (int)block_size != 0) return -1;
    const float inv_scale = 1.0f / sqrtf((float)in);                 /* :76 */
    const uint32_t seed_p = seeds[0], seed_r = seeds[1];
    const size_t total = (size_t)out * (size_t)in;
    const size_t res_total = (size_t)out * (size_t)residual_cols;

    int has_residual = 0;                                            /* :118-128 */
    for (size_t i = 0; i < res_total; ++i) if (pr[i] != 0) { has_residual = 1; break; }
    const int shared = (seed_r == 0 && has_residual);                /* :133 */

    if (shared && !primary_5bit) {
        /* path A (:136-184): 256-entry table, zero where p >= n_cbp, filled by the
         * reference's loop as written (:144-150): the index is cast to uint8_t, so a
         * primary codebook of more than 16 entries on nibble planes writes entry
         * p >= 16 over ((r | 1) << 4) | (p & 15), later writes winning.  The
         * reference reads r_centroids[r] for all r < 16 without a bound check;
         * a shorter residual codebook is clamped here. */
        float lut[256];
        memset(lut, 0, sizeof lut);
        for (int r = 0; r < 16; ++r)
            for (int p = 0; p < n_cbp; ++p)
                lut[(uint8_t)((r << 4) | p)] = cbp[p] + cbr[r < n_cbr ? r : n_cbr - 1];
#pragma omp parallel for num_threads(g_threads) schedule(static)
        for (int row = 0; row < out; ++row) {
            for (int b = 0; b < primary_cols; ++b) {
                size_t off = (size_t)row * primary_cols + b;
                uint8_t p_byte = pp[off], r_byte = pr[off];
                size_t col_even = (size_t)row * in + (size_t)b * 2;
                uint8_t ce = (uint8_t)((p_byte & 0x0F) | ((r_byte & 0x0F) << 4));
                uint8_t co = (uint8_t)(((p_byte >> 4) & 0x0F) | (r_byte & 0xF0));
                W[col_even]     = lut[ce] * inv_scale;
                W[col_even + 1] = lut[co] * inv_scale;
            }
        }
        tqo_wht_inverse(W, W, out, in, seed_p, block_size);
    } else {
        /* primary lookup (:83-106) */
#pragma omp parallel for num_threads(g_threads) schedule(static)
        for (size_t i = 0; i < total; ++i) {
            size_t idx;
            if (primary_5bit) idx = pp[i];
            else idx = (i & 1) ? ((pp[i >> 1] >> 4) & 0x0F) : (pp[i >> 1] & 0x0F);
            if (idx >= (size_t)n_cbp) idx = (size_t)n_cbp - 1;
            W[i] = cbp[idx];
        }
        if (shared) {
            /* path B (:186-212) */
#pragma omp parallel for num_threads(g_threads) schedule(static)
            for (size_t i = 0; i < total; ++i) {
                size_t q = (i & 1) ? ((pr[i >> 1] >> 4) & 0x0F) : (pr[i >> 1] & 0x0F);
                if (q >= (size_t)n_cbr) q = (size_t)n_cbr - 1;
                float combined = W[i] + cbr[q];
                W[i] = combined * inv_scale;
            }
            tqo_wht_inverse(W, W, out, in, seed_p, block_size);
        } else {
            /* path C (:215-246) */
            scale_inplace(W, total, inv_scale);
            tqo_wht_inverse(W, W, out, in, seed_p, block_size);
            if (has_residual) {
                float* R = (float*)malloc(sizeof(float) * total);
                if (!R) return -1;
#pragma omp parallel for num_threads(g_threads) schedule(static)
                for (size_t i = 0; i < total; ++i) {
                    size_t q = (i & 1) ? ((pr[i >> 1] >> 4) & 0x0F) : (pr[i >> 1] & 0x0F);
                    if (q >= (size_t)n_cbr) q = (size_t)n_cbr - 1;
                    R[i] = cbr[q] * inv_scale;
                }
                tqo_wht_inverse(R, R, out, in, seed_r, block_size);
#pragma omp parallel for num_threads(g_threads) schedule(static)
                for (size_t i = 0; i < total; ++i) W[i] = W[i] + R[i];
                free(R);
            }
        }
    }

    /* norms (:251-253) */
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int r = 0; r < out; ++r) {
        float* row = W + (size_t)r * in;
        const float nr = norms[r];
        for (int j = 0; j < in; ++j) row[j] *= nr;
    }
    return 0;
}

/* ---- x . W^T: tests/integration/test_linear.cpp:102-107 ----------------- */

void tqo_matmul_xwT(const float* x, const float* w, int batch, int in, int out,
                    float* y, int acc_double) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int r = 0; r < out; ++r) {
        const float* wr = w + (size_t)r * in;
        for (int b = 0; b < batch; ++b) {
            const float* xb = x + (size_t)b * in;
            if (acc_double) {
                double acc = 0.0;
                for (int k = 0; k < in; ++k) acc += (double)xb[k] * (double)wr[k];
                y[(size_t)b * out + r] = (float)acc;
            } else {
                float acc = 0.0f;
                for (int k = 0; k < in; ++k) { float p = xb[k] * wr[k]; acc += p; }
                y[(size_t)b * out + r] = acc;
            }
        }
    }
}

/* ---- bf16 helpers -------------------------------------------------------- */

uint16_t tqo_f32_to_bf16(float f) {
    uint32_t u; memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

float tqo_bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16; float f; memcpy(&f, &u, 4); return f;
}
