#ifndef TURBOQUANT_C_H
#define TURBOQUANT_C_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * TurboQuant C API -- the 25 entry points of the reference's
 * include/turboquant_c/turboquant_c.h:25-136 with the same names, signatures, ownership
 * (every tq_*_create / load has a matching tq_*_free, every free accepts NULL) and error
 * conventions (no exception crosses the boundary: NULL / -1 / non-zero on failure).
 *
 * What is behind them here:
 *   tq_model_dequant            TQ8 safetensors -> fp16/bf16 safetensors; the weights are
 *                               reconstructed by the GPU dequant kernel.
 *   tq_model_load/forward/free  as the reference (src/turboquant_c.cpp:56-83): a directory
 *                               check and a forward stub that returns NULL.
 *   tq_distributed_init_local,  single-node coordinator (rank 0 of 1) and the memory-proportional
 *   tq_cluster_*                layer planner, pure host logic.
 *   tq_distributed_init,        outside the quantized-linear path: always fail the way the
 *   tq_kv_cache_*               reference does on error (NULL / 0 / no-op).
 * The per-layer entry points the reference lacks are in tq_linear.h and tq_quantizer.h.
 */

/* Opaque handle types */
typedef struct tq_model_s* tq_model_t;
typedef struct tq_kv_cache_s* tq_kv_cache_t;
typedef struct tq_coordinator_s* tq_coordinator_t;
typedef struct tq_cluster_s* tq_cluster_t;

/* -- Model (reference turboquant_c.h:27-34) ------------------------------ */

/* NULL unless model_path names an existing directory. */
tq_model_t tq_model_load(const char* model_path);
/* Always NULL (stub in the reference as well, src/turboquant_c.cpp:71-77). */
void* tq_model_forward(tq_model_t model, const void* input_array);
void tq_model_free(tq_model_t model);

/* -- KV cache (reference turboquant_c.h:38-70): not part of this library -- */

tq_kv_cache_t tq_kv_cache_create(int num_layers, int num_heads, int head_dim,
                                 int kv_bits, int max_context, int decode_window);   /* NULL */
void tq_kv_cache_append(tq_kv_cache_t cache, int layer, const void* keys_array, const void* values_array);
void* tq_kv_cache_get_keys_fp16(tq_kv_cache_t cache, int layer, int start, int end);      /* NULL */
void* tq_kv_cache_get_values_fp16(tq_kv_cache_t cache, int layer, int start, int end);    /* NULL */
void* tq_kv_cache_attention(tq_kv_cache_t cache, int layer, const void* queries_array,
                            int compressed_start, int compressed_end);                    /* NULL */
int tq_kv_cache_seq_length(tq_kv_cache_t cache);                                         /* 0 */
void tq_kv_cache_free(tq_kv_cache_t cache);

/* -- Distributed (reference turboquant_c.h:74-87) ------------------------ */

tq_coordinator_t tq_distributed_init(const char* hostfile, const char* backend);   /* NULL: one GPU only */
tq_coordinator_t tq_distributed_init_local(void);
int tq_distributed_rank(tq_coordinator_t coord);          /* 0 for NULL */
int tq_distributed_world_size(tq_coordinator_t coord);    /* 1 for NULL */
void tq_distributed_free(tq_coordinator_t coord);

/* -- Cluster planning (reference turboquant_c.h:91-121) ------------------ */

tq_cluster_t tq_cluster_create(int num_layers, int num_heads, int head_dim);
int tq_cluster_add_node(tq_cluster_t cluster, const char* hostname, double memory_gb);
int tq_cluster_plan(tq_cluster_t cluster);
int tq_cluster_node_count(tq_cluster_t cluster);
int tq_cluster_get_layer_start(tq_cluster_t cluster, int rank);
int tq_cluster_get_layer_end(tq_cluster_t cluster, int rank);
void tq_cluster_free(tq_cluster_t cluster);

/* -- Dequantization (reference turboquant_c.h:125-131, src/turboquant_c_dequant.cpp:20-191) -- */

/* Rebuild a standard model directory from a TQ8 one: copies the non-safetensors files, strips
 * "quantization_config" from config.json, and for every TQ8 shard writes {layer}.weight in the
 * source model's element type (bf16 unless the shard's *_passthrough.safetensors says otherwise)
 * plus the passthrough tensors.  Returns 0 on success, non-zero on error. */
int tq_model_dequant(const char* tq_model_path, const char* output_path);

/* -- Utility (reference turboquant_c.h:135-139) -------------------------- */

void tq_array_free(void* array);
const char* tq_version(void);

#ifdef __cplusplus
}
#endif

#endif /* TURBOQUANT_C_H */
