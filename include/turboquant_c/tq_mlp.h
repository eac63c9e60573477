#ifndef TURBOQUANT_C_TQ_MLP_H
#define TURBOQUANT_C_TQ_MLP_H

/*
 * Gated MLP block over three TQ8 linears:  y = down( silu(gate(x)) * up(x) ),
 * with the SiLU gate evaluated in fp32 between the linears.
 *
 * The reference has no block-level operator: callers chain TurboQuantLinear::forward
 * (include/turboquant/linear.h:21-23) and the activation themselves, which costs one
 * launch, one allocation and two host synchronisations per layer
 * (src/dequantizer.cpp:606-721).  This entry point keeps the intermediates in buffers
 * owned by the block and enqueues the whole block on one stream without allocating,
 * so it can be captured in a HIP graph.  gate and up have their own seeds and
 * codebooks, so each rotates the activation for itself.  Batch 1: the gate is folded
 * into the store of the up projection (three kernels in all).  Two or more rows: the
 * three layers run on the matrix cores with one elementwise kernel in between, the
 * activation handed on as fp32.
 */

#include "tq_linear.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tq_mlp_s* tq_mlp_t;

/* gate, up: [intermediate, hidden]; down: [out, intermediate].  The layers are borrowed:
 * they must outlive the block.  Intermediates are sized for max_batch rows.  NULL on error. */
tq_mlp_t tq_mlp_create(tq_linear_t gate, tq_linear_t up, tq_linear_t down, int max_batch);

/* x_dev [batch, hidden] -> y_dev [batch, out]; device pointers, TQ_DTYPE_* element types,
 * stream = hipStream_t or NULL.  Asynchronous.  Returns 0 on success. */
int tq_mlp_forward(tq_mlp_t mlp, const void* x_dev, int x_dtype, int batch,
                   void* y_dev, int y_dtype, void* stream);

/* Frees the intermediates (not the layers).  NULL is a no-op. */
void tq_mlp_free(tq_mlp_t mlp);

#ifdef __cplusplus
}
#endif

#endif /* TURBOQUANT_C_TQ_MLP_H */
