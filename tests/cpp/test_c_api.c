/* C99 checks of the handle-based C API (no GPU work): model, cluster planner, local
 * coordinator and the entry points that always fail.  Cases follow the reference's
 * tests/c_api/test_c_api_{model,cluster,distributed,kv_cache}.c. */
#include "turboquant_c/turboquant_c.h"
#include "turboquant_c/tq_linear.h"
#include "turboquant_c/tq_quantizer.h"

#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static int failures = 0;
#define CHECK(cond) do { if (!(cond)) { printf("  FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond); ++failures; } } while (0)

static void model_api(const char* existing_dir) {
    tq_model_t m = tq_model_load(existing_dir);
    CHECK(m != NULL);
    CHECK(tq_model_forward(m, NULL) == NULL);
    tq_model_free(m);
    CHECK(tq_model_load("/nonexistent/path") == NULL);
    CHECK(tq_model_load(NULL) == NULL);
    tq_model_free(NULL);
    CHECK(tq_version() != NULL && strcmp(tq_version(), "0.1.0") == 0);
    tq_array_free(NULL);
    CHECK(tq_model_dequant(NULL, "/tmp/x") != 0);
    CHECK(tq_model_dequant("/nonexistent/path", "/tmp/x") != 0);
}

static tq_cluster_t three_nodes(void) {
    tq_cluster_t c = tq_cluster_create(64, 28, 128);
    CHECK(c != NULL);
    CHECK(tq_cluster_add_node(c, "a.local", 128.0) == 0);
    CHECK(tq_cluster_add_node(c, "b.local", 64.0) == 0);
    CHECK(tq_cluster_add_node(c, "c.local", 32.0) == 0);
    return c;
}

static void cluster_api(void) {
    static const int bad[6][3] = {{0, 28, 128}, {-1, 28, 128}, {64, 0, 128}, {64, -1, 128}, {64, 28, 0}, {64, 28, -1}};
    int i;
    tq_cluster_t c;
    for (i = 0; i < 6; ++i) CHECK(tq_cluster_create(bad[i][0], bad[i][1], bad[i][2]) == NULL);

    c = tq_cluster_create(64, 28, 128);
    CHECK(tq_cluster_node_count(c) == 0);
    CHECK(tq_cluster_add_node(NULL, "h", 64.0) == -1);
    CHECK(tq_cluster_add_node(c, NULL, 64.0) == -1);
    CHECK(tq_cluster_add_node(c, "h", 0.0) == -1);
    CHECK(tq_cluster_add_node(c, "h", -16.0) == -1);
    CHECK(tq_cluster_node_count(c) == 0);
    CHECK(tq_cluster_plan(c) == -1);                       /* no nodes */
    CHECK(tq_cluster_add_node(c, "h", 128.0) == 0);
    CHECK(tq_cluster_get_layer_start(c, 0) == -1);         /* not planned yet */
    CHECK(tq_cluster_get_layer_end(c, 0) == -1);
    CHECK(tq_cluster_plan(c) == 0);
    CHECK(tq_cluster_get_layer_start(c, 0) == 0 && tq_cluster_get_layer_end(c, 0) == 64);   /* one node: all */
    CHECK(tq_cluster_plan(c) == -1);                       /* only once */
    CHECK(tq_cluster_add_node(c, "late", 64.0) == -1);     /* frozen after planning */
    tq_cluster_free(c);

    c = three_nodes();
    CHECK(tq_cluster_node_count(c) == 3);
    CHECK(tq_cluster_plan(c) == 0);
    /* 64 layers over 128:64:32 GB -> round(36.57)=37, round(18.29)=18, remainder 9 */
    CHECK(tq_cluster_get_layer_start(c, 0) == 0 && tq_cluster_get_layer_end(c, 0) == 37);
    CHECK(tq_cluster_get_layer_start(c, 1) == 37 && tq_cluster_get_layer_end(c, 1) == 55);
    CHECK(tq_cluster_get_layer_start(c, 2) == 55 && tq_cluster_get_layer_end(c, 2) == 64);
    CHECK(tq_cluster_get_layer_start(c, 3) == -1 && tq_cluster_get_layer_end(c, 3) == -1);
    CHECK(tq_cluster_get_layer_start(c, -1) == -1 && tq_cluster_get_layer_end(c, -1) == -1);
    tq_cluster_free(c);
    tq_cluster_free(NULL);
    CHECK(tq_cluster_node_count(NULL) == 0);
    CHECK(tq_cluster_plan(NULL) == -1);
}

static void distributed_api(void) {
    tq_coordinator_t co = tq_distributed_init_local();
    CHECK(co != NULL);
    CHECK(tq_distributed_rank(co) == 0);
    CHECK(tq_distributed_world_size(co) == 1);
    tq_distributed_free(co);
    tq_distributed_free(NULL);
    CHECK(tq_distributed_init(NULL, "auto") == NULL);
    CHECK(tq_distributed_init("/nonexistent/hostfile.json", "ring") == NULL);
    CHECK(tq_distributed_rank(NULL) == 0);
    CHECK(tq_distributed_world_size(NULL) == 1);
}

static void kv_cache_api(void) {
    tq_kv_cache_t kv = tq_kv_cache_create(2, 4, 64, 3, 128, 16);
    CHECK(kv == NULL);                                     /* not part of this library */
    tq_kv_cache_append(NULL, 0, NULL, NULL);
    CHECK(tq_kv_cache_get_keys_fp16(NULL, 0, 0, 1) == NULL);
    CHECK(tq_kv_cache_get_values_fp16(NULL, 0, 0, 1) == NULL);
    CHECK(tq_kv_cache_attention(NULL, 0, NULL, 0, 1) == NULL);
    CHECK(tq_kv_cache_seq_length(NULL) == 0);
    tq_kv_cache_free(NULL);
}

static void host_only_helpers(void) {
    float c[32], b[32];
    CHECK(tq_generate_codebook(4, c, b) == 16);
    CHECK(c[0] + c[15] == 0.0f && b[7] == 0.0f);
    CHECK(tq_generate_codebook(0, c, b) < 0);
    CHECK(tq_generate_codebook(6, c, b) < 0);
    CHECK(tq_best_block_size(4096, 512) == 512u);
    CHECK(tq_best_block_size(896, 512) == 128u);
    CHECK(tq_best_block_size(4864, 512) == 256u);
    tq_linear_free(NULL);
    CHECK(tq_linear_in_features(NULL) == 0);
}

int main(int argc, char** argv) {
    model_api(argc > 1 ? argv[1] : "/tmp");
    cluster_api();
    distributed_api();
    kv_cache_api();
    host_only_helpers();
    if (failures) { printf("%d check(s) failed\n", failures); return 1; }
    printf("c api ok\n");
    return 0;
}
