// tq-dequant-model: TQ8 model directory -> fp16/bf16 safetensors directory
// (reference tools/tq_dequant_model.cpp:19-211: same two positional arguments).  The work is
// tq_model_dequant of the C API; the weights are rebuilt by the GPU dequant kernel.
#include "turboquant_c/turboquant_c.h"
#include <cstdio>

int main(int argc, char** argv) {
    if (argc != 3) {
        std::printf("Usage: %s <tq-model-dir> <output-dir>\n", argv[0]);
        std::printf("Dequant a TQ model back to fp16 safetensors for PPL evaluation.\n");
        return 1;
    }
    if (tq_model_dequant(argv[1], argv[2]) != 0) {
        std::fprintf(stderr, "Error: dequantisation of %s failed\n", argv[1]);
        return 1;
    }
    std::printf("Done.\n");
    return 0;
}
