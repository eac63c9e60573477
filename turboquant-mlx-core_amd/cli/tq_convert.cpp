// tq-convert: HuggingFace model directory -> TQ8 directory (reference tools/tq_convert.cpp:1-101;
// same options and defaults, plus --shared-rotation for the one-rotation layout the fused kernels
// are fastest on).
#include "turboquant/converter.h"
#include "turboquant/turboquant.h"
#include <cstdio>
#include <cstdlib>
#include <string>

static void print_usage() {
    std::printf("Usage: tq-convert --model <path> [--bits 4] [--residual-bits 4] [--output <path>]\n\n"
                "Convert a HuggingFace model to TurboQuant format.\n\n"
                "Options:\n"
                "  --model <path>         Path to source model directory\n"
                "  --bits <n>             Primary quantization bits (default: 4)\n"
                "  --residual-bits <n>    Residual quantization bits (default: 4, 0 to disable)\n"
                "  --block-size <n>       WHT block size (default: 512)\n"
                "  --sensitive-layers <n> Keep first and last N transformer layers at fp16 (default: 0)\n"
                "  --per-layer-codebooks  Fit Lloyd-Max codebooks to each layer's distribution\n"
                "  --shared-rotation      One rotation for both passes (seeds[1] = 0)\n"
                "  --output <path>        Output directory (default: <model>-tq<bits>)\n"
                "  --version              Print version and exit\n");
}

int main(int argc, char* argv[]) {
    if (argc < 2) { print_usage(); return 1; }
    std::string model_path, output_path;
    int bits = 4, residual_bits = 4, block_size = 512, sensitive_layers = 0;
    bool per_layer_codebooks = false, shared_rotation = false;
    for (int i = 1; i < argc; i++) {
        const std::string arg = argv[i];
        if (arg == "--model" && i + 1 < argc) model_path = argv[++i];
        else if (arg == "--bits" && i + 1 < argc) bits = std::atoi(argv[++i]);
        else if (arg == "--residual-bits" && i + 1 < argc) residual_bits = std::atoi(argv[++i]);
        else if (arg == "--block-size" && i + 1 < argc) block_size = std::atoi(argv[++i]);
        else if (arg == "--sensitive-layers" && i + 1 < argc) sensitive_layers = std::atoi(argv[++i]);
        else if (arg == "--per-layer-codebooks") per_layer_codebooks = true;
        else if (arg == "--shared-rotation") shared_rotation = true;
        else if (arg == "--output" && i + 1 < argc) output_path = argv[++i];
        else if (arg == "--version") { std::printf("tq-convert %s\n", turboquant::version()); return 0; }
        else if (arg == "--help" || arg == "-h") { print_usage(); return 0; }
    }
    if (model_path.empty()) {
        std::fprintf(stderr, "Error: --model is required\n");
        print_usage();
        return 1;
    }
    if (output_path.empty()) output_path = model_path + "-tq" + std::to_string(bits);

    turboquant::ConversionConfig config;
    config.input_path = model_path;
    config.output_path = output_path;
    config.quantizer.primary_bits = static_cast<uint8_t>(bits);
    config.quantizer.residual_bits = static_cast<uint8_t>(residual_bits);
    config.quantizer.block_size = static_cast<uint32_t>(block_size);
    config.quantizer.shared_rotation = shared_rotation;
    config.quantizer.sensitive_layers_start = sensitive_layers;
    config.quantizer.sensitive_layers_end = sensitive_layers;
    config.per_layer_codebooks = per_layer_codebooks;
    config.progress_callback = [](int current, int total, const std::string& name) {
        std::printf("[%d/%d] Converting %s\n", current, total, name.c_str());
    };
    std::printf("Converting: %s -> %s (TQ%d+%d)\n", model_path.c_str(), output_path.c_str(), bits, residual_bits);
    try {
        if (!turboquant::convert_model(config)) {
            std::fprintf(stderr, "Error: conversion failed\n");
            return 1;
        }
    } catch (const std::exception& e) {
        std::fprintf(stderr, "Error: %s\n", e.what());
        return 1;
    }
    if (!turboquant::validate_converted_model(output_path)) {
        std::fprintf(stderr, "Error: the output carries no TurboQuant metadata\n");
        return 1;
    }
    std::printf("Done: %s\n", output_path.c_str());
    return 0;
}
