// Host-only tool for the safetensors tests: load a file with this library's reader and write
// it back with its writer, or print the metadata of a file.
//   st_roundtrip copy <in> <out>
//   st_roundtrip meta <in>
#include "turboquant/serialization.h"

#include <cstdio>
#include <map>
#include <string>

int main(int argc, char** argv) {
    try {
        const std::string mode = argc > 1 ? argv[1] : "";
        if (mode == "copy" && argc == 4) {
            auto loaded = turboquant::load_safetensors(argv[2]);
            turboquant::save_safetensors(argv[3], loaded.first, loaded.second);
            std::printf("%zu tensors\n", loaded.first.size());
            return 0;
        }
        if (mode == "meta" && argc == 3) {
            const auto md = turboquant::read_tq_metadata(argv[2]);
            for (const auto& kv : std::map<std::string, std::string>(md.begin(), md.end()))
                std::printf("%s=%s\n", kv.first.c_str(), kv.second.c_str());
            return 0;
        }
        std::fprintf(stderr, "usage: st_roundtrip copy <in> <out> | meta <in>\n");
        return 2;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "error: %s\n", e.what());
        return 1;
    }
}
