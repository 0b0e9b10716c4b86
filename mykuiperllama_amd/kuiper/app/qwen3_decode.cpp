// kx_qwen3_decode [--graph] [--max-positions N] file.safetensors token [token ...]
//
// Feeds the tokens one by one to model::Qwen3Decoder from an empty KV cache (token i at position i)
// and prints one line per step:
//     position token next_token fnv1a64-of-the-bf16-logits
// With --graph the step is captured in a HIP graph first and every token replays it.  The model's
// sizes are read off the checkpoint's tensors.
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "model/qwen3_decoder.h"

int main(int argc, char** argv) {
    bool graph = false;
    int32_t max_positions = 0;
    std::string path;
    std::vector<int32_t> tokens;
    for (int i = 1; i < argc; i++) {
        if (std::strcmp(argv[i], "--graph") == 0) {
            graph = true;
        } else if (std::strcmp(argv[i], "--max-positions") == 0 && i + 1 < argc) {
            max_positions = static_cast<int32_t>(std::strtol(argv[++i], nullptr, 10));
        } else if (path.empty()) {
            path = argv[i];
        } else {
            tokens.push_back(static_cast<int32_t>(std::strtol(argv[i], nullptr, 10)));
        }
    }
    if (path.empty() || tokens.empty()) {
        std::fprintf(stderr, "usage: %s [--graph] [--max-positions N] file.safetensors token [token ...]\n", argv[0]);
        return 2;
    }
    if (max_positions <= 0) max_positions = static_cast<int32_t>(tokens.size());

    model::SafetensorsFile file;
    base::Status st = file.open(path);
    model::Qwen3Config config;
    if (st) st = model::Qwen3Config::from_file(file, config);
    if (!st) {
        std::fprintf(stderr, "%s\n", st.get_err_msg().c_str());
        return 1;
    }
    std::fprintf(stderr, "layers %d hidden %d intermediate %d q heads %d kv heads %d vocab %d group %d\n", config.layers,
                 config.hidden, config.intermediate, config.n_q_heads, config.n_kv_heads, config.vocab,
                 config.group_size);
    model::Qwen3Decoder decoder(config, max_positions);
    st = decoder.load(file);
    if (st && graph) st = decoder.capture();
    if (!st) {
        std::fprintf(stderr, "%s\n", st.get_err_msg().c_str());
        return 1;
    }
    file.close();  // the weights are on the GPU
    std::fprintf(stderr, "%d launches per step%s\n", decoder.launches_per_step(), graph ? ", one graph" : "");
    for (size_t i = 0; i < tokens.size(); i++) {
        int32_t next = -1;
        st = decoder.step(tokens[i], static_cast<int32_t>(i), &next);
        if (!st) {
            std::fprintf(stderr, "%s\n", st.get_err_msg().c_str());
            return 1;
        }
        const std::vector<uint16_t> logits = decoder.logits();
        uint64_t h = 1469598103934665603ull;
        const unsigned char* p = reinterpret_cast<const unsigned char*>(logits.data());
        for (size_t b = 0; b < logits.size() * sizeof(uint16_t); b++) {
            h ^= p[b];
            h *= 1099511628211ull;
        }
        std::printf("%zu %d %d %016" PRIx64 "\n", i, tokens[i], next, h);
    }
    return 0;
}
