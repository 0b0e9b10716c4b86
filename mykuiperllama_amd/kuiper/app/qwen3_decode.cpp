// kx_qwen3_decode [--graph] [--layers | --operators] [--max-positions N] [--generate N] file.safetensors token [token ...]
// kx_qwen3_decode [--graph] [--layers | --operators] --random qwen3-8b|qwen3-32b|tiny --context C [--steps S] [--warmup W]
//
// First form: feeds the tokens one by one to model::Qwen3Decoder from an empty KV cache (token i at
// position i) and prints one line per step:
//     position token next_token fnv1a64-of-the-bf16-logits
// The model's sizes are read off the checkpoint's tensors.  With --generate N the greedy token is fed
// back N more times after the last given token (lines continue in the same format).
// Second form: random-init weights of the named architecture, caches filled with N(0,1) up to the
// context length, then S steps at position C timed back to back; prints one JSON line with
// ms_per_step and tokens_per_s (batch 1, lm_head and argmax included).
// With --graph the step is captured in a HIP graph first and every step replays it.  With --layers every
// launch of the step is the forward() of a kuiper layer, the projections in their fused form (the same five or
// six launches per decoder layer as the fused entry points called directly); with --operators the step is one
// kuiper layer forward() per operator (ten launches per decoder layer).
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "model/qwen3_decoder.h"

namespace {

const char* path_name(model::DecodePath p) {
    return p == model::DecodePath::Layers ? "layers" : (p == model::DecodePath::Operators ? "operators" : "fused");
}

int run_random(const std::string& name, int32_t context, int32_t steps, int32_t warmup, bool graph,
               model::DecodePath decode_path) {
    model::Qwen3Config c;
    if (name == "qwen3-8b") {
        c.layers = 36, c.hidden = 4096, c.intermediate = 12288, c.n_q_heads = 32, c.n_kv_heads = 8, c.vocab = 151936;
    } else if (name == "qwen3-32b") {
        c.layers = 64, c.hidden = 5120, c.intermediate = 25600, c.n_q_heads = 64, c.n_kv_heads = 8, c.vocab = 151936;
    } else if (name == "tiny") {
        c.layers = 2, c.hidden = 512, c.intermediate = 1024, c.n_q_heads = 4, c.n_kv_heads = 2, c.vocab = 1024;
    } else {
        std::fprintf(stderr, "unknown architecture %s (qwen3-8b, qwen3-32b, tiny)\n", name.c_str());
        return 2;
    }
    if (context < 0 || steps < 1 || warmup < 0) {
        std::fprintf(stderr, "--context C (>= 0), --steps S (>= 1) and --warmup W (>= 0) are needed with --random\n");
        return 2;
    }
    model::Qwen3Decoder decoder(c, context + 1, decode_path);
    decoder.init_random(20251125);
    decoder.fill_cache_random(context, 7);
    base::Status st = graph ? decoder.capture() : base::error::success();
    double ms = 0.0;
    if (st) st = decoder.time_steps(17 % c.vocab, context, steps, warmup, &ms);
    if (!st) {
        std::fprintf(stderr, "%s\n", st.get_err_msg().c_str());
        return 1;
    }
    std::printf("{\"model\": \"%s\", \"weights\": \"random-init\", \"context\": %d, \"graph\": %s, \"path\": \"%s\", "
                "\"launches_per_step\": %d, \"steps\": %d, \"warmup\": %d, \"ms_per_step\": %.4f, "
                "\"tokens_per_s\": %.2f}\n",
                name.c_str(), context, graph ? "true" : "false", path_name(decode_path), decoder.launches_per_step(), steps,
                warmup, ms,
                1000.0 / ms);
    return 0;
}

}  // namespace

int main(int argc, char** argv) {
    bool graph = false;
    model::DecodePath decode_path = model::DecodePath::Fused;
    int32_t max_positions = 0, context = -1, steps = 50, warmup = 10, generate = 0;
    std::string path, random_model;
    std::vector<int32_t> tokens;
    auto number = [&](int& i) { return static_cast<int32_t>(std::strtol(argv[++i], nullptr, 10)); };
    for (int i = 1; i < argc; i++) {
        if (std::strcmp(argv[i], "--graph") == 0) {
            graph = true;
        } else if (std::strcmp(argv[i], "--layers") == 0) {
            decode_path = model::DecodePath::Layers;
        } else if (std::strcmp(argv[i], "--operators") == 0) {
            decode_path = model::DecodePath::Operators;
        } else if (std::strcmp(argv[i], "--max-positions") == 0 && i + 1 < argc) {
            max_positions = number(i);
        } else if (std::strcmp(argv[i], "--generate") == 0 && i + 1 < argc) {
            generate = number(i);
        } else if (std::strcmp(argv[i], "--context") == 0 && i + 1 < argc) {
            context = number(i);
        } else if (std::strcmp(argv[i], "--steps") == 0 && i + 1 < argc) {
            steps = number(i);
        } else if (std::strcmp(argv[i], "--warmup") == 0 && i + 1 < argc) {
            warmup = number(i);
        } else if (std::strcmp(argv[i], "--random") == 0 && i + 1 < argc) {
            random_model = argv[++i];
        } else if (path.empty()) {
            path = argv[i];
        } else {
            tokens.push_back(static_cast<int32_t>(std::strtol(argv[i], nullptr, 10)));
        }
    }
    if (!random_model.empty()) return run_random(random_model, context, steps, warmup, graph, decode_path);
    if (path.empty() || tokens.empty()) {
        std::fprintf(stderr,
                     "usage: %s [--graph] [--layers | --operators] [--max-positions N] [--generate N] file.safetensors token [token ...]\n"
                     "       %s [--graph] [--layers | --operators] --random qwen3-8b|qwen3-32b|tiny --context C [--steps S] [--warmup W]\n",
                     argv[0], argv[0]);
        return 2;
    }
    if (generate < 0) generate = 0;
    const size_t total = tokens.size() + static_cast<size_t>(generate);
    if (max_positions <= 0) max_positions = static_cast<int32_t>(total);
    if (static_cast<size_t>(max_positions) < total) {
        std::fprintf(stderr, "--max-positions %d is less than the %zu positions asked for\n", max_positions, total);
        return 2;
    }

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
    model::Qwen3Decoder decoder(config, max_positions, decode_path);
    st = decoder.load(file);
    if (st && graph) st = decoder.capture();
    if (!st) {
        std::fprintf(stderr, "%s\n", st.get_err_msg().c_str());
        return 1;
    }
    file.close();  // the weights are on the GPU
    std::fprintf(stderr, "%d launches per step%s\n", decoder.launches_per_step(), graph ? ", one graph" : "");
    for (size_t i = 0; i < total; i++) {
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
        if (i + 1 == tokens.size() && tokens.size() < total) tokens.push_back(next);  // greedy continuation
    }
    return 0;
}
