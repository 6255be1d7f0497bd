// Entry point of the token loop (the reference's src/main.cu:61-136 without
// the chat REPL and tokenizer): build or load a model, move it to the device,
// run a prompt and a fixed number of greedy decode steps, report tokens/s.
//
//   llama3_main [--config tiny|8b] [--seed S] [--weights a.safetensors[,b,...]]
//               [--prompt-len N] [--decode N] [--max-pos N] [--no-graph]
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "llama3_host.h"
#include "llmcu_hip.h"

int main(int argc, char **argv) {
    std::string config = "tiny", weights;
    uint64_t seed = 1234;
    int prompt_len = 16, decode = 32, max_pos = 0, graph = 1;
    for (int i = 1; i < argc; ++i) {
        std::string a = argv[i];
        auto next = [&]() -> const char * {
            if (i + 1 >= argc) {
                printf("Error: %s needs a value\n", a.c_str());
                exit(1);
            }
            return argv[++i];
        };
        if (a == "--config") config = next();
        else if (a == "--seed") seed = strtoull(next(), nullptr, 10);
        else if (a == "--weights") weights = next();
        else if (a == "--prompt-len") prompt_len = atoi(next());
        else if (a == "--decode") decode = atoi(next());
        else if (a == "--max-pos") max_pos = atoi(next());
        else if (a == "--no-graph") graph = 0;
        else {
            printf("Error: unknown option %s\n", a.c_str());
            return 1;
        }
    }
    ModelConfig cfg = config == "8b" ? llama3_config_8b() : llama3_config_tiny();
    if (max_pos > 0) cfg.max_pos = max_pos;
    int need = (prompt_len + decode + 63) / 64 * 64;
    if (cfg.max_pos < need) cfg.max_pos = need;

    if (llm_init(0) != LLM_OK) {
        printf("Error: %s\n", llm_last_error());
        return 1;
    }
    Llama3 *model = init_llama3(cfg.n_layers);
    printf("Model has been allocated with %d layers\n", model->n_layers);
    if (weights.empty()) {
        seeded_fill_model(model, &cfg, seed);
        printf("[CPU] Seeded synthetic weights (seed %llu)\n", (unsigned long long)seed);
        to_cuda(model);
    } else {
        // shards named on the command line (main.cu:73-76 loads four), streamed to the device
        std::vector<std::string> names;
        size_t b = 0;
        while (b <= weights.size()) {
            size_t e = weights.find(',', b);
            if (e == std::string::npos) e = weights.size();
            names.push_back(weights.substr(b, e - b));
            b = e + 1;
        }
        std::vector<const char *> ptrs;
        for (const std::string &n : names) ptrs.push_back(n.c_str());
        load_safetensor_weights_streaming(model, ptrs.data(), (int)ptrs.size());
        printf("[CPU] Read %d shard(s)\n", (int)ptrs.size());
    }
    printf("[HIP] Loaded to the device, parameters converted to FP16\n");
    CudaCache *cache = init_cache_cfg(model, &cfg);
    llama3_set_use_graph(cache, graph);

    std::vector<int> prompt(prompt_len), out(decode);
    seeded_tokens(seed, prompt_len, cfg.vocab, prompt.data());
    GenStats st;
    llama3_generate(model, cache, prompt.data(), prompt_len, decode, out.data(), &st);
    printf("tokens:");
    for (int t : out) printf(" %d", t);
    printf("\nprefill: %d tokens in %.3f ms (%.1f tok/s)\n", st.n_prompt, st.prefill_ms,
           st.n_prompt / (st.prefill_ms * 1e-3));
    if (st.n_decode_steps > 0)
        printf("decode: %d steps in %.3f ms (%.1f tok/s)\n", st.n_decode_steps, st.decode_ms,
               st.n_decode_steps / (st.decode_ms * 1e-3));
    free_cache(cache);
    free_llama3(model);
    return 0;
}
