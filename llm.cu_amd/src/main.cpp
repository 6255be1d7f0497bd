// Entry point of the token loop (the reference's src/main.cu:61-136 without
// the chat REPL and tokenizer): build or load a model, move it to the device,
// run a prompt and a fixed number of greedy decode steps, report tokens/s.
//
//   llama3_main [--config tiny|8b] [--seed S] [--weights a.safetensors[,b,...]]
//               [--prompt-len N] [--decode N] [--max-pos N] [--no-graph]
//               [--tokenizer tokenizer.json --text "question" [--sample]]
// With --tokenizer and --text the reference's chat turn runs instead (main.cu:98-130): chat template,
// tokenize, inference() per token until a special id (>= 128000) or the context limit, decoded text
// printed as it comes; --sample uses the reference's sampler instead of the argmax.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "llama3_host.h"
#include "llmcu_hip.h"

int main(int argc, char **argv) {
    std::string config = "tiny", weights, tokenizer_path, text;
    bool sample = false;
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
        else if (a == "--tokenizer") tokenizer_path = next();
        else if (a == "--text") text = next();
        else if (a == "--sample") sample = true;
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

    if (!tokenizer_path.empty()) {
        Llama3Tokenizer *tk = load_tokenizer_from(tokenizer_path.c_str(), cfg.vocab);
        char *input = llama3_chat_prompt(text.c_str());
        int *tokens = tokenize(tk, input);
        const int limit = cfg.max_pos < 2048 ? cfg.max_pos : 2048;
        llama3_set_sampling(cache, sample ? 1 : 0);
        Tensor *X = (Tensor *)calloc(1, sizeof(Tensor));
        int *d_tokens = tokens_to_cuda(tokens, cfg.d_model, X);
        const int first_special = cfg.vocab > 128000 ? 128000 : cfg.vocab; // main.cu:113
        int next_token = 0, produced = 0;
        while (next_token < first_special && tokens[0] <= limit && produced < decode) {
            next_token = inference(model, X, d_tokens, tokens, cache);
            if (next_token < first_special && tk->decode[next_token]) {
                printf("%s", tk->decode[next_token]);
                fflush(stdout);
            }
            if (tokens[0] > 2048) break;
            tokens[tokens[0]] = next_token;
            tokens[0] = tokens[0] + 1;
            ++produced;
        }
        printf("\n");
        free(tokens);
        free(input);
        _free_tensor(X);
        llm_free(d_tokens);
        free_tokenizer(tk, cfg.vocab);
        free_cache(cache);
        free_llama3(model);
        return 0;
    }

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
