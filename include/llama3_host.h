/*
 * llama3_host.h -- host-side interface of the MI355X LLaMA3 token loop.
 *
 * The functions and structs below keep the names, argument meaning and error
 * behaviour (print a message, exit(1)) of the reference's host API, so that a
 * caller written against the reference's headers links against this library
 * unchanged.  Reference declarations replaced:
 *   Tensor / Llama3Layer / Llama3          src/llama3/llama3.cuh:10-50
 *   init_llama3, free_llama3, _free_tensor src/llama3/llama3.cuh:58-78
 *   to_cuda                                src/llama3/llama3.cuh:80-90, llama3.cu:156-161
 *   load_safetensor_weights                src/safetensor/safetensor.cuh:26-40, safetensor.cu:16-31
 *   CudaCache, init_cache, inference       src/inference/inference.cuh:19-34,71, inference.cu:110-193
 *   tokens_to_cuda                         src/tokenizer/tokenizer.cuh:66, tokenizer.cu:157-198
 * Everything after "extensions" has no counterpart in the reference: a shape
 * configuration (the reference hard-codes LLaMA3-8B in its kernels), the KV
 * cache controls, greedy generation, seeded synthetic checkpoints and timing.
 *
 * The library is C-ABI throughout (extern "C", plain pointers and sizes).
 */
#ifndef LLAMA3_HOST_H
#define LLAMA3_HOST_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint16_t llm_half; /* fp16 bit pattern (the reference's __half) */

/* src/llama3/llama3.cuh:10-23 -- same fields, same order. */
typedef struct {
    int *ndim;
    int *mem_len;
    int *shape;
    uint16_t *bf16_tensor;

    int *d_ndim;
    int *d_mem_len;
    int *d_shape;
    uint16_t *d_bf16_tensor;
    llm_half *d_fp16_tensor;
} Tensor;

/* src/llama3/llama3.cuh:28-39 */
typedef struct {
    int layernum;
    Tensor *input_layernorm;
    Tensor *mlp_down_proj;
    Tensor *mlp_gate_proj;
    Tensor *mlp_up_proj;
    Tensor *post_attention_layernorm;
    Tensor *self_attn_k_proj;
    Tensor *self_attn_o_proj;
    Tensor *self_attn_q_proj;
    Tensor *self_attn_v_proj;
} Llama3Layer;

/* src/llama3/llama3.cuh:44-50 (+ one trailing private field) */
typedef struct {
    Tensor *embed_tokens;
    Tensor *lm_head;
    Tensor *norm;
    Llama3Layer **layers;
    int n_layers;
    void *device_slab; /* extension: the single HBM allocation that backs every weight */
} Llama3;

/* src/inference/inference.cuh:19-34 -- the reference's fields first, then the engine. */
typedef struct {
    Tensor *PN_X;
    Tensor *Q;
    Tensor *K;
    Tensor *V;
    float *d_attention_score_cache; /* always NULL: attention never materialises [H,T,T] */
    llm_half *d_feedforward_cache_upgate;
    llm_half *d_token_probdist; /* device fp16 logits of the last row */
    llm_half *h_token_probdist;
    float *f_token_probdist;
    void *engine; /* extension: opaque engine state (KV cache, scratch, stream, graph) */
} CudaCache;

/* src/inference/inference.cuh:46-49 */
typedef struct {
    float probability;
    int index;
} ProbIndex;

/* src/tokenizer/tokenizer.cuh:14-32 */
typedef struct TrieNode {
    int _max_childs;
    int child_len;
    char *child_char;
    struct TrieNode **child_node;
    int token;
} TrieNode;

typedef struct {
    TrieNode *root;
    char **decode;
} Llama3Tokenizer;

/* ---- reference API ---------------------------------------------------- */
Llama3 *init_llama3(int n_layers);
void free_llama3(Llama3 *llama3);
void _free_tensor(Tensor *tensor);
void load_safetensor_weights(Llama3 *llama3_model, const char *filename);
void to_cuda(Llama3 *llama3);
CudaCache *init_cache(Llama3 *llama3_model);
int *tokens_to_cuda(int *tokens, int embed_size, Tensor *token_tensor);
/* h_tokens[0] = n+1, ids in h_tokens[1..n]; returns the next token id. */
int inference(Llama3 *llama3_model, Tensor *X, int *d_tokens, int *h_tokens, CudaCache *Cache);

/* Host sampler, src/inference/inference.cuh:418-426, inference.cu:1030-1161: temperature 0.7, top-k 50
 * (renormalises the head of the sorted array in place, its own draw is discarded), top-p 0.9 picks the
 * token; rand() unseeded.  tensor: vocab floats of scratch, half_tensor: the fp16 logits. */
int sample_next_token(float *tensor, llm_half *half_tensor);
/* the same token through the reference's exact sequence of calls (full-vocabulary qsort per token);
 * sample_next_token() reaches it by selecting only the top_k head when that is provably equivalent */
int sample_next_token_reference(float *tensor, llm_half *half_tensor);
ProbIndex *temperature_softmax(float *tensor, llm_half *half_tensor, float temperature);
int _compare_desc(const void *a, const void *b);
int top_k_sampling(ProbIndex *prob_dist_array, int k);
int top_p_sampling(ProbIndex *prob_dist_array, float p);

/* Tokenizer, src/tokenizer/tokenizer.cuh:44-150: byte trie over the vocabulary, greedy longest match,
 * decode table.  load_tokenizer() reads model_weights/modified_tokenizer.json as the reference does. */
Llama3Tokenizer *load_tokenizer(void);
int *tokenize(Llama3Tokenizer *tokenizer, char *input_str); /* [0] = count + 1, ids from [1], malloc'd */
char *read_tokenizer_json(Llama3Tokenizer *tokenizer, const char *filename);
long _get_file_size(const char *filename);
TrieNode *init_trienode(void);
void _build_trie(TrieNode *node, char *token_string, int token_int);
int _find_child(TrieNode *node, char str, TrieNode **result);
void _memexpand_child_nodes(TrieNode *node);
void _build_decoder(char **decoder, char *token_string, int token_int);

/* ---- extensions -------------------------------------------------------- */
/* load_tokenizer() with the file and the decode-table size as arguments; release; the chat template
 * of src/main.cu:26-59 around one user turn (malloc'd string). */
Llama3Tokenizer *load_tokenizer_from(const char *filename, int decode_size);
void free_tokenizer(Llama3Tokenizer *tokenizer, int decode_size);
char *llama3_chat_prompt(const char *user_input);

/* The reference fixes vocab 128256, temperature 0.7, top-k 50, top-p 0.9 at compile time
 * (inference.cu:24-29).  llama3_sampler_config() sets all four for the reference-named sampler
 * functions above when they are called directly (one process-wide setting, as in the reference).
 * inference() does not read that setting: every CudaCache carries its own (the vocabulary of its
 * configuration, the reference's other three constants), changed with llama3_cache_sampler_config(). */
void llama3_sampler_config(int vocab, float temperature, int top_k, float top_p);
void llama3_cache_sampler_config(CudaCache *c, float temperature, int top_k, float top_p);
/* sample_next_token() with the four settings as arguments: tensor is float[vocab] scratch, half_tensor
 * the fp16 logits [vocab].  Reads and writes no process-wide setting. */
int llama3_sample_with(int vocab, float temperature, int top_k, float top_p, float *tensor, llm_half *half_tensor);
/* inference() returns the greedy id (0, default) or sample_next_token() of the logits as the
 * reference does (1). */
void llama3_set_sampling(CudaCache *c, int on);
/* With sampling on and settings under which only the k most probable ids can be drawn (0 < top_k <
 * vocab, 0 < top_p <= 0.99), the exponentials' sum and the k candidates are computed on the device
 * (llm_sample_candidates) and the host draws from k pairs instead of exponentiating, normalising and
 * ordering the vocabulary; the ids drawn are those of sample_next_token() for the same rand() stream.
 * f_token_probdist is then not written.  0 turns this off (every draw on the host); default 1.  The
 * counts say how many draws of this cache went which way (the device hands a draw back when a logit is
 * NaN, an exponential or their sum overflows, or the sum is zero). */
void llama3_set_device_sampling(CudaCache *c, int on);
void llama3_sampler_draw_counts(const CudaCache *c, long *device_draws, long *host_draws);
/* The cache's sampler (settings, device selection) applied to fp16 logits [vocab] in device memory. */
int llama3_sample_device_logits(CudaCache *c, const llm_half *logits_dev);
typedef struct {
    int n_layers;
    int d_model;
    int n_heads;
    int n_kv_heads;
    int head_dim;
    int ffn_dim;
    int vocab;
    int max_pos;
    double rms_eps;
    float rope_theta;
} ModelConfig;

/* LLaMA3-8B shapes with the reference's 2048-token limit. */
ModelConfig llama3_config_8b(void);
/* The CPU-runnable tiny model (2 layers, d 256, 8/2 heads, head_dim 32, FFN 768, vocab 4096). */
ModelConfig llama3_config_tiny(void);

/* init_cache with explicit shapes (init_cache() derives them from the tensor
 * shapes, head_dim 128, max_pos 2048). */
CudaCache *init_cache_cfg(Llama3 *llama3_model, const ModelConfig *cfg);
void free_cache(CudaCache *Cache);

/* load_safetensor_weights() for every file followed by to_cuda(), streamed: headers first, then every
 * tensor through two pinned 64 MiB buffers (read of one chunk overlaps the upload and BF16->FP16 of the
 * previous), so host memory never holds the checkpoint.  Same device contents as the two-step path. */
void load_safetensor_weights_streaming(Llama3 *llama3_model, const char *const *filenames, int n_files);

/* KV-cached token loop.  prefill appends n tokens (any n >= 1) at the current
 * position and returns the greedy next token; decode appends one. */
int llama3_prefill(Llama3 *m, CudaCache *c, const int *tokens, int n);
int llama3_decode(Llama3 *m, CudaCache *c, int token);
void llama3_cache_reset(CudaCache *c);
int llama3_cache_pos(const CudaCache *c);

/* One decode step for `batch` (<= 16) independent sequences, each with its own cache (created with the
 * same configuration, filled by llama3_prefill): tokens[b] is appended to sequence b, next_tokens[b]
 * receives its greedy continuation.  Every weight matrix is streamed once per step for the whole batch.
 * llama3_read_batch_logits copies the fp16 logits of sequence b of the last step (caches[0] of that step). */
void llama3_decode_batch(Llama3 *m, CudaCache *const *caches, const int *tokens, int batch, int *next_tokens);
void llama3_read_batch_logits(CudaCache *cache0, int b, llm_half *logits);

typedef struct {
    double prefill_ms;     /* wall time of the prompt pass (HIP events) */
    double decode_ms;      /* wall time of all decode steps */
    int n_prompt;
    int n_decode_steps;    /* steps timed in decode_ms */
} GenStats;

/* Greedy generation with the token id and position resident on the device:
 * prompt pass, then n_decode-1 replays of one captured decode step.
 * out_tokens receives n_decode ids (the first comes from the prompt pass). */
int llama3_generate(Llama3 *m, CudaCache *c, const int *prompt, int n_prompt, int n_decode,
                    int *out_tokens, GenStats *stats);

/* Parity hooks: after the next prefill/decode call, hidden receives the
 * residual stream after every layer for the rows of that call
 * ([n_layers][n][d_model] fp16 bits, host memory); pass NULL to switch off.
 * llama3_read_logits copies the fp16 logits of the last processed row. */
void llama3_set_hidden_trace(CudaCache *c, llm_half *hidden);
void llama3_read_logits(CudaCache *c, llm_half *logits);
/* Teacher forcing for per-layer parity: during the next prefill/decode call,
 * layer l >= 1 starts from rows hidden[l-1] ([n_layers][n][d_model] fp16 bits,
 * host memory, e.g. another implementation's trace) instead of this engine's
 * own layer l-1 output, so each layer is compared on identical input and
 * rounding differences do not compound across layers. */
void llama3_set_hidden_inject(CudaCache *c, const llm_half *hidden);

/* Choose between one hipGraph replay per decode step (1, default) and plain
 * stream launches (0). */
void llama3_set_use_graph(CudaCache *c, int on);

/* The decode step's launches that hand the attention output to the output projection inside one kernel
 * (llm_attn_decode_rope_oproj, llm_attn_decode_rope_long_oproj) bound the projection's wait.  When a wait
 * gives up -- only seen when other work holds the device's CUs for the whole wait -- the step's results are
 * discarded, the step (for llama3_generate: its run of decode steps) is redone with one launch per
 * operation, a line goes to stderr, and the cache keeps the one-launch-per-operation form from then on:
 * the same token ids either way, a slower step instead of a failed one.
 * llama3_set_handover: on = 1 puts a cache back into the hand-over form (0 takes it out); spin_limit is
 * the bound of the wait in polling rounds, negative for the kernels' default.
 * llama3_handover_stats: waits that gave up and steps redone so far, and whether the form is in use.
 * llama3_test_mark_handover_timeout: the next step is treated as if one wait had given up (for tests of
 * the redo path; every kernel still runs to its normal end). */
void llama3_set_handover(CudaCache *c, int on, int spin_limit);
void llama3_handover_stats(const CudaCache *c, long *timeouts, long *recoveries, int *active);
void llama3_test_mark_handover_timeout(CudaCache *c);

/* Error hook.  Default prints the message and calls exit(1) as the reference
 * does; tests install a handler that records instead. */
typedef void (*llama3_error_fn)(const char *msg);
void llama3_set_error_handler(llama3_error_fn fn);

/* ---- seeded synthetic checkpoints -------------------------------------- */
/* Counter-based generator: the value of element i of tensor id depends on
 * (seed, id, i) only.  Matrices are N(0, 0.02) quantised through a 65536-level
 * inverse-CDF table and rounded to bf16; RMSNorm gains are 1. */
void seeded_normal_bf16(uint64_t seed, uint64_t tensor_id, size_t n, float sigma, uint16_t *out);
void seeded_tokens(uint64_t seed, int n, int vocab, int *out);
const uint16_t *seeded_unit_table_bf16(float sigma); /* 65536 entries */
/* Fill every tensor of an init_llama3() model with host bf16 data of the
 * shapes cfg implies (as load_safetensor_weights would leave it). */
void seeded_fill_model(Llama3 *m, const ModelConfig *cfg, uint64_t seed);
/* Write the same tensors as one safetensors file with HF LLaMA3 key names. */
int seeded_write_safetensors(const ModelConfig *cfg, uint64_t seed, const char *path);
uint64_t seeded_tensor_id(int layer, int slot);

#ifdef __cplusplus
}
#endif
#endif
