// Settings-carrying form of the host sampler (src/inference/inference.cu:1030-1161 of the reference):
// the reference-named entry points use one process-wide SamplerParams, a CudaCache its own.
#pragma once
#include "llama3_host.h"

struct SamplerParams {
    int vocab = 128256;        // VOCAB_SIZE, inference.cu:24
    float temperature = 0.7f;  // TEMPERATURE, inference.cu:27
    int top_k = 50;            // TOP_K, inference.cu:28
    float top_p = 0.9f;        // TOP_P, inference.cu:29
};

// tensor: float[vocab] scratch (left holding the probabilities), half_tensor: fp16 logits [vocab].
int sampler_draw(const SamplerParams &sp, float *tensor, const llm_half *half_tensor);
int sampler_draw_reference(const SamplerParams &sp, float *tensor, const llm_half *half_tensor);

// The device-assisted form (llm_sample_candidates picks the head of the sorted array):
// settings for which only the k largest probabilities can be drawn (the same condition under which
// sampler_draw avoids the full sort)
bool sampler_head_suffices(const SamplerParams &sp);
// table[b] = expf(fp16(b) / temperature) for every fp16 bit pattern b, with this host's expf.  Returns
// whether the finite entries do not decrease with the value of b (what the device selection relies on).
bool sampler_fill_exp_table(float temperature, float *table65536);
// The draws of sample_next_token from the k entries a stable descending sort would put first, given in
// any order (sorted here by probability descending, index ascending).
int sampler_draw_from_head(const SamplerParams &sp, ProbIndex *head, int k);
