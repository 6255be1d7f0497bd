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
