// Internal helpers of the model/weight layer (public structs live in
// include/llama3_host.h).
#pragma once
#include "llama3_host.h"

// Sets ndim / shape / mem_len of a host tensor descriptor (allocating the
// three small heap ints the reference's Tensor carries).
void tensor_set_host_shape(Tensor *t, int ndim, const int *shape);

// Visits every tensor in the reference's order: embed, lm_head, norm, then
// per layer input_ln, down, gate, up, post_ln, k, o, q, v
// (src/llama3/llama3.cu:257-277).
void _m_component_tensor_operation(Llama3 *llama3, void (*_func)(Tensor *));

// True when p lies inside a weight slab owned by some Llama3 (such pointers
// are released with the slab, not one by one).
bool llama3_pointer_in_slab(const void *p);

// One HBM slab for all tensors whose shapes are set; d_fp16_tensor of each points into it.  Returns the
// element count of the largest tensor.
size_t llama3_plan_slab(Llama3 *m);
