// Model / weight structs, upload and the BF16->FP16 pass at load time.
// Host structure follows src/llama3/llama3.cu of the reference; device work
// goes through the HIP C-ABI (llmcu_hip.h) only.
#include "llama3/llama3.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <vector>

#include "common/fail.h"
#include "llmcu_hip.h"

namespace {
struct Slab {
    char *base;
    size_t bytes;
};
std::mutex g_mu;
std::vector<Slab> g_slabs;

Tensor *new_tensor() {
    // calloc, not malloc: _free_tensor reads the device fields, which the
    // reference leaves uninitialised (src/llama3/llama3.cu:20-22,43-51).
    Tensor *t = (Tensor *)calloc(1, sizeof(Tensor));
    if (!t) llama3_fail("Memory allocation failed for a Tensor structure");
    return t;
}
size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
} // namespace

bool llama3_pointer_in_slab(const void *p) {
    std::lock_guard<std::mutex> lk(g_mu);
    for (const Slab &s : g_slabs)
        if ((const char *)p >= s.base && (const char *)p < s.base + s.bytes) return true;
    return false;
}

void tensor_set_host_shape(Tensor *t, int ndim, const int *shape) {
    free(t->ndim);
    free(t->shape);
    free(t->mem_len);
    t->ndim = (int *)malloc(sizeof(int));
    t->shape = (int *)malloc(sizeof(int) * (ndim > 0 ? ndim : 1));
    t->mem_len = (int *)malloc(sizeof(int));
    if (!t->ndim || !t->shape || !t->mem_len)
        llama3_fail("An Error Occurred while allocating memory for the component shape");
    *t->ndim = ndim;
    long long n = 1;
    for (int i = 0; i < ndim; ++i) {
        t->shape[i] = shape[i];
        n *= shape[i];
    }
    if (n <= 0 || n > 0x7fffffffLL) llama3_fail("tensor has %lld elements; mem_len is an int", n);
    *t->mem_len = (int)n;
}

// src/llama3/llama3.cu:9-69
extern "C" Llama3 *init_llama3(int n_layers) {
    Llama3 *m = (Llama3 *)calloc(1, sizeof(Llama3));
    if (!m) llama3_fail("Memory allocation failed for Llama3 structure");
    m->n_layers = n_layers;
    m->embed_tokens = new_tensor();
    m->norm = new_tensor();
    m->lm_head = new_tensor();
    m->layers = (Llama3Layer **)calloc(n_layers > 0 ? n_layers : 1, sizeof(Llama3Layer *));
    if (!m->layers) llama3_fail("Memory allocation failed for layers array");
    for (int i = 0; i < n_layers; ++i) {
        Llama3Layer *l = (Llama3Layer *)calloc(1, sizeof(Llama3Layer));
        if (!l) llama3_fail("Memory allocation failed for layer %d", i);
        l->layernum = i;
        l->input_layernorm = new_tensor();
        l->mlp_down_proj = new_tensor();
        l->mlp_gate_proj = new_tensor();
        l->mlp_up_proj = new_tensor();
        l->post_attention_layernorm = new_tensor();
        l->self_attn_k_proj = new_tensor();
        l->self_attn_o_proj = new_tensor();
        l->self_attn_q_proj = new_tensor();
        l->self_attn_v_proj = new_tensor();
        m->layers[i] = l;
    }
    return m;
}

// src/llama3/llama3.cu:120-154
extern "C" void _free_tensor(Tensor *t) {
    if (!t) return;
    free(t->ndim);
    free(t->mem_len);
    free(t->shape);
    free(t->bf16_tensor);
    if (t->d_ndim) llm_free(t->d_ndim);
    if (t->d_mem_len) llm_free(t->d_mem_len);
    if (t->d_shape) llm_free(t->d_shape);
    if (t->d_bf16_tensor) llm_free(t->d_bf16_tensor);
    if (t->d_fp16_tensor && !llama3_pointer_in_slab(t->d_fp16_tensor)) llm_free(t->d_fp16_tensor);
    free(t);
}

// src/llama3/llama3.cu:71-118
extern "C" void free_llama3(Llama3 *m) {
    if (!m) return;
    _free_tensor(m->embed_tokens);
    _free_tensor(m->norm);
    _free_tensor(m->lm_head);
    for (int i = 0; i < m->n_layers; ++i) {
        Llama3Layer *l = m->layers[i];
        if (!l) continue;
        _free_tensor(l->input_layernorm);
        _free_tensor(l->mlp_down_proj);
        _free_tensor(l->mlp_gate_proj);
        _free_tensor(l->mlp_up_proj);
        _free_tensor(l->post_attention_layernorm);
        _free_tensor(l->self_attn_k_proj);
        _free_tensor(l->self_attn_o_proj);
        _free_tensor(l->self_attn_q_proj);
        _free_tensor(l->self_attn_v_proj);
        free(l);
    }
    free(m->layers);
    if (m->device_slab) {
        {
            std::lock_guard<std::mutex> lk(g_mu);
            for (size_t i = 0; i < g_slabs.size(); ++i)
                if (g_slabs[i].base == (char *)m->device_slab) {
                    g_slabs.erase(g_slabs.begin() + i);
                    break;
                }
        }
        llm_free(m->device_slab);
    }
    free(m);
}

void _m_component_tensor_operation(Llama3 *m, void (*f)(Tensor *)) {
    f(m->embed_tokens);
    f(m->lm_head);
    f(m->norm);
    for (int i = 0; i < m->n_layers; ++i) {
        Llama3Layer *l = m->layers[i];
        f(l->input_layernorm);
        f(l->mlp_down_proj);
        f(l->mlp_gate_proj);
        f(l->mlp_up_proj);
        f(l->post_attention_layernorm);
        f(l->self_attn_k_proj);
        f(l->self_attn_o_proj);
        f(l->self_attn_q_proj);
        f(l->self_attn_v_proj);
    }
}

// Lays every tensor out in one HBM slab (shapes must be known: mem_len set) and points d_fp16_tensor
// into it.  Returns the element count of the largest tensor.
size_t llama3_plan_slab(Llama3 *m) {
    std::vector<Tensor *> order; // slab order
    for (int i = 0; i < m->n_layers; ++i) {
        Llama3Layer *l = m->layers[i];
        Tensor *ts[] = {l->input_layernorm, l->self_attn_q_proj, l->self_attn_k_proj,
                        l->self_attn_v_proj, l->self_attn_o_proj, l->post_attention_layernorm,
                        l->mlp_gate_proj,   l->mlp_up_proj,      l->mlp_down_proj};
        for (Tensor *t : ts) order.push_back(t);
    }
    order.push_back(m->embed_tokens);
    order.push_back(m->norm);
    order.push_back(m->lm_head);

    size_t total = 0, largest = 0;
    std::vector<size_t> offs;
    for (Tensor *t : order) {
        if (!t || !t->mem_len || *t->mem_len <= 0)
            llama3_fail("to_cuda: a tensor was not loaded (missing from the checkpoint)");
        offs.push_back(total);
        size_t bytes = sizeof(llm_half) * (size_t)*t->mem_len;
        total += align_up(bytes, 256);
        if ((size_t)*t->mem_len > largest) largest = (size_t)*t->mem_len;
    }
    void *slab = nullptr;
    llama3_check(llm_malloc(&slab, total), "llm_malloc(weight slab)");
    {
        std::lock_guard<std::mutex> lk(g_mu);
        g_slabs.push_back({(char *)slab, total});
    }
    m->device_slab = slab;
    for (size_t i = 0; i < order.size(); ++i) order[i]->d_fp16_tensor = (llm_half *)((char *)slab + offs[i]);
    return largest;
}

// to_cuda (src/llama3/llama3.cu:156-254): fp16 device storage for every
// tensor, H2D of the bf16 payload, BF16->FP16 on the device, host payload
// freed.  Differences in mechanism, not in result: one HBM slab instead of
// four cudaMallocs per tensor (q/k/v and gate/up of a layer end up adjacent so
// one projection launch covers them), one reusable bf16 staging buffer
// instead of a malloc/free per tensor, and no device copies of
// ndim/mem_len/shape (no kernel reads them).
extern "C" void to_cuda(Llama3 *m) {
    _m_component_tensor_operation(m, [](Tensor *t) {
        if (!t || !t->bf16_tensor) llama3_fail("to_cuda: a tensor was not loaded (missing from the checkpoint)");
    });
    const size_t largest = llama3_plan_slab(m);
    void *stage = nullptr;
    llama3_check(llm_malloc(&stage, largest * sizeof(uint16_t)), "llm_malloc(bf16 staging)");

    // upload + convert in the reference's visitor order
    struct Ctx {
        void *stage;
    };
    static thread_local Ctx ctx;
    ctx.stage = stage;
    _m_component_tensor_operation(m, [](Tensor *t) {
        size_t n = (size_t)*t->mem_len;
        llama3_check(llm_memcpy_h2d(ctx.stage, t->bf16_tensor, n * 2, nullptr), "H2D of bf16 weights");
        free(t->bf16_tensor);
        t->bf16_tensor = nullptr;
        llama3_check(llm_bf16_to_fp16((const uint16_t *)ctx.stage, t->d_fp16_tensor, n, nullptr),
                     "llm_bf16_to_fp16");
        llama3_check(llm_device_sync(), "device sync");
    });
    llama3_check(llm_free(stage), "llm_free(bf16 staging)");
}

extern "C" ModelConfig llama3_config_8b(void) {
    ModelConfig c;
    c.n_layers = 32;
    c.d_model = 4096;
    c.n_heads = 32;
    c.n_kv_heads = 8;
    c.head_dim = 128;
    c.ffn_dim = 14336;
    c.vocab = 128256;
    c.max_pos = 2048;
    c.rms_eps = 1e-5;
    c.rope_theta = 500000.0f;
    return c;
}

extern "C" ModelConfig llama3_config_tiny(void) {
    ModelConfig c;
    c.n_layers = 2;
    c.d_model = 256;
    c.n_heads = 8;
    c.n_kv_heads = 2;
    c.head_dim = 32;
    c.ffn_dim = 768;
    c.vocab = 4096;
    c.max_pos = 64;
    c.rms_eps = 1e-5;
    c.rope_theta = 500000.0f;
    return c;
}
