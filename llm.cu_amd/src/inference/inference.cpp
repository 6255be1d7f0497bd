// Forward / generation driver.  Keeps the reference's entry points
// (init_cache, inference; src/inference/inference.cu:110-193) and adds what the
// token loop needs on top: an fp16 KV cache, a prompt pass that processes many
// rows at once, a one-row decode step captured as a hipGraph, greedy argmax on
// the device.  All device work goes through llmcu_hip.h.
//
// Layer graph (inference.cu:157-186), with the reference's extra passes folded
// into neighbours where the result is the same bits:
//   save residual + norm      -> llm_rmsnorm into a second buffer (x stays the residual);
//                                for one row, folded into the next projection
//   Q, K, V (3 launches)      -> one projection over the adjacent q|k|v weights
//   RoPE(Q), RoPE(K)          -> llm_rope_kv_append (also writes the KV cache)
//   scores, softmax, P.V      -> llm_attn_prefill / llm_attn_decode over the cache
//   copy + O projection, add  -> llm_linear with the residual in its epilogue
//   gate/up+SiLU, down, add   -> llm_linear_swiglu, llm_linear with residual
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "common/fail.h"
#include "llama3/llama3.h"
#include "llama3_host.h"
#include "llmcu_hip.h"
#include "sampler.h"

namespace {

struct Engine {
    ModelConfig cfg;
    const Llama3 *model = nullptr; // whose weight pointers the captured graphs hold
    const void *model_slab = nullptr;
    SamplerParams sampler;         // this cache's own settings (vocab = cfg.vocab)
    llm_stream_t stream = nullptr;
    void *splitk_ws = nullptr;     // fp32 partial tiles of split-K projections issued on `stream`
    size_t splitk_bytes = 0;
    // pinned staging: [0] token in, [1] position in, [2] token out.  Reused by every step; safe because
    // each step ends in a stream sync before the next one writes them.
    int32_t *h_stage = nullptr;
    // what the device holds after the last step: *d_pos == pos and d_tokens[pos] == dev_next (or -1)
    bool dev_pos_valid = false;
    int dev_next = -1;
    int qkv_dim = 0;
    // activations, sized for max_pos rows
    llm_half *x = nullptr, *xn = nullptr, *qkv = nullptr, *attn = nullptr, *ffn = nullptr;
    llm_half *logits = nullptr;
    // KV cache: K [L][Hkv][max_pos][hd], V [L][Hkv][hd][max_pos]
    llm_half *kc = nullptr, *vc = nullptr;
    size_t kv_layer_elems = 0;
    float *rope_table = nullptr;
    int32_t *d_tokens = nullptr; // [max_pos + 1]
    int32_t *d_pos = nullptr;    // tokens cached so far; d_tokens[*d_pos] is the next input
    int32_t *d_token = nullptr;  // [0] last argmax, [1] waits of the fused attention + projection launch that gave up
    llm_half *ao_ring = nullptr; // one attention-output buffer per layer for llm_attn_decode_rope_oproj (null: not used)
    bool ao_long = false;        // the ring also serves llm_attn_decode_rope_long_oproj
    // The launches that hand the attention output over inside the kernel are used while handover_on; a step in
    // which a bounded wait gave up is redone with one launch per operation and the cache stays in that form.
    bool handover_on = true;
    int handover_spin_limit = -1; // < 0: the kernels' default
    bool handover_test_mark = false; // tests: count one timeout into the next step as if a wait had given up
    long handover_timeouts = 0, handover_recoveries = 0;
    void *ws_attn = nullptr, *ws_lm = nullptr;
    llm_half *trace_dev = nullptr;
    size_t trace_rows = 0;
    llm_half *trace_host = nullptr;
    const llm_half *inject_host = nullptr; // teacher forcing: layer l >= 1 starts from these rows
    llm_half *inject_dev = nullptr;
    size_t inject_rows = 0;
    std::vector<int> tokens; // ids whose K/V are cached
    int pos = 0;
    bool use_graph = true;
    bool sampling = false; // inference() samples like the reference instead of returning the argmax
    // device half of the sampler (llm_sample_candidates): the host's exp table for table_temperature, the
    // selection's output and its pinned mirror, sized for table_k pairs
    bool device_select = true;   // use it whenever the settings allow
    bool select_pending = false; // the step being issued also selects candidates
    bool table_ok = false;       // the table is monotone (else every draw takes the host path)
    float table_temperature = 0.0f;
    int select_cap = 0;
    float *d_exp_table = nullptr;
    uint32_t *d_select = nullptr, *h_select = nullptr;
    long device_draws = 0, host_draws = 0;
    // one captured decode step per attention form: [0] single launch (up to 512 cached positions),
    // [1] span + merge launches (beyond)
    llm_graph_t graph[2] = {nullptr, nullptr};
    bool long_attn = false; // form used by the next decode step that is issued
    // scratch of llama3_decode_batch (allocated by the first call on this cache as sequence 0)
    int batch_cap = 0;
    llm_half *b_logits = nullptr; // [batch][vocab]
    int32_t *b_ids = nullptr;     // [batch] input ids, then the argmax results
    void *b_ws_attn = nullptr, *b_ws_argmax = nullptr;
    // the sequences' caches and positions where the kernels of a batched step read them, its pinned mirror, pinned
    // staging for the ids in and out; one captured step per (batch size, attention form), taken into use once that
    // combination has run with plain launches
    llm_batch_desc *b_desc = nullptr, *b_desc_host = nullptr;
    int32_t *b_ids_host = nullptr;
    llm_graph_t b_graph[17][2] = {};
    bool b_ran[17][2] = {};
    llm_event_t ev[4] = {nullptr, nullptr, nullptr, nullptr};
};

const int LONG_ATTN_FROM = 512; // cached positions from which the span + merge attention is faster
// Prompt passes of this many rows and more leave the rotation of the queries to the attention kernel (one pass over Q
// in memory less: 134 MB per layer at 8192 rows); below, the rotation in the attention's prologue (its first tile loads
// wait for queries and angles, about 4 us per launch) costs more than the smaller RoPE launch saves (5 us at any size
// up to a thousand rows).  Same bits either way.
constexpr int ROPE_IN_ATTENTION_FROM = 4096;

Engine *eng(const CudaCache *c) {
    if (!c || !c->engine) llama3_fail("CudaCache was not created by init_cache");
    return (Engine *)c->engine;
}

template <typename T> T *dmalloc(size_t n, const char *what) {
    void *p = nullptr;
    llama3_check(llm_malloc(&p, n * sizeof(T)), what);
    return (T *)p;
}

struct LayerW {
    const llm_half *in_ln, *post_ln, *wq, *wk, *wv, *wo, *wg, *wu, *wd;
};

LayerW layer_w(const Llama3 *m, int l) {
    const Llama3Layer *L = m->layers[l];
    return {L->input_layernorm->d_fp16_tensor,  L->post_attention_layernorm->d_fp16_tensor,
            L->self_attn_q_proj->d_fp16_tensor, L->self_attn_k_proj->d_fp16_tensor,
            L->self_attn_v_proj->d_fp16_tensor, L->self_attn_o_proj->d_fp16_tensor,
            L->mlp_gate_proj->d_fp16_tensor,    L->mlp_up_proj->d_fp16_tensor,
            L->mlp_down_proj->d_fp16_tensor};
}

void check_shapes(const Llama3 *m, const ModelConfig &c) {
    auto want = [](const Tensor *t, int r, int cc, const char *name) {
        if (!t || !t->shape || !t->d_fp16_tensor) llama3_fail("%s is not on the device (call to_cuda first)", name);
        int rows = t->shape[0], cols = *t->ndim > 1 ? t->shape[1] : 0;
        if (rows != r || cols != cc) llama3_fail("%s is [%d,%d], the configuration needs [%d,%d]", name, rows, cols, r, cc);
    };
    const int d = c.d_model, qd = c.n_heads * c.head_dim, kvd = c.n_kv_heads * c.head_dim;
    if (m->n_layers != c.n_layers) llama3_fail("model has %d layers, configuration %d", m->n_layers, c.n_layers);
    want(m->embed_tokens, c.vocab, d, "embed_tokens");
    want(m->lm_head, c.vocab, d, "lm_head");
    want(m->norm, d, 0, "norm");
    for (int l = 0; l < c.n_layers; ++l) {
        const Llama3Layer *L = m->layers[l];
        want(L->input_layernorm, d, 0, "input_layernorm");
        want(L->post_attention_layernorm, d, 0, "post_attention_layernorm");
        want(L->self_attn_q_proj, qd, d, "q_proj");
        want(L->self_attn_k_proj, kvd, d, "k_proj");
        want(L->self_attn_v_proj, kvd, d, "v_proj");
        want(L->self_attn_o_proj, d, qd, "o_proj");
        want(L->mlp_gate_proj, c.ffn_dim, d, "gate_proj");
        want(L->mlp_up_proj, c.ffn_dim, d, "up_proj");
        want(L->mlp_down_proj, d, c.ffn_dim, "down_proj");
    }
}

void drop_graph(Engine *e) {
    for (int f = 0; f < 2; ++f) {
        if (!e->graph[f]) continue;
        llm_graph_destroy(e->graph[f]);
        e->graph[f] = nullptr;
    }
    for (auto &per_batch : e->b_graph)
        for (llm_graph_t &g : per_batch) {
            if (g) llm_graph_destroy(g);
            g = nullptr;
        }
}

// The captured decode graphs hold the weight pointers of the model they were captured with.  A call
// with another model (or the same struct after its weights were reloaded) is checked against the
// configuration like the first one and the graphs are captured again.
void bind_model(Engine *e, const Llama3 *m) {
    const void *slab = m && m->embed_tokens ? (const void *)m->embed_tokens->d_fp16_tensor : nullptr;
    if (m == e->model && slab == e->model_slab) return;
    check_shapes(m, e->cfg);
    drop_graph(e);
    e->model = m;
    e->model_slab = slab;
}

// Issues one pass over T rows on the engine's stream.  With dev_pos the row
// position comes from *d_pos (T must be 1): that form is what gets captured.
void issue_pass(Engine *e, const Llama3 *m, int T, int pos0, bool dev_pos, bool trace, bool inject = false) {
    const ModelConfig &c = e->cfg;
    const int d = c.d_model, hd = c.head_dim, Hq = c.n_heads, Hkv = c.n_kv_heads, F = c.ffn_dim;
    const int qd = Hq * hd, kvd = Hkv * hd, QKV = e->qkv_dim;
    llm_stream_t s = e->stream;
    const int32_t *pd = dev_pos ? e->d_pos : nullptr;
    const int p0 = dev_pos ? 0 : pos0;

    // decode step over a fused Q/K/V matrix: the first projection gathers the embedding row itself
    bool embed_folded = false;
    if (T == 1 && c.n_layers > 0) {
        const LayerW w0 = layer_w(m, 0);
        embed_folded = w0.wk == w0.wq + (size_t)qd * d && w0.wv == w0.wk + (size_t)kvd * d;
    }
    if (!embed_folded)
        llama3_check(llm_embed_gather(m->embed_tokens->d_fp16_tensor, e->d_tokens + p0, pd, e->x, T, d, c.vocab, s),
                     "llm_embed_gather");
    const llm_half *final_gain = m->norm->d_fp16_tensor;
    if (T == 1) {
        // decode step: 4 launches per layer, 5 at long contexts (norm folded into the projections, RoPE + cache
        // append folded into the attention, residual adds in the projection epilogues)
        for (int l = 0; l < c.n_layers; ++l) {
            const LayerW w = layer_w(m, l);
            llm_half *kc = e->kc + (size_t)l * e->kv_layer_elems, *vc = e->vc + (size_t)l * e->kv_layer_elems;
            if (inject && l > 0)
                llama3_check(llm_memcpy_d2d(e->x, e->inject_dev + (size_t)(l - 1) * d, sizeof(llm_half) * (size_t)d, s),
                             "inject copy");
            if (l == 0 && embed_folded) {
                llama3_check(llm_embed_norm_linear(m->embed_tokens->d_fp16_tensor, e->d_tokens + p0, pd, c.vocab, e->x,
                                                   w.in_ln, c.rms_eps, w.wq, e->qkv, QKV, d, s),
                             "llm_embed_norm_linear(qkv)");
            } else if (w.wk == w.wq + (size_t)qd * d && w.wv == w.wk + (size_t)kvd * d) {
                llama3_check(llm_norm_linear(e->x, w.in_ln, c.rms_eps, w.wq, e->qkv, QKV, d, s), "llm_norm_linear(qkv)");
            } else {
                llama3_check(llm_norm_linear(e->x, w.in_ln, c.rms_eps, w.wq, e->qkv, qd, d, s), "llm_norm_linear(q)");
                llama3_check(llm_norm_linear(e->x, w.in_ln, c.rms_eps, w.wk, e->qkv + qd, kvd, d, s), "llm_norm_linear(k)");
                llama3_check(llm_norm_linear(e->x, w.in_ln, c.rms_eps, w.wv, e->qkv + qd + kvd, kvd, d, s),
                             "llm_norm_linear(v)");
            }
            if (!e->long_attn && e->ao_ring && e->handover_on) {
                // attention and output projection in one launch: the projection's weights stream while the
                // attention runs.  Layer l hands over through ring buffer l and re-arms the next one.
                llama3_check(llm_attn_decode_rope_oproj(e->qkv, kc, vc, e->ao_ring + (size_t)l * qd,
                                                        e->ao_ring + (size_t)((l + 1) % c.n_layers) * qd, p0, pd,
                                                        e->rope_table, Hq, Hkv, hd, c.max_pos, w.wo, e->x, e->x, d,
                                                        e->d_token + 1, e->handover_spin_limit, s),
                             "llm_attn_decode_rope_oproj");
            } else if (e->long_attn && e->ao_ring && e->ao_long && e->handover_on) {
                // long contexts: spans, then merge + output projection in one launch (same ring, same re-arming)
                llama3_check(llm_attn_decode_rope_long_oproj(e->qkv, kc, vc, e->ao_ring + (size_t)l * qd,
                                                             e->ao_ring + (size_t)((l + 1) % c.n_layers) * qd, p0, pd,
                                                             e->rope_table, Hq, Hkv, hd, c.max_pos, e->ws_attn, w.wo, e->x,
                                                             e->x, d, e->d_token + 1, e->handover_spin_limit, s),
                             "llm_attn_decode_rope_long_oproj");
            } else {
                llama3_check((e->long_attn ? llm_attn_decode_rope_long : llm_attn_decode_rope)(
                                 e->qkv, kc, vc, e->attn, p0, pd, e->rope_table, Hq, Hkv, hd, c.max_pos, e->ws_attn, s),
                             "llm_attn_decode_rope");
                llama3_check(llm_linear(e->attn, qd, w.wo, e->x, d, e->x, d, 1, d, qd, s), "llm_linear(o)");
            }
            llama3_check(llm_norm_linear_swiglu(e->x, w.post_ln, c.rms_eps, w.wg, w.wu, e->ffn, F, d, s),
                         "llm_norm_linear_swiglu");
            llama3_check(llm_linear(e->ffn, F, w.wd, e->x, d, e->x, d, 1, d, F, s), "llm_linear(down)");
            if (trace)
                llama3_check(llm_memcpy_d2d(e->trace_dev + (size_t)l * d, e->x, sizeof(llm_half) * (size_t)d, s),
                             "trace copy");
        }
    } else {
        for (int l = 0; l < c.n_layers; ++l) {
            const LayerW w = layer_w(m, l);
            llm_half *kc = e->kc + (size_t)l * e->kv_layer_elems, *vc = e->vc + (size_t)l * e->kv_layer_elems;
            if (inject && l > 0)
                llama3_check(llm_memcpy_d2d(e->x, e->inject_dev + (size_t)(l - 1) * T * d,
                                            sizeof(llm_half) * (size_t)T * d, s),
                             "inject copy");
            llama3_check(llm_rmsnorm(e->x, w.in_ln, e->xn, T, d, c.rms_eps, s), "llm_rmsnorm");
            if (w.wk == w.wq + (size_t)qd * d && w.wv == w.wk + (size_t)kvd * d) {
                llama3_check(llm_linear(e->xn, d, w.wq, nullptr, 0, e->qkv, QKV, T, QKV, d, s), "llm_linear(qkv)");
            } else {
                llama3_check(llm_linear(e->xn, d, w.wq, nullptr, 0, e->qkv, QKV, T, qd, d, s), "llm_linear(q)");
                llama3_check(llm_linear(e->xn, d, w.wk, nullptr, 0, e->qkv + qd, QKV, T, kvd, d, s), "llm_linear(k)");
                llama3_check(llm_linear(e->xn, d, w.wv, nullptr, 0, e->qkv + qd + kvd, QKV, T, kvd, d, s), "llm_linear(v)");
            }
            if (!pd && T >= ROPE_IN_ATTENTION_FROM && llm_attn_prefill_rope_q_supported(T, Hq, Hkv, hd, c.max_pos)) {
                // the attention rotates the queries it loads: no pass over Q in memory
                llama3_check(llm_rope_k_append(e->qkv, kc, vc, T, Hq, Hkv, hd, p0, e->rope_table, c.max_pos, s),
                             "llm_rope_k_append");
                llama3_check(llm_attn_prefill_rope_q(e->qkv, QKV, kc, vc, e->attn, qd, T, p0, e->rope_table, Hq, Hkv, hd,
                                                     c.max_pos, s),
                             "llm_attn_prefill_rope_q");
            } else {
                llama3_check(llm_rope_kv_append(e->qkv, kc, vc, T, Hq, Hkv, hd, p0, pd, e->rope_table, c.max_pos, s),
                             "llm_rope_kv_append");
                llama3_check(llm_attn_prefill(e->qkv, QKV, kc, vc, e->attn, qd, T, p0, Hq, Hkv, hd, c.max_pos, s),
                             "llm_attn_prefill");
            }
            llama3_check(llm_linear(e->attn, qd, w.wo, e->x, d, e->x, d, T, d, qd, s), "llm_linear(o)");
            llama3_check(llm_rmsnorm(e->x, w.post_ln, e->xn, T, d, c.rms_eps, s), "llm_rmsnorm");
            llama3_check(llm_linear_swiglu(e->xn, d, w.wg, w.wu, e->ffn, F, T, F, d, s), "llm_linear_swiglu");
            llama3_check(llm_linear(e->ffn, F, w.wd, e->x, d, e->x, d, T, d, F, s), "llm_linear(down)");
            if (trace)
                llama3_check(llm_memcpy_d2d(e->trace_dev + (size_t)l * T * d, e->x, sizeof(llm_half) * (size_t)T * d, s),
                             "trace copy");
        }
    }
    // final norm on the last row only (the reference norms all rows and reads the last), folded into the LM head
    llama3_check(llm_norm_lmhead_argmax(e->x + (size_t)(T - 1) * d, final_gain, c.rms_eps, m->lm_head->d_fp16_tensor,
                                        e->logits, e->d_token, e->d_tokens, e->d_pos, c.vocab, d, e->ws_lm, s),
                 "llm_norm_lmhead_argmax");
}

// h_stage[3] mirrors d_token[1]: waits inside llm_attn_decode_rope_oproj that ran into their limit.  Any
// such wait means a projection used an incomplete attention output, so everything the step computed behind it
// is invalid.  Returns false when the step is clean.  Otherwise the cache leaves the hand-over launches for
// good (one launch per operation from here on: a device whose CUs are held by other work would run into the
// limit again), the count is cleared, the buffers are armed again, the captured steps are dropped, and the
// caller redoes the step: K and V rows of the position are simply written again.
bool handover_gave_up(Engine *e) {
    if (e->h_stage[3] == 0) return false;
    if (!e->handover_on) llama3_fail("hand-over timeouts counted (%d) although no hand-over launch is in use", e->h_stage[3]);
    fprintf(stderr, "[llama3] attention/projection hand-over gave up %d time(s) at position %d: redoing the step with one launch "
                    "per operation (this cache keeps that form)\n", e->h_stage[3], e->pos);
    e->handover_timeouts += e->h_stage[3];
    ++e->handover_recoveries;
    e->handover_on = false;
    drop_graph(e);
    llama3_check(llm_fill_zero(e->d_token + 1, sizeof(int32_t), e->stream), "zero timeout count");
    llama3_check(llm_attn_oproj_buffer_init(e->ao_ring, e->cfg.n_layers * e->cfg.n_heads * e->cfg.head_dim, e->stream),
                 "llm_attn_oproj_buffer_init");
    e->h_stage[3] = 0;
    return true;
}

// tests: the next step sees one counted timeout (the count only ever grows inside a step)
void apply_test_mark(Engine *e) {
    if (!e->handover_test_mark || !e->handover_on || !e->ao_ring) return;
    e->handover_test_mark = false;
    e->h_stage[4] = 1;
    llama3_check(llm_memcpy_h2d(e->d_token + 1, &e->h_stage[4], sizeof(int32_t), e->stream), "H2D timeout mark");
}

// Brings the exp table and the selection buffers in line with the cache's sampler settings; false when
// the settings or the table rule the device selection out.
bool prepare_selection(Engine *e) {
    const SamplerParams &sp = e->sampler;
    if (!e->device_select || !sampler_head_suffices(sp) || sp.vocab > llm_sample_candidates_max_vocab()) return false;
    if (!e->d_exp_table || e->table_temperature != sp.temperature) {
        std::vector<float> table(65536);
        e->table_ok = sampler_fill_exp_table(sp.temperature, table.data());
        if (!e->d_exp_table) e->d_exp_table = dmalloc<float>(65536, "llm_malloc(exp table)");
        llama3_check(llm_memcpy_h2d(e->d_exp_table, table.data(), sizeof(float) * 65536, e->stream), "H2D exp table");
        llama3_check(llm_stream_sync(e->stream), "stream sync"); // `table` goes out of scope
        e->table_temperature = sp.temperature;
    }
    if (!e->table_ok) return false;
    if (sp.top_k > e->select_cap) {
        if (e->d_select) llm_free(e->d_select);
        if (e->h_select) llm_free_host(e->h_select);
        e->d_select = (uint32_t *)dmalloc<char>(llm_sample_candidates_bytes(e->cfg.vocab, sp.top_k),
                                                "llm_malloc(sampler candidates)");
        void *hp = nullptr;
        llama3_check(llm_malloc_host(&hp, llm_sample_candidates_head_bytes(sp.top_k)), "llm_malloc_host(sampler candidates)");
        e->h_select = (uint32_t *)hp;
        e->select_cap = sp.top_k;
    }
    return true;
}

// After the LM head of a step, in stream order: select the sampler's candidates from `logits` and bring
// them to the host behind the token id.
void enqueue_selection(Engine *e, const llm_half *logits) {
    llama3_check(llm_sample_candidates(logits, e->d_exp_table, e->cfg.vocab, e->sampler.top_k, e->d_select, e->stream),
                 "llm_sample_candidates");
    llama3_check(llm_memcpy_d2h(e->h_select, e->d_select, llm_sample_candidates_head_bytes(e->sampler.top_k), e->stream),
                 "D2H sampler candidates");
}

// The draw from what enqueue_selection brought back (after the stream sync); -1 when the device left the
// decision to the host.
int draw_from_selection(Engine *e) {
    const uint32_t *h = e->h_select;
    const int k = e->sampler.top_k;
    if (h[2] != 0 || (int)h[1] != k) return -1;
    std::vector<ProbIndex> head((size_t)k);
    for (int i = 0; i < k; ++i) {
        memcpy(&head[i].probability, &h[4 + 2 * i], sizeof(float));
        head[i].index = (int)h[5 + 2 * i];
    }
    return sampler_draw_from_head(e->sampler, head.data(), k);
}

// Appends n host tokens at e->pos with one multi-row pass.  Leaves
// d_pos = pos + n and d_tokens[pos + n] = the greedy next token.
// logits_host (may be null): pinned host memory that receives the fp16 logits before the pass's one sync.
int run_pass(Engine *e, const Llama3 *m, const int *tokens, int n, llm_half *logits_host = nullptr) {
    const ModelConfig &c = e->cfg;
    bind_model(e, m);
    if (n < 1) llama3_fail("a pass needs at least one token");
    if (e->pos + n > c.max_pos) llama3_fail("sequence of %d tokens exceeds max_pos %d", e->pos + n, c.max_pos);
    for (int i = 0; i < n; ++i)
        if (tokens[i] < 0 || tokens[i] >= c.vocab) llama3_fail("token id %d outside the vocabulary", tokens[i]);
    llm_stream_t s = e->stream;
    llama3_check(llm_memcpy_h2d(e->d_tokens + e->pos, tokens, sizeof(int) * (size_t)n, s), "H2D tokens");
    e->h_stage[1] = e->pos + n - 1;
    llama3_check(llm_memcpy_h2d(e->d_pos, &e->h_stage[1], sizeof(int32_t), s), "H2D position");
    llama3_check(llm_stream_sync(s), "stream sync"); // `tokens` is the caller's (pageable) memory
    const bool trace = e->trace_host != nullptr;
    if (trace) {
        size_t need = (size_t)c.n_layers * n * c.d_model;
        if (need > e->trace_rows) {
            if (e->trace_dev) llm_free(e->trace_dev);
            e->trace_dev = dmalloc<llm_half>(need, "llm_malloc(trace)");
            e->trace_rows = need;
        }
    }
    const bool inject = e->inject_host != nullptr;
    if (inject) {
        size_t need = (size_t)c.n_layers * n * c.d_model;
        if (need > e->inject_rows) {
            if (e->inject_dev) llm_free(e->inject_dev);
            e->inject_dev = dmalloc<llm_half>(need, "llm_malloc(inject)");
            e->inject_rows = need;
        }
        llama3_check(llm_memcpy_h2d(e->inject_dev, e->inject_host, sizeof(llm_half) * need, s), "H2D inject");
    }
    for (int attempt = 0;; ++attempt) {
        if (attempt) // the first attempt's argmax advanced *d_pos
            llama3_check(llm_memcpy_h2d(e->d_pos, &e->h_stage[1], sizeof(int32_t), s), "H2D position");
        if (n == 1) apply_test_mark(e); // passes over several rows use no hand-over launch
        e->long_attn = n == 1 && e->pos >= LONG_ATTN_FROM; // single rows go through the decode kernels
        issue_pass(e, m, n, e->pos, false, trace, inject);
        llama3_check(llm_memcpy_d2h(&e->h_stage[2], e->d_token, sizeof(int32_t) * 2, s), "D2H token");
        if (trace)
            llama3_check(llm_memcpy_d2h(e->trace_host, e->trace_dev, sizeof(llm_half) * (size_t)c.n_layers * n * c.d_model, s),
                         "D2H trace");
        if (logits_host)
            llama3_check(llm_memcpy_d2h(logits_host, e->logits, sizeof(llm_half) * (size_t)c.vocab, s), "D2H logits");
        if (e->select_pending) enqueue_selection(e, e->logits);
        llama3_check(llm_stream_sync(s), "stream sync");
        if (!handover_gave_up(e)) break;
    }
    e->trace_host = nullptr;
    e->inject_host = nullptr;
    e->tokens.insert(e->tokens.end(), tokens, tokens + n);
    e->pos += n;
    // the pass left *d_pos == pos and its pick in d_tokens[pos]
    e->dev_pos_valid = true;
    e->dev_next = e->h_stage[2];
    return (int)e->h_stage[2];
}

// One decode step from device state (d_tokens[*d_pos] in, next token out).
void capture_decode_graph(Engine *e, const Llama3 *m, int form) {
    if (e->graph[form]) return;
    e->long_attn = form == 1;
    llama3_check(llm_graph_capture_begin(e->stream), "graph capture begin");
    issue_pass(e, m, 1, 0, true, false);
    llama3_check(llm_graph_capture_end(e->stream, &e->graph[form]), "graph capture end");
}

// pos: position of the token this step processes (known on the host although the kernels read it
// from device memory), which selects the attention form
void launch_decode_step(Engine *e, const Llama3 *m, int pos) {
    const int form = pos >= LONG_ATTN_FROM ? 1 : 0;
    if (e->use_graph) {
        capture_decode_graph(e, m, form);
        llama3_check(llm_graph_launch(e->graph[form], e->stream), "graph launch");
    } else {
        e->long_attn = form == 1;
        issue_pass(e, m, 1, 0, true, false);
    }
}

// One cached decode step with a single host round trip: the token id and the position go up only when
// the device does not already hold them (after a greedy step it does: the argmax kernel stored its pick
// at d_tokens[pos] and advanced *d_pos), the result (and, when asked for, the logits) come back through
// pinned memory, one stream sync at the end.
int step_one(Engine *e, const Llama3 *m, int token, llm_half *logits_host) {
    if (e->trace_host || e->inject_host) return run_pass(e, m, &token, 1, logits_host);
    const ModelConfig &c = e->cfg;
    bind_model(e, m);
    if (e->pos + 1 > c.max_pos) llama3_fail("sequence of %d tokens exceeds max_pos %d", e->pos + 1, c.max_pos);
    if (token < 0 || token >= c.vocab) llama3_fail("token id %d outside the vocabulary", token);
    llm_stream_t s = e->stream;
    for (int attempt = 0;; ++attempt) {
        if (attempt) e->dev_pos_valid = false; // a step that is redone starts from the host's view of the sequence
        if (!e->dev_pos_valid || e->dev_next != token) {
            e->h_stage[0] = token;
            llama3_check(llm_memcpy_h2d(e->d_tokens + e->pos, &e->h_stage[0], sizeof(int32_t), s), "H2D token");
        }
        if (!e->dev_pos_valid) {
            e->h_stage[1] = e->pos;
            llama3_check(llm_memcpy_h2d(e->d_pos, &e->h_stage[1], sizeof(int32_t), s), "H2D position");
        }
        apply_test_mark(e);
        launch_decode_step(e, m, e->pos);
        llama3_check(llm_memcpy_d2h(&e->h_stage[2], e->d_token, sizeof(int32_t) * 2, s), "D2H token");
        if (logits_host)
            llama3_check(llm_memcpy_d2h(logits_host, e->logits, sizeof(llm_half) * (size_t)c.vocab, s), "D2H logits");
        if (e->select_pending) enqueue_selection(e, e->logits);
        llama3_check(llm_stream_sync(s), "stream sync");
        if (!handover_gave_up(e)) break;
    }
    e->tokens.push_back(token);
    e->pos += 1;
    e->dev_pos_valid = true;
    e->dev_next = e->h_stage[2];
    return (int)e->h_stage[2];
}

// One batched decode step on e0's stream from device state: ids in e0->b_ids, caches and positions in e0->b_desc;
// leaves the greedy ids in e0->b_ids and the logits in e0->b_logits.  Nothing in it depends on host values that
// change from step to step, so it can be captured.  form: 0 every position below LONG_ATTN_FROM, 1 otherwise.
void issue_batch_step(Engine *e0, const Llama3 *m, int batch, int form) {
    const ModelConfig &c = e0->cfg;
    const int d = c.d_model, hd = c.head_dim, Hq = c.n_heads, Hkv = c.n_kv_heads, F = c.ffn_dim;
    const int qd = Hq * hd, kvd = Hkv * hd, QKV = e0->qkv_dim;
    llm_stream_t s = e0->stream;
    llama3_check(llm_embed_gather(m->embed_tokens->d_fp16_tensor, e0->b_ids, nullptr, e0->x, batch, d, c.vocab, s),
                 "llm_embed_gather");
    for (int l = 0; l < c.n_layers; ++l) {
        const LayerW w = layer_w(m, l);
        llama3_check(llm_rmsnorm(e0->x, w.in_ln, e0->xn, batch, d, c.rms_eps, s), "llm_rmsnorm");
        if (w.wk == w.wq + (size_t)qd * d && w.wv == w.wk + (size_t)kvd * d) {
            llama3_check(llm_linear(e0->xn, d, w.wq, nullptr, 0, e0->qkv, QKV, batch, QKV, d, s), "llm_linear(qkv)");
        } else {
            llama3_check(llm_linear(e0->xn, d, w.wq, nullptr, 0, e0->qkv, QKV, batch, qd, d, s), "llm_linear(q)");
            llama3_check(llm_linear(e0->xn, d, w.wk, nullptr, 0, e0->qkv + qd, QKV, batch, kvd, d, s), "llm_linear(k)");
            llama3_check(llm_linear(e0->xn, d, w.wv, nullptr, 0, e0->qkv + qd + kvd, QKV, batch, kvd, d, s), "llm_linear(v)");
        }
        llama3_check(llm_attn_decode_rope_batch_dev(e0->qkv, QKV, e0->b_desc, (size_t)l * e0->kv_layer_elems, batch, form, e0->attn,
                                                    qd, e0->rope_table, Hq, Hkv, hd, c.max_pos, e0->b_ws_attn, s),
                     "llm_attn_decode_rope_batch_dev");
        llama3_check(llm_linear(e0->attn, qd, w.wo, e0->x, d, e0->x, d, batch, d, qd, s), "llm_linear(o)");
        llama3_check(llm_rmsnorm(e0->x, w.post_ln, e0->xn, batch, d, c.rms_eps, s), "llm_rmsnorm");
        llama3_check(llm_linear_swiglu(e0->xn, d, w.wg, w.wu, e0->ffn, F, batch, F, d, s), "llm_linear_swiglu");
        llama3_check(llm_linear(e0->ffn, F, w.wd, e0->x, d, e0->x, d, batch, d, F, s), "llm_linear(down)");
    }
    llama3_check(llm_rmsnorm(e0->x, m->norm->d_fp16_tensor, e0->xn, batch, d, c.rms_eps, s), "llm_rmsnorm");
    llama3_check(llm_linear(e0->xn, d, m->lm_head->d_fp16_tensor, nullptr, 0, e0->b_logits, c.vocab, batch, c.vocab, d, s),
                 "llm_linear(lm_head)");
    llama3_check(llm_argmax_f16_rows(e0->b_logits, c.vocab, batch, c.vocab, e0->b_ids, e0->b_ws_argmax, s),
                 "llm_argmax_f16_rows");
}

} // namespace

// ---------------------------------------------------------------------------
extern "C" CudaCache *init_cache_cfg(Llama3 *m, const ModelConfig *cfg) {
    const ModelConfig &c = *cfg;
    if (c.max_pos <= 0 || c.max_pos % 64) llama3_fail("max_pos %d must be a positive multiple of 64", c.max_pos);
    if (c.n_kv_heads <= 0 || c.n_heads % c.n_kv_heads) llama3_fail("heads %d/%d", c.n_heads, c.n_kv_heads);
    check_shapes(m, c);
    Engine *e = new Engine;
    e->cfg = c;
    e->model = m;
    e->model_slab = m->embed_tokens->d_fp16_tensor;
    e->sampler.vocab = c.vocab; // temperature 0.7, top-k 50, top-p 0.9 as in inference.cu:27-29
    const int d = c.d_model, qd = c.n_heads * c.head_dim, kvd = c.n_kv_heads * c.head_dim;
    e->qkv_dim = qd + 2 * kvd;
    const size_t R = (size_t)c.max_pos;
    llama3_check(llm_stream_create(&e->stream), "llm_stream_create");
    e->x = dmalloc<llm_half>(R * d, "llm_malloc(x)");
    e->xn = dmalloc<llm_half>(R * d, "llm_malloc(xn)");
    e->qkv = dmalloc<llm_half>(R * e->qkv_dim, "llm_malloc(qkv)");
    e->attn = dmalloc<llm_half>(R * qd, "llm_malloc(attn)");
    e->ffn = dmalloc<llm_half>(R * c.ffn_dim, "llm_malloc(ffn)");
    e->logits = dmalloc<llm_half>((size_t)c.vocab, "llm_malloc(logits)");
    e->kv_layer_elems = (size_t)c.n_kv_heads * R * c.head_dim;
    e->kc = dmalloc<llm_half>(e->kv_layer_elems * c.n_layers, "llm_malloc(K cache)");
    e->vc = dmalloc<llm_half>(e->kv_layer_elems * c.n_layers, "llm_malloc(V cache)");
    llama3_check(llm_fill_zero(e->kc, sizeof(llm_half) * e->kv_layer_elems * c.n_layers, e->stream), "zero K cache");
    llama3_check(llm_fill_zero(e->vc, sizeof(llm_half) * e->kv_layer_elems * c.n_layers, e->stream), "zero V cache");
    {
        size_t n = R * (c.head_dim / 2) * 2;
        std::vector<float> tab(n);
        llama3_check(llm_rope_table_host(tab.data(), c.max_pos, c.head_dim, c.rope_theta), "llm_rope_table_host");
        e->rope_table = dmalloc<float>(n, "llm_malloc(rope table)");
        llama3_check(llm_memcpy_h2d(e->rope_table, tab.data(), sizeof(float) * n, nullptr), "H2D rope table");
    }
    e->d_tokens = dmalloc<int32_t>(R + 1, "llm_malloc(tokens)");
    e->d_pos = dmalloc<int32_t>(1, "llm_malloc(pos)");
    e->d_token = dmalloc<int32_t>(2, "llm_malloc(token)");
    llama3_check(llm_fill_zero(e->d_token, sizeof(int32_t) * 2, e->stream), "zero token");
    if (c.n_layers >= 2 && llm_attn_oproj_supported(c.n_heads, c.n_kv_heads, c.head_dim, d)) {
        e->ao_ring = dmalloc<llm_half>((size_t)c.n_layers * qd, "llm_malloc(attention hand-over ring)");
        llama3_check(llm_attn_oproj_buffer_init(e->ao_ring, c.n_layers * qd, e->stream), "llm_attn_oproj_buffer_init");
        e->ao_long = llm_attn_long_oproj_supported(c.n_heads, c.n_kv_heads, c.head_dim, d) == 1;
    }
    llama3_check(llm_fill_zero(e->d_tokens, sizeof(int32_t) * (R + 1), e->stream), "zero tokens");
    llama3_check(llm_fill_zero(e->d_pos, sizeof(int32_t), e->stream), "zero pos");
    size_t wa = llm_attn_decode_workspace_bytes(c.n_heads, c.head_dim);
    wa = (wa + 3) / 4 * 4;
    llama3_check(llm_malloc(&e->ws_attn, wa), "llm_malloc(attention workspace)");
    llama3_check(llm_fill_zero(e->ws_attn, wa, e->stream), "zero attention workspace");
    llama3_check(llm_malloc(&e->ws_lm, llm_lmhead_workspace_bytes(c.vocab)), "llm_malloc(lm head workspace)");
    for (auto &ev : e->ev) llama3_check(llm_event_create(&ev), "llm_event_create");
    {
        void *hs = nullptr;
        llama3_check(llm_malloc_host(&hs, sizeof(int32_t) * 8), "llm_malloc_host(staging)");
        e->h_stage = (int32_t *)hs;
    }
    llama3_check(llm_stream_sync(e->stream), "stream sync");

    CudaCache *C = (CudaCache *)calloc(1, sizeof(CudaCache));
    if (!C) llama3_fail("Memory allocation failed for CudaCache");
    C->d_feedforward_cache_upgate = e->ffn;
    C->d_token_probdist = e->logits;
    // pinned, so that the logits of a step come back asynchronously behind its token id
    void *hp = nullptr;
    llama3_check(llm_malloc_host(&hp, sizeof(llm_half) * (size_t)c.vocab), "llm_malloc_host(h_token_probdist)");
    C->h_token_probdist = (llm_half *)hp;
    C->f_token_probdist = (float *)malloc(sizeof(float) * (size_t)c.vocab);
    if (!C->f_token_probdist) llama3_fail("Memory allocation failed for f_token_probdist");
    C->engine = e;
    return C;
}

// inference.cu:110-145.  Shapes come from the loaded tensors; head_dim 128 and
// the 2048-token limit are the reference's constants (inference.cu:122,700).
extern "C" CudaCache *init_cache(Llama3 *m) {
    ModelConfig c = llama3_config_8b();
    if (!m || !m->embed_tokens || !m->embed_tokens->shape) llama3_fail("init_cache: the model holds no tensors");
    c.n_layers = m->n_layers;
    c.vocab = m->embed_tokens->shape[0];
    c.d_model = m->embed_tokens->shape[1];
    c.ffn_dim = m->layers[0]->mlp_gate_proj->shape[0];
    c.head_dim = 128;
    c.n_heads = m->layers[0]->self_attn_q_proj->shape[0] / c.head_dim;
    c.n_kv_heads = m->layers[0]->self_attn_k_proj->shape[0] / c.head_dim;
    c.max_pos = 2048;
    return init_cache_cfg(m, &c);
}

extern "C" void free_cache(CudaCache *C) {
    if (!C) return;
    Engine *e = (Engine *)C->engine;
    if (e) {
        llm_stream_sync(e->stream);
        drop_graph(e);
        void *bufs[] = {e->x, e->xn, e->qkv, e->attn, e->ffn, e->logits, e->kc, e->vc, e->rope_table,
                        e->d_tokens, e->d_pos, e->d_token, e->ao_ring, e->ws_attn, e->ws_lm, e->trace_dev, e->inject_dev,
                        e->b_logits, e->b_ids, e->b_ws_attn, e->b_ws_argmax, e->b_desc};
        for (void *b : bufs) llm_free(b);
        for (auto ev : e->ev) llm_event_destroy(ev);
        llm_stream_destroy(e->stream);
        llm_free_host(e->h_stage);
        if (e->b_desc_host) llm_free_host(e->b_desc_host);
        if (e->b_ids_host) llm_free_host(e->b_ids_host);
        if (e->h_select) llm_free_host(e->h_select);
        if (e->d_select) llm_free(e->d_select);
        if (e->d_exp_table) llm_free(e->d_exp_table);
        delete e;
    }
    llm_free_host(C->h_token_probdist);
    free(C->f_token_probdist);
    free(C);
}

// tokenizer.cu:157-198: the activation tensor X ([2048, embed] fp16, zeroed)
// and the device token array.  The engine keeps its own activations; X and
// d_tokens exist so that callers written for the reference keep working.
extern "C" int *tokens_to_cuda(int *tokens, int embed_size, Tensor *X) {
    (void)tokens;
    memset(X, 0, sizeof(Tensor));
    int shape[2] = {2048, embed_size};
    tensor_set_host_shape(X, 2, shape);
    void *p = nullptr;
    llama3_check(llm_malloc(&p, sizeof(llm_half) * (size_t)*X->mem_len), "llm_malloc(X)");
    X->d_fp16_tensor = (llm_half *)p;
    llama3_check(llm_fill_zero(p, sizeof(llm_half) * (size_t)*X->mem_len, nullptr), "zero X");
    void *dt = nullptr;
    llama3_check(llm_malloc(&dt, sizeof(int) * 2048), "llm_malloc(d_tokens)");
    llama3_check(llm_device_sync(), "device sync");
    return (int *)dt;
}

extern "C" void llama3_cache_reset(CudaCache *C) {
    Engine *e = eng(C);
    e->pos = 0;
    e->tokens.clear();
    e->dev_pos_valid = false;
    e->dev_next = -1;
}

extern "C" int llama3_cache_pos(const CudaCache *C) { return eng(C)->pos; }

extern "C" int llama3_prefill(Llama3 *m, CudaCache *C, const int *tokens, int n) {
    return run_pass(eng(C), m, tokens, n);
}

extern "C" int llama3_decode(Llama3 *m, CudaCache *C, int token) { return step_one(eng(C), m, token, nullptr); }

extern "C" int llama3_generate(Llama3 *m, CudaCache *C, const int *prompt, int n_prompt, int n_decode,
                               int *out_tokens, GenStats *stats) {
    Engine *e = eng(C);
    const ModelConfig &c = e->cfg;
    bind_model(e, m);
    if (n_decode < 1) llama3_fail("llama3_generate: n_decode must be at least 1");
    if (e->pos + n_prompt + n_decode - 1 > c.max_pos)
        llama3_fail("prompt %d + %d decode steps exceed max_pos %d", e->pos + n_prompt, n_decode - 1, c.max_pos);
    llm_stream_t s = e->stream;
    const int start = e->pos;
    llama3_check(llm_event_record(e->ev[0], s), "event record");
    int first = run_pass(e, m, prompt, n_prompt); // syncs
    llama3_check(llm_event_record(e->ev[1], s), "event record");
    // capture outside the timed decode region
    if (e->use_graph && n_decode > 1) {
        const int first_pos = start + n_prompt, last_pos = start + n_prompt + n_decode - 2;
        if (first_pos < LONG_ATTN_FROM) capture_decode_graph(e, m, 0);
        if (last_pos >= LONG_ATTN_FROM) capture_decode_graph(e, m, 1);
    }
    out_tokens[0] = first;
    for (int attempt = 0;; ++attempt) {
        if (attempt) {
            // a wait gave up somewhere in the run of steps: all of them again from the first decode position
            // (d_tokens[first position] still holds the prompt pass's pick), now with one launch per operation
            e->h_stage[1] = start + n_prompt;
            llama3_check(llm_memcpy_h2d(e->d_pos, &e->h_stage[1], sizeof(int32_t), s), "H2D position");
        }
        if (n_decode > 1) apply_test_mark(e);
        llama3_check(llm_event_record(e->ev[2], s), "event record");
        for (int i = 1; i < n_decode; ++i) launch_decode_step(e, m, start + n_prompt + i - 1);
        llama3_check(llm_event_record(e->ev[3], s), "event record");
        llama3_check(llm_stream_sync(s), "stream sync");
        if (n_decode <= 1) break;
        llama3_check(llm_memcpy_d2h(out_tokens + 1, e->d_tokens + start + n_prompt + 1,
                                    sizeof(int32_t) * (size_t)(n_decode - 1), s),
                     "D2H tokens");
        llama3_check(llm_memcpy_d2h(&e->h_stage[2], e->d_token, sizeof(int32_t) * 2, s), "D2H token");
        llama3_check(llm_stream_sync(s), "stream sync");
        if (!handover_gave_up(e)) break;
    }
    // host mirror: the decode steps consumed out_tokens[0..n_decode-2]
    for (int i = 0; i + 1 < n_decode; ++i) e->tokens.push_back(out_tokens[i]);
    e->pos += n_decode - 1;
    e->dev_pos_valid = true; // every replayed step advanced *d_pos and stored its pick at d_tokens[pos]
    e->dev_next = out_tokens[n_decode - 1];
    if (stats) {
        float a = 0.f, b = 0.f;
        llm_event_elapsed_ms(e->ev[0], e->ev[1], &a);
        llm_event_elapsed_ms(e->ev[2], e->ev[3], &b);
        stats->prefill_ms = a;
        stats->decode_ms = b;
        stats->n_prompt = n_prompt;
        stats->n_decode_steps = n_decode - 1;
    }
    return 0;
}

// ---------------------------------------------------------------------------
// One decode step for `batch` independent sequences (no counterpart in the reference, which serves one):
// the activations of all sequences form a [batch, d] matrix, so every weight matrix is streamed once per
// step for all of them (the 2..16-row MFMA kernel that reads weights once), while each sequence keeps its
// own KV cache and position.  caches[0] lends its activation buffers.  Per-row arithmetic is that of a
// one-token prompt pass (separate RMSNorm, same rounding points as the single-sequence step).
// ---------------------------------------------------------------------------
extern "C" void llama3_decode_batch(Llama3 *m, CudaCache *const *caches, const int *tokens, int batch, int *next_tokens) {
    if (batch < 1 || batch > 16) llama3_fail("llama3_decode_batch: batch %d (1..16)", batch);
    Engine *e0 = eng(caches[0]);
    const ModelConfig &c = e0->cfg;
    bind_model(e0, m);
    const int d = c.d_model, hd = c.head_dim, Hq = c.n_heads;
    llm_stream_t s = e0->stream;
    Engine *es[16];
    int pos[16];
    for (int b = 0; b < batch; ++b) {
        es[b] = eng(caches[b]);
        for (int a = 0; a < b; ++a)
            if (es[a] == es[b]) llama3_fail("llama3_decode_batch: sequence %d and %d share a cache", a, b);
        const ModelConfig &cb = es[b]->cfg;
        if (cb.max_pos != c.max_pos || cb.d_model != d || cb.n_layers != c.n_layers || cb.vocab != c.vocab ||
            cb.n_kv_heads != c.n_kv_heads || cb.head_dim != c.head_dim)
            llama3_fail("llama3_decode_batch: cache %d has a different configuration", b);
        if (es[b]->pos + 1 > c.max_pos) llama3_fail("sequence of %d tokens exceeds max_pos %d", es[b]->pos + 1, c.max_pos);
        if (tokens[b] < 0 || tokens[b] >= c.vocab) llama3_fail("token id %d outside the vocabulary", tokens[b]);
        pos[b] = es[b]->pos;
        if (b > 0) llama3_check(llm_stream_sync(es[b]->stream), "stream sync"); // its prompt pass has finished
    }
    if (c.max_pos < batch) llama3_fail("llama3_decode_batch: max_pos %d below the batch size", c.max_pos);
    if (e0->batch_cap < batch) {
        if (e0->b_logits) llm_free(e0->b_logits);
        if (e0->b_ids) llm_free(e0->b_ids);
        if (e0->b_ws_attn) llm_free(e0->b_ws_attn);
        if (e0->b_ws_argmax) llm_free(e0->b_ws_argmax);
        e0->b_logits = dmalloc<llm_half>((size_t)16 * c.vocab, "llm_malloc(batch logits)");
        e0->b_ids = dmalloc<int32_t>(16, "llm_malloc(batch ids)");
        const size_t wsb = llm_attn_decode_workspace_bytes(Hq, hd);
        e0->b_ws_attn = dmalloc<char>(wsb * 16, "llm_malloc(batch attention workspace)");
        llama3_check(llm_fill_zero(e0->b_ws_attn, wsb * 16, s), "zero workspace");
        e0->b_ws_argmax = dmalloc<char>((size_t)16 * 1024 * 8, "llm_malloc(batch argmax candidates)");
        if (!e0->b_desc) {
            e0->b_desc = dmalloc<llm_batch_desc>(1, "llm_malloc(batch descriptor)");
            void *hp = nullptr;
            llama3_check(llm_malloc_host(&hp, sizeof(llm_batch_desc)), "llm_malloc_host(batch descriptor)");
            e0->b_desc_host = (llm_batch_desc *)hp;
            llama3_check(llm_malloc_host(&hp, sizeof(int32_t) * 16), "llm_malloc_host(batch ids)");
            e0->b_ids_host = (int32_t *)hp;
        }
        e0->batch_cap = 16;
    }
    // ids, caches and positions to the device through pinned staging, in stream order in front of the step
    bool long_form = false;
    for (int b = 0; b < batch; ++b) {
        e0->b_ids_host[b] = tokens[b];
        e0->b_desc_host->k_cache[b] = es[b]->kc;
        e0->b_desc_host->v_cache[b] = es[b]->vc;
        e0->b_desc_host->pos[b] = pos[b];
        long_form = long_form || pos[b] >= LONG_ATTN_FROM;
    }
    llama3_check(llm_memcpy_h2d(e0->b_ids, e0->b_ids_host, sizeof(int32_t) * (size_t)batch, s), "H2D ids");
    llama3_check(llm_memcpy_h2d(e0->b_desc, e0->b_desc_host, sizeof(llm_batch_desc), s), "H2D batch descriptor");
    const int form = long_form ? 1 : 0;
    if (e0->use_graph && e0->b_ran[batch][form]) {
        llm_graph_t &g = e0->b_graph[batch][form];
        if (!g) {
            llama3_check(llm_graph_capture_begin(s), "graph capture begin");
            issue_batch_step(e0, m, batch, form);
            llama3_check(llm_graph_capture_end(s, &g), "graph capture end");
        }
        llama3_check(llm_graph_launch(g, s), "graph launch");
    } else {
        issue_batch_step(e0, m, batch, form);
        e0->b_ran[batch][form] = true;
    }
    llama3_check(llm_memcpy_d2h(e0->b_ids_host, e0->b_ids, sizeof(int32_t) * (size_t)batch, s), "D2H tokens");
    llama3_check(llm_stream_sync(s), "stream sync");
    for (int b = 0; b < batch; ++b) {
        next_tokens[b] = (int)e0->b_ids_host[b];
        es[b]->tokens.push_back(tokens[b]);
        es[b]->pos += 1;
        es[b]->dev_pos_valid = false; // the batched step keeps no per-cache position on the device
    }
}

// fp16 logits of sequence b after the last llama3_decode_batch() in which caches[0] was this cache
extern "C" void llama3_read_batch_logits(CudaCache *C0, int b, llm_half *logits) {
    Engine *e = eng(C0);
    if (!e->b_logits || b < 0 || b >= e->batch_cap) llama3_fail("llama3_read_batch_logits: no batch step has run");
    llama3_check(llm_memcpy_d2h(logits, e->b_logits + (size_t)b * e->cfg.vocab, sizeof(llm_half) * (size_t)e->cfg.vocab,
                                e->stream),
                 "D2H logits");
    llama3_check(llm_stream_sync(e->stream), "stream sync");
}

extern "C" void llama3_set_hidden_trace(CudaCache *C, llm_half *hidden) { eng(C)->trace_host = hidden; }

extern "C" void llama3_set_hidden_inject(CudaCache *C, const llm_half *hidden) { eng(C)->inject_host = hidden; }

extern "C" void llama3_read_logits(CudaCache *C, llm_half *logits) {
    Engine *e = eng(C);
    llama3_check(llm_memcpy_d2h(logits, e->logits, sizeof(llm_half) * (size_t)e->cfg.vocab, e->stream), "D2H logits");
    llama3_check(llm_stream_sync(e->stream), "stream sync");
}

// Hand-over launches of the decode step (attention and output projection in one launch): spin_limit < 0
// restores the kernels' default bound of their wait, on != 0 puts a cache that left the form back into it.
extern "C" void llama3_set_handover(CudaCache *C, int on, int spin_limit) {
    Engine *e = eng(C);
    const bool want = on != 0;
    if (want != e->handover_on || spin_limit != e->handover_spin_limit) {
        llama3_check(llm_stream_sync(e->stream), "stream sync");
        drop_graph(e);
    }
    e->handover_on = want;
    e->handover_spin_limit = spin_limit;
}

extern "C" void llama3_handover_stats(const CudaCache *C, long *timeouts, long *recoveries, int *active) {
    const Engine *e = eng(C);
    if (timeouts) *timeouts = e->handover_timeouts;
    if (recoveries) *recoveries = e->handover_recoveries;
    if (active) *active = (e->handover_on && e->ao_ring) ? 1 : 0;
}

extern "C" void llama3_test_mark_handover_timeout(CudaCache *C) { eng(C)->handover_test_mark = true; }

extern "C" void llama3_set_use_graph(CudaCache *C, int on) {
    Engine *e = eng(C);
    e->use_graph = on != 0;
    if (!e->use_graph) drop_graph(e);
}

// inference.cu:149-193.  h_tokens[0] = n + 1, ids in h_tokens[1..n].  The
// reference recomputes all n rows on every call; here rows whose K/V are
// already cached (same leading ids as the previous call) are not recomputed,
// which yields the same next token because the recompute is causal.
extern "C" int inference(Llama3 *m, Tensor *X, int *d_tokens, int *h_tokens, CudaCache *C) {
    (void)X;
    Engine *e = eng(C);
    const int n = h_tokens[0] - 1;
    const int *ids = h_tokens + 1;
    if (n < 1) llama3_fail("inference: empty token list");
    bool extend = n > e->pos;
    for (int i = 0; extend && i < e->pos; ++i) extend = ids[i] == e->tokens[i];
    if (!extend) llama3_cache_reset(C);
    if (d_tokens) {
        // the reference's H2D of the token array (inference.cu:150); nothing here reads it back, so only
        // the entries that changed since the last call go up (the count and the new ids), in stream order
        const int first_new = e->pos + 1, last = n < 2047 ? n : 2047;
        llama3_check(llm_memcpy_h2d(d_tokens, h_tokens, sizeof(int), e->stream), "H2D token count");
        if (last >= first_new)
            llama3_check(llm_memcpy_h2d(d_tokens + first_new, h_tokens + first_new,
                                        sizeof(int) * (size_t)(last - first_new + 1), e->stream),
                         "H2D tokens");
    }
    const int fresh = n - e->pos;
    // h_token_probdist holds the step's logits on return, as after the reference's compute_lm_head
    // (inference.cu:1021-1026); they travel behind the token id in the same stream, one sync per call
    e->select_pending = e->sampling && prepare_selection(e);
    int tok = fresh == 1 ? step_one(e, m, ids[n - 1], C->h_token_probdist)
                         : run_pass(e, m, ids + e->pos, fresh, C->h_token_probdist);
    if (e->sampling) { // sample_next_token, inference.cu:1028
        int drawn = -1;
        if (e->select_pending) {
            e->select_pending = false;
            drawn = draw_from_selection(e);
        }
        if (drawn >= 0) {
            ++e->device_draws;
        } else {
            drawn = sampler_draw(e->sampler, C->f_token_probdist, C->h_token_probdist);
            ++e->host_draws;
        }
        tok = drawn;
    }
    return tok;
}

extern "C" void llama3_set_sampling(CudaCache *C, int on) { eng(C)->sampling = on != 0; }

extern "C" void llama3_set_device_sampling(CudaCache *C, int on) { eng(C)->device_select = on != 0; }

extern "C" void llama3_sampler_draw_counts(const CudaCache *C, long *device_draws, long *host_draws) {
    if (device_draws) *device_draws = eng(C)->device_draws;
    if (host_draws) *host_draws = eng(C)->host_draws;
}

// The cache's sampler applied to fp16 logits that already sit on the device.
extern "C" int llama3_sample_device_logits(CudaCache *C, const llm_half *logits_dev) {
    Engine *e = eng(C);
    if (!logits_dev) llama3_fail("llama3_sample_device_logits: null logits");
    int drawn = -1;
    if (prepare_selection(e)) {
        enqueue_selection(e, logits_dev);
        llama3_check(llm_stream_sync(e->stream), "stream sync");
        drawn = draw_from_selection(e);
    }
    if (drawn >= 0) {
        ++e->device_draws;
        return drawn;
    }
    llama3_check(llm_memcpy_d2h(C->h_token_probdist, logits_dev, sizeof(llm_half) * (size_t)e->cfg.vocab, e->stream),
                 "D2H logits");
    llama3_check(llm_stream_sync(e->stream), "stream sync");
    ++e->host_draws;
    return sampler_draw(e->sampler, C->f_token_probdist, C->h_token_probdist);
}

extern "C" void llama3_cache_sampler_config(CudaCache *C, float temperature, int top_k, float top_p) {
    Engine *e = eng(C);
    e->sampler.temperature = temperature;
    e->sampler.top_k = top_k;
    e->sampler.top_p = top_p;
}
