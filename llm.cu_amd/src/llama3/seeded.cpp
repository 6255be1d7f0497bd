// Seeded synthetic checkpoints: a counter-based generator so that a tensor's
// bits depend on (seed, tensor id, element index) only, whether it is written
// to a safetensors file or filled straight into host memory.  No LLaMA3
// weights ship with the reference (model_weights/ holds a README only), so
// every configuration runs on these.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "common/fail.h"
#include "llama3/llama3.h"
#include "llama3_host.h"

static inline uint64_t mix64(uint64_t z) { // splitmix64 finaliser
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

static inline uint16_t f32_to_bf16_rne(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// Inverse normal CDF: Acklam's rational approximation, then one Halley step
// against erfc, which brings it to double precision.
static double inv_norm_cdf(double p) {
    static const double a[] = {-3.969683028665376e+01, 2.209460984245205e+02, -2.759285104469687e+02,
                               1.383577518672690e+02,  -3.066479806614716e+01, 2.506628277459239e+00};
    static const double b[] = {-5.447609879822406e+01, 1.615858368580409e+02, -1.556989798598866e+02,
                               6.680131188771972e+01,  -1.328068155288572e+01};
    static const double c[] = {-7.784894002430293e-03, -3.223964580411365e-01, -2.400758277161838e+00,
                               -2.549732539343734e+00, 4.374664141464968e+00,  2.938163982698783e+00};
    static const double d[] = {7.784695709041462e-03, 3.224671290700398e-01, 2.445134137142996e+00,
                               3.754408661907416e+00};
    const double plow = 0.02425, phigh = 1.0 - plow;
    double x;
    if (p < plow) {
        double q = std::sqrt(-2.0 * std::log(p));
        x = (((((c[0] * q + c[1]) * q + c[2]) * q + c[3]) * q + c[4]) * q + c[5]) /
            ((((d[0] * q + d[1]) * q + d[2]) * q + d[3]) * q + 1.0);
    } else if (p <= phigh) {
        double q = p - 0.5, r = q * q;
        x = (((((a[0] * r + a[1]) * r + a[2]) * r + a[3]) * r + a[4]) * r + a[5]) * q /
            (((((b[0] * r + b[1]) * r + b[2]) * r + b[3]) * r + b[4]) * r + 1.0);
    } else {
        double q = std::sqrt(-2.0 * std::log(1.0 - p));
        x = -(((((c[0] * q + c[1]) * q + c[2]) * q + c[3]) * q + c[4]) * q + c[5]) /
            ((((d[0] * q + d[1]) * q + d[2]) * q + d[3]) * q + 1.0);
    }
    double e = 0.5 * std::erfc(-x / std::sqrt(2.0)) - p;
    double u = e * std::sqrt(2.0 * M_PI) * std::exp(x * x / 2.0);
    return x - u / (1.0 + x * u / 2.0);
}

namespace {
struct Table {
    float sigma;
    std::vector<uint16_t> v;
};
std::mutex g_mu;
std::vector<Table *> g_tables;
} // namespace

// tab[j] = bf16(sigma * Phi^-1((j + 0.5) / 65536)): 65536 equiprobable strata.
extern "C" const uint16_t *seeded_unit_table_bf16(float sigma) {
    std::lock_guard<std::mutex> lk(g_mu);
    for (Table *t : g_tables)
        if (t->sigma == sigma) return t->v.data();
    Table *t = new Table;
    t->sigma = sigma;
    t->v.resize(65536);
    for (int j = 0; j < 65536; ++j)
        t->v[j] = f32_to_bf16_rne((float)((double)sigma * inv_norm_cdf((j + 0.5) / 65536.0)));
    g_tables.push_back(t);
    return t->v.data();
}

// Element i takes bits [16*(i%4), 16*(i%4)+16) of mix64(key + (i/4) * golden).
extern "C" void seeded_normal_bf16(uint64_t seed, uint64_t tensor_id, size_t n, float sigma,
                                   uint16_t *out) {
    const uint16_t *tab = seeded_unit_table_bf16(sigma);
    const uint64_t key = mix64(mix64(seed) ^ tensor_id);
    const size_t groups = (n + 3) / 4;
#pragma omp parallel for schedule(static)
    for (size_t g = 0; g < groups; ++g) {
        uint64_t h = mix64(key + g * 0x9E3779B97F4A7C15ull);
        size_t base = g * 4;
        size_t lim = n - base < 4 ? n - base : 4;
        for (size_t j = 0; j < lim; ++j) out[base + j] = tab[(h >> (16 * j)) & 0xffffu];
    }
}

extern "C" void seeded_tokens(uint64_t seed, int n, int vocab, int *out) {
    const uint64_t key = mix64(mix64(seed) ^ 0x746f6b656e73ull); // "tokens"
    for (int i = 0; i < n; ++i) {
        uint64_t h = mix64(key + (uint64_t)i * 0x9E3779B97F4A7C15ull);
        out[i] = (int)(((h >> 32) * (uint64_t)vocab) >> 32);
    }
}

// ids: 0 embed, 1 lm_head, 2 norm, then 16 + 16*layer + slot.
extern "C" uint64_t seeded_tensor_id(int layer, int slot) {
    return layer < 0 ? (uint64_t)slot : 16ull + 16ull * (uint64_t)layer + (uint64_t)slot;
}

namespace {
struct Spec {
    std::string key;
    uint64_t id;
    int rows, cols; // cols == 0: 1-d
    bool gain;
    Tensor *(*slot)(Llama3 *, int);
    int layer;
};

std::vector<Spec> specs(const ModelConfig *c) {
    std::vector<Spec> s;
    const int d = c->d_model, qd = c->n_heads * c->head_dim, kvd = c->n_kv_heads * c->head_dim;
    s.push_back({"model.embed_tokens.weight", seeded_tensor_id(-1, 0), c->vocab, d, false,
                 [](Llama3 *m, int) { return m->embed_tokens; }, -1});
    for (int l = 0; l < c->n_layers; ++l) {
        std::string p = "model.layers." + std::to_string(l) + ".";
        s.push_back({p + "input_layernorm.weight", seeded_tensor_id(l, 0), d, 0, true,
                     [](Llama3 *m, int i) { return m->layers[i]->input_layernorm; }, l});
        s.push_back({p + "mlp.down_proj.weight", seeded_tensor_id(l, 1), d, c->ffn_dim, false,
                     [](Llama3 *m, int i) { return m->layers[i]->mlp_down_proj; }, l});
        s.push_back({p + "mlp.gate_proj.weight", seeded_tensor_id(l, 2), c->ffn_dim, d, false,
                     [](Llama3 *m, int i) { return m->layers[i]->mlp_gate_proj; }, l});
        s.push_back({p + "mlp.up_proj.weight", seeded_tensor_id(l, 3), c->ffn_dim, d, false,
                     [](Llama3 *m, int i) { return m->layers[i]->mlp_up_proj; }, l});
        s.push_back({p + "post_attention_layernorm.weight", seeded_tensor_id(l, 4), d, 0, true,
                     [](Llama3 *m, int i) { return m->layers[i]->post_attention_layernorm; }, l});
        s.push_back({p + "self_attn.k_proj.weight", seeded_tensor_id(l, 5), kvd, d, false,
                     [](Llama3 *m, int i) { return m->layers[i]->self_attn_k_proj; }, l});
        s.push_back({p + "self_attn.o_proj.weight", seeded_tensor_id(l, 6), d, qd, false,
                     [](Llama3 *m, int i) { return m->layers[i]->self_attn_o_proj; }, l});
        s.push_back({p + "self_attn.q_proj.weight", seeded_tensor_id(l, 7), qd, d, false,
                     [](Llama3 *m, int i) { return m->layers[i]->self_attn_q_proj; }, l});
        s.push_back({p + "self_attn.v_proj.weight", seeded_tensor_id(l, 8), kvd, d, false,
                     [](Llama3 *m, int i) { return m->layers[i]->self_attn_v_proj; }, l});
    }
    s.push_back({"model.norm.weight", seeded_tensor_id(-1, 2), d, 0, true,
                 [](Llama3 *m, int) { return m->norm; }, -1});
    s.push_back({"lm_head.weight", seeded_tensor_id(-1, 1), c->vocab, d, false,
                 [](Llama3 *m, int) { return m->lm_head; }, -1});
    return s;
}

void fill(const Spec &sp, uint64_t seed, uint16_t *dst) {
    size_t n = (size_t)sp.rows * (sp.cols ? sp.cols : 1);
    if (sp.gain) {
        for (size_t i = 0; i < n; ++i) dst[i] = 0x3F80u; // bf16 1.0
    } else {
        seeded_normal_bf16(seed, sp.id, n, 0.02f, dst);
    }
}
} // namespace

extern "C" void seeded_fill_model(Llama3 *m, const ModelConfig *cfg, uint64_t seed) {
    if (m->n_layers != cfg->n_layers) llama3_fail("seeded_fill_model: layer count mismatch");
    for (const Spec &sp : specs(cfg)) {
        Tensor *t = sp.slot(m, sp.layer < 0 ? 0 : sp.layer);
        int shape[2] = {sp.rows, sp.cols};
        tensor_set_host_shape(t, sp.cols ? 2 : 1, shape);
        t->bf16_tensor = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)*t->mem_len);
        if (!t->bf16_tensor) llama3_fail("An Error Occurred while allocating memory for the component Tensor");
        fill(sp, seed, t->bf16_tensor);
    }
}

extern "C" int seeded_write_safetensors(const ModelConfig *cfg, uint64_t seed, const char *path) {
    std::vector<Spec> sp = specs(cfg);
    std::string hdr = "{\"__metadata__\":{\"format\":\"pt\"}";
    size_t off = 0;
    for (const Spec &s : sp) {
        size_t bytes = 2 * (size_t)s.rows * (s.cols ? s.cols : 1);
        hdr += ",\"" + s.key + "\":{\"dtype\":\"BF16\",\"shape\":[" + std::to_string(s.rows);
        if (s.cols) hdr += "," + std::to_string(s.cols);
        hdr += "],\"data_offsets\":[" + std::to_string(off) + "," + std::to_string(off + bytes) + "]}";
        off += bytes;
    }
    hdr += "}";
    while (hdr.size() % 8) hdr += ' ';
    FILE *fp = fopen(path, "wb");
    if (!fp) return -1;
    uint64_t n = hdr.size();
    fwrite(&n, 8, 1, fp);
    fwrite(hdr.data(), 1, hdr.size(), fp);
    std::vector<uint16_t> buf;
    for (const Spec &s : sp) {
        size_t cnt = (size_t)s.rows * (s.cols ? s.cols : 1);
        buf.resize(cnt);
        fill(s, seed, buf.data());
        if (fwrite(buf.data(), 2, cnt, fp) != cnt) {
            fclose(fp);
            return -1;
        }
    }
    fclose(fp);
    return 0;
}
