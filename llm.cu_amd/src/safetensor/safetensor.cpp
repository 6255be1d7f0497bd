// Safetensors loader: file -> host bf16 tensors of a Llama3.
// Follows src/safetensor/safetensor.cu of the reference: u64 little-endian
// header length, JSON header {name: {dtype, shape, data_offsets:[b,e]}}, data
// at 8 + header_len + b; entries lacking any of the three keys (e.g.
// __metadata__) are skipped (:71); slot chosen by the first matching substring
// in the reference's order (:99-123); layer index = atoi of the third
// dot-separated token of the key (:83,164-191).
// Stricter than the reference in three places where it reads out of bounds or
// silently loads garbage: dtype must be BF16, the layer index must exist, and
// a short read is an error.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

#include "common/fail.h"
#include "llama3/llama3.h"
#include "llama3_host.h"
#include "safetensor/json.h"

namespace {

struct SafeTensorFile {
    FILE *fp = nullptr;
    uint64_t header_size = 0;
    char *header = nullptr;
};

// safetensor.cu:164-191
int get_llama3_decoder_layer_num(const char *layer_key, int index) {
    std::string s(layer_key);
    size_t pos = 0;
    for (int i = 0;; ++i) {
        // strtok semantics: skip leading delimiters, token runs to the next '.'
        while (pos < s.size() && s[pos] == '.') ++pos;
        if (pos >= s.size()) return -1;
        size_t end = s.find('.', pos);
        if (end == std::string::npos) end = s.size();
        if (i == index) return atoi(s.substr(pos, end - pos).c_str());
        pos = end;
    }
}

// safetensor.cu:33-50
void safetensor_load_header(SafeTensorFile *stf, const char *filename) {
    uint64_t n = 0;
    if (fread(&n, sizeof(uint64_t), 1, stf->fp) != 1)
        llama3_fail("%s is too short to hold a safetensors header", filename);
    fseek(stf->fp, 0, SEEK_END);
    long fsize = ftell(stf->fp);
    fseek(stf->fp, 8, SEEK_SET);
    if (fsize < 8 || n > (uint64_t)(fsize - 8))
        llama3_fail("%s: header length %llu exceeds the file size", filename, (unsigned long long)n);
    stf->header_size = n;
    stf->header = (char *)malloc(n + 1);
    if (!stf->header)
        llama3_fail("An Error Occurred while allocating memory for the safetensor file header data");
    if (fread(stf->header, 1, n, stf->fp) != n) llama3_fail("%s: short read of the header", filename);
    stf->header[n] = '\0';
}

// safetensor.cu:82-162
void llama3_load_layer(const std::string &key, const minijson::Value &entry, SafeTensorFile *stf,
                       Llama3 *m, const char *filename) {
    int layer_num = get_llama3_decoder_layer_num(key.c_str(), 2);
    const minijson::Value *dtype = entry.get("dtype");
    const minijson::Value *shape = entry.get("shape");
    const minijson::Value *offs = entry.get("data_offsets");

    const char *k = key.c_str();
    bool per_layer = true;
    Tensor *Llama3Layer::*slot = nullptr;
    Tensor *component = nullptr;
    if (strstr(k, "input_layernorm")) slot = &Llama3Layer::input_layernorm;
    else if (strstr(k, "down_proj")) slot = &Llama3Layer::mlp_down_proj;
    else if (strstr(k, "gate_proj")) slot = &Llama3Layer::mlp_gate_proj;
    else if (strstr(k, "up_proj")) slot = &Llama3Layer::mlp_up_proj;
    else if (strstr(k, "post_attention_layernorm")) slot = &Llama3Layer::post_attention_layernorm;
    else if (strstr(k, "k_proj")) slot = &Llama3Layer::self_attn_k_proj;
    else if (strstr(k, "o_proj")) slot = &Llama3Layer::self_attn_o_proj;
    else if (strstr(k, "q_proj")) slot = &Llama3Layer::self_attn_q_proj;
    else if (strstr(k, "v_proj")) slot = &Llama3Layer::self_attn_v_proj;
    else {
        per_layer = false;
        if (strstr(k, "embed_tokens")) component = m->embed_tokens;
        else if (strstr(k, "model.norm")) component = m->norm;
        else if (strstr(k, "lm_head")) component = m->lm_head;
    }
    if (per_layer) {
        if (layer_num < 0 || layer_num >= m->n_layers)
            llama3_fail("%s names layer %d but the model has %d layers", k, layer_num, m->n_layers);
        component = m->layers[layer_num]->*slot;
    }
    if (component == nullptr) llama3_fail("Component not allocated or not initialized properly.");

    if (dtype->kind != minijson::Value::String || dtype->str != "BF16")
        llama3_fail("%s: dtype %s is not BF16", k, dtype->kind == minijson::Value::String ? dtype->str.c_str() : "?");
    if (shape->kind != minijson::Value::Array || offs->kind != minijson::Value::Array || offs->arr.empty())
        llama3_fail("%s: malformed shape or data_offsets", k);

    int ndim = (int)shape->arr.size();
    int dims[8];
    if (ndim > 8) llama3_fail("%s: %d dimensions", k, ndim);
    for (int i = 0; i < ndim; ++i) dims[i] = (int)shape->arr[i].num;
    tensor_set_host_shape(component, ndim, dims);
    size_t mem_len = (size_t)*component->mem_len;

    free(component->bf16_tensor);
    component->bf16_tensor = (uint16_t *)malloc(sizeof(uint16_t) * mem_len);
    if (component->bf16_tensor == nullptr)
        llama3_fail("An Error Occurred while allocating memory for the component Tensor");

    long offset = 8L + (long)stf->header_size + (long)offs->arr[0].num;
    fseek(stf->fp, offset, SEEK_SET);
    size_t got = fread(component->bf16_tensor, sizeof(uint16_t), mem_len, stf->fp);
    if (got != mem_len) llama3_fail("%s: %s holds %zu of %zu elements", filename, k, got, mem_len);
}

// safetensor.cu:52-80
void safetensor_read_header(SafeTensorFile *stf, Llama3 *m, const char *filename) {
    minijson::Value json;
    minijson::Parser parser(stf->header, stf->header_size);
    if (!parser.parse(json) || json.kind != minijson::Value::Object) {
        printf("Error: Error parsing JSON\n"); // the reference prints and returns (:56-59)
        return;
    }
    for (const auto &kv : json.obj) {
        const minijson::Value &e = kv.second;
        if (e.kind != minijson::Value::Object) continue;
        if (e.get("dtype") && e.get("shape") && e.get("data_offsets"))
            llama3_load_layer(kv.first, e, stf, m, filename);
    }
}

} // namespace

// safetensor.cu:16-31
extern "C" void load_safetensor_weights(Llama3 *llama3_model, const char *filename) {
    SafeTensorFile stf;
    stf.fp = fopen(filename, "rb");
    if (stf.fp == nullptr) llama3_fail("An Error Occurred while opening %s", filename);
    safetensor_load_header(&stf, filename);
    safetensor_read_header(&stf, llama3_model, filename);
    fclose(stf.fp);
    free(stf.header);
}
