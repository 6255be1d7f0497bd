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
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "common/fail.h"
#include "llama3/llama3.h"
#include "llama3_host.h"
#include "llmcu_hip.h"
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

// Placement of one header entry (safetensor.cu:82-127 and the shape part of :128-150): which tensor of
// the model it fills, with its shape recorded in the descriptor, and where its bytes start in the file.
struct Placement {
    Tensor *component;
    long offset;
    size_t mem_len;
};

Placement resolve_entry(const std::string &key, const minijson::Value &entry, const SafeTensorFile *stf, Llama3 *m) {
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
    Placement p;
    p.component = component;
    p.mem_len = (size_t)*component->mem_len;
    p.offset = 8L + (long)stf->header_size + (long)offs->arr[0].num;
    return p;
}

// safetensor.cu:128-162: the payload into a fresh host buffer
void llama3_load_layer(const std::string &key, const minijson::Value &entry, SafeTensorFile *stf,
                       Llama3 *m, const char *filename) {
    const Placement p = resolve_entry(key, entry, stf, m);
    Tensor *component = p.component;
    free(component->bf16_tensor);
    component->bf16_tensor = (uint16_t *)malloc(sizeof(uint16_t) * p.mem_len);
    if (component->bf16_tensor == nullptr)
        llama3_fail("An Error Occurred while allocating memory for the component Tensor");
    fseek(stf->fp, p.offset, SEEK_SET);
    size_t got = fread(component->bf16_tensor, sizeof(uint16_t), p.mem_len, stf->fp);
    if (got != p.mem_len) llama3_fail("%s: %s holds %zu of %zu elements", filename, key.c_str(), got, p.mem_len);
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

// ---------------------------------------------------------------------------
// Streaming load: the same device state as load_safetensor_weights() for every file followed by
// to_cuda(), without ever holding the checkpoint in host memory.  Pass 1 reads only the headers (shapes
// and file offsets), the HBM slab is laid out, pass 2 moves every tensor through two pinned 64 MiB
// buffers: while one chunk is on its way to the device (async copy, then BF16->FP16 on the same
// stream) the next is read from the file.  Peak host memory: the two buffers.
// ---------------------------------------------------------------------------
extern "C" void load_safetensor_weights_streaming(Llama3 *m, const char *const *filenames, int n_files) {
    struct Job {
        int file;
        std::string key;
        Placement p;
    };
    std::vector<SafeTensorFile> files((size_t)n_files);
    std::vector<Job> jobs;
    for (int f = 0; f < n_files; ++f) {
        SafeTensorFile &stf = files[(size_t)f];
        stf.fp = fopen(filenames[f], "rb");
        if (stf.fp == nullptr) llama3_fail("An Error Occurred while opening %s", filenames[f]);
        safetensor_load_header(&stf, filenames[f]);
        minijson::Value json;
        minijson::Parser parser(stf.header, stf.header_size);
        if (!parser.parse(json) || json.kind != minijson::Value::Object)
            llama3_fail("%s: Error parsing JSON", filenames[f]);
        for (const auto &kv : json.obj) {
            const minijson::Value &e = kv.second;
            if (e.kind != minijson::Value::Object) continue;
            if (e.get("dtype") && e.get("shape") && e.get("data_offsets"))
                jobs.push_back({f, kv.first, resolve_entry(kv.first, e, &stf, m)});
        }
    }
    llama3_plan_slab(m); // fails if a tensor of the model appeared in no header
    // ascending offsets keep the reads sequential within a shard whatever order the header lists the keys in
    std::stable_sort(jobs.begin(), jobs.end(), [](const Job &a, const Job &b) {
        return a.file != b.file ? a.file < b.file : a.p.offset < b.p.offset;
    });

    const size_t CHUNK = (size_t)32 << 20; // elements: 64 MiB of bf16
    uint16_t *host[2] = {nullptr, nullptr};
    void *dev[2] = {nullptr, nullptr};
    llm_event_t done[2] = {nullptr, nullptr};
    llm_stream_t s = nullptr;
    llama3_check(llm_stream_create(&s), "llm_stream_create");
    for (int b = 0; b < 2; ++b) {
        llama3_check(llm_malloc_host((void **)&host[b], CHUNK * 2), "llm_malloc_host(staging)");
        llama3_check(llm_malloc(&dev[b], CHUNK * 2), "llm_malloc(bf16 staging)");
        llama3_check(llm_event_create(&done[b]), "llm_event_create");
    }
    bool used[2] = {false, false};
    int b = 0;
    for (const Job &j : jobs) {
        SafeTensorFile &stf = files[(size_t)j.file];
        fseek(stf.fp, j.p.offset, SEEK_SET);
        for (size_t at = 0; at < j.p.mem_len; at += CHUNK) {
            const size_t n = j.p.mem_len - at < CHUNK ? j.p.mem_len - at : CHUNK;
            if (used[b]) llama3_check(llm_event_sync(done[b]), "event sync"); // buffer b is free again
            const size_t got = fread(host[b], sizeof(uint16_t), n, stf.fp);
            if (got != n)
                llama3_fail("%s: %s holds %zu of %zu elements", filenames[j.file], j.key.c_str(), at + got, j.p.mem_len);
            llama3_check(llm_memcpy_h2d(dev[b], host[b], n * 2, s), "H2D of bf16 weights");
            llama3_check(llm_bf16_to_fp16((const uint16_t *)dev[b], j.p.component->d_fp16_tensor + at, n, s),
                         "llm_bf16_to_fp16");
            llama3_check(llm_event_record(done[b], s), "event record");
            used[b] = true;
            b ^= 1;
        }
    }
    llama3_check(llm_stream_sync(s), "stream sync");
    for (int i = 0; i < 2; ++i) {
        llama3_check(llm_event_destroy(done[i]), "llm_event_destroy");
        llama3_check(llm_free(dev[i]), "llm_free(bf16 staging)");
        llama3_check(llm_free_host(host[i]), "llm_free_host(staging)");
    }
    llama3_check(llm_stream_destroy(s), "llm_stream_destroy");
    for (SafeTensorFile &stf : files) {
        fclose(stf.fp);
        free(stf.header);
    }
}
