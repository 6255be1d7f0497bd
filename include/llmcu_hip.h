/*
 * llmcu_hip.h -- thin C-ABI over the hand-written gfx950 (MI355X) kernels of
 * the LLaMA3 token loop.  One entry point per kernel family; every pointer
 * marked "device" is HBM memory, fp16 tensors are passed as uint16_t bit
 * patterns, `stream` is a hipStream_t (NULL = the default stream).  All entry
 * points return LLM_OK or an error code; llm_last_error() gives the text.
 * Nothing here is asynchronous with respect to the given stream order.
 *
 * Each entry point names the launcher/kernel of the reference it replaces
 * (paths under src/ of abhisheknair10/LLM.cu).  The host layer
 * (llama3_host.h) is written against this header only and never includes the
 * HIP runtime.
 */
#ifndef LLMCU_HIP_H
#define LLMCU_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    LLM_OK = 0,
    LLM_ERR_INVALID = 1, /* bad argument or a shape the kernels do not cover */
    LLM_ERR_HIP = 2,     /* the HIP runtime reported an error */
    LLM_ERR_NO_DEVICE = 3
};

typedef void *llm_stream_t;
typedef void *llm_event_t;
typedef void *llm_graph_t;

/* ---- runtime (replaces the reference's direct cudart calls) ------------ */
const char *llm_last_error(void);
int llm_device_count(int *count);
int llm_init(int device);                 /* select the device; fails unless it is gfx950 */
int llm_device_name(char *buf, size_t n); /* e.g. "gfx950:sramecc+:xnack-" */
int llm_device_cu_count(int *n);
int llm_malloc(void **ptr, size_t bytes);           /* cudaMalloc   (inference.cu:101-108) */
int llm_free(void *ptr);                            /* cudaFree */
int llm_mem_info(size_t *free_bytes, size_t *total_bytes); /* cudaMemGetInfo (inference.cu:46-62) */
int llm_malloc_host(void **ptr, size_t bytes);      /* pinned host memory */
int llm_free_host(void *ptr);
int llm_memcpy_h2d(void *dst, const void *src, size_t bytes, llm_stream_t stream);
int llm_memcpy_d2h(void *dst, const void *src, size_t bytes, llm_stream_t stream);
int llm_memcpy_d2d(void *dst, const void *src, size_t bytes, llm_stream_t stream);
int llm_fill_zero(void *dst, size_t bytes, llm_stream_t stream); /* a fill kernel, graph-safe */
int llm_stream_create(llm_stream_t *stream);
int llm_stream_destroy(llm_stream_t stream);
int llm_stream_sync(llm_stream_t stream);
int llm_device_sync(void);                          /* cudaDeviceSynchronize */
int llm_event_create(llm_event_t *ev);
int llm_event_destroy(llm_event_t ev);
int llm_event_record(llm_event_t ev, llm_stream_t stream);
int llm_event_sync(llm_event_t ev);
int llm_event_elapsed_ms(llm_event_t start, llm_event_t stop, float *ms);
int llm_graph_capture_begin(llm_stream_t stream);
int llm_graph_capture_end(llm_stream_t stream, llm_graph_t *graph_exec);
int llm_graph_launch(llm_graph_t graph_exec, llm_stream_t stream);
int llm_graph_destroy(llm_graph_t graph_exec);

/* ---- BF16 -> FP16 weight conversion ------------------------------------ */
/* Replaces _kernel_wrapper_bf16_to_fp16 / _kernel_bf16_to_fp16
 * (src/llama3/llama3.cu:219-254): dst[i] = fp16_rne(float(src[i] << 16)),
 * NaN -> 0x7FFF.  Bit-exact.  4 algorithmic bytes per element. */
int llm_bf16_to_fp16(const uint16_t *src_dev, uint16_t *dst_dev, size_t n, llm_stream_t stream);

/* ---- embedding gather ---------------------------------------------------- */
/* Replaces tokens_to_embeddings / kernel_tokens_to_embeddings
 * (src/inference/inference.cu:196-223): out[t,:] = table[ids[t],:].
 * ids are int32 on the device; an id outside [0, vocab) is rejected by
 * writing a row of fp16 NaN (the reference reads out of bounds).
 * ids_offset_dev (may be NULL): device int added to the index into ids_dev,
 * so a captured graph can walk a token buffer. */
int llm_embed_gather(const uint16_t *table_dev, const int32_t *ids_dev, const int32_t *ids_offset_dev,
                     uint16_t *out_dev, int T, int d, int vocab, llm_stream_t stream);

/* ---- RMSNorm --------------------------------------------------------------- */
/* Replaces compute_layer_norm / kernel_compute_rms_norm
 * (src/inference/inference.cu:282-363): y = fp16(x * g / sqrtf(eps + ss/d)),
 * ss summed in the reference's own order (4-element partials, stride-halving
 * tree), eps added in double as the reference's literal 1e-5 is.  y may alias
 * x (the reference normalises in place).  Requires d % 4 == 0, d/4 a power of
 * two, 64 <= d/4 <= 4096. */
int llm_rmsnorm(const uint16_t *x_dev, const uint16_t *gain_dev, uint16_t *y_dev, int T, int d,
                double eps, llm_stream_t stream);

/* ---- residual add ---------------------------------------------------------- */
/* Replaces add_norm / kernel_add_norm (src/inference/inference.cu:366-390):
 * x = fp16(float(x) + float(res)). */
int llm_add_residual(uint16_t *x_dev, const uint16_t *res_dev, size_t n, llm_stream_t stream);

/* ---- RoPE -------------------------------------------------------------------- */
/* Host helper: fills table[pos][i] = (cosf(a), sinf(a)), a = pos * 1/powf(theta, 2i/head_dim),
 * i < head_dim/2, pos < max_pos, with the host libm -- the reference evaluates
 * the same expression per element inside its kernel (inference.cu:673-678). */
int llm_rope_table_host(float *table_host, int max_pos, int head_dim, float theta);
/* Replaces rope_scaling / kernel_rope_scaling (src/inference/inference.cu:621-695):
 * adjacent pairs (x[2p], x[2p+1]) of every head rotated in place by the
 * angle of (pos0 + t, p % (head_dim/2)).  buf: [T, row_stride] fp16 with
 * n_heads*head_dim leading columns used.  pos_dev (may be NULL): device int
 * added to pos0, so a captured graph can advance without new arguments.
 * table_dev: [max_pos][head_dim/2][2] floats from llm_rope_table_host. */
int llm_rope(uint16_t *buf_dev, int T, int n_heads, int head_dim, int row_stride, int pos0,
             const int32_t *pos_dev, const float *table_dev, int max_pos, llm_stream_t stream);
/* Fused form used by the engine: rotates Q in place inside qkv ([T, (Hq+2Hkv)*hd]),
 * rotates K and writes it into the K cache ([Hkv][max_pos][hd] per layer,
 * rows pos0+t), and stores V into the V cache, which is kept transposed
 * ([Hkv][hd][max_pos], columns pos0+t) so that P.V streams contiguous memory. */
int llm_rope_kv_append(uint16_t *qkv_dev, uint16_t *k_cache_dev, uint16_t *v_cache_dev, int T,
                       int n_heads, int n_kv_heads, int head_dim, int pos0, const int32_t *pos_dev,
                       const float *table_dev, int max_pos, llm_stream_t stream);
/* The same without the pass over Q: K is rotated into the K cache and V stored into the V cache, the queries in qkv
 * stay as the projection left them -- for a prompt pass whose attention rotates the queries itself
 * (llm_attn_prefill_rope_q).  At least 16 rows, positions known on the host. */
int llm_rope_k_append(uint16_t *qkv_dev, uint16_t *k_cache_dev, uint16_t *v_cache_dev, int T, int n_heads,
                      int n_kv_heads, int head_dim, int pos0, const float *table_dev, int max_pos, llm_stream_t stream);

/* ---- projections -------------------------------------------------------------- */
/* Replaces kernel_standard_tiled_gemm and its launchers compute_qkv_tensors,
 * compute_output, the down projection of compute_feedforward
 * (src/inference/inference.cu:393-449,561-618,967-976):
 * out[t,n] = fp16(sum_k x[t,k] * w[n,k] (+ float(residual[t,n]))), fp32
 * accumulation, w is [N,K] row-major.  With residual != NULL the result is
 * fp16(fp16(sum) + residual), the reference's add_norm applied to the stored
 * projection (inference.cu:377-390).  ldx/ldo/ldr are row strides in elements.
 * T == 1 runs the bandwidth-bound GEMV, 2 <= T <= 16 the skinny kernel, larger
 * T the MFMA GEMM.  K % 64 == 0 and N % 16 == 0 are required.
 * Device memory the call may take: passes of 17 to 1024 rows split k over several workgroups and keep fp32
 * partial tiles in a 64 MiB buffer that belongs to the (device, stream) pair.  llm_init allocates the default
 * stream's; any other stream gets its own at its first such launch (a hipMalloc inside llm_linear) and returns
 * it in llm_stream_destroy -- a stream that was not created by llm_stream_create keeps its buffer until the
 * process ends.  When the buffer cannot be had (no memory, or that first launch falls inside a graph capture)
 * the launch runs unsplit, slower and with the same results up to summation order;
 * llm_linear_unsplit_fallbacks() counts such launches since the library was loaded. */
int llm_linear(const uint16_t *x_dev, int ldx, const uint16_t *w_dev, const uint16_t *residual_dev,
               int ldr, uint16_t *out_dev, int ldo, int T, int N, int K, llm_stream_t stream);
/* Replaces kernel_standard_tiled_gemm_ffn_swiglu (src/inference/inference.cu:455-519):
 * out[t,n] = fp16(SiLU(sum_k x.wgate) * (sum_k x.wup)), neither sum rounded on its own. */
long llm_linear_unsplit_fallbacks(void);
int llm_linear_swiglu(const uint16_t *x_dev, int ldx, const uint16_t *wgate_dev,
                      const uint16_t *wup_dev, uint16_t *out_dev, int ldo, int T, int N, int K,
                      llm_stream_t stream);

/* One-row projections with the RMSNorm of the input folded in (the decode
 * step): out = linear(rmsnorm(x, gain, eps), w).  Replaces compute_layer_norm
 * followed by compute_qkv_tensors, resp. by the gate/up launch of
 * compute_feedforward (src/inference/inference.cu:160-163,179-182) for T = 1;
 * same bits as llm_rmsnorm followed by llm_linear / llm_linear_swiglu. */
int llm_norm_linear(const uint16_t *x_dev, const uint16_t *gain_dev, double eps, const uint16_t *w_dev,
                    uint16_t *out_dev, int N, int K, llm_stream_t stream);
int llm_norm_linear_swiglu(const uint16_t *x_dev, const uint16_t *gain_dev, double eps,
                           const uint16_t *wgate_dev, const uint16_t *wup_dev, uint16_t *out_dev, int N,
                           int K, llm_stream_t stream);

/* The first projection of a decode step with the embedding gather folded in: the input row is
 * table[ids[ids_offset ? *ids_offset : 0]] (a row of 0x7fff NaNs for an id outside [0, vocab), as
 * llm_embed_gather writes), out = linear(rmsnorm(row, gain, eps), w), and x_out receives the row itself (the
 * residual stream of the first layer).  Replaces tokens_to_embeddings followed by compute_layer_norm and
 * compute_qkv_tensors of layer 0 (src/inference/inference.cu:149-163) for T = 1; same bits as
 * llm_embed_gather followed by llm_norm_linear, one launch fewer. */
int llm_embed_norm_linear(const uint16_t *table_dev, const int32_t *ids_dev, const int32_t *ids_offset_dev, int vocab,
                          uint16_t *x_out_dev, const uint16_t *gain_dev, double eps, const uint16_t *w_dev,
                          uint16_t *out_dev, int N, int K, llm_stream_t stream);

/* ---- attention ------------------------------------------------------------------ */
/* Replaces compute_attention and its three kernels
 * (src/inference/inference.cu:698-947) for one new row: causal GQA attention
 * of the query at position ctx-1 over cache rows 0..ctx-1, kv_head = q_head /
 * (Hq/Hkv), scores scaled by 1/sqrtf(head_dim), softmax and P.V in fp32.
 * q: [Hq*hd] fp16; K cache [Hkv][max_pos][hd], V cache [Hkv][hd][max_pos];
 * out: [Hq*hd] fp16.  ctx = ctx_host + (ctx_dev ? *ctx_dev : 0).
 * max_pos % 64 == 0.  workspace: llm_attn_decode_workspace_bytes, zeroed once
 * with llm_fill_zero before its first use (every call leaves it reusable);
 * calls that share a workspace must not overlap. */
size_t llm_attn_decode_workspace_bytes(int n_heads, int head_dim);
int llm_attn_decode(const uint16_t *q_dev, const uint16_t *k_cache_dev, const uint16_t *v_cache_dev,
                    uint16_t *out_dev, int ctx_host, const int32_t *ctx_dev, int n_heads,
                    int n_kv_heads, int head_dim, int max_pos, void *workspace_dev,
                    llm_stream_t stream);
/* No counterpart in the reference: llm_attn_decode for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  Same
 * arguments without the workspace: the partial results and counters live in an array built into the
 * library's device code (llm_attn_decode_noalloc_max_bytes() = 4 259 968 bytes on each GPU the
 * library runs on, held until the process ends), whose device address llm_init looks up once per
 * device.  Calls no hipMalloc/hipFree.  Limits: n_heads <= 32 and head_dim <= 128, otherwise
 * LLM_ERR_INVALID.  All calls on one GPU share the array: calls that overlap on one GPU (two
 * streams, two threads) race; serialise them or use llm_attn_decode with separate workspaces. */
size_t llm_attn_decode_noalloc_max_bytes(void);
int llm_attn_decode_noalloc(const uint16_t *q_dev, const uint16_t *k_cache_dev, const uint16_t *v_cache_dev,
                            uint16_t *out_dev, int ctx_host, const int32_t *ctx_dev, int n_heads,
                            int n_kv_heads, int head_dim, int max_pos, llm_stream_t stream);
/* The decode step's form: takes the raw projection row qkv ([(Hq+2Hkv)*hd],
 * not rotated), applies RoPE for position pos = pos_host + (pos_dev ? *pos_dev : 0)
 * to Q and K, appends K and V to the caches at that position, and attends over
 * rows 0..pos.  One launch for rope_scaling + compute_attention
 * (src/inference/inference.cu:621-734).  qkv is left unmodified. */
int llm_attn_decode_rope(const uint16_t *qkv_dev, uint16_t *k_cache_dev, uint16_t *v_cache_dev,
                         uint16_t *out_dev, int pos_host, const int32_t *pos_dev, const float *table_dev,
                         int n_heads, int n_kv_heads, int head_dim, int max_pos, void *workspace_dev,
                         llm_stream_t stream);
/* llm_attn_decode_rope and the projection that consumes its result (compute_output + add_norm,
 * src/inference/inference.cu:600-618,366-390) in one launch, for positions below 512: the first
 * workgroups compute the attention into attn_out_dev ([Hq*hd]) exactly as llm_attn_decode_rope does;
 * all others fetch their rows of w ([N, Hq*hd]) while the attention runs, wait for its output, and
 * write out[n] = fp16(fp16(sum_k attn[k] * w[n,k]) + residual[n]) (residual may be NULL or alias out).
 * Same bits as llm_attn_decode_rope followed by llm_linear with T = 1 (a NaN result of the attention
 * may differ in its payload bits).
 * attn_out_dev must hold the "empty" pattern when the launch starts: llm_attn_oproj_buffer_init() once,
 * after that every launch refills attn_out_next_dev, the buffer that the next such launch in stream
 * order will pass as attn_out_dev (a ring of two or more buffers; never the same as attn_out_dev).
 * The wait of the projection workgroups is bounded: after spin_limit polling rounds (a negative value selects
 * the default, 2^18 rounds, a few tenths of a second) a workgroup gives up, reduces whatever the buffer holds
 * and adds one to *timeouts_dev (one int32, zeroed by the caller).  A non-zero count after the launch means
 * out_dev is invalid: fill attn_out_dev and attn_out_next_dev with llm_attn_oproj_buffer_init again, zero the
 * count and redo the operation (llm_attn_decode_rope + llm_linear give the same bits).  The wait relies on the
 * hardware handing out the workgroups of a launch in id order, so the attention workgroups run before any
 * projection workgroup waits for them; that also holds when launches of several streams share the device.
 * Something else that keeps every CU busy for the whole wait (another process's long kernel) shows up as a
 * counted timeout, never as a hang.
 * Launches that share these buffers must not overlap.  Limits: Hq*hd <= 4096, N <= 24 * (CUs - Hkv*4). */
int llm_attn_oproj_supported(int n_heads, int n_kv_heads, int head_dim, int N); /* 1 or 0, current device */
int llm_attn_oproj_buffer_init(uint16_t *buf_dev, int n, llm_stream_t stream);
int llm_attn_decode_rope_oproj(const uint16_t *qkv_dev, uint16_t *k_cache_dev, uint16_t *v_cache_dev,
                               uint16_t *attn_out_dev, uint16_t *attn_out_next_dev, int pos_host,
                               const int32_t *pos_dev, const float *table_dev, int n_heads, int n_kv_heads,
                               int head_dim, int max_pos, const uint16_t *w_dev, const uint16_t *residual_dev,
                               uint16_t *out_dev, int N, int32_t *timeouts_dev, int spin_limit, llm_stream_t stream);
/* The same operation as two launches: one workgroup per (KV head, 256-position span) leaves partial
 * softmax statistics and P.V, a second kernel (one workgroup per query head) merges them.  Correct at
 * any position; faster than the single launch beyond 512 cached positions (no in-kernel merge tail). */
int llm_attn_decode_rope_long(const uint16_t *qkv_dev, uint16_t *k_cache_dev, uint16_t *v_cache_dev,
                         uint16_t *out_dev, int pos_host, const int32_t *pos_dev, const float *table_dev,
                         int n_heads, int n_kv_heads, int head_dim, int max_pos, void *workspace_dev,
                         llm_stream_t stream);
/* llm_attn_decode_rope_long and the projection that consumes its result in two launches instead of three
 * (compute_output + add_norm, src/inference/inference.cu:600-618,366-390): the span kernel as above, then one
 * launch whose first Hq workgroups merge one query head each while all others fetch their rows of w and wait
 * for the merged vector.  Buffers, hand-over, timeouts_dev, spin_limit and the bits of the result as for
 * llm_attn_decode_rope_oproj (the two entry points may share one ring of buffers); any position below max_pos.
 * Limits: Hq*hd <= 4096, N <= 24 * (CUs - Hq). */
int llm_attn_long_oproj_supported(int n_heads, int n_kv_heads, int head_dim, int N); /* 1 or 0, current device */
int llm_attn_decode_rope_long_oproj(const uint16_t *qkv_dev, uint16_t *k_cache_dev, uint16_t *v_cache_dev,
                                    uint16_t *attn_out_dev, uint16_t *attn_out_next_dev, int pos_host,
                                    const int32_t *pos_dev, const float *table_dev, int n_heads, int n_kv_heads,
                                    int head_dim, int max_pos, void *workspace_dev, const uint16_t *w_dev,
                                    const uint16_t *residual_dev, uint16_t *out_dev, int N, int32_t *timeouts_dev,
                                    int spin_limit, llm_stream_t stream);
/* The same step for `batch` (<= 16) independent sequences in one launch: row z of qkv_dev belongs to the
 * sequence with caches k_caches[z], v_caches[z] (host arrays of device pointers) at position positions[z];
 * workspace_dev holds batch * llm_attn_decode_workspace_bytes().  No counterpart in the reference (it
 * serves one sequence). */
int llm_attn_decode_rope_batch(const uint16_t *qkv_dev, int ldq, uint16_t *const *k_caches, uint16_t *const *v_caches,
                               const int *positions, int batch, uint16_t *out_dev, int ldo, const float *table_dev,
                               int n_heads, int n_kv_heads, int head_dim, int max_pos, void *workspace_dev,
                               llm_stream_t stream);
/* The same with the caches and positions of the sequences read from device memory when the kernels run, so that
 * the launch can be captured once and replayed while the sequences advance: desc_dev points to an llm_batch_desc in
 * device memory (the caller rewrites it between replays, in stream order); cache_offset is added, in elements, to
 * every cache pointer (a layer's part of caches that hold all layers).  long_form: 0 when every position is below
 * 512 (one launch), 1 otherwise (span + merge launches, grids sized for any position below max_pos); positions are
 * clamped to what the chosen form serves. */
#define LLM_MAX_BATCH 16
typedef struct {
    uint16_t *k_cache[LLM_MAX_BATCH], *v_cache[LLM_MAX_BATCH];
    int32_t pos[LLM_MAX_BATCH];
} llm_batch_desc;
int llm_attn_decode_rope_batch_dev(const uint16_t *qkv_dev, int ldq, const llm_batch_desc *desc_dev, size_t cache_offset,
                                   int batch, int long_form, uint16_t *out_dev, int ldo, const float *table_dev, int n_heads,
                                   int n_kv_heads, int head_dim, int max_pos, void *workspace_dev, llm_stream_t stream);
/* Same attention for T query rows at positions pos0..pos0+T-1 (prompt pass),
 * streaming softmax on MFMA tiles; never materialises [H,T,T].
 * q: [T, ldq] with head h at columns h*hd; out: [T, ldo].  Cache rows beyond
 * the written positions must hold finite values (zero the caches once). */
int llm_attn_prefill(const uint16_t *q_dev, int ldq, const uint16_t *k_cache_dev,
                     const uint16_t *v_cache_dev, uint16_t *out_dev, int ldo, int T, int pos0,
                     int n_heads, int n_kv_heads, int head_dim, int max_pos, llm_stream_t stream);
/* llm_attn_prefill on queries that have not been rotated yet (rope_scaling of Q, src/inference/inference.cu:621-695,
 * folded into the attention): every wavefront rotates the query fragments it has just loaded by the angles of
 * their rows' positions (table_dev as for llm_rope) -- the arithmetic of llm_rope on the same elements, so the
 * result has the bits of llm_rope on Q followed by llm_attn_prefill, and Q is not read and written once more
 * (134 MB per layer of an 8192-token pass).  Served by the pipelined kernel only: head size 128, four query heads
 * per KV head, at least 64 rows (llm_attn_prefill_rope_q_supported says 1); other shapes return LLM_ERR_INVALID. */
int llm_attn_prefill_rope_q_supported(int T, int n_heads, int n_kv_heads, int head_dim, int max_pos);
int llm_attn_prefill_rope_q(const uint16_t *q_dev, int ldq, const uint16_t *k_cache_dev, const uint16_t *v_cache_dev,
                            uint16_t *out_dev, int ldo, int T, int pos0, const float *table_dev, int n_heads,
                            int n_kv_heads, int head_dim, int max_pos, llm_stream_t stream);

/* ---- sampler candidates --------------------------------------------------------------------------- */
/* Device half of sample_next_token (src/inference/inference.cu:1030-1161): what temperature_softmax's
 * loop and its qsort of the whole vocabulary (:1043-1072) decide for the first k entries, without moving
 * the logits to the host.  exp_table_dev: 65536 floats, entry b = expf(fp16(b) / temperature) as the HOST
 * computes it (the caller fills it, so that the values are the host library's, bit for bit), monotone in
 * the logit.  out_dev: llm_sample_candidates_bytes(vocab, k) bytes, 16-byte aligned; only its first
 * llm_sample_candidates_head_bytes(k) bytes are the result (the rest is the kernel's scratch space and
 * need not travel to the host).  The result is four 32-bit words --
 * the float32 denominator (the running sum of the table values in index order, rounded after every
 * addition as the host loop rounds), the number of pairs n (k, or 0), a flag, the number of groups
 * of 8 entries the sum had to add one by one -- and n pairs {float probability, int32 index}: the k entries that a
 * stable descending sort by probability puts first, unordered among the larger ones, by index among those
 * equal to the k-th.  flag != 0 (a NaN or infinite value, a zero or infinite denominator, a table that is
 * not monotone, a wait inside the kernel that gave up): nothing was selected and the caller falls back to
 * the host path.  1 <= k < vocab <= llm_sample_candidates_max_vocab().  Two launches (a clear of the scratch
 * space and the selection, whose workgroups wait for one another); calls that share out_dev must not overlap. */
size_t llm_sample_candidates_bytes(int vocab, int k);
size_t llm_sample_candidates_head_bytes(int k);
int llm_sample_candidates_max_vocab(void); /* larger vocabularies are rejected */
int llm_sample_candidates(const uint16_t *logits_dev, const float *exp_table_dev, int vocab, int k,
                          void *out_dev, llm_stream_t stream);

/* ---- LM head + argmax ------------------------------------------------------------ */
/* Replaces compute_lm_head (src/inference/inference.cu:1003-1028) with the
 * north-star's greedy selection instead of the host sampler: logits =
 * fp16(x . w^T) for one row, token = argmax over the fp16 logits, lowest index
 * on ties, NaN never selected.  logits_dev: [vocab] fp16 (kept, as the
 * reference keeps d_token_probdist).  token_dev: device int32 result.
 * tokens_dev/pos_dev (may be NULL): when given, the token is also stored at
 * tokens_dev[*pos_dev + 1] and *pos_dev is incremented, which lets a captured
 * decode step feed the next one. */
size_t llm_lmhead_workspace_bytes(int vocab);
int llm_lmhead_argmax(const uint16_t *x_dev, const uint16_t *w_dev, uint16_t *logits_dev,
                      int32_t *token_dev, int32_t *tokens_dev, int32_t *pos_dev, int vocab, int K,
                      void *workspace_dev, llm_stream_t stream);
/* Same with the final RMSNorm of x folded in (compute_layer_norm(model->norm)
 * + compute_lm_head, src/inference/inference.cu:188-190). */
int llm_norm_lmhead_argmax(const uint16_t *x_dev, const uint16_t *gain_dev, double eps, const uint16_t *w_dev,
                           uint16_t *logits_dev, int32_t *token_dev, int32_t *tokens_dev, int32_t *pos_dev,
                           int vocab, int K, void *workspace_dev, llm_stream_t stream);
/* argmax alone over fp16 values (same tie/NaN rule); workspace as for the LM head of n rows. */
int llm_argmax_f16(const uint16_t *logits_dev, int n, int32_t *token_dev, void *workspace_dev,
                   llm_stream_t stream);
/* The same for every row of a [rows, ld] matrix in two launches: tokens_dev[r] = argmax of row r.
 * workspace_dev: rows * min(1024, ceil(n / 256)) * 8 bytes. */
int llm_argmax_f16_rows(const uint16_t *logits_dev, int ld, int rows, int n, int32_t *tokens_dev,
                        void *workspace_dev, llm_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif
