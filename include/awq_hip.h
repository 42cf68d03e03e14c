/*
 * awq_hip.h -- C-ABI of libawq_hip.so: AWQ int4 group-128 weight-only batch-1
 * decode on one AMD gfx950 GPU.
 *
 * The reference (llama_cu_awq) has no FFI or plugin interface: its host code
 * launches kernels through a set of static launcher functions in one
 * translation unit.  This header cuts the seam there.  Each entry point below
 * names the reference launcher / call site it replaces (paths relative to the
 * reference checkout) and keeps that launcher's argument meaning.
 *
 * Conventions (the reference's):
 *   - every op is asynchronous on the context's single stream and never
 *     synchronises; only awq_stream_sync() and the blocking copies wait;
 *   - the caller owns every buffer; ops own nothing;
 *   - the sequence position is passed as a DEVICE pointer and read inside the
 *     kernels, so that a recorded launch sequence can be replayed;
 *   - fp16 tensors are passed as uint16_t* (IEEE binary16 bit patterns);
 *   - a packed matrix with reduction length K and N outputs is three arrays,
 *     one row per output n:
 *       weight[n*pwh + k/8]  uint32, element k in bits 4*(k%8), pwh = ceil(K/32)*4
 *       zeros [n*pzh + g/8]  uint32, group g = k/128 in bits 4*(g%8), pzh = ceil(ceil(K/128)/8)
 *       scales[n*sh  + g]    fp16,   sh = ceil(K/128)
 *     (common.h:26-30, llama2_q4.cu:106-129, weight_packer.cpp:114-124).
 *
 * Every function returns AWQ_OK (0) or a negative status; it never exits the
 * process.  Where the reference prints "Unsupported matmul size. Exiting" and
 * exits (K or N not a multiple of 8), this library returns AWQ_ERR_SHAPE and
 * launches nothing.  The library is thread-agnostic: a context may be used
 * from any one thread at a time; there is no thread-local state.
 */
#ifndef AWQ_HIP_H
#define AWQ_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AWQ_OK 0
#define AWQ_ERR_ARG (-1)    /* null pointer / bad argument */
#define AWQ_ERR_SHAPE (-2)  /* the reference's "Unsupported matmul size" guard, or a size a kernel cannot take */
#define AWQ_ERR_HIP (-3)    /* a HIP runtime call failed; see awq_last_error() */
#define AWQ_ERR_IO (-4)     /* model file missing / short / bad header */

typedef struct awq_ctx awq_ctx;                 /* device ordinal + stream + library workspace */
typedef struct awq_transformer awq_transformer; /* weights + run state of one model on one GPU */

/* Text of the most recent error recorded by any call in this process. */
const char* awq_last_error(void);

/* ---- device enumeration: get_and_print_gpu_info(), llama2_q4.cu:817-837 (cudaGetDeviceCount/Properties). */
int awq_device_count(int* count);
int awq_device_info(int device, char* name, size_t name_bytes, size_t* global_mem_bytes, int* compute_units);

/* ---- context: cudaSetDevice + cudaStreamCreate (llama2_q4.cu:685, 695) and the
 *      global `streams[rank]` (llama2_q4.cu:338-345). */
int awq_ctx_create(int device, awq_ctx** out);
/* Same, but enqueue on a stream the caller owns (a hipStream_t), e.g. torch's current stream. */
int awq_ctx_create_on_stream(int device, void* hip_stream, awq_ctx** out);
int awq_ctx_destroy(awq_ctx* ctx);
/* cudaStreamSynchronize (llama2_q4.cu:713, 737). */
int awq_stream_sync(awq_ctx* ctx);
/* Raw hipStream_t of the context. */
void* awq_ctx_stream(awq_ctx* ctx);

/* ---- memory: cudaMalloc / cudaFree / cudaMallocHost / cudaFreeHost / cudaMemcpyAsync /
 *      cudaMemset (llama2_q4.cu:62-74, 93-104, 114-136, 249, 703). */
int awq_malloc(awq_ctx* ctx, void** ptr, size_t bytes);
int awq_free(awq_ctx* ctx, void* ptr);
int awq_malloc_host(awq_ctx* ctx, void** ptr, size_t bytes); /* pinned, GPU-visible */
int awq_free_host(awq_ctx* ctx, void* ptr);
int awq_memcpy_h2d_async(awq_ctx* ctx, void* dst, const void* src, size_t bytes);
int awq_memcpy_h2d(awq_ctx* ctx, void* dst, const void* src, size_t bytes); /* blocking */
int awq_memcpy_d2h(awq_ctx* ctx, void* dst, const void* src, size_t bytes); /* blocking, ordered after the stream */
int awq_memcpy_d2d_async(awq_ctx* ctx, void* dst, const void* src, size_t bytes);
/* (hipMemsetAsync on the context's stream.  Not for a stream that is being captured into a graph: memset nodes have
 * given wrong results on replays after the first on this platform; inside a capture clear memory with a kernel, as the
 * library's own recorded sequences do.) */
int awq_memset_async(awq_ctx* ctx, void* dst, int value, size_t bytes);

/* ---- timing on the context's stream (cudaEvent pair, llama2_q4.cu:545-550, 592-600). */
int awq_event_create(awq_ctx* ctx, void** event);
int awq_event_destroy(awq_ctx* ctx, void* event);
int awq_event_record(awq_ctx* ctx, void* event);
int awq_event_elapsed_ms(awq_ctx* ctx, void* start, void* stop, float* ms); /* waits for `stop` */

typedef struct awq_qweight { /* QWeight, common.h:26-30 (device pointers) */
    const uint32_t* weight;
    const uint32_t* zeros;
    const uint16_t* scales;
} awq_qweight;

/* ---- ops: the launchers of llama2_q4.cu:347-427 and sampler.h:77-84 ---- */

/* copy_embedding_kernel launch, llama2_q4.cu:441: x[i] = table[tokens[*pos]*dim + i].
 * `tokens` may be pinned host memory (as in the reference) or device memory. */
int awq_embed(awq_ctx* ctx, uint16_t* x, const uint16_t* table, int dim, const int* tokens, const int* pos);

/* rmsnorm(), llama2_q4.cu:347-350: o = half(x * (rsqrt(mean(x^2)+1e-5) * weight)); o may alias x. */
int awq_rmsnorm(awq_ctx* ctx, uint16_t* o, const uint16_t* x, const uint16_t* weight, int size);

/* matmul(QWeight), llama2_q4.cu:367-376: out = half(W x), fp32 accumulation.
 * accum != 0: out = half(W x + out/gpu_count) (fused residual; gpu_count is 1 on one GPU).
 * loff != -1: the result row is written at out + loff + (*pos)*N (KV-cache row); pos may be NULL when loff == -1. */
int awq_matvec_int4(awq_ctx* ctx, uint16_t* out, const uint16_t* x, const awq_qweight* w, int K, int N,
                    int accum, int gpu_count, int loff, const int* pos);

/* qkv_matvec(), llama2_q4.cu:378-391: q = Wq x; key_cache[loff + pos*N ..] = Wk x; value_cache[...] = Wv x. */
int awq_qkv_matvec(awq_ctx* ctx, uint16_t* q, uint16_t* key_cache, uint16_t* value_cache, const uint16_t* x,
                   const awq_qweight* qw, const awq_qweight* kw, const awq_qweight* vw, int K, int N, int loff,
                   const int* pos);

/* ffn_matvec_silu(), llama2_q4.cu:393-404: out = half(silu(Wgate x) * (Wup x)), both products kept in fp32. */
int awq_ffn_matvec_silu(awq_ctx* ctx, uint16_t* out, const uint16_t* x, const awq_qweight* gate_w,
                        const awq_qweight* up_w, int K, int N);

/* rmsnorm() followed by ffn_matvec_silu() (llama2_q4.cu:496-498) as ONE launch, the form the fused schedule issues:
 * out = half(silu(Wgate xn) * (Wup xn)) with xn = half(x * (rsqrt(mean(x^2) + 1e-5) * norm_weight)) formed while x
 * is staged; xn never travels through memory.  Same rounding points as the two separate calls. */
int awq_rmsnorm_ffn_matvec_silu(awq_ctx* ctx, uint16_t* out, const uint16_t* x, const uint16_t* norm_weight,
                                const awq_qweight* gate_w, const awq_qweight* up_w, int K, int N);

/* RoPERotation(), llama2_q4.cu:406-408: rotate-half RoPE, pairs (i, i+head/2), in place on q (all heads)
 * and on the K row at k + loff + (*pos)*num_kv_heads*head_size (first num_kv_heads heads). */
int awq_rope(awq_ctx* ctx, uint16_t* q, uint16_t* k, int num_heads, int num_kv_heads, int head_size, const int* pos,
             int loff, float rope_theta);

/* MultiHeadAttention(), llama2_q4.cu:410-427.  key_cache / value_cache point at the layer's
 * (seq_len, num_heads*head_size/kv_mul) block.  att is a scratch of num_heads*max_seq_len halves; on return it
 * holds the fp16 scores with the reference's compact row stride (*pos + 1) (the reference overwrites them with
 * the probabilities, which nothing reads afterwards).  max_seq_len only sizes the launch (any value > *pos);
 * the live length is read from *pos on the device.  head_size must be 64, 128 or 256. */
int awq_attention(awq_ctx* ctx, uint16_t* output, const uint16_t* q, const uint16_t* key_cache,
                  const uint16_t* value_cache, uint16_t* att, int num_heads, int head_size, int kv_mul,
                  int max_seq_len, const int* pos);

/* The two halves of MultiHeadAttention + the O projection (llama2_q4.cu:410-427, 487) as the fused schedule runs them
 * at long contexts.  awq_attention_partial: scores as awq_attention, then the probability-weighted sum of the value
 * rows split over `*chunks` contiguous ranges of positions (chosen by the library, at most AWQ_ATTENTION_MAX_CHUNKS),
 * written as fp32 partial sums part[chunk][num_heads * head_size]; the probabilities are the reference's (softmax over
 * all positions, rounded to fp16).  awq_matvec_int4_parts: out = half(W x [+ out]) where x = half(part[0] + part[1] +
 * ... ) is formed while the input vector is staged (the reference's fp16 rounding of the attention output).
 * part: AWQ_ATTENTION_MAX_CHUNKS * num_heads * head_size floats.  K <= 8192. */
#define AWQ_ATTENTION_MAX_CHUNKS 4
int awq_attention_partial(awq_ctx* ctx, float* part, int* chunks, const uint16_t* q, const uint16_t* key_cache,
                          const uint16_t* value_cache, uint16_t* att, int num_heads, int head_size, int kv_mul, int max_seq_len,
                          const int* pos);
int awq_matvec_int4_parts(awq_ctx* ctx, uint16_t* out, const float* part, int parts, const awq_qweight* w, int K, int N,
                          int accum);

/* matmul(half), llama2_q4.cu:357-365 as used for the classifier (:530): out[r] = half(sum_j w[r*n+j] x[j]),
 * w row-major (d, n).  The batch/stride/alpha generality of the reference launcher is unused on its live path. */
int awq_matvec_f16(awq_ctx* ctx, uint16_t* out, const uint16_t* x, const uint16_t* w, int n, int d);

/* sample() greedy branch, sampler.h:77-84 (argmax_kernel, gpu_kernels.h:456-501): index of the largest logit
 * (lowest index on ties); p = *pos_dev + 1; if write_token, tokens[p] = argmax; *pos_host = *pos_dev = p.
 * tokens and pos_host are pinned host memory in the reference; any GPU-visible memory works. */
int awq_argmax_advance(awq_ctx* ctx, const uint16_t* logits, int size, int* tokens, volatile int* pos_host,
                       int* pos_dev, int write_token);

/* Dequantise a packed matrix to fp16, out[n*K + k] = half_rne((q - z) * scale): the arithmetic of
 * gpu_kernels.h:204-205 materialised (no launcher in the reference; used by the prefill path and by tests). */
int awq_dequant(awq_ctx* ctx, uint16_t* out, const awq_qweight* w, int K, int N);

/* ---- model level: build_transformer / run_transformer / free_transformer ---- */

typedef struct awq_config { /* Config, common.h:15-24 = the 32-byte file header */
    int dim, hidden_dim, n_layers, n_heads, n_kv_heads, vocab_size, seq_len;
    float rope_theta;
} awq_config;

typedef struct awq_run_state { /* RunState, common.h:62-78 (device pointers; shared_* are pinned host) */
    uint16_t *x, *xb, *hb, *q, *att, *logits, *key_cache, *value_cache;
    int* pos;                  /* device copy of the position */
    volatile int* shared_pos;  /* SharedData.pos  (common.h:57-60) */
    int* shared_tokens;        /* SharedData.tokens */
} awq_run_state;

typedef struct awq_layer_weights { /* PerLayerWeight, common.h:32-42 */
    const uint16_t* rms_att_weight;
    const uint16_t* rms_ffn_weight;
    awq_qweight wq_q, wq_k, wq_v, wq_o, wq_gate, wq_up, wq_down;
} awq_layer_weights;

/* build_transformer(), llama2_q4.cu:625-659, single GPU: read the header and every tensor of a weight_packer
 * .bin file (order llama2_q4.cu:220-246) to the GPU and allocate the run state (llama2_q4.cu:62-91). */
int awq_transformer_load_file(awq_ctx* ctx, const char* checkpoint_path, awq_transformer** out);
/* Same from a file image in host memory (synthetic models, tests). */
int awq_transformer_load_image(awq_ctx* ctx, const void* image, size_t bytes, awq_transformer** out);
/* free_transformer(), llama2_q4.cu:668-678. */
int awq_transformer_free(awq_transformer* t);
int awq_transformer_config(const awq_transformer* t, awq_config* out);
int awq_transformer_state(const awq_transformer* t, awq_run_state* out);
int awq_transformer_layer(const awq_transformer* t, int layer, awq_layer_weights* out);
/* token_embedding_table, wcls, rms_final_weight (common.h:44-54). */
int awq_transformer_globals(const awq_transformer* t, const uint16_t** embed, const uint16_t** wcls,
                            const uint16_t** rms_final);

/* Position bookkeeping of the model-level calls.  The reference sizes each pass from the pinned position after a
 * stream synchronisation (llama2_q4.cu:552, 713).  Here the transformer counts on the host the passes it has ISSUED
 * (reset: 0; set_pos: pos; forward / accept / sample: +1; prefill: +n_tokens), and that count sizes the attention
 * launch, selects the recorded sequence and bounds the position by seq_len.  Passes may therefore be issued back to
 * back without synchronising.  A caller that advances the device position of a transformer's run state by other means
 * (awq_argmax_advance or awq_sampler_sample on its buffers) must call awq_transformer_set_pos before the next
 * model-level call. */

/* Start a sequence (llama2_q4.cu:703-705): position 0, prompt copied into the shared token list. */
int awq_transformer_reset(awq_transformer* t, const int* prompt_tokens, int num_prompt_tokens);
/* Start at position `pos` with caller-provided KV-cache contents below it; `token` is consumed next. */
int awq_transformer_set_pos(awq_transformer* t, int pos, int token);

/* run_transformer(), llama2_q4.cu:541-601, with the greedy sampler: one token through the network
 * (run_llama_network, llama2_q4.cu:430-538, gpu_count 1) followed by argmax-and-advance.
 * gen_token: write the sampled token into the shared list (false while the prompt is being consumed).
 * use_graph != 0 replays a recorded launch sequence keyed by sequence-length bin (the USE_CUDA_GRAPHS path,
 * llama2_q4.cu:553-575); 0 launches eagerly.  mode selects the schedule: AWQ_SCHEDULE_REFERENCE issues the
 * reference's op sequence one launcher at a time; AWQ_SCHEDULE_FUSED merges RMSNorm into the consuming
 * matrix-vector kernels (same rounding points) and is the one to use.
 * AWQ_SCHEDULE_PERSISTENT is EXPERIMENTAL and about 2.3x SLOWER than FUSED (379 against 869 tokens/s at the 7B shape):
 * the whole token, sampler included, as ONE launch of a persistent kernel (one workgroup per CU, grid barriers between
 * the steps, weights prefetched across steps).  It produces the same tokens, ignores use_graph and returns
 * AWQ_ERR_SHAPE for models whose shape its work split cannot take (the other two schedules run every model).  Kept
 * as a record of what a grid barrier costs on this part (as much as a kernel boundary); not tuned further. */
#define AWQ_SCHEDULE_REFERENCE 0
#define AWQ_SCHEDULE_FUSED 1
#define AWQ_SCHEDULE_PERSISTENT 2
int awq_transformer_forward(awq_transformer* t, int gen_token, int use_graph, int mode);

/* Record and instantiate ahead of time the launch sequences that awq_transformer_forward and
 * awq_transformer_forward_logits (use_graph != 0) replay for positions below max_positions (per sequence-length bin,
 * llama2_q4.cu:553-575, one with the greedy sampler behind the network and one without; the reference records a bin
 * on its first visit, inside the decode loop).  Executes nothing; the run state is untouched.  mode: REFERENCE or
 * FUSED. */
int awq_transformer_capture(awq_transformer* t, int mode, int max_positions);

/* Per-launch GPU time of the fused schedule measured in place (the reference's DUMP_PER_TOKEN_TIMINGS switch,
 * llama2_q4.cu:32, 545-600, times whole tokens; this times each launch of one).  Runs the network of the CURRENT
 * position `passes` times eagerly (after one untimed run), every kernel launched with an event pair that the runtime
 * stamps with the kernel's own start and end, and returns, per launch kind, the mean kernel duration in microseconds
 * and the number of kernels averaged: AWQ_LAUNCH_EMBED, _QKV (RMSNorm + q/k/v products + RoPE), _ATTENTION (each of
 * its kernels on its own), _OPROJ, _GATE_UP (RMSNorm + gate/up products + SiLU), _DOWN, _CLASSIFIER (RMSNorm + fp16
 * product).  The gaps between dependent kernels are not part of these figures.  The position is not advanced: the pass rewrites the KV-cache
 * rows of the current position and the logits with the values a forward call would write.  Both arrays hold
 * AWQ_LAUNCH_KINDS entries. */
#define AWQ_LAUNCH_EMBED 0
#define AWQ_LAUNCH_QKV 1
#define AWQ_LAUNCH_ATTENTION 2
#define AWQ_LAUNCH_OPROJ 3
#define AWQ_LAUNCH_GATE_UP 4
#define AWQ_LAUNCH_DOWN 5
#define AWQ_LAUNCH_CLASSIFIER 6
#define AWQ_LAUNCH_KINDS 7
int awq_transformer_time_launches(awq_transformer* t, int passes, float* us_by_kind, int* launches_by_kind);

/* run_llama_network() alone (llama2_q4.cu:430-538): the token's logits without any sampler, for callers that sample
 * on their own (the non-greedy branch of sample(), sampler.h:85-115).  mode: REFERENCE or FUSED.  use_graph != 0
 * replays a recording of the network for the position's sequence-length bin, made on first use (what run_transformer()
 * does, llama2_q4.cu:552-590); awq_transformer_capture records those ahead of time as well. */
int awq_transformer_forward_logits(awq_transformer* t, int use_graph, int mode);
/* The tail of the reference's samplers (gpu_kernels.h:490-500, 582-591) for a token chosen by the caller:
 * p = pos + 1; if write_token, tokens[p] = token; pos = p (pinned-host and device copies). */
int awq_transformer_accept(awq_transformer* t, int token, int write_token);

/* ---- temperature / top-p sampling on the GPU (the non-greedy branch of sample(), sampler.h:85-115) ---- */

/* softmax_logits_kernel (gpu_kernels.h:507-557), in place: logits = half(logits / temperature), then
 * p = half(float(half(expf(l - max))) / sum) with the sum taken over the unrounded exponentials in fp32. */
int awq_softmax_logits(awq_ctx* ctx, uint16_t* logits, int size, float temperature);
/* The reference's sort + prefix sum + sample_top_p_kernel (sampler.h:94-115, gpu_kernels.h:562-592) in one launch:
 * sorted != 0 orders the fp16 probabilities descending (stable, as the reference's radix sort), sorted == 0 keeps
 * index order; the token is the first position whose inclusive prefix sum, rounded to fp16, is >= threshold
 * (position size-1 when none is).  The prefix sums are exact (fp16 values are multiples of 2^-24) and rounded once;
 * the reference's CUB scan adds in fp16 in an unspecified order.  Then p = pos + 1; tokens[p] = token; pos = p
 * (pinned-host and device copies).  probs is left untouched.  size <= 1048576 (above 65535 entries a slower,
 * plain form of the kernels runs). */
int awq_sample_top_p(awq_ctx* ctx, const uint16_t* probs, int size, float threshold, int sorted, int* tokens,
                     volatile int* pos_host, int* pos_dev);

/* Sampler (sampler.h:10-47): hyperparameters and the xorshift* state (sampler.h:65-74). */
typedef struct awq_sampler awq_sampler;
int awq_sampler_create(awq_ctx* ctx, int vocab_size, float temperature, float topp, unsigned long long rng_seed,
                       awq_sampler** out);
int awq_sampler_destroy(awq_sampler* sampler);
/* sample() (sampler.h:77-115): draws the coin (every call, as the reference does), then the greedy kernel when
 * temperature == 0 or gen_token == 0, else softmax + top-p (threshold coin * topp) or plain sampling (threshold coin
 * when topp <= 0 or >= 1).  logits are overwritten on the non-greedy branch. */
int awq_sampler_sample(awq_sampler* sampler, uint16_t* logits, int* tokens, volatile int* pos_host, int* pos_dev,
                       int gen_token);
/* The same on a transformer's own logits and token list (also keeps the device mirror of the token list current):
 * run_transformer() = awq_transformer_forward_logits + awq_transformer_sample (llama2_q4.cu:541-601). */
int awq_transformer_sample(awq_transformer* t, awq_sampler* sampler, int gen_token);

/* ---- multi-token prefill.  No counterpart in the reference, which consumes the prompt one token per forward pass
 * (llama2_q4.cu:716-735); the contract is the state that loop would leave. ---- */

/* out[m*ldo + n] = half(sum_k a[m*lda + k] * W[n][k]) for M rows at once on the fp16 matrix cores, the weights
 * dequantised to fp16 exactly as awq_dequant does; accum != 0 adds the previous contents of out (fused residual).
 * K multiple of 32, N multiple of 128, lda multiple of 8. */
int awq_gemm_int4(awq_ctx* ctx, uint16_t* out, int ldo, const uint16_t* a, int lda, int M, const awq_qweight* w, int K, int N,
                  int accum);

/* awq_gemm_int4 for callers that cannot allocate device memory (code recorded into a HIP graph, serving loops and
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, shapes and results as
 * awq_gemm_int4; the workspace of the split-K form (matrices with fewer than 256 output tiles of 128 x 128: fp32
 * partial tiles and arrival counters, up to 32 MiB) lives in a device array inside the library instead of being
 * allocated on first use, so this call makes no hipMalloc / hipFree and configures nothing (that happens per device
 * when a context is created).  All calls on one GPU share that array: calls that overlap on one GPU (two streams,
 * two contexts) race and must be serialised by the caller; calls on one stream are safe.  A shape whose split form
 * would need more tiles than the array holds is refused with AWQ_ERR_SHAPE. */
int awq_gemm_int4_static(awq_ctx* ctx, uint16_t* out, int ldo, const uint16_t* a, int lda, int M, const awq_qweight* w, int K,
                         int N, int accum);

/* Consume the n_tokens tokens at positions pos .. pos+n_tokens-1 of the shared token list in one batched pass:
 * afterwards the KV cache rows, the logits (of the last token), the token list and the position are those that
 * n_tokens calls of awq_transformer_forward (gen_token false for all but the last, `gen_token` for the last) would
 * leave.  Needs dim, kv_dim and hidden_dim to be multiples of 128.  The batched attention holds a score row per
 * query in LDS and takes contexts of up to 1920 positions with 128-wide heads (5048 / 4856 with 64 / 256); prompt
 * tokens beyond that are run one at a time through the matrix-vector path inside this call. */
int awq_transformer_prefill(awq_transformer* t, int n_tokens, int gen_token);

/* Diagnostics of the persistent schedule (no counterpart in the reference; its DUMP_PER_TOKEN_TIMINGS switch,
 * llama2_q4.cu:32, 545-600, times whole tokens only).  enable != 0 makes later persistent launches record, for
 * workgroup 0, five 100-MHz wall-clock stamps per step (start, input staged, products done, results published,
 * grid barrier passed); host_out (may be NULL) receives the stamps of the most recent launch first. */
int awq_transformer_trace(awq_transformer* t, int enable, long long* host_out, int max_entries, int* nphases);

#ifdef __cplusplus
}
#endif
#endif /* AWQ_HIP_H */
