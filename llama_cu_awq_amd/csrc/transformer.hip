// Model level of libawq_hip: load a weight_packer .bin image to the GPU,
// allocate the run state, and push one token through the network.
//
// Follows the reference's single-GPU flow: build_transformer /
// init_transformer (llama2_q4.cu:613-659), malloc_run_state (:62-91), the file
// order of checkpoint_init_weights (:220-246), run_llama_network (:430-538),
// run_transformer incl. its seq-len-binned graph replay (:541-601) and the
// greedy branch of sample() (sampler.h:77-84).
#include <stdlib.h>
#include <string.h>

#include <vector>

#include "common.hpp"
#include "token_kernel.hpp"

int awq_launch_matvec_int4(awq_ctx* ctx, uint16_t* out, const uint16_t* x, const awq_qweight* w, int K, int N, int accum,
                           int gpu_count, int loff, const int* pos, const uint16_t* norm_w, uint16_t* norm_out);
int awq_launch_qkv(awq_ctx* ctx, uint16_t* q, uint16_t* key_cache, uint16_t* value_cache, const uint16_t* x,
                   const awq_qweight* qw, const awq_qweight* kw, const awq_qweight* vw, int K, int N, int loff,
                   const int* pos, const uint16_t* norm_w, uint16_t* norm_out, const float2* rope, int head_size, int Nkv);
int awq_launch_ffn(awq_ctx* ctx, uint16_t* out, const uint16_t* x, const awq_qweight* gate_w, const awq_qweight* up_w, int K,
                   int N, const uint16_t* norm_w, uint16_t* norm_out);
int awq_launch_matvec_f16(awq_ctx* ctx, uint16_t* out, const uint16_t* x, const uint16_t* w, int n, int d,
                          const uint16_t* norm_w, uint16_t* norm_out);
int awq_attention_partial_chunks(const awq_ctx* ctx, int num_heads, int head_size);
int awq_launch_attention_partial(awq_ctx* ctx, float* part, int* chunks_out, const uint16_t* q, const uint16_t* key_cache,
                                 const uint16_t* value_cache, uint16_t* att, int num_heads, int head_size, int kv_mul,
                                 int max_seq_len, const int* pos);
int awq_launch_matvec_int4_parts(awq_ctx* ctx, uint16_t* out, const float* part, int parts, const awq_qweight* w, int K, int N,
                                 int accum);
int awq_launch_argmax(awq_ctx* ctx, const uint16_t* logits, int size, int* tokens, volatile int* pos_host, int* pos_dev,
                      int write_token, int* tokens_mirror);
// sampler.hip
int awq_sampler_run(awq_sampler* s, uint16_t* logits, int* tokens, volatile int* pos_host, int* pos_dev, int gen_token,
                    int* mirror);
// prefill.hip
int awq_launch_gemm_single(awq_ctx* ctx, uint16_t* out, long long ldo, const uint16_t* A, int lda, int M, const awq_qweight* w,
                           int K, int N, int accum, bool static_ws, bool a_perm);
int awq_launch_gemm_qkv(awq_ctx* ctx, uint16_t* q, uint16_t* key_cache, uint16_t* value_cache, long long kv_row0_off,
                        const uint16_t* A, int lda, int M, const awq_qweight* qw, const awq_qweight* kw, const awq_qweight* vw,
                        int K, int Nq, int Nkv, const float2* rope128, int pos0, bool a_perm);
int awq_launch_gemm_ffn(awq_ctx* ctx, uint16_t* hb, const uint16_t* A, int lda, int M, const awq_qweight* gate_w,
                        const awq_qweight* up_w, int K, int N, bool a_perm, bool out_perm);
int awq_launch_embed_rows(awq_ctx* ctx, uint16_t* x, const uint16_t* table, int dim, const int* tokens, int pos0, int M);
int awq_launch_rmsnorm_rows(awq_ctx* ctx, uint16_t* o, const uint16_t* x, const uint16_t* w, int size, int M, int perm);
int awq_launch_rope_rows(awq_ctx* ctx, uint16_t* q, uint16_t* kcache_layer, int nh, int nkv, int hs, int pos0, float theta, int M,
                         const float2* table);
int awq_launch_attn_prefill(awq_ctx* ctx, uint16_t* out, const uint16_t* q, const uint16_t* kc, const uint16_t* vc, int nh, int hs,
                            int kv_mul, int M, int pos0, int out_perm);
int awq_launch_set_pos(awq_ctx* ctx, int* pos_dev, volatile int* pos_host, int value);
int awq_prefill_attention_max_positions(int head_size);
int awq_launch_copy_row(awq_ctx* ctx, uint16_t* dst, const uint16_t* src, int n);

namespace {

// (cos, sin) of pos * theta^(-2i/head) for every position and pair index, with the arithmetic of the RoPE kernel
// (gpu_kernels.h:346-350), so that the fused QKV epilogue rotates with exactly the values that kernel would compute.
__global__ void rope_table_kernel(float2* table, int half, int head_size, float rope_theta) {
    const int pos = blockIdx.x;
    const int i = threadIdx.x;
    const int head_dim = (i * 2) % head_size;
    const float freq = 1.0f / powf(rope_theta, head_dim / (float)head_size);
    const float val = pos * freq;
    table[(size_t)pos * half + i] = make_float2(cosf(val), sinf(val));
}

// p = *pos + 1; if (write_token) tokens[p] = token; *pos_host = *pos_dev = p  (the tail of the reference's samplers,
// gpu_kernels.h:490-500 and :582-591, for a token chosen on the host)
__global__ void accept_kernel(int token, int* tokens_host, int* tokens_dev, volatile int* pos_host, int* pos_dev, int write_token) {
    const int p = *pos_dev + 1;
    if (write_token) {
        tokens_host[p] = token;
        tokens_dev[p] = token;
    }
    *pos_host = p;
    *pos_dev = p;
}

constexpr int kMaxSeqLen = 128 * 1024;  // SharedData.tokens capacity, common.h:13
constexpr int kMaxGraphs = 8;           // llama2_q4.cu:337

struct SharedData {  // common.h:57-60, pinned host memory
    volatile int pos;
    int tokens[kMaxSeqLen];
};

}  // namespace

struct awq_transformer {
    awq_ctx* ctx;
    awq_config cfg;
    uint8_t* blob;  // every tensor of the file, in file order, in one device allocation
    size_t blob_bytes;
    const uint16_t* embed;
    const uint16_t* wcls;
    const uint16_t* rms_final;
    std::vector<awq_layer_weights> layers;
    awq_run_state s;
    SharedData* shared;
    // Position the next pass will run at, counted on the host as passes are ISSUED (the pinned copy in `shared` is
    // only current after the stream has drained).  Sizes the attention launch, selects the graph bin and bounds
    // the sequence; kept by reset / set_pos / forward / accept / sample / prefill.
    int issued_pos;
    hipGraphExec_t graphs[2][kMaxGraphs];      // network + greedy sampler, per schedule and sequence-length bin
    bool captured[2][kMaxGraphs];
    hipGraphExec_t graphs_net[2][kMaxGraphs];  // the network alone (what the reference itself records, llama2_q4.cu:560-575)
    bool captured_net[2][kMaxGraphs];
    int* tokens_dev;  // device mirror of SharedData.tokens (the persistent kernel reads its input token here)
    float2* rope_table;  // [seq_len][head_size/2] (cos, sin)
    float* attn_part;    // [kAttnMaxChunks][dim] fp32 partial attention outputs of the position-split form
    // plan of the persistent per-token kernel
    bool tk_ok;
    char tk_why[160];  // why the persistent kernel cannot run this model, when !tk_ok
    tk::Args tk_args;
    size_t tk_lds_bytes;
    tk::Phase* tk_phases;
    tk::Sync* tk_sync;
    int* tk_err_host;
    long long* tk_trace;  // device buffer of per-phase time stamps when tracing is on, else null
    // prefill workspace: activations of up to pf_rows tokens
    int pf_rows;
    uint16_t *pf_x, *pf_xb, *pf_q, *pf_att, *pf_hb;
};

namespace {

size_t qweight_bytes(int K, int N) {
    return (size_t)packed_weight_height(K) * N * 4 + (size_t)packed_zeros_height(K) * N * 4 + (size_t)scales_height(K) * N * 2;
}

size_t model_payload_bytes(const awq_config& c) {
    const int kv_dim = (c.dim * c.n_kv_heads) / c.n_heads;
    size_t b = 2 * (size_t)c.vocab_size * c.dim * 2 + (size_t)c.dim * 2;
    size_t layer = 2 * qweight_bytes(c.dim, c.dim) + 2 * qweight_bytes(c.dim, kv_dim) + 2 * qweight_bytes(c.dim, c.hidden_dim) +
                   qweight_bytes(c.hidden_dim, c.dim) + 2 * (size_t)c.dim * 2;
    return b + layer * c.n_layers;
}

int check_config(const awq_config& c) {
    AWQ_REQUIRE(c.dim > 0 && c.hidden_dim > 0 && c.n_layers > 0 && c.n_heads > 0 && c.n_kv_heads > 0 && c.vocab_size > 0 &&
                    c.seq_len > 0,
                AWQ_ERR_IO, "bad header: non-positive field");
    AWQ_REQUIRE(c.seq_len <= kMaxSeqLen - 1, AWQ_ERR_IO, "bad header: seq_len above 128K");
    AWQ_REQUIRE(c.n_heads % c.n_kv_heads == 0 && c.dim % c.n_heads == 0, AWQ_ERR_IO, "bad header: head counts do not divide");
    const int kv_dim = (c.dim * c.n_kv_heads) / c.n_heads;
    // The packer writes ceil(K/8) dwords per row and the loader expects ceil(K/32)*4: only K % 32 == 0 files
    // load correctly in the reference (weight_packer.cpp:156 vs llama2_q4.cu:111).
    AWQ_REQUIRE(c.dim % 32 == 0 && c.hidden_dim % 32 == 0, AWQ_ERR_SHAPE, "dim and hidden_dim must be multiples of 32");
    AWQ_REQUIRE((kv_dim & 7) == 0 && (c.vocab_size & 7) == 0, AWQ_ERR_SHAPE, "kv_dim and vocab_size must be multiples of 8");
    AWQ_REQUIRE(c.dim <= kMaxStagedK && c.hidden_dim <= kMaxStagedKInt4, AWQ_ERR_SHAPE, "dim/hidden_dim above the staged maximum");
    const int head = c.dim / c.n_heads;
    AWQ_REQUIRE(head == 64 || head == 128 || head == 256, AWQ_ERR_SHAPE, "head size must be 64, 128 or 256");
    AWQ_REQUIRE(c.n_heads <= kAttnMaxHeads, AWQ_ERR_SHAPE, "too many heads");
    return AWQ_OK;
}

const uint8_t* take_qweight(awq_qweight* w, const uint8_t* p, int K, int N) {
    w->weight = reinterpret_cast<const uint32_t*>(p);
    p += (size_t)packed_weight_height(K) * N * 4;
    w->zeros = reinterpret_cast<const uint32_t*>(p);
    p += (size_t)packed_zeros_height(K) * N * 4;
    w->scales = reinterpret_cast<const uint16_t*>(p);
    p += (size_t)scales_height(K) * N * 2;
    return p;
}

void map_tensors(awq_transformer* t) {
    const awq_config& c = t->cfg;
    const int kv_dim = (c.dim * c.n_kv_heads) / c.n_heads;
    const uint8_t* p = t->blob;
    t->embed = reinterpret_cast<const uint16_t*>(p);
    p += (size_t)c.vocab_size * c.dim * 2;
    t->wcls = reinterpret_cast<const uint16_t*>(p);
    p += (size_t)c.vocab_size * c.dim * 2;
    t->rms_final = reinterpret_cast<const uint16_t*>(p);
    p += (size_t)c.dim * 2;
    t->layers.resize(c.n_layers);
    for (int l = 0; l < c.n_layers; l++) {
        awq_layer_weights& L = t->layers[l];
        p = take_qweight(&L.wq_q, p, c.dim, c.dim);
        p = take_qweight(&L.wq_k, p, c.dim, kv_dim);
        p = take_qweight(&L.wq_v, p, c.dim, kv_dim);
        p = take_qweight(&L.wq_o, p, c.dim, c.dim);
        p = take_qweight(&L.wq_up, p, c.dim, c.hidden_dim);  // file order: up before gate (llama2_q4.cu:236-237)
        p = take_qweight(&L.wq_gate, p, c.dim, c.hidden_dim);
        p = take_qweight(&L.wq_down, p, c.hidden_dim, c.dim);
        L.rms_att_weight = reinterpret_cast<const uint16_t*>(p);
        p += (size_t)c.dim * 2;
        L.rms_ffn_weight = reinterpret_cast<const uint16_t*>(p);
        p += (size_t)c.dim * 2;
    }
}

int alloc_state(awq_transformer* t) {
    const awq_config& c = t->cfg;
    const size_t kv_dim = ((size_t)c.dim * c.n_kv_heads) / c.n_heads;
    awq_run_state& s = t->s;
    AWQ_HIP_TRY(hipMalloc((void**)&s.x, (size_t)c.dim * 2));
    AWQ_HIP_TRY(hipMalloc((void**)&s.xb, (size_t)c.dim * 2));
    AWQ_HIP_TRY(hipMalloc((void**)&s.hb, (size_t)c.hidden_dim * 2));
    AWQ_HIP_TRY(hipMalloc((void**)&s.q, (size_t)c.dim * 2));
    AWQ_HIP_TRY(hipMalloc((void**)&s.att, (size_t)c.n_heads * c.seq_len * 2));
    AWQ_HIP_TRY(hipMalloc((void**)&s.logits, (size_t)c.vocab_size * 2));
    const size_t kv_bytes = (size_t)c.n_layers * c.seq_len * kv_dim * 2;
    AWQ_HIP_TRY(hipMalloc((void**)&s.key_cache, kv_bytes));
    AWQ_HIP_TRY(hipMalloc((void**)&s.value_cache, kv_bytes));
    AWQ_HIP_TRY(hipMalloc((void**)&s.pos, sizeof(int)));
    AWQ_HIP_TRY(hipMemset(s.key_cache, 0, kv_bytes));
    AWQ_HIP_TRY(hipMemset(s.value_cache, 0, kv_bytes));
    AWQ_HIP_TRY(hipMemset(s.pos, 0, sizeof(int)));
    AWQ_HIP_TRY(hipHostMalloc((void**)&t->shared, sizeof(SharedData), hipHostMallocDefault));
    memset((void*)t->shared, 0, sizeof(SharedData));
    AWQ_HIP_TRY(hipMalloc((void**)&t->tokens_dev, (size_t)(c.seq_len + 8) * sizeof(int)));
    AWQ_HIP_TRY(hipMemset(t->tokens_dev, 0, (size_t)(c.seq_len + 8) * sizeof(int)));
    const int head = c.dim / c.n_heads;
    AWQ_HIP_TRY(hipMalloc((void**)&t->rope_table, (size_t)c.seq_len * (head / 2) * sizeof(float2)));
    AWQ_HIP_TRY(hipMalloc((void**)&t->attn_part, (size_t)kAttnMaxChunks * c.dim * sizeof(float)));
    hipLaunchKernelGGL(rope_table_kernel, dim3(c.seq_len), dim3(head / 2), 0, t->ctx->stream, t->rope_table, head / 2, head, c.rope_theta);
    if (int r = awq_check_launch("rope_table")) return r;
    s.shared_pos = &t->shared->pos;
    s.shared_tokens = t->shared->tokens;
    return AWQ_OK;
}

void release(awq_transformer* t) {
    if (!t) return;
    for (int m = 0; m < 2; m++)
        for (int i = 0; i < kMaxGraphs; i++)
        {
            if (t->captured[m][i]) (void)hipGraphExecDestroy(t->graphs[m][i]);
            if (t->captured_net[m][i]) (void)hipGraphExecDestroy(t->graphs_net[m][i]);
        }
    (void)hipFree(t->blob);
    (void)hipFree(t->s.x);
    (void)hipFree(t->s.xb);
    (void)hipFree(t->s.hb);
    (void)hipFree(t->s.q);
    (void)hipFree(t->s.att);
    (void)hipFree(t->s.logits);
    (void)hipFree(t->s.key_cache);
    (void)hipFree(t->s.value_cache);
    (void)hipFree(t->s.pos);
    if (t->shared) (void)hipHostFree(t->shared);
    (void)hipFree(t->tokens_dev);
    (void)hipFree(t->rope_table);
    (void)hipFree(t->attn_part);
    (void)hipFree(t->tk_phases);
    (void)hipFree(t->tk_sync);
    (void)hipFree(t->tk_trace);
    (void)hipFree(t->pf_x);
    (void)hipFree(t->pf_xb);
    (void)hipFree(t->pf_q);
    (void)hipFree(t->pf_att);
    (void)hipFree(t->pf_hb);
    if (t->tk_err_host) (void)hipHostFree(t->tk_err_host);
    delete t;
}

awq_transformer* new_transformer(awq_ctx* ctx) {
    awq_transformer* t = new awq_transformer();
    t->ctx = ctx;
    t->blob = nullptr;
    t->blob_bytes = 0;
    t->shared = nullptr;
    t->tokens_dev = nullptr;
    t->rope_table = nullptr;
    t->attn_part = nullptr;
    t->tk_ok = false;
    t->tk_why[0] = 0;
    t->tk_phases = nullptr;
    t->tk_sync = nullptr;
    t->tk_err_host = nullptr;
    t->tk_trace = nullptr;
    t->pf_rows = 0;
    t->pf_x = t->pf_xb = t->pf_q = t->pf_att = t->pf_hb = nullptr;
    t->issued_pos = 0;
    memset(&t->s, 0, sizeof(t->s));
    memset(t->captured, 0, sizeof(t->captured));
    return t;
}


// Plan the persistent per-token kernel for this model: choose the grid, lay out LDS, build the phase list.
// Leaves t->tk_ok false (with the reason in t->tk_why) when the model's shape does not fit the kernel's
// work split; the multi-kernel schedules still run such a model.
#define TK_REQUIRE(cond, why)                                   \
    do {                                                        \
        if (!(cond)) {                                          \
            snprintf(t->tk_why, sizeof(t->tk_why), "%s", why);  \
            return AWQ_OK;                                      \
        }                                                       \
    } while (0)

int plan_token_kernel(awq_transformer* t) {
    const awq_config& c = t->cfg;
    const int dim = c.dim, hidden = c.hidden_dim;
    const int hs = dim / c.n_heads;
    const int kv_dim = (dim * c.n_kv_heads) / c.n_heads;
    hipDeviceProp_t prop;
    AWQ_HIP_TRY(hipGetDeviceProperties(&prop, t->ctx->device));
    int G = prop.multiProcessorCount < tk::kMaxWorkgroups ? prop.multiProcessorCount : tk::kMaxWorkgroups;
    // every workgroup takes the same number of rows of every matrix
    while (G >= 32 && !((dim / 2) % G == 0 && (kv_dim / 2) % G == 0 && hidden % G == 0)) G--;
    TK_REQUIRE(G >= 32, "no grid size divides dim/2, kv_dim/2 and hidden_dim");
    TK_REQUIRE(c.n_heads <= G, "more heads than workgroups");
    TK_REQUIRE(hs == 64 || hs == 128 || hs == 256, "head size must be 64, 128 or 256");
    TK_REQUIRE((scales_height(dim) & 1) == 0 && (scales_height(hidden) & 1) == 0, "odd number of groups per row");
    TK_REQUIRE(dim <= 20480 && hidden <= 20480, "reduction length above 20480");
    const int ppw = dim / 2 / G, kpw = kv_dim / 2 / G, vpw = kv_dim / G;
    TK_REQUIRE(ppw + kpw + vpw <= 256 && 2 * hidden / G <= 512 && dim / G <= 256, "too many rows per workgroup");
    const int cls_rows = div_up(c.vocab_size, G);
    TK_REQUIRE(cls_rows <= 256, "too many classifier rows per workgroup");

    auto passes = [](int K) { return div_up(div_up(K, 32), 64); };
    const int cls_passes = div_up(dim / 8, 64);
    int max_units = 1024;  // attention borrows 4 x 256 floats of this area
    auto upd = [&](int v) { if (v > max_units) max_units = v; };
    upd((2 * ppw + 2 * kpw + vpw) * passes(dim));
    upd((dim / G) * passes(dim));
    upd((2 * hidden / G) * passes(dim));
    upd((dim / G) * passes(hidden));
    upd(cls_rows * cls_passes);
    const int cmax = div_up(dim > hidden ? dim : hidden, 32);
    int xs_bytes = cmax * 64;
    if (dim * 2 > xs_bytes) xs_bytes = dim * 2;
    if (c.seq_len * 4 > xs_bytes) xs_bytes = c.seq_len * 4;
    xs_bytes = (xs_bytes + 255) & ~255;
    const int ab_bytes = (cmax * 8 + 255) & ~255;
    const int part_bytes = (max_units * 4 + 255) & ~255;
    const int misc_bytes = 1024;
    const int lds_total = 160 * 1024;
    const int fixed = xs_bytes + ab_bytes + part_bytes + misc_bytes;
    int depth = (lds_total - fixed) / (tk::NSW * tk::UNIT_BYTES);
    if (depth > 16) depth = 16;
    TK_REQUIRE(depth >= 4, "not enough LDS left for the weight ring");

    std::vector<tk::Phase> ph;
    auto int4_phase = [&](int kind, int in_sel, int K, int N, int rows_per_wg, const uint16_t* norm_w, long long kvoff) {
        tk::Phase p;
        memset(&p, 0, sizeof(p));
        p.kind = kind;
        p.in_sel = in_sel;
        p.K = K;
        p.C = div_up(K, 32);
        p.P = div_up(p.C, 64);
        p.N = N;
        p.rows_per_wg = rows_per_wg;
        p.pzh = packed_zeros_height(K);
        p.sh = scales_height(K);
        p.kv_layer_off = kvoff;
        p.norm_w = norm_w;
        return p;
    };
    auto set_mat = [](tk::Phase& p, int i, const awq_qweight& w) {
        p.w[i] = w.weight;
        p.z[i] = w.zeros;
        p.s[i] = w.scales;
    };
    for (int l = 0; l < c.n_layers; l++) {
        const awq_layer_weights& L = t->layers[l];
        const long long kvoff = (long long)l * c.seq_len * kv_dim;
        tk::Phase q = int4_phase(tk::KIND_QKV, l == 0 ? tk::IN_EMBED : tk::IN_X, dim, dim, 2 * ppw + 2 * kpw + vpw, L.rms_att_weight, kvoff);
        q.ppw = ppw;
        q.kpw = kpw;
        q.vpw = vpw;
        set_mat(q, 0, L.wq_q);
        set_mat(q, 1, L.wq_k);
        set_mat(q, 2, L.wq_v);
        ph.push_back(q);
        tk::Phase at;
        memset(&at, 0, sizeof(at));
        at.kind = tk::KIND_ATTN;
        at.kv_layer_off = kvoff;
        ph.push_back(at);
        tk::Phase o = int4_phase(tk::KIND_OPROJ, tk::IN_XB, dim, dim, dim / G, nullptr, kvoff);
        set_mat(o, 0, L.wq_o);
        ph.push_back(o);
        tk::Phase f = int4_phase(tk::KIND_FFN, tk::IN_X, dim, hidden, 2 * hidden / G, L.rms_ffn_weight, kvoff);
        set_mat(f, 0, L.wq_gate);
        set_mat(f, 1, L.wq_up);
        ph.push_back(f);
        tk::Phase d = int4_phase(tk::KIND_DOWN, tk::IN_HB, hidden, dim, dim / G, nullptr, kvoff);
        set_mat(d, 0, L.wq_down);
        ph.push_back(d);
    }
    tk::Phase cl;
    memset(&cl, 0, sizeof(cl));
    cl.kind = tk::KIND_CLS;
    cl.in_sel = tk::IN_X;
    cl.K = dim;
    cl.C = 0;
    cl.P = cls_passes;
    cl.N = c.vocab_size;
    cl.rows_per_wg = cls_rows;
    cl.w[0] = reinterpret_cast<const uint32_t*>(t->wcls);
    cl.norm_w = t->rms_final;
    ph.push_back(cl);
    tk::Phase am;
    memset(&am, 0, sizeof(am));
    am.kind = tk::KIND_ARGMAX;
    ph.push_back(am);

    AWQ_HIP_TRY(hipMalloc((void**)&t->tk_phases, ph.size() * sizeof(tk::Phase)));
    AWQ_HIP_TRY(hipMemcpy(t->tk_phases, ph.data(), ph.size() * sizeof(tk::Phase), hipMemcpyHostToDevice));
    AWQ_HIP_TRY(hipMalloc((void**)&t->tk_sync, sizeof(tk::Sync)));
    AWQ_HIP_TRY(hipMemset(t->tk_sync, 0, sizeof(tk::Sync)));
    AWQ_HIP_TRY(hipHostMalloc((void**)&t->tk_err_host, sizeof(int), hipHostMallocDefault));
    *t->tk_err_host = 0;

    tk::Args& a = t->tk_args;
    memset(&a, 0, sizeof(a));
    a.phases = t->tk_phases;
    a.nphases = (int)ph.size();
    a.G = G;
    a.depth = depth;
    a.dim = dim;
    a.hidden = hidden;
    a.n_heads = c.n_heads;
    a.n_kv_heads = c.n_kv_heads;
    a.head_size = hs;
    a.half_head_shift = hs == 64 ? 5 : (hs == 128 ? 6 : 7);
    a.vocab = c.vocab_size;
    a.rope_theta = c.rope_theta;
    a.x = t->s.x;
    a.xb = t->s.xb;
    a.hb = t->s.hb;
    a.q = t->s.q;
    a.logits = t->s.logits;
    a.key_cache = t->s.key_cache;
    a.value_cache = t->s.value_cache;
    a.embed = t->embed;
    a.pos_dev = t->s.pos;
    a.pos_host = t->s.shared_pos;
    a.tokens_host = t->s.shared_tokens;
    a.tokens_dev = t->tokens_dev;
    a.sync = t->tk_sync;
    a.err_host = t->tk_err_host;
    a.spin_limit = 50000000LL;  // 0.5 s of the 100 MHz wall clock
    a.lds_xs = 0;
    a.lds_ab = xs_bytes;
    a.lds_part = a.lds_ab + ab_bytes;
    a.lds_misc = a.lds_part + part_bytes;
    a.lds_ring = a.lds_misc + misc_bytes;
    t->tk_lds_bytes = (size_t)a.lds_ring + (size_t)tk::NSW * depth * tk::UNIT_BYTES;
    t->tk_ok = true;
    return AWQ_OK;
}

// One token, the reference's launcher sequence with gpu_count = 1.
int network_reference(awq_transformer* t, int seq_len_bin) {
    awq_ctx* ctx = t->ctx;
    const awq_config& p = t->cfg;
    awq_run_state& s = t->s;
    const int dim = p.dim, hidden_dim = p.hidden_dim;
    const int head_size = dim / p.n_heads;
    const int kv_dim = (p.dim * p.n_kv_heads) / p.n_heads;
    const int kv_mul = p.n_heads / p.n_kv_heads;
    int* pPos = s.pos;
    int r;
    if ((r = awq_embed(ctx, s.x, t->embed, dim, s.shared_tokens, pPos))) return r;
    for (int l = 0; l < p.n_layers; l++) {
        const awq_layer_weights& L = t->layers[l];
        if ((r = awq_rmsnorm(ctx, s.xb, s.x, L.rms_att_weight, dim))) return r;
        const int loff = l * p.seq_len * kv_dim;
        if (dim == kv_dim) {
            if ((r = awq_qkv_matvec(ctx, s.q, s.key_cache, s.value_cache, s.xb, &L.wq_q, &L.wq_k, &L.wq_v, dim, dim, loff, pPos)))
                return r;
        } else {
            if ((r = awq_matvec_int4(ctx, s.q, s.xb, &L.wq_q, dim, dim, 0, 1, -1, nullptr))) return r;
            if ((r = awq_matvec_int4(ctx, s.key_cache, s.xb, &L.wq_k, dim, kv_dim, 0, 1, loff, pPos))) return r;
            if ((r = awq_matvec_int4(ctx, s.value_cache, s.xb, &L.wq_v, dim, kv_dim, 0, 1, loff, pPos))) return r;
        }
        if ((r = awq_rope(ctx, s.q, s.key_cache, p.n_heads, p.n_kv_heads, head_size, pPos, loff, p.rope_theta))) return r;
        if ((r = awq_attention(ctx, s.xb, s.q, s.key_cache + loff, s.value_cache + loff, s.att, p.n_heads, head_size, kv_mul,
                               seq_len_bin, pPos)))
            return r;
        if ((r = awq_matvec_int4(ctx, s.x, s.xb, &L.wq_o, dim, dim, 1, 1, -1, nullptr))) return r;
        if ((r = awq_rmsnorm(ctx, s.xb, s.x, L.rms_ffn_weight, dim))) return r;
        if ((r = awq_ffn_matvec_silu(ctx, s.hb, s.xb, &L.wq_gate, &L.wq_up, dim, hidden_dim))) return r;
        if ((r = awq_matvec_int4(ctx, s.x, s.hb, &L.wq_down, hidden_dim, dim, 1, 1, -1, nullptr))) return r;
    }
    if ((r = awq_rmsnorm(ctx, s.x, s.x, t->rms_final, dim))) return r;
    return awq_matvec_f16(ctx, s.logits, s.x, t->wcls, dim, p.vocab_size);
}

// Launch kinds of the fused schedule, as awq_transformer_time_launches reports them.
enum { LK_EMBED = 0, LK_QKV = 1, LK_ATTENTION = 2, LK_OPROJ = 3, LK_GATE_UP = 4, LK_DOWN = 5, LK_CLASSIFIER = 6, LK_COUNT = 7 };

// Names the schedule step whose launches follow, for a timing run (see awq_launch in common.hpp); otherwise free.
struct LaunchProbe {
    LaunchProbe(awq_transformer* t, int kind) {
        if (t->ctx->probe) t->ctx->probe->kind = kind;
    }
};

// Same arithmetic with RMSNorm folded into the staging of the consuming
// matrix-vector kernels (the normalised vector never travels through memory).
int network_fused(awq_transformer* t, int seq_len_bin) {
    awq_ctx* ctx = t->ctx;
    const awq_config& p = t->cfg;
    awq_run_state& s = t->s;
    const int dim = p.dim, hidden_dim = p.hidden_dim;
    const int head_size = dim / p.n_heads;
    const int kv_dim = (p.dim * p.n_kv_heads) / p.n_heads;
    const int kv_mul = p.n_heads / p.n_kv_heads;
    int* pPos = s.pos;
    int r;
    // the token list's device mirror (kept by reset / set_pos / accept / the sampler) saves a read over PCIe
    {
        LaunchProbe probe(t, LK_EMBED);
        if ((r = awq_embed(ctx, s.x, t->embed, dim, t->tokens_dev, pPos))) return r;
    }
    for (int l = 0; l < p.n_layers; l++) {
        const awq_layer_weights& L = t->layers[l];
        const int loff = l * p.seq_len * kv_dim;
        {
            LaunchProbe probe(t, LK_QKV);
            // one launch for the three matrices, RMSNorm in its staging and the rotation in its epilogue; with grouped
            // queries (the reference then makes three launches and the rotation, llama2_q4.cu:457-464) the K and V
            // matrices have kv_dim rows and the workgroups past them leave at once
            if ((r = awq_launch_qkv(ctx, s.q, s.key_cache, s.value_cache, s.x, &L.wq_q, &L.wq_k, &L.wq_v, dim, dim, loff, pPos,
                                    L.rms_att_weight, nullptr, t->rope_table, head_size, kv_dim)))
                return r;
        }
        // Long launch sizes: P.V split over positions too, its fp32 partial sums added up (and rounded to fp16, the
        // reference's rounding point) while the O projection stages its input; xb is not written on this path.
        // (Measured: +1.4 % tokens/s at 1.6 K positions of the 13B shape; just above 256 positions the split costs
        // 2 us per layer more than it saves, so it starts at the 1024 bin.)
        // ... and it needs ranges long enough to pay for the partial sums: with four ranges (32 heads) the 1024 bin is
        // faster unsplit (7B shape at positions 600-664: 743 against 719 tokens/s), with three (40 heads) it is not
        // (13B shape: 448 against 453); from the 2048 bin on the split wins at both
        const bool split = seq_len_bin >= kAttnSplitMinSeq && dim <= 8192 &&
                           seq_len_bin / awq_attention_partial_chunks(ctx, p.n_heads, head_size) >= kAttnSplitMinRange;
        int parts = 0;
        {
            LaunchProbe probe(t, LK_ATTENTION);
            if (split)
                r = awq_launch_attention_partial(ctx, t->attn_part, &parts, s.q, s.key_cache + loff, s.value_cache + loff, s.att,
                                                 p.n_heads, head_size, kv_mul, seq_len_bin, pPos);
            else
                r = awq_attention(ctx, s.xb, s.q, s.key_cache + loff, s.value_cache + loff, s.att, p.n_heads, head_size, kv_mul,
                                  seq_len_bin, pPos);
            if (r) return r;
        }
        {
            LaunchProbe probe(t, LK_OPROJ);
            if (split)
                r = awq_launch_matvec_int4_parts(ctx, s.x, t->attn_part, parts, &L.wq_o, dim, dim, 1);
            else
                r = awq_launch_matvec_int4(ctx, s.x, s.xb, &L.wq_o, dim, dim, 1, 1, -1, nullptr, nullptr, nullptr);
            if (r) return r;
        }
        {
            LaunchProbe probe(t, LK_GATE_UP);
            if ((r = awq_launch_ffn(ctx, s.hb, s.x, &L.wq_gate, &L.wq_up, dim, hidden_dim, L.rms_ffn_weight, nullptr))) return r;
        }
        {
            LaunchProbe probe(t, LK_DOWN);
            if ((r = awq_launch_matvec_int4(ctx, s.x, s.hb, &L.wq_down, hidden_dim, dim, 1, 1, -1, nullptr, nullptr, nullptr)))
                return r;
        }
    }
    LaunchProbe probe(t, LK_CLASSIFIER);
    return awq_launch_matvec_f16(ctx, s.logits, s.x, t->wcls, dim, p.vocab_size, t->rms_final, nullptr);
}

int network(awq_transformer* t, int seq_len_bin, int mode) {
    return mode == AWQ_SCHEDULE_FUSED ? network_fused(t, seq_len_bin) : network_reference(t, seq_len_bin);
}

// llama2_q4.cu:553-558: sequence-length bins 128, 256, ..., the last one being the model's seq_len.  Returns the
// index of the bin that a pass over seq_len positions replays and stores the bin's launch size.
int graph_bin(const awq_config& cfg, int seq_len, int* seq_len_bin_out) {
    int graph_index;
    int seq_len_bin = 128;
    for (graph_index = 0; graph_index < kMaxGraphs - 1; seq_len_bin *= 2, graph_index++)
        if (seq_len <= seq_len_bin) break;
    if (seq_len > seq_len_bin || graph_index == kMaxGraphs - 1 || seq_len_bin > cfg.seq_len) seq_len_bin = cfg.seq_len;
    *seq_len_bin_out = seq_len_bin;
    return graph_index;
}

// Record and instantiate the launch sequence of one bin (the network, with or without the greedy sampler behind it),
// unless that is done already.  Recording executes nothing and leaves the run state untouched.
int ensure_captured(awq_transformer* t, int mode, int graph_index, int seq_len_bin, bool with_sampler = true) {
    bool* done = with_sampler ? &t->captured[mode][graph_index] : &t->captured_net[mode][graph_index];
    hipGraphExec_t* exec = with_sampler ? &t->graphs[mode][graph_index] : &t->graphs_net[mode][graph_index];
    if (*done) return AWQ_OK;
    awq_ctx* ctx = t->ctx;
    hipGraph_t graph = nullptr;
    AWQ_HIP_TRY(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed));
    int r = network(t, seq_len_bin, mode);
    if (r == AWQ_OK && with_sampler)
        r = awq_launch_argmax(ctx, t->s.logits, t->cfg.vocab_size, t->s.shared_tokens, t->s.shared_pos, t->s.pos, 1, t->tokens_dev);
    hipError_t e = hipStreamEndCapture(ctx->stream, &graph);
    if (r) {
        if (graph) (void)hipGraphDestroy(graph);
        return r;
    }
    if (e != hipSuccess) {
        awq_set_error("hipStreamEndCapture failed: %s", hipGetErrorString(e));
        return AWQ_ERR_HIP;
    }
    e = hipGraphInstantiate(exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) {
        awq_set_error("hipGraphInstantiate failed: %s", hipGetErrorString(e));
        return AWQ_ERR_HIP;
    }
    // (the first replay of an instantiated graph otherwise pays for its upload to the device, a few milliseconds)
    (void)hipGraphUpload(*exec, ctx->stream);
    *done = true;
    return AWQ_OK;
}

}  // namespace

extern "C" {

int awq_transformer_load_image(awq_ctx* ctx, const void* image, size_t bytes, awq_transformer** out) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_REQUIRE(image && out, AWQ_ERR_ARG, "null pointer");
    AWQ_REQUIRE(bytes >= sizeof(awq_config), AWQ_ERR_IO, "Invalid header size");
    awq_transformer* t = new_transformer(ctx);
    memcpy(&t->cfg, image, sizeof(awq_config));
    int r = check_config(t->cfg);
    if (r) {
        release(t);
        return r;
    }
    t->blob_bytes = model_payload_bytes(t->cfg);
    if (bytes < sizeof(awq_config) + t->blob_bytes) {
        awq_set_error("error reading weights: image holds %zu bytes, config needs %zu", bytes, sizeof(awq_config) + t->blob_bytes);
        release(t);
        return AWQ_ERR_IO;
    }
    hipError_t e = hipMalloc((void**)&t->blob, t->blob_bytes);
    if (e == hipSuccess)
        e = hipMemcpy(t->blob, (const uint8_t*)image + sizeof(awq_config), t->blob_bytes, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        awq_set_error("weight upload failed: %s", hipGetErrorString(e));
        release(t);
        return AWQ_ERR_HIP;
    }
    map_tensors(t);
    r = alloc_state(t);
    if (r == AWQ_OK) r = plan_token_kernel(t);
    if (r) {
        release(t);
        return r;
    }
    if (hipError_t e = hipDeviceSynchronize(); e != hipSuccess) {
        awq_set_error("model set-up failed: %s", hipGetErrorString(e));
        release(t);
        return AWQ_ERR_HIP;
    }
    *out = t;
    return AWQ_OK;
}

int awq_transformer_load_file(awq_ctx* ctx, const char* checkpoint_path, awq_transformer** out) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_REQUIRE(checkpoint_path && out, AWQ_ERR_ARG, "null pointer");
    FILE* f = fopen(checkpoint_path, "rb");
    if (!f) {
        awq_set_error("Couldn't open file %s", checkpoint_path);
        return AWQ_ERR_IO;
    }
    awq_transformer* t = new_transformer(ctx);
    if (fread(&t->cfg, sizeof(awq_config), 1, f) != 1) {
        awq_set_error("Invalid header size");
        fclose(f);
        release(t);
        return AWQ_ERR_IO;
    }
    int r = check_config(t->cfg);
    if (r) {
        fclose(f);
        release(t);
        return r;
    }
    t->blob_bytes = model_payload_bytes(t->cfg);
    hipError_t e = hipMalloc((void**)&t->blob, t->blob_bytes);
    if (e != hipSuccess) {
        awq_set_error("weight allocation failed: %s", hipGetErrorString(e));
        fclose(f);
        release(t);
        return AWQ_ERR_HIP;
    }
    // Stream the file through two pinned staging buffers so that disk reads overlap the uploads.
    const size_t chunk = (size_t)64 << 20;
    uint8_t* stage[2] = {nullptr, nullptr};
    hipEvent_t done[2];
    bool ok = true;
    for (int i = 0; i < 2 && ok; i++) {
        ok = hipHostMalloc((void**)&stage[i], chunk, hipHostMallocDefault) == hipSuccess && hipEventCreate(&done[i]) == hipSuccess;
    }
    size_t off = 0;
    int which = 0;
    bool used[2] = {false, false};
    while (ok && off < t->blob_bytes) {
        const size_t n = (t->blob_bytes - off < chunk) ? t->blob_bytes - off : chunk;
        if (used[which]) ok = hipEventSynchronize(done[which]) == hipSuccess;
        if (ok && fread(stage[which], 1, n, f) != n) {
            awq_set_error("error reading weights");
            r = AWQ_ERR_IO;
            ok = false;
            break;
        }
        if (ok) ok = hipMemcpyAsync(t->blob + off, stage[which], n, hipMemcpyHostToDevice, ctx->stream) == hipSuccess;
        if (ok) ok = hipEventRecord(done[which], ctx->stream) == hipSuccess;
        used[which] = true;
        which ^= 1;
        off += n;
    }
    (void)hipStreamSynchronize(ctx->stream);
    for (int i = 0; i < 2; i++) {
        if (stage[i]) {
            (void)hipHostFree(stage[i]);
            (void)hipEventDestroy(done[i]);
        }
    }
    fclose(f);
    if (!ok) {
        if (r == AWQ_OK) {
            awq_set_error("weight upload failed");
            r = AWQ_ERR_HIP;
        }
        release(t);
        return r;
    }
    map_tensors(t);
    r = alloc_state(t);
    if (r == AWQ_OK) r = plan_token_kernel(t);
    if (r) {
        release(t);
        return r;
    }
    if (hipError_t e = hipDeviceSynchronize(); e != hipSuccess) {
        awq_set_error("model set-up failed: %s", hipGetErrorString(e));
        release(t);
        return AWQ_ERR_HIP;
    }
    *out = t;
    return AWQ_OK;
}

int awq_transformer_free(awq_transformer* t) {
    AWQ_REQUIRE(t, AWQ_ERR_ARG, "null transformer");
    if (int r = awq_bind(t->ctx)) return r;
    (void)hipStreamSynchronize(t->ctx->stream);
    release(t);
    return AWQ_OK;
}

int awq_transformer_config(const awq_transformer* t, awq_config* out) {
    AWQ_REQUIRE(t && out, AWQ_ERR_ARG, "null pointer");
    *out = t->cfg;
    return AWQ_OK;
}

int awq_transformer_state(const awq_transformer* t, awq_run_state* out) {
    AWQ_REQUIRE(t && out, AWQ_ERR_ARG, "null pointer");
    *out = t->s;
    return AWQ_OK;
}

int awq_transformer_layer(const awq_transformer* t, int layer, awq_layer_weights* out) {
    AWQ_REQUIRE(t && out, AWQ_ERR_ARG, "null pointer");
    AWQ_REQUIRE(layer >= 0 && layer < t->cfg.n_layers, AWQ_ERR_ARG, "no such layer");
    *out = t->layers[layer];
    return AWQ_OK;
}

int awq_transformer_globals(const awq_transformer* t, const uint16_t** embed, const uint16_t** wcls, const uint16_t** rms_final) {
    AWQ_REQUIRE(t, AWQ_ERR_ARG, "null pointer");
    if (embed) *embed = t->embed;
    if (wcls) *wcls = t->wcls;
    if (rms_final) *rms_final = t->rms_final;
    return AWQ_OK;
}

int awq_transformer_reset(awq_transformer* t, const int* prompt_tokens, int num_prompt_tokens) {
    AWQ_REQUIRE(t && prompt_tokens, AWQ_ERR_ARG, "null pointer");
    AWQ_REQUIRE(num_prompt_tokens >= 1 && num_prompt_tokens <= t->cfg.seq_len, AWQ_ERR_ARG, "prompt length out of range");
    if (int r = awq_bind(t->ctx)) return r;
    AWQ_HIP_TRY(hipStreamSynchronize(t->ctx->stream));
    AWQ_HIP_TRY(hipMemset(t->s.pos, 0, sizeof(int)));
    t->shared->pos = 0;
    memcpy(t->shared->tokens, prompt_tokens, sizeof(int) * (size_t)num_prompt_tokens);
    AWQ_HIP_TRY(hipMemcpy(t->tokens_dev, prompt_tokens, sizeof(int) * (size_t)num_prompt_tokens, hipMemcpyHostToDevice));
    t->issued_pos = 0;
    if (t->tk_err_host) *t->tk_err_host = 0;
    // After a barrier time-out the flag and release words hold epochs of a launch that never finished; start the
    // persistent kernel's synchronisation state from scratch (all zero = the state of a fresh model).
    if (t->tk_sync) AWQ_HIP_TRY(hipMemset(t->tk_sync, 0, sizeof(tk::Sync)));
    return AWQ_OK;
}

int awq_transformer_set_pos(awq_transformer* t, int pos, int token) {
    AWQ_REQUIRE(t, AWQ_ERR_ARG, "null pointer");
    AWQ_REQUIRE(pos >= 0 && pos < t->cfg.seq_len, AWQ_ERR_ARG, "pos out of range");
    if (int r = awq_bind(t->ctx)) return r;
    AWQ_HIP_TRY(hipStreamSynchronize(t->ctx->stream));
    AWQ_HIP_TRY(hipMemcpy(t->s.pos, &pos, sizeof(int), hipMemcpyHostToDevice));
    t->shared->pos = pos;
    t->shared->tokens[pos] = token;
    AWQ_HIP_TRY(hipMemcpy(t->tokens_dev + pos, &token, sizeof(int), hipMemcpyHostToDevice));
    t->issued_pos = pos;
    return AWQ_OK;
}


int awq_transformer_prefill(awq_transformer* t, int n_tokens, int gen_token) {
    AWQ_REQUIRE(t, AWQ_ERR_ARG, "null transformer");
    awq_ctx* ctx = t->ctx;
    if (int r = awq_bind(ctx)) return r;
    const awq_config& p = t->cfg;
    const int dim = p.dim, hidden = p.hidden_dim;
    const int hs = dim / p.n_heads;
    const int kv_dim = (dim * p.n_kv_heads) / p.n_heads;
    const int kv_mul = p.n_heads / p.n_kv_heads;
    AWQ_REQUIRE(n_tokens >= 1, AWQ_ERR_ARG, "n_tokens must be >= 1");
    if ((dim & 127) || (kv_dim & 127) || (hidden & 127)) {
        awq_set_error("prefill needs dim, kv_dim and hidden_dim to be multiples of 128 (got %d, %d, %d)", dim, kv_dim, hidden);
        return AWQ_ERR_SHAPE;
    }
    const int pos_start = t->issued_pos;
    AWQ_REQUIRE(pos_start + n_tokens <= p.seq_len, AWQ_ERR_ARG, "prompt runs past seq_len");
    // The batched attention keeps a score row per query in LDS, which bounds the context it can take; tokens past
    // that bound go through the matrix-vector path one at a time (the definition of what prefill must leave behind).
    const int max_ctx = awq_prefill_attention_max_positions(hs);
    int n_batched = max_ctx - pos_start;
    if (n_batched > n_tokens) n_batched = n_tokens;
    if (n_batched < 0) n_batched = 0;
    const int chunk = 512;
    if (n_batched > 0 && t->pf_rows == 0) {
        const int rows = p.seq_len < chunk ? p.seq_len : chunk;
        uint16_t** bufs[5] = {&t->pf_x, &t->pf_xb, &t->pf_q, &t->pf_att, &t->pf_hb};
        const size_t widths[5] = {(size_t)dim, (size_t)dim, (size_t)dim, (size_t)dim, (size_t)hidden};
        for (int i = 0; i < 5; i++) {
            hipError_t e = hipMalloc((void**)bufs[i], (size_t)rows * widths[i] * 2);
            if (e != hipSuccess) {  // leave no half-allocated workspace behind
                for (int j = 0; j < i; j++) {
                    (void)hipFree(*bufs[j]);
                    *bufs[j] = nullptr;
                }
                *bufs[i] = nullptr;
                awq_set_error("prefill workspace allocation failed: %s", hipGetErrorString(e));
                return AWQ_ERR_HIP;
            }
        }
        t->pf_rows = rows;
    }
    int r;
    for (int done = 0; done < n_batched; done += t->pf_rows) {
        const int M = (n_batched - done < t->pf_rows) ? n_batched - done : t->pf_rows;
        const int pos0 = pos_start + done;
        if ((r = awq_launch_embed_rows(ctx, t->pf_x, t->embed, dim, t->tokens_dev, pos0, M))) return r;
        // The activations that feed a GEMM (xb, att, hb) are written with every 8 values in the order the packed weights
        // dequantise in, so that the GEMMs multiply them without reordering either operand; x, q and the KV cache
        // keep the natural order.
        for (int l = 0; l < p.n_layers; l++) {
            const awq_layer_weights& L = t->layers[l];
            const long long loff = (long long)l * p.seq_len * kv_dim;
            if ((r = awq_launch_rmsnorm_rows(ctx, t->pf_xb, t->pf_x, L.rms_att_weight, dim, M, 1))) return r;
            // 128-wide heads: the QKV GEMM rotates q and k in its epilogue; other head sizes run the RoPE kernel
            const float2* rope128 = (hs == 128) ? t->rope_table : nullptr;
            if ((r = awq_launch_gemm_qkv(ctx, t->pf_q, t->s.key_cache, t->s.value_cache, loff + (long long)pos0 * kv_dim, t->pf_xb,
                                         dim, M, &L.wq_q, &L.wq_k, &L.wq_v, dim, dim, kv_dim, rope128, pos0, true)))
                return r;
            if (!rope128 && (r = awq_launch_rope_rows(ctx, t->pf_q, t->s.key_cache + loff, p.n_heads, p.n_kv_heads, hs, pos0,
                                                      p.rope_theta, M, t->rope_table)))
                return r;
            if ((r = awq_launch_attn_prefill(ctx, t->pf_att, t->pf_q, t->s.key_cache + loff, t->s.value_cache + loff, p.n_heads, hs,
                                             kv_mul, M, pos0, 1)))
                return r;
            if ((r = awq_launch_gemm_single(ctx, t->pf_x, dim, t->pf_att, dim, M, &L.wq_o, dim, dim, 1, false, true))) return r;
            if ((r = awq_launch_rmsnorm_rows(ctx, t->pf_xb, t->pf_x, L.rms_ffn_weight, dim, M, 1))) return r;
            if ((r = awq_launch_gemm_ffn(ctx, t->pf_hb, t->pf_xb, dim, M, &L.wq_gate, &L.wq_up, dim, hidden, true, true))) return r;
            if ((r = awq_launch_gemm_single(ctx, t->pf_x, dim, t->pf_hb, hidden, M, &L.wq_down, hidden, dim, 1, false, true))) return r;
        }
        if (done + M == n_tokens) {
            // last token: final norm, classifier and the greedy sampler exactly as the decode path does them
            if ((r = awq_launch_copy_row(ctx, t->s.x, t->pf_x + (size_t)(M - 1) * dim, dim))) return r;
            if ((r = awq_launch_set_pos(ctx, t->s.pos, t->s.shared_pos, pos_start + n_tokens - 1))) return r;
            if ((r = awq_launch_matvec_f16(ctx, t->s.logits, t->s.x, t->wcls, dim, p.vocab_size, t->rms_final, nullptr))) return r;
            if ((r = awq_launch_argmax(ctx, t->s.logits, p.vocab_size, t->s.shared_tokens, t->s.shared_pos, t->s.pos, gen_token,
                                       t->tokens_dev)))
                return r;
        }
    }
    if (n_batched < n_tokens) {
        if (n_batched > 0 && (r = awq_launch_set_pos(ctx, t->s.pos, t->s.shared_pos, pos_start + n_batched))) return r;
        for (int i = n_batched; i < n_tokens; i++) {
            if ((r = network(t, pos_start + i + 1, AWQ_SCHEDULE_FUSED))) return r;
            if ((r = awq_launch_argmax(ctx, t->s.logits, p.vocab_size, t->s.shared_tokens, t->s.shared_pos, t->s.pos,
                                       i == n_tokens - 1 ? gen_token : 0, t->tokens_dev)))
                return r;
        }
    }
    t->issued_pos = pos_start + n_tokens;
    return AWQ_OK;
}

int awq_transformer_trace(awq_transformer* t, int enable, long long* host_out, int max_entries, int* nphases) {
    AWQ_REQUIRE(t, AWQ_ERR_ARG, "null transformer");
    if (int r = awq_bind(t->ctx)) return r;
    AWQ_REQUIRE(t->tk_ok, AWQ_ERR_SHAPE, "persistent schedule unavailable for this model");
    const size_t n = (size_t)t->tk_args.nphases * 5;
    if (nphases) *nphases = t->tk_args.nphases;
    if (host_out && t->tk_trace) {
        AWQ_HIP_TRY(hipStreamSynchronize(t->ctx->stream));
        const size_t m = n < (size_t)max_entries ? n : (size_t)max_entries;
        AWQ_HIP_TRY(hipMemcpy(host_out, t->tk_trace, m * sizeof(long long), hipMemcpyDeviceToHost));
    }
    if (enable && !t->tk_trace) {
        AWQ_HIP_TRY(hipMalloc((void**)&t->tk_trace, n * sizeof(long long)));
        AWQ_HIP_TRY(hipMemset(t->tk_trace, 0, n * sizeof(long long)));
    } else if (!enable && t->tk_trace) {
        AWQ_HIP_TRY(hipStreamSynchronize(t->ctx->stream));
        AWQ_HIP_TRY(hipFree(t->tk_trace));
        t->tk_trace = nullptr;
    }
    return AWQ_OK;
}

int awq_transformer_forward_logits(awq_transformer* t, int use_graph, int mode) {
    AWQ_REQUIRE(t, AWQ_ERR_ARG, "null transformer");
    AWQ_REQUIRE(mode == AWQ_SCHEDULE_REFERENCE || mode == AWQ_SCHEDULE_FUSED, AWQ_ERR_ARG,
                "forward_logits runs the reference or the fused schedule");
    awq_ctx* ctx = t->ctx;
    if (int r = awq_bind(ctx)) return r;
    const int seq_len = t->issued_pos + 1;
    AWQ_REQUIRE(seq_len <= t->cfg.seq_len, AWQ_ERR_ARG, "position beyond seq_len");
    if (use_graph) {  // run_transformer(), llama2_q4.cu:552-590: the network of the position's bin, recorded on first use
        int seq_len_bin;
        const int graph_index = graph_bin(t->cfg, seq_len, &seq_len_bin);
        if (int r = ensure_captured(t, mode, graph_index, seq_len_bin, false)) return r;
        AWQ_HIP_TRY(hipGraphLaunch(t->graphs_net[mode][graph_index], ctx->stream));
        return AWQ_OK;
    }
    return network(t, seq_len, mode);
}

int awq_transformer_accept(awq_transformer* t, int token, int write_token) {
    AWQ_REQUIRE(t, AWQ_ERR_ARG, "null transformer");
    AWQ_REQUIRE(token >= 0 && token < t->cfg.vocab_size, AWQ_ERR_ARG, "token out of range");
    awq_ctx* ctx = t->ctx;
    if (int r = awq_bind(ctx)) return r;
    AWQ_REQUIRE(t->issued_pos + 1 <= t->cfg.seq_len, AWQ_ERR_ARG, "position beyond seq_len");
    hipLaunchKernelGGL(accept_kernel, dim3(1), dim3(1), 0, ctx->stream, token, t->s.shared_tokens, t->tokens_dev, t->s.shared_pos,
                       t->s.pos, write_token);
    if (int r = awq_check_launch("accept")) return r;
    t->issued_pos++;
    return AWQ_OK;
}

int awq_transformer_sample(awq_transformer* t, awq_sampler* sampler, int gen_token) {
    AWQ_REQUIRE(t && sampler, AWQ_ERR_ARG, "null transformer or sampler");
    awq_ctx* ctx = t->ctx;
    if (int r = awq_bind(ctx)) return r;
    AWQ_REQUIRE(t->issued_pos + 1 <= t->cfg.seq_len, AWQ_ERR_ARG, "position beyond seq_len");
    if (int r = awq_sampler_run(sampler, t->s.logits, t->s.shared_tokens, t->s.shared_pos, t->s.pos, gen_token, t->tokens_dev)) return r;
    t->issued_pos++;
    return AWQ_OK;
}

int awq_transformer_time_launches(awq_transformer* t, int passes, float* us_by_kind, int* launches_by_kind) {
    AWQ_REQUIRE(t && us_by_kind && launches_by_kind, AWQ_ERR_ARG, "null pointer");
    AWQ_REQUIRE(passes >= 1 && passes <= 64, AWQ_ERR_ARG, "passes must be 1 .. 64");
    awq_ctx* ctx = t->ctx;
    if (int r = awq_bind(ctx)) return r;
    const int seq_len = t->issued_pos + 1;
    AWQ_REQUIRE(seq_len <= t->cfg.seq_len, AWQ_ERR_ARG, "position beyond seq_len");
    awq_launch_probe probe;
    int r = network_fused(t, seq_len);  // untimed: code objects loaded, caches in their steady state
    ctx->probe = &probe;
    for (int i = 0; i < passes && r == AWQ_OK; i++) r = network_fused(t, seq_len);
    ctx->probe = nullptr;
    hipError_t e = hipStreamSynchronize(ctx->stream);
    double sum[LK_COUNT] = {0};
    int count[LK_COUNT] = {0};
    if (r == AWQ_OK && e == hipSuccess) {
        for (size_t i = 0; i < probe.kinds.size(); i++) {
            float ms = 0.0f;
            if (hipEventElapsedTime(&ms, probe.events[2 * i], probe.events[2 * i + 1]) == hipSuccess) {
                sum[probe.kinds[i]] += ms * 1e3;
                count[probe.kinds[i]]++;
            }
        }
    }
    for (hipEvent_t ev : probe.events) (void)hipEventDestroy(ev);
    if (r) return r;
    if (e != hipSuccess) {
        awq_set_error("timing run failed: %s", hipGetErrorString(e));
        return AWQ_ERR_HIP;
    }
    for (int k = 0; k < LK_COUNT; k++) {
        us_by_kind[k] = count[k] ? (float)(sum[k] / count[k]) : 0.0f;
        launches_by_kind[k] = count[k];
    }
    return AWQ_OK;
}

int awq_transformer_capture(awq_transformer* t, int mode, int max_positions) {
    AWQ_REQUIRE(t, AWQ_ERR_ARG, "null transformer");
    AWQ_REQUIRE(mode == AWQ_SCHEDULE_REFERENCE || mode == AWQ_SCHEDULE_FUSED, AWQ_ERR_ARG,
                "only the reference and the fused schedule replay recorded sequences");
    AWQ_REQUIRE(max_positions >= 1 && max_positions <= t->cfg.seq_len, AWQ_ERR_ARG, "max_positions out of range");
    if (int r = awq_bind(t->ctx)) return r;
    int last = -1;
    for (int seq_len = 1; seq_len <= max_positions; seq_len++) {
        int seq_len_bin;
        const int graph_index = graph_bin(t->cfg, seq_len, &seq_len_bin);
        if (graph_index != last) {
            if (int r = ensure_captured(t, mode, graph_index, seq_len_bin, true)) return r;
            if (int r = ensure_captured(t, mode, graph_index, seq_len_bin, false)) return r;
            last = graph_index;
        }
        seq_len = (seq_len_bin < max_positions ? seq_len_bin : max_positions);  // jump to the end of this bin
    }
    return AWQ_OK;
}

int awq_transformer_forward(awq_transformer* t, int gen_token, int use_graph, int mode) {
    AWQ_REQUIRE(t, AWQ_ERR_ARG, "null transformer");
    AWQ_REQUIRE(mode == AWQ_SCHEDULE_REFERENCE || mode == AWQ_SCHEDULE_FUSED || mode == AWQ_SCHEDULE_PERSISTENT, AWQ_ERR_ARG,
                "unknown schedule");
    awq_ctx* ctx = t->ctx;
    if (int r = awq_bind(ctx)) return r;
    if (mode == AWQ_SCHEDULE_PERSISTENT) {
        if (!t->tk_ok) {
            awq_set_error("persistent schedule unavailable for this model: %s", t->tk_why);
            return AWQ_ERR_SHAPE;
        }
        if (*t->tk_err_host) {
            awq_set_error("persistent kernel: a grid barrier timed out (workgroups not co-resident?)");
            return AWQ_ERR_HIP;
        }
        AWQ_REQUIRE(t->issued_pos + 1 <= t->cfg.seq_len, AWQ_ERR_ARG, "position beyond seq_len");
        tk::Args a = t->tk_args;
        a.write_token = gen_token;
        a.trace = t->tk_trace;
        if (int r = tk_launch(ctx->stream, a, t->tk_lds_bytes)) return r;
        t->issued_pos++;
        return AWQ_OK;
    }
    // llama2_q4.cu:552 sizes the attention launch from the pinned position after a synchronisation; the count of
    // issued passes is the same number and does not need one
    const int seq_len = t->issued_pos + 1;
    AWQ_REQUIRE(seq_len <= t->cfg.seq_len, AWQ_ERR_ARG, "position beyond seq_len");
    int r;
    if (use_graph) {
        int seq_len_bin;
        const int graph_index = graph_bin(t->cfg, seq_len, &seq_len_bin);
        if ((r = ensure_captured(t, mode, graph_index, seq_len_bin))) return r;
        // The recorded sampler always writes its token; while the prompt is being consumed the next prompt
        // token must survive, so those steps replay the recording of the network alone and launch the sampler
        // (which then only advances the position) behind it.
        if (gen_token) {
            AWQ_HIP_TRY(hipGraphLaunch(t->graphs[mode][graph_index], ctx->stream));
            t->issued_pos++;
            return AWQ_OK;
        }
        if ((r = ensure_captured(t, mode, graph_index, seq_len_bin, false))) return r;
        AWQ_HIP_TRY(hipGraphLaunch(t->graphs_net[mode][graph_index], ctx->stream));
        r = AWQ_OK;
    } else {
        r = network(t, seq_len, mode);
    }
    if (r) return r;
    if ((r = awq_launch_argmax(ctx, t->s.logits, t->cfg.vocab_size, t->s.shared_tokens, t->s.shared_pos, t->s.pos, gen_token,
                               t->tokens_dev)))
        return r;
    t->issued_pos++;
    return AWQ_OK;
}

}  // extern "C"
