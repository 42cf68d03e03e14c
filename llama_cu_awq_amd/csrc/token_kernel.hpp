// Descriptors shared by the persistent per-token kernel and the host code that plans its launch.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tk {

constexpr int NSW = 8;                // streaming waves per workgroup
constexpr int NHW = 4;                // helper waves per workgroup
constexpr int NT = (NSW + NHW) * 64;  // threads per workgroup
constexpr int UNIT_BYTES = 1024 + 64; // ring slot: 64 lanes x 16 B of weights + scales/zeros of the pass
constexpr int kMaxWorkgroups = 256;

enum Kind { KIND_QKV = 0, KIND_ATTN = 1, KIND_OPROJ = 2, KIND_FFN = 3, KIND_DOWN = 4, KIND_CLS = 5, KIND_ARGMAX = 6 };
enum Input { IN_X = 0, IN_XB = 1, IN_HB = 2, IN_EMBED = 3 };

struct Phase {
    int kind;
    int in_sel;           // which vector is staged as the input of the phase
    int K;                // reduction length
    int C;                // 32-element chunks per row (int4 phases)
    int P;                // 64-lane passes per row
    int N;                // rows per matrix
    int rows_per_wg;      // stacked rows owned by one workgroup
    int ppw, kpw, vpw;    // QKV: Q pairs, K pairs and V rows per workgroup
    int pzh, sh;          // zero-point dwords / scale halves per row
    long long kv_layer_off;  // element offset of the layer's block in the KV cache
    const uint32_t* w[3];
    const uint32_t* z[3];
    const uint16_t* s[3];
    const uint16_t* norm_w;  // RMSNorm weights applied while staging the input, or null
};

struct Sync {
    uint32_t flags[kMaxWorkgroups];   // arrival epoch of each workgroup
    uint32_t release[8 * 32];         // one 128-byte line per leader workgroup
    uint32_t amax_bits[kMaxWorkgroups];
    int amax_idx[kMaxWorkgroups];
    uint32_t epoch_base;              // continues from launch to launch
    int error;                        // non-zero after a barrier wait exceeded its spin limit
};

struct Args {
    const Phase* phases;
    int nphases;
    int G;       // workgroups = grid size
    int depth;   // ring slots per streaming wave
    int dim, hidden, n_heads, n_kv_heads, head_size, vocab;
    int half_head_shift;  // log2(head_size / 2)
    float rope_theta;
    uint16_t *x, *xb, *hb, *q, *logits, *key_cache, *value_cache;
    const uint16_t* embed;
    int* pos_dev;
    volatile int* pos_host;
    int* tokens_host;
    int* tokens_dev;
    int write_token;
    Sync* sync;
    int* err_host;         // pinned host word set to 1 when a barrier wait times out
    long long spin_limit;  // barrier wait limit in 100 MHz ticks
    long long* trace;      // optional: per-phase wall-clock stamps of workgroup 0 (5 per phase), or null
    int lds_ring, lds_xs, lds_ab, lds_part, lds_misc;  // byte offsets into dynamic LDS
};

}  // namespace tk

int tk_launch(hipStream_t stream, const tk::Args& args, size_t lds_bytes);
