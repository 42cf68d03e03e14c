// AWQ int4 group-128 matrix-vector kernels for gfx950 (wave64).
//
// What they compute is the reference's mat_vec_kernel_int4 family
// (gpu_kernels.h:179-283): per output row n,
//     sum_k (q[n,k] - z[n,k/128]) * s[n,k/128] * x[k]   in fp32,
// followed by one of the epilogues (plain store, KV-cache row store, fused
// residual add, SiLU(gate)*up).
//
// How: a workgroup of W waves (8, or 16 for long rows) stages the activation vector once in LDS (optionally applying
// RMSNorm on the way in), pre-permuted so that a lane's 32 consecutive K elements (one 16-byte load of packed
// weights, the same lane ownership as the reference's uint4 load) meet their activations as packed fp16 pairs.
// Each wave owns R consecutive rows (one gate/up pair in the fused FFN form) and walks them in passes of 64 x 16
// bytes with D passes in flight.  Loads return in order, so a wave first requests its share of the activations,
// then its first D passes of weights, and stages the activations while the weights are still on their way.
// Nibbles are used as fp16 denormals (a shift and a mask put q * 2^-20 into an fp16 lane: that is the whole conversion),
// products are accumulated in fp32 by v_dot2_f32_f16, the zero point enters through a per-chunk constant, and the group
// scale (times 2^20) is applied once per 32 elements.
#include <math.h>

#include <mutex>
#include <set>
#include <utility>

#include "common.hpp"
#include "gemv_core.hpp"

namespace {

using namespace gemv;

struct Int4Mat {
    const uint32_t* w;
    const uint32_t* z;
    const uint16_t* s;
};

struct GemvParams {
    Int4Mat m[3];            // [0] for the single form; q,k,v; gate,up
    uint16_t* out[3];
    const uint16_t* x;
    const uint16_t* norm_w;  // RMSNorm weights when the norm is fused into staging
    uint16_t* norm_out;      // optional: block 0 also stores the normalised vector here
    int K, N;
    int Nkv;                 // QKV form: rows of the K and V matrices (grouped-query models have fewer than N); else = N
    int C;                   // 32-element chunks per row = ceil(K/32)
    int pzh, sh;             // zeros dwords / scale halves per row
    int accum;
    float inv_gpu_count;
    int loff[3];             // -1: none; else out += loff + *pos * N
    const int* pos;
    const float2* rope;      // fused RoPE: (cos, sin) table [position][head_size/2], or null
    int head_size;           // for the fused RoPE row pairing
    const float* xpart;      // PARTS form: x is the sum of `xparts` fp32 vectors K floats apart, rounded to fp16
    int xparts;
    // Filled in by launch().  Everything a wave needs before it can request its first packed weights is a handful of
    // scalar instructions on these: the compute unit's one scalar unit serves all of its waves, and with 16 to 24 waves
    // arriving at once every scalar instruction of the prologue costs all of them a cycle (a division by the grid size
    // and 64-bit row offsets had put the first weight request 0.8 us, in the QKV kernel 1.6 us, behind the wave's start).
    int gx;                  // workgroups along x (= gridDim.x, without the trip to the dispatch packet)
    int groups_q, groups_rem;  // row groups per workgroup: groups_q, and one more for workgroups below groups_rem
    int half_shift;          // log2(head_size / 2) for the fused RoPE pairing (head sizes are powers of two there)
    uint32_t wbytes, zbytes, sbytes;  // bytes per row of weights, zeros, scales (32-bit offsets: a matrix is below 4 GiB)
#ifdef AWQ_STAMPS
    long long* stamps;       // instrumented build: 6 wall-clock stamps (10 ns ticks) per workgroup, or null
#endif
};

#ifdef AWQ_STAMPS
#define AWQ_STAMP(i) do { if (p.stamps && threadIdx.x == 0) stamp_[i] = wall_clock64(); } while (0)
#else
#define AWQ_STAMP(i) do { } while (0)
#endif

enum { KIND_SINGLE = 0, KIND_QKV = 1, KIND_FFN = 2 };

// Logical index li of a workgroup's row space -> matrix row.  With ROPE, consecutive indices (2j, 2j+1) are the two
// rows (i, i + head/2) of one rotation pair, so that one wave holds both.
template <bool ROPE>
__device__ __forceinline__ int map_row(int li, int half_shift) {
    if (!ROPE) return li;
    const int pi = li >> 1;
    return ((pi >> half_shift) << (half_shift + 1)) + (pi & ((1 << half_shift) - 1)) + ((li & 1) << half_shift);
}

// SPLIT (1, 2 or 4): a row takes 64 / SPLIT lanes, and the SPLIT parts of a wave work on SPLIT rows side by side (QKV
// with RoPE: rotation pairs; FFN: gate/up pairs), so a pass covers 64 / SPLIT chunks of each.  A row whose chunk count
// leaves at most half (a quarter) of a 64-lane pass over (K = 5120: 2.5 passes, 11008: 5.375; K = 6656: 3.25) then
// takes ceil(C * SPLIT / 64) passes per SPLIT rows instead of SPLIT * ceil(C / 64): the kernels' time follows the
// number of passes, not the bytes (K = 11008 and K = 12288 took the same 6.9 us; 10240: 6.4).  R then counts the row
// sets of a wave.
template <int W, int R, int D, int KIND, bool NORM, bool ROPE, bool PARTS = false, int SPLIT = 1>
__global__ __launch_bounds__(W * 64) void gemv_int4_kernel(const GemvParams p) {
    static_assert(!PARTS || (!NORM && KIND == KIND_SINGLE), "partial-sum input only for the plain single-matrix form");
    extern __shared__ u32x4 xs[];
    __shared__ float red[W + 1];
#ifdef AWQ_STAMPS
    long long stamp_[6] = {0, 0, 0, 0, 0, 0};
#endif
    AWQ_STAMP(0);  // entry
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform: row addresses stay scalar
    const int C = p.C;
    static_assert(SPLIT == 1 || SPLIT == 2 || SPLIT == 4, "a row takes 64, 32 or 16 lanes");
    constexpr bool HALF = SPLIT > 1;        // (the name from when two was the only split)
    constexpr int LPR = 64 / SPLIT;        // lanes per row
    constexpr int RW = SPLIT * R;          // rows (FFN: gate/up pairs) of a wave per row group
    const int hf = HALF ? lane / LPR : 0;  // which of the wave's SPLIT rows this lane works on
    const int ll = HALF ? lane % LPR : lane;
    const int P = (int)(((uint32_t)C + LPR - 1) / LPR);  // passes per row (per SPLIT rows)
    float* ca = reinterpret_cast<float*>(xs + 4 * C);
    const int which = (KIND == KIND_QKV) ? blockIdx.y : 0;
    const int N = (KIND == KIND_QKV && which != 0) ? p.Nkv : p.N;  // rows of this workgroup's matrix
    // (the grid is sized for the Q matrix; workgroups beyond the K and V rows of a grouped-query model have nothing to do)
    if (KIND == KIND_QKV && (int)blockIdx.x * (W * SPLIT * R) >= N) return;
    const bool rope_here = ROPE && which != 2;
    constexpr bool RES = KIND == KIND_SINGLE;

    constexpr int NS = (KIND == KIND_FFN) ? 2 * R : R;
    const Int4Mat m0 = (KIND == KIND_QKV) ? (which == 0 ? p.m[0] : (which == 1 ? p.m[1] : p.m[2])) : p.m[0];
    const Int4Mat m1 = p.m[1];  // FFN: up
    uint16_t* out_base = (KIND == KIND_QKV) ? (which == 0 ? p.out[0] : (which == 1 ? p.out[1] : p.out[2])) : p.out[0];
    // The position (row of the KV cache, rotation angle) is only needed in the epilogue.  Read as a scalar it is waited
    // for right here, a round trip before anything else is requested; read as the kernel's first vector load (through
    // an address the compiler cannot prove uniform) it returns ahead of everything else and nothing waits for it.
    int loff = (KIND == KIND_QKV) ? (which == 0 ? p.loff[0] : (which == 1 ? p.loff[1] : p.loff[2])) : p.loff[0];
    if (RES && p.accum && loff != -1) {
        // adding to a row that depends on the position: the old values are requested along with the weights
        out_base += (size_t)loff + (size_t)(*p.pos) * p.N;
        loff = -1;
    }
    // (it is the first load of the wave, so whether the branch is taken changes nothing for the loads counted behind it)
    int pos_now = 0;
    if (KIND != KIND_FFN && p.pos) {
        int zero = 0;
        asm volatile("" : "+v"(zero));
        pos_now = p.pos[zero];
    }

    // This workgroup's row groups (W waves x R rows each).  A wave walks its rows as a sequence of stages (group-major,
    // then pass); D stages are in flight at any time.  The sequence is padded to a multiple of D with repeats of the
    // last stage, which are loaded (same addresses again) but not accumulated, so that the number of loads between a
    // stage's request and its use is a compile-time constant.
    // The workgroup takes row groups blockIdx.x, blockIdx.x + gridDim.x, ... (x is staged once for all of them).
    const int g_begin = blockIdx.x, g_stride = p.gx;
    const int total = (p.groups_q + ((int)blockIdx.x < p.groups_rem ? 1 : 0)) * P;

    // ---- load cursor
    const uint32_t* wrow[NS];
    const uint32_t* zrow[NS];
    const uint16_t* srow[NS];
    const uint16_t* resrow[R];
    // SPLIT > 1: the row pointers are those of the first part's row; the other parts add the distance to their own rows
    // (0 when the indices are clamped to the last row), as byte offsets on top of the lane's offset in the row
    uint32_t hoff_w[R], hoff_z[R], hoff_s[R], hoff_r[R];
    int lg = g_begin, lp = 0, ls = 0;
    auto set_rows = [&](int g) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int li = min((g * W + wave) * RW + SPLIT * r, N - 1);  // indices past N are recomputed, never stored
            const int row = rope_here ? map_row<true>(li, p.half_shift) : li;
            if (HALF) {
                const int li_own = min((g * W + wave) * RW + SPLIT * r + hf, N - 1);
                const int drow = (rope_here ? map_row<true>(li_own, p.half_shift) : li_own) - row;
                hoff_w[r] = (uint32_t)drow * p.wbytes;
                hoff_z[r] = (uint32_t)drow * p.zbytes;
                hoff_s[r] = (uint32_t)drow * p.sbytes;
                hoff_r[r] = (uint32_t)(drow * 2);
            }
            resrow[r] = reinterpret_cast<const uint16_t*>(reinterpret_cast<const char*>(out_base) + (uint32_t)row * 2u);  // (the residual form never writes KV-cache rows: no position offset)
            // (byte offsets formed in 32 bits: one scalar multiply and one 64-bit add per pointer)
            const uint32_t ow = (uint32_t)row * p.wbytes, oz = (uint32_t)row * p.zbytes, os = (uint32_t)row * p.sbytes;
            auto at = [](const auto* base, uint32_t off) { return reinterpret_cast<decltype(base)>(reinterpret_cast<const char*>(base) + off); };
            if (KIND == KIND_FFN) {
                wrow[2 * r] = at(m0.w, ow);
                zrow[2 * r] = at(m0.z, oz);
                srow[2 * r] = at(m0.s, os);
                wrow[2 * r + 1] = at(m1.w, ow);
                zrow[2 * r + 1] = at(m1.z, oz);
                srow[2 * r + 1] = at(m1.s, os);
            } else {
                wrow[r] = at(m0.w, ow);
                zrow[r] = at(m0.z, oz);
                srow[r] = at(m0.s, os);
            }
        }
    };
    auto issue = [&](Stage<NS>& st) {
        const int c = min(lp * LPR + ll, C - 1);  // lanes past the row end repeat its last chunk; consume() drops them
        // byte offsets as unsigned 32-bit values on top of wave-uniform row pointers: the loads take the scalar-base
        // form and need no 64-bit address arithmetic per lane
        const uint32_t off_w = (uint32_t)c << 4, off_z = (uint32_t)(c >> 5) << 2, off_s = (uint32_t)(c >> 2) << 1;
#pragma unroll
        for (int i = 0; i < NS; i++) {
            const int r = (KIND == KIND_FFN) ? i >> 1 : i;  // gate and up of a pair are the same row of two matrices
            const uint32_t ow = HALF ? off_w + hoff_w[r] : off_w, oz = HALF ? off_z + hoff_z[r] : off_z, os = HALF ? off_s + hoff_s[r] : off_s;
            st.w[i] = load_nt(reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(wrow[i]) + ow));
            st.zw[i] = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const char*>(zrow[i]) + oz);
            st.s[i] = *reinterpret_cast<const uint16_t*>(reinterpret_cast<const char*>(srow[i]) + os);
        }
        if (RES) {
#pragma unroll
            for (int r = 0; r < R; r++)
                st.res[r] = *reinterpret_cast<const uint16_t*>(reinterpret_cast<const char*>(resrow[r]) + (HALF ? hoff_r[r] : 0u));
        }
        ls++;
        if (ls < total) {
            lp++;
            if (lp == P) {
                lp = 0;
                lg += g_stride;
                set_rows(lg);
            }
        }
    };

    float sum[NS];
#pragma unroll
    for (int i = 0; i < NS; i++) sum[i] = 0.0f;

    // ---- consume cursor
    int cg = g_begin, cp = 0, cs = 0;
    auto finish_group = [&](const Stage<NS>& st) {
        // chunk_dot works in units of 2^-20; with SPLIT > 1 every lane ends up with the sum of its own part of the wave
#pragma unroll
        for (int i = 0; i < NS; i++) {
            float v = sum[i];
            if (SPLIT == 1) v = wave_sum(v);
            else if (SPLIT == 2) v = lane_xor_sum<16>(row16_sum(v));
            else v = row16_sum(v);
            sum[i] = v * kChunkDotUnscale;
        }
        const int li0 = (cg * W + wave) * RW;
        if (rope_here) {
            // q/k are rounded to fp16 and then rotated, as the separate RoPE kernel does (gpu_kernels.h:351-361);
            // the two rows of a pair are two streams of the wave, or (SPLIT > 1) two neighbouring parts of it: the even
            // part's first lane takes the odd part's sum from LPR lanes further on
            float second[R];
#pragma unroll
            for (int r = 0; r < R; r++) {
                second[r] = 0.0f;
                if (HALF) second[r] = __shfl_xor(sum[r], LPR);
            }
            if (ll == 0 && (hf & 1) == 0 && li0 + hf < N) {
                uint16_t* out = out_base;
                if (loff != -1) out += (size_t)loff + (size_t)pos_now * N;
                const int half = p.head_size >> 1;
                const float2* cs_tab = p.rope + (size_t)pos_now * half;
#pragma unroll
                for (int r = 0; r < (HALF ? R : R - 1); r += (HALF ? 1 : 2)) {
                    const int li = li0 + (HALF ? SPLIT * r + hf : r);
                    if (li < N) {
                        const int row = map_row<true>(li, p.half_shift);
                        const float v0 = half_bits_to_float(float_to_half_bits(sum[r]));
                        const float v1 = half_bits_to_float(float_to_half_bits(HALF ? second[r] : sum[HALF ? r : r + 1]));
                        const float2 c = cs_tab[row % half];
                        float r0, r1;
                        rope_rotate(v0, v1, c.x, c.y, r0, r1);
                        out[row] = float_to_half_bits(r0);
                        out[row + half] = float_to_half_bits(r1);
                    }
                }
            }
        } else if (ll == 0) {
            uint16_t* out = out_base;
            if (loff != -1) out += (size_t)loff + (size_t)pos_now * N;
#pragma unroll
            for (int r = 0; r < R; r++) {
                const int row = li0 + (HALF ? SPLIT * r + hf : r);
                if (row < N) {
                    float v;
                    if (KIND == KIND_FFN) {
                        // gate = stream 2r, up = stream 2r+1 (gpu_kernels.h:276-281)
                        float g = sum[2 * r];
                        g *= 1.0f / (1.0f + expf(-g));
                        v = g * sum[2 * r + 1];
                    } else {
                        v = sum[r];
                        if (RES && p.accum) v += half_bits_to_float(st.res[r]) * p.inv_gpu_count;
                    }
                    out[row] = float_to_half_bits(v);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < NS; i++) sum[i] = 0.0f;
    };
    auto consume = [&](const Stage<NS>& st) {
        if (cs < total) {
            const int c = cp * LPR + ll;
            const int cc = min(c, C - 1);
            u32x4 xq[4];
#pragma unroll
            for (int qi = 0; qi < 4; qi++) xq[qi] = xs[qi * C + cc];
            const float cA = ca[cc];
            const int zshift = ((cc >> 2) & 7) * 4;
#pragma unroll
            for (int i = 0; i < NS; i++) {
                const float zf = (float)((st.zw[i] >> zshift) & 0xFu);
                const float acc = chunk_dot(st.w[i], zf, xq, cA);
                const float sc = c < C ? half_bits_to_float(st.s[i]) : 0.0f;
                sum[i] = fmaf(sc, acc, sum[i]);
            }
            cs++;
            cp++;
            if (cp == P) {
                finish_group(st);
                cp = 0;
                cg += g_stride;
            }
        }
    };

    // Packed weights are requested before x is staged (all D stages in the plain forms, D - 1 in the norm-fused ones), so
    // that their HBM latency overlaps the staging (and the RMSNorm reduction).
    const XArgs xa{p.x, p.norm_w, p.norm_out, p.K, p.C, p.xpart, p.xparts};
    XPieces<NORM, pieces_for(W)> xr;
    PartPieces pr;
    if constexpr (PARTS)
        load_parts<W>(pr, xa);
    else
        load_x<W, NORM>(xr, xa);
    AWQ_STAMP(1);  // x requested
    // Norm-fused forms: every wave's share of x is requested before any wave of the workgroup requests weights.  The
    // staging needs all shares, and a share requested behind another wave's weights waits in the compute unit's queue
    // until those have been delivered (+0.7 % tokens/s at 7B; the plain forms, whose staging is short, lose by it).
    if (NORM) __builtin_amdgcn_s_barrier();
    Stage<NS> st[D];
    set_rows(lg);
    // ... and for the same reason they request the last of their D stages only after the staging: one pass fewer queued
    // ahead of the other workgroups' activations on the compute unit (7B shape +1.5 % tokens/s, 13B +0.6 %, 33B
    // unchanged; with nothing requested ahead of the staging the weights' own latency shows: -0.4 %; the plain forms lose
    // by any delay)
    constexpr int DE = NORM ? D - 1 : D;  // stages requested before the staging
#pragma unroll
    for (int d = 0; d < DE; d++) {
        issue(st[d]);
#ifdef AWQ_STAMPS
        if (d == 0) AWQ_STAMP(2);  // first stage requested
#endif
    }
    AWQ_STAMP(3);  // the stages that go ahead of the staging requested
    if constexpr (PARTS) combine_x<W>(xr, pr, xa);
    stage_x<W, NORM>(xs, ca, xa, red, xr);
    AWQ_STAMP(4);  // x staged
#pragma unroll
    for (int d = DE; d < D; d++) issue(st[d]);
    const int rounds = (total + D - 1) / D;
    for (int r = 1; r < rounds; r++) {
#pragma unroll
        for (int d = 0; d < D; d++) {
            consume(st[d]);
            issue(st[d]);
        }
    }
#pragma unroll
    for (int d = 0; d < D; d++) consume(st[d]);
#ifdef AWQ_STAMPS
    if (p.stamps && threadIdx.x == 0) {
        stamp_[5] = wall_clock64();  // results stored
        long long* o = p.stamps + 6 * (size_t)(blockIdx.y * gridDim.x + blockIdx.x);
        for (int i = 0; i < 6; i++) o[i] = stamp_[i];
    }
#endif
}

// out[n*K + k] = half_rne((q - z) * s): exact fp32 product, one rounding.
__global__ __launch_bounds__(256) void dequant_kernel(uint16_t* out, Int4Mat m, int K, int N, int pwh, int pzh, int sh) {
    const size_t total8 = (size_t)N * (K >> 3);
    for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < total8; e += (size_t)gridDim.x * 256) {
        const int n = (int)(e / (size_t)(K >> 3));
        const int k8 = (int)(e % (size_t)(K >> 3));
        const int g = k8 >> 4;
        uint32_t d = m.w[(size_t)n * pwh + k8];
        const float z = (float)((m.z[(size_t)n * pzh + (g >> 3)] >> (4 * (g & 7))) & 0xFu);
        const float s = half_bits_to_float(m.s[(size_t)n * sh + g]);
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float w0 = ((float)(d & 0xFu) - z) * s;
            const float w1 = ((float)((d >> 4) & 0xFu) - z) * s;
            d >>= 8;
            o[i] = (uint32_t)float_to_half_bits(w0) | ((uint32_t)float_to_half_bits(w1) << 16);
        }
        *reinterpret_cast<u32x4*>(out + (size_t)n * K + (size_t)k8 * 8) = o;
    }
}

int check_shape(int K, int N) {
    // llama2_q4.cu:368: "Unsupported matmul size"
    if (K <= 0 || N <= 0 || (K & 7) || (N & 7)) {
        awq_set_error("unsupported matmul size K=%d N=%d (both must be positive multiples of 8)", K, N);
        return AWQ_ERR_SHAPE;
    }
    if ((size_t)N * (size_t)div_up(K, 32) * 16 >= ((size_t)1 << 32)) {
        awq_set_error("matrix of K=%d N=%d exceeds the 4 GiB that 32-bit row offsets address", K, N);
        return AWQ_ERR_SHAPE;
    }
    if (K > kMaxStagedKInt4) {
        awq_set_error("K=%d exceeds the %d activations the kernels stage in LDS", K, kMaxStagedKInt4);
        return AWQ_ERR_SHAPE;
    }
    return AWQ_OK;
}

void fill_common(GemvParams& p, const uint16_t* x, int K, int N) {
    p.x = x;
    p.norm_w = nullptr;
    p.norm_out = nullptr;
    p.K = K;
    p.N = N;
    p.Nkv = N;
    p.C = div_up(K, 32);
    p.pzh = packed_zeros_height(K);
    p.sh = scales_height(K);
    p.accum = 0;
    p.inv_gpu_count = 1.0f;
    p.loff[0] = p.loff[1] = p.loff[2] = -1;
    p.pos = nullptr;
    p.rope = nullptr;
    p.head_size = 0;
    p.xpart = nullptr;
    p.xparts = 0;
}

Int4Mat to_mat(const awq_qweight* w) { return Int4Mat{w->weight, w->zeros, w->scales}; }

bool qw_ok(const awq_qweight* w) { return w && w->weight && w->zeros && w->scales; }

// Launch geometry of one matrix-vector product.
struct GemvPlan {
    int waves;   // waves per workgroup (4, 8)
    int rows;    // rows per wave (1, 2, 4)
    int depth;   // stages in flight per wave (2, 3, 4)
};

#ifdef AWQ_STAMPS
long long* g_stamps_base = nullptr;
int g_stamps_stride = 0, g_stamps_launches = 0, g_stamps_next = 0;
int g_stamps_grid[4096], g_stamps_bytes[4096];
#endif

// Rows above 30 K elements need more dynamic LDS than a kernel may take by default (64 KB): the limit of the kernel
// about to be launched is raised, once per device and kernel.
std::mutex g_lds_mutex;
std::set<std::pair<int, const void*>> g_lds_raised;
int ensure_lds_limit(awq_ctx* ctx, const void* kernel, size_t lds, const char* what) {
    if (lds <= 64 * 1024) return AWQ_OK;
    std::lock_guard<std::mutex> lock(g_lds_mutex);
    const auto key = std::make_pair(ctx->device, kernel);
    if (g_lds_raised.count(key)) return AWQ_OK;
    const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)((size_t)(kMaxStagedKInt4 / 32) * 68));
    if (e != hipSuccess) {
        awq_set_error("%s: hipFuncSetAttribute(dynamic LDS) failed: %s", what, hipGetErrorString(e));
        return AWQ_ERR_HIP;
    }
    g_lds_raised.insert(key);
    return AWQ_OK;
}

template <int W, int R, int D, int KIND, bool ROPE, int SPLIT = 1>
int launch(awq_ctx* ctx, GemvParams& p, int grid_y, const char* what) {
    const int groups_total = div_up(p.N, W * R * SPLIT);
    int gx = groups_total;
    // The norm-fused gate/up kernel stages (and normalises) x in every workgroup, and that work is what bounds it:
    // three 4-wave workgroups per compute unit walk the row groups between them (measured best at the 7B shape; the
    // plain kernels are faster with one group per workgroup).
    if (p.norm_w && KIND == KIND_FFN) {
        const int cus = ctx->cus;
        if (gx > 3 * cus) gx = 3 * cus;
    }
    // Rows so long that their staged activations leave room for one workgroup per compute unit (more than 64 KB of LDS):
    // one workgroup per compute unit walks the row groups and stages the activations once, instead of once per group
    // (K = 53248, N = 16384: 100 -> 93 us).
    if ((size_t)p.C * 68 > 64 * 1024 && grid_y == 1 && gx > ctx->cus) gx = ctx->cus;
    p.gx = gx;
    p.groups_q = groups_total / gx;
    p.groups_rem = groups_total % gx;
    p.half_shift = 0;
    if (ROPE) {
        while ((2 << p.half_shift) < p.head_size) p.half_shift++;
        if ((2 << p.half_shift) != p.head_size) {
            awq_set_error("%s: the fused rotation needs a power-of-two head size (got %d)", what, p.head_size);
            return AWQ_ERR_SHAPE;
        }
    }
    p.wbytes = (uint32_t)p.C * 16u;
    p.zbytes = (uint32_t)p.pzh * 4u;
    p.sbytes = (uint32_t)p.sh * 2u;
#ifdef AWQ_STAMPS
    p.stamps = nullptr;
    if (g_stamps_base && g_stamps_next < g_stamps_launches && (int)(gx * grid_y) <= g_stamps_stride) {
        p.stamps = g_stamps_base + (size_t)g_stamps_next * g_stamps_stride * 6;
        g_stamps_grid[g_stamps_next] = gx * grid_y;
        g_stamps_bytes[g_stamps_next] = KIND * 1000 + W;
        g_stamps_next++;
    }
#endif
    const dim3 grid(gx, grid_y);
    const size_t lds = (size_t)p.C * 68;  // activations + per-chunk constant
    if constexpr (KIND == KIND_SINGLE && !ROPE && R == 1 && (W == 8 || W == 10 || W == 13)) {  // (partial-sum input comes with K <= 8192)
        if (p.xpart) {
            if (int r = ensure_lds_limit(ctx, (const void*)gemv_int4_kernel<W, R, D, KIND, false, false, true, SPLIT>, lds, what)) return r;
            awq_launch(ctx, gemv_int4_kernel<W, R, D, KIND, false, false, true, SPLIT>, grid, dim3(W * 64), lds, p);
            return awq_check_launch(what);
        }
    }
    if (p.xpart) {
        awq_set_error("%s: no kernel takes partial-sum input in this geometry", what);
        return AWQ_ERR_ARG;
    }
    if (p.norm_w) {
        if (int r = ensure_lds_limit(ctx, (const void*)gemv_int4_kernel<W, R, D, KIND, true, ROPE, false, SPLIT>, lds, what)) return r;
        awq_launch(ctx, gemv_int4_kernel<W, R, D, KIND, true, ROPE, false, SPLIT>, grid, dim3(W * 64), lds, p);
    } else {
        if (int r = ensure_lds_limit(ctx, (const void*)gemv_int4_kernel<W, R, D, KIND, false, ROPE, false, SPLIT>, lds, what)) return r;
        awq_launch(ctx, gemv_int4_kernel<W, R, D, KIND, false, ROPE, false, SPLIT>, grid, dim3(W * 64), lds, p);
    }
    return awq_check_launch(what);
}

// The split forms: one set of SPLIT rows per wave (SPLIT gate/up pairs in the FFN form), `depth` passes of the set in
// flight.
template <int W, int KIND, bool ROPE, int SPLIT>
int dispatch_split(awq_ctx* ctx, GemvParams& p, int grid_y, const char* what, int depth) {
    if (depth == 2) return launch<W, 1, 2, KIND, ROPE, SPLIT>(ctx, p, grid_y, what);
    return launch<W, 1, 3, KIND, ROPE, SPLIT>(ctx, p, grid_y, what);
}

template <int W, int R, int KIND, bool ROPE>
int dispatch_depth(awq_ctx* ctx, GemvParams& p, int grid_y, const char* what, const GemvPlan& plan) {
    constexpr int NS = (KIND == KIND_FFN) ? 2 * R : R;
    int depth = plan.depth;
    while (depth > 2 && (NS * depth > 16 || depth > 4)) depth--;  // what the register file affords
    switch (depth) {
        case 2: return launch<W, R, 2, KIND, ROPE>(ctx, p, grid_y, what);
        case 3: if constexpr (NS * 3 <= 16) return launch<W, R, 3, KIND, ROPE>(ctx, p, grid_y, what); break;
        case 4: if constexpr (NS * 4 <= 16) return launch<W, R, 4, KIND, ROPE>(ctx, p, grid_y, what); break;
    }
    awq_set_error("no int4 matrix-vector kernel with %d stages in flight for %d streams", plan.depth, NS);
    return AWQ_ERR_ARG;
}


// Measured on MI355X at the 7B shapes: one row (one gate/up pair) per wave, two passes in flight, 8 waves sharing the
// staged activations; long rows (K > 8192) want 16 waves for the staging and a third pass in flight.
GemvPlan plan_for(int K, int rows) {
    GemvPlan plan;
    plan.waves = K > 8192 ? 16 : 8;
    plan.rows = rows;
    // The stage sequence of a wave is padded to a multiple of the depth with loads that are not used: a row of three
    // passes is requested whole (two in flight would pad it to four), and long rows take whichever of two and three
    // pads less (K = 13824, seven passes: eight stages instead of nine, down projection 11.9 -> 11.2 us at the 13B
    // shape; K = 11008 and 17920, six and nine passes, keep three; four in flight measured slower everywhere).
    const int passes = (div_up(K, 32) + 63) / 64;
    if (K > 8192)
        plan.depth = (3 - passes % 3) % 3 <= passes % 2 ? 3 : 2;
    else
        plan.depth = passes == 3 ? 3 : 2;
    return plan;
}

template <int KIND, bool ROPE>
int dispatch(awq_ctx* ctx, GemvParams& p, int grid_y, const char* what, GemvPlan plan) {
    if (p.norm_w && KIND == KIND_FFN && p.K <= 8192) plan.waves = 4;  // see launch()
    if (plan.waves == 16 && plan.rows == 1) {
        // Long rows, one per wave: every workgroup is resident at once, so the kernel takes as long as the compute unit
        // with the most workgroups.  16-wave workgroups suit 4096 rows on 256 compute units (one each); 5120 rows are
        // 320 workgroups, two on a quarter of the compute units and one on the rest, and go better as 640 of 8 waves
        // (13B down projection 11.2 -> 10.7 us); 6656 rows are as uneven either way and keep 16 (measured).
        const double per_cu16 = (double)div_up(p.N, 16) / ctx->cus, per_cu8 = (double)div_up(p.N, 8) / ctx->cus;
        if (ceil(per_cu8) / per_cu8 < ceil(per_cu16) / per_cu16 - 0.05) plan.waves = 8;
    }
    if (ROPE && plan.rows < 2) plan.rows = 2;  // a rotation pair lives in one wave
    // Rows that leave at most half of a 64-lane pass over go two to a wave, 32 lanes each (see the kernel).  Measured
    // at the 13B and 33B shapes (K = 5120, 6656): gate/up -6 %, O projection -7 %, QKV -2 % with two passes in flight
    // and even with three, tokens/s +3 %.  Rows above 8192 (K = 11008: 16 waves, or 8, at any depth) lose: two rows per
    // wave halve the workgroups of a matrix that has few rows to begin with.
    const int tail = p.C & 63;
    const bool split2 = tail != 0 && tail <= 32 && plan.rows <= 2 && p.K <= 8192;
    if constexpr (KIND == KIND_SINGLE) {
        // The workgroups of a single-matrix product are all resident at once, and the kernel takes as long as the
        // compute unit that holds the most of them.  Workgroups of 10 or 13 waves are taken where they make the count a
        // multiple of the compute units and the usual size does not (5120 rows: 256 workgroups of 10 two-row waves
        // instead of 320 of 8, O projection from partial sums 7.8 -> 6.1 us, and 512 of 10 one-row waves instead of 640
        // of 8, down projection 10.6 -> 9.9 us, at the 13B shape; 6656 rows: 13 waves).
        if (plan.rows == 1 && (split2 || p.K > 8192)) {
            const int cus = ctx->cus;
            const int waves_total = div_up(p.N, split2 ? 2 : 1);
            auto unevenness = [&](int w) {
                const double per_cu = (double)div_up(waves_total, w) / cus;
                return ceil(per_cu) / per_cu;
            };
            int best = plan.waves;
            for (int w : {10, 13})
                if (unevenness(w) < unevenness(best) - 0.15) best = w;
            if (best == 10 || best == 13) {
                if (split2) {
                    if (best == 10) return dispatch_split<10, KIND, ROPE, 2>(ctx, p, grid_y, what, 3);
                    return dispatch_split<13, KIND, ROPE, 2>(ctx, p, grid_y, what, 3);
                }
                if (best == 10) return dispatch_depth<10, 1, KIND, ROPE>(ctx, p, grid_y, what, plan);
                return dispatch_depth<13, 1, KIND, ROPE>(ctx, p, grid_y, what, plan);
            }
        }
    }
    if (split2) {
        const int depth = KIND == KIND_QKV ? 2 : 3;
        // at most a quarter of a pass over (K = 6656): four rows to a wave pays for the QKV kernel (16.3 -> 15.6 us at the
        // 33B shape); the O projection is unchanged by it and the gate/up kernel loses (21.8 -> 23.2: half as many row
        // groups for its workgroups to walk)
        if constexpr (KIND == KIND_QKV) {
            if (tail <= 16) {
                // all workgroups are resident at once here too: 6656 rows x 3 are 624 workgroups of 8 waves (2.4 per
                // compute unit, so three on some) or 501 of 10 (two on each): 16.5 -> 16.1 us, +0.75 % tokens/s at the
                // 33B shape
                auto unevenness = [&](int w) {
                    const double per_cu = (double)(div_up(p.N, w * 4) + (grid_y - 1) * div_up(p.Nkv, w * 4)) / ctx->cus;
                    return ceil(per_cu) / per_cu;
                };
                if (unevenness(10) < unevenness(8) - 0.15) return dispatch_split<10, KIND, ROPE, 4>(ctx, p, grid_y, what, depth);
                return dispatch_split<8, KIND, ROPE, 4>(ctx, p, grid_y, what, depth);
            }
        }
        if (plan.waves == 4) return dispatch_split<4, KIND, ROPE, 2>(ctx, p, grid_y, what, depth);
        return dispatch_split<8, KIND, ROPE, 2>(ctx, p, grid_y, what, depth);
    }
    if constexpr (KIND == KIND_QKV) {
        // grouped-query models: the K and V matrices add few workgroups to those of Q, and the sum can fall badly on the
        // compute units (4096 + 2 x 1024 rows: 384 workgroups of 8 waves, two on half of the compute units, against 768
        // of 4 waves, three on each: 7.1 -> 6.6 us, +1.6 % tokens/s).  Not beyond three per compute unit: every workgroup
        // stages the activations (8192 + 2 x 1024 rows: 1280 workgroups of 4 waves, 12.0 -> 13.7 us).
        if (plan.waves == 8 && plan.rows == 2 && p.Nkv != p.N) {
            auto per_cu = [&](int w) { return (double)(div_up(p.N, w * 2) + (grid_y - 1) * div_up(p.Nkv, w * 2)) / ctx->cus; };
            auto unevenness = [&](int w) { return ceil(per_cu(w)) / per_cu(w); };
            if (unevenness(4) < unevenness(8) - 0.15 && per_cu(4) <= 3.0) plan.waves = 4;
        }
    }
#define AWQ_CASE(W_, R_) \
    if (plan.waves == W_ && plan.rows == R_) return dispatch_depth<W_, R_, KIND, ROPE>(ctx, p, grid_y, what, plan);
    AWQ_CASE(4, 2) AWQ_CASE(4, 4) AWQ_CASE(8, 2) AWQ_CASE(8, 4) AWQ_CASE(16, 2)
    if constexpr (!ROPE) {
        AWQ_CASE(4, 1) AWQ_CASE(8, 1) AWQ_CASE(16, 1)
    }
#undef AWQ_CASE
    awq_set_error("no int4 matrix-vector kernel for %d waves x %d rows", plan.waves, plan.rows);
    return AWQ_ERR_ARG;
}

}  // namespace

// Internal launchers shared with the fused schedule (norm_w != nullptr fuses
// RMSNorm into the staging of x; norm_out optionally receives the normalised vector).
int awq_launch_matvec_int4(awq_ctx* ctx, uint16_t* out, const uint16_t* x, const awq_qweight* w, int K, int N, int accum,
                           int gpu_count, int loff, const int* pos, const uint16_t* norm_w, uint16_t* norm_out) {
    GemvParams p;
    fill_common(p, x, K, N);
    p.m[0] = to_mat(w);
    p.out[0] = out;
    p.accum = accum;
    p.inv_gpu_count = 1.0f / (float)gpu_count;
    p.loff[0] = loff;
    p.pos = pos;
    p.norm_w = norm_w;
    p.norm_out = norm_out;
    return dispatch<KIND_SINGLE, false>(ctx, p, 1, "gemv_int4", plan_for(K, 1));
}

// out = half(W x [+ out]) with x = half(part[0] + part[1] + ...): the O projection behind the position-split attention.
int awq_launch_matvec_int4_parts(awq_ctx* ctx, uint16_t* out, const float* part, int parts, const awq_qweight* w, int K, int N,
                                 int accum) {
    if (parts < 1 || parts > kMaxParts || K > XP * 8 * 64 * 8) {  // every piece of x travels in registers (8-wave workgroups)
        awq_set_error("matvec with partial-sum input: %d parts, K = %d not supported", parts, K);
        return AWQ_ERR_SHAPE;
    }
    GemvParams p;
    fill_common(p, nullptr, K, N);
    p.m[0] = to_mat(w);
    p.out[0] = out;
    p.accum = accum;
    p.xpart = part;
    p.xparts = parts;
    return dispatch<KIND_SINGLE, false>(ctx, p, 1, "gemv_int4_parts", plan_for(K, 1));
}

int awq_launch_qkv(awq_ctx* ctx, uint16_t* q, uint16_t* key_cache, uint16_t* value_cache, const uint16_t* x,
                   const awq_qweight* qw, const awq_qweight* kw, const awq_qweight* vw, int K, int N, int loff,
                   const int* pos, const uint16_t* norm_w, uint16_t* norm_out, const float2* rope, int head_size, int Nkv) {
    GemvParams p;
    fill_common(p, x, K, N);
    p.Nkv = Nkv;  // = N in the reference's qkv_matvec_kernel (llama2_q4.cu:454); fewer rows in grouped-query models
    p.rope = rope;
    p.head_size = head_size;
    p.m[0] = to_mat(qw);
    p.m[1] = to_mat(kw);
    p.m[2] = to_mat(vw);
    p.out[0] = q;
    p.out[1] = key_cache;
    p.out[2] = value_cache;
    p.loff[1] = loff;
    p.loff[2] = loff;
    p.pos = pos;
    p.norm_w = norm_w;
    p.norm_out = norm_out;
    if (rope) return dispatch<KIND_QKV, true>(ctx, p, 3, "qkv_matvec_rope", plan_for(K, 2));
    return dispatch<KIND_QKV, false>(ctx, p, 3, "qkv_matvec", plan_for(K, 2));
}

int awq_launch_ffn(awq_ctx* ctx, uint16_t* out, const uint16_t* x, const awq_qweight* gate_w, const awq_qweight* up_w, int K,
                   int N, const uint16_t* norm_w, uint16_t* norm_out) {
    GemvParams p;
    fill_common(p, x, K, N);
    p.m[0] = to_mat(gate_w);
    p.m[1] = to_mat(up_w);
    p.out[0] = out;
    p.norm_w = norm_w;
    p.norm_out = norm_out;
    return dispatch<KIND_FFN, false>(ctx, p, 1, "ffn_matvec_silu", plan_for(K, 1));
}

#ifdef AWQ_STAMPS
// Instrumented build only: every int4 matrix-vector launch from now on writes its workgroups' stamps to
// buf[launch][wg_stride][6]; returns how many launches have been recorded so far and their grid sizes / kinds.
extern "C" int awq_debug_stamps(long long* buf, int wg_stride, int max_launches, int* grids_out, int* kinds_out) {
    const int n = g_stamps_next;
    if (grids_out) for (int i = 0; i < n; i++) { grids_out[i] = g_stamps_grid[i]; kinds_out[i] = g_stamps_bytes[i]; }
    g_stamps_base = buf;
    g_stamps_stride = wg_stride;
    g_stamps_launches = max_launches > 4096 ? 4096 : max_launches;
    g_stamps_next = 0;
    return n;
}
#endif

extern "C" {

int awq_matvec_int4(awq_ctx* ctx, uint16_t* out, const uint16_t* x, const awq_qweight* w, int K, int N, int accum,
                    int gpu_count, int loff, const int* pos) {
    if (int r = awq_bind(ctx)) return r;
    if (int r = check_shape(K, N)) return r;
    AWQ_REQUIRE(out && x && qw_ok(w), AWQ_ERR_ARG, "null pointer");
    AWQ_REQUIRE(gpu_count >= 1, AWQ_ERR_ARG, "gpu_count must be >= 1");
    AWQ_REQUIRE(loff == -1 || (loff >= 0 && pos), AWQ_ERR_ARG, "loff needs a position pointer");
    return awq_launch_matvec_int4(ctx, out, x, w, K, N, accum, gpu_count, loff, pos, nullptr, nullptr);
}

int awq_qkv_matvec(awq_ctx* ctx, uint16_t* q, uint16_t* key_cache, uint16_t* value_cache, const uint16_t* x,
                   const awq_qweight* qw, const awq_qweight* kw, const awq_qweight* vw, int K, int N, int loff,
                   const int* pos) {
    if (int r = awq_bind(ctx)) return r;
    if (int r = check_shape(K, N)) return r;
    AWQ_REQUIRE(q && key_cache && value_cache && x && qw_ok(qw) && qw_ok(kw) && qw_ok(vw), AWQ_ERR_ARG, "null pointer");
    AWQ_REQUIRE(loff >= 0 && pos, AWQ_ERR_ARG, "qkv needs loff >= 0 and a position pointer");
    return awq_launch_qkv(ctx, q, key_cache, value_cache, x, qw, kw, vw, K, N, loff, pos, nullptr, nullptr, nullptr, 0, N);
}

int awq_ffn_matvec_silu(awq_ctx* ctx, uint16_t* out, const uint16_t* x, const awq_qweight* gate_w, const awq_qweight* up_w,
                        int K, int N) {
    if (int r = awq_bind(ctx)) return r;
    if (int r = check_shape(K, N)) return r;
    AWQ_REQUIRE(out && x && qw_ok(gate_w) && qw_ok(up_w), AWQ_ERR_ARG, "null pointer");
    return awq_launch_ffn(ctx, out, x, gate_w, up_w, K, N, nullptr, nullptr);
}

int awq_matvec_int4_parts(awq_ctx* ctx, uint16_t* out, const float* part, int parts, const awq_qweight* w, int K, int N,
                          int accum) {
    if (int r = awq_bind(ctx)) return r;
    if (int r = check_shape(K, N)) return r;
    AWQ_REQUIRE(out && part && qw_ok(w), AWQ_ERR_ARG, "null pointer");
    return awq_launch_matvec_int4_parts(ctx, out, part, parts, w, K, N, accum);
}

int awq_rmsnorm_ffn_matvec_silu(awq_ctx* ctx, uint16_t* out, const uint16_t* x, const uint16_t* norm_weight,
                                const awq_qweight* gate_w, const awq_qweight* up_w, int K, int N) {
    if (int r = awq_bind(ctx)) return r;
    if (int r = check_shape(K, N)) return r;
    AWQ_REQUIRE(out && x && norm_weight && qw_ok(gate_w) && qw_ok(up_w), AWQ_ERR_ARG, "null pointer");
    return awq_launch_ffn(ctx, out, x, gate_w, up_w, K, N, norm_weight, nullptr);
}

int awq_dequant(awq_ctx* ctx, uint16_t* out, const awq_qweight* w, int K, int N) {
    if (int r = awq_bind(ctx)) return r;
    if (K <= 0 || N <= 0 || (K & 7) || (N & 7)) {
        awq_set_error("unsupported matmul size K=%d N=%d", K, N);
        return AWQ_ERR_SHAPE;
    }
    AWQ_REQUIRE(out && qw_ok(w), AWQ_ERR_ARG, "null pointer");
    const size_t total8 = (size_t)N * (K >> 3);
    const int grid = (int)((total8 + 255) / 256 < 65536 ? (total8 + 255) / 256 : 65536);
    hipLaunchKernelGGL(dequant_kernel, dim3(grid), dim3(256), 0, ctx->stream, out, to_mat(w), K, N, packed_weight_height(K),
                       packed_zeros_height(K), scales_height(K));
    return awq_check_launch("dequant");
}

}  // extern "C"
