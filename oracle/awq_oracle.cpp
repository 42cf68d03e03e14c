// TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's hot path.
//
// This file is the parity oracle and the CPU baseline.  It is never linked
// into, imported by or called from the shipped HIP library or its host
// driver; only the tests, the smoke check and the benchmark's cpu_baseline
// leg load it.
//
// It restates, in scalar C++ (OpenMP over output rows / heads), the
// arithmetic of the reference's CUDA kernels with the reference's rounding
// points, and the per-token schedule and decode loop around them.  Every
// function cites the reference lines it follows (paths relative to the
// reference checkout).
//
// How each function is pinned (the reference ships no tests or vectors):
//   half <-> float           : hardware F16C vs the software routine below vs
//                              numpy.float16 on all 65536 patterns / random floats
//   unpack + dequant         : numpy restatement from the layout definition;
//                              pack/unpack round trip; compiled reference
//                              weight_packer output (oracle/_ref)
//   int4 / fp16 matvec       : fp64 dot of exactly dequantised weights (numpy)
//   residual / KV epilogues  : identities (zero weights, address arithmetic)
//   rmsnorm, silu, softmax   : fp64 closed forms and invariants
//   rope                     : fp64 closed form, pos 0 identity, norm preserved
//   attention                : fp64 softmax(qK^T/sqrt(d))V brute force
//   argmax                   : brute force; ties -> lowest index (the
//                              reference's tie winner is a write race)
//   softmax of logits, top-p : fp64 softmax; numpy stable argsort + integer
//                              cumulative sums; hand-built distributions whose
//                              crossing index is known (the fp16 prefix sum of
//                              the reference's CUB scan is order dependent:
//                              "parity unpinned", the exact sum rounded once is
//                              used instead)
//   schedule / decode loop   : hand-traced toy model built from the above
// The fp32 summation ORDER of the CUDA block/warp reductions comes from CUB,
// which is not vendored in the reference: that order is "parity unpinned" and
// is covered by tolerance against the fp64 forms only.

#include <stdint.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#include <immintrin.h>
#ifdef _OPENMP
#include <omp.h>
#endif

typedef uint16_t h16;

// ---------------------------------------------------------------- fp16 helpers
static inline float h2f(h16 h) { return _cvtsh_ss(h); }
static inline h16 f2h(float f) { return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC); }

extern "C" {

// Software IEEE binary16 -> binary32 (exact).
float orc_half_to_float_sw(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {  // subnormal: normalise
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

// Software binary32 -> binary16, round to nearest even (what CUDA's (half)
// cast of a float does).
uint16_t orc_float_to_half_sw(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7FFFFFFFu;
    if (ax >= 0x7F800000u) {  // inf / nan
        return (uint16_t)(sign | 0x7C00u | ((ax > 0x7F800000u) ? (0x200u | ((ax >> 13) & 0x3FFu)) : 0u));
    }
    if (ax >= 0x477FF000u) {  // >= 65520 -> inf
        return (uint16_t)(sign | 0x7C00u);
    }
    if (ax < 0x33000001u) {  // <= 2^-25 -> 0 (tie at 2^-25 goes to even = 0)
        return (uint16_t)sign;
    }
    int e = (int)(ax >> 23) - 127;
    uint32_t m = (ax & 0x7FFFFFu) | 0x800000u;
    int shift = (e < -14) ? (13 + (-14 - e)) : 13;
    uint32_t half_m = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (half_m & 1u))) half_m++;
    uint32_t out;
    if (e < -14) {
        out = half_m;  // subnormal (may carry into the smallest normal)
    } else {
        out = ((uint32_t)(e + 15) << 10) + (half_m - 0x400u);  // carry propagates into exponent
    }
    return (uint16_t)(sign | out);
}

float orc_half_to_float(uint16_t h) { return h2f(h); }
uint16_t orc_float_to_half(float f) { return f2h(f); }

int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

// ---------------------------------------------------------------- layout
// Derived strides of a packed matrix with reduction length K
// (llama2_q4.cu:106-112, 121-129, 367-372).
static inline int div_up(int a, int b) { return (a - 1) / b + 1; }
static inline int packed_weight_height(int K) { return div_up(K, 32) * 4; }  // dwords per row
static inline int scales_height(int K) { return div_up(K, 128); }           // halves per row
static inline int packed_zeros_height(int K) { return div_up(scales_height(K), 8); }  // dwords per row

typedef struct {
    const uint32_t* weight;
    const uint32_t* zeros;
    const h16* scales;
} QW;

// Dequantise a packed matrix to fp16, row n / column k of the logical
// (N x K) matrix at out[n*K + k].  Element k of row n sits in nibble k%8 of
// weight[n*pwh + k/8]; its group g = k/128 has its zero in nibble g%8 of
// zeros[n*pzh + g/8] and its scale at scales[n*sh + g]
// (gpu_kernels.h:184-207 read side; weight_packer.cpp:114-124 write side).
// w16 = half_rne((float)(q - z) * (float)scale): the fp32 product is exact.
void orc_dequant(uint16_t* out, const uint32_t* weight, const uint32_t* zeros, const uint16_t* scales, int K, int N) {
    const int pwh = packed_weight_height(K), sh = scales_height(K), pzh = packed_zeros_height(K);
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; n++) {
        for (int k = 0; k < K; k++) {
            uint32_t q = (weight[(size_t)n * pwh + k / 8] >> (4 * (k % 8))) & 0xFu;
            int g = k / 128;
            uint32_t z = (zeros[(size_t)n * pzh + g / 8] >> (4 * (g % 8))) & 0xFu;
            float s = h2f(scales[(size_t)n * sh + g]);
            out[(size_t)n * K + k] = f2h(((float)q - (float)z) * s);
        }
    }
}

// ---------------------------------------------------------------- int4 dot
// Diagnostic switch (off by default): matrix-vector sums in double precision instead of the reference's fp32 order.
static int g_exact_sums = 0;
extern "C" void orc_set_exact_sums(int on) { g_exact_sums = on; }

// One output row of the fused unpack/dequant/dot, with the reference's
// lane structure: 32 lanes, lane L owns the uint4 (32 consecutive K
// elements) at dword ygq*128 + L*4 of each 1024-element tile; fp32
// w = (q - z) * scale; sum = fma(w, x, sum); then a shuffle-down tree over the
// 32 lane sums (gpu_kernels.h:179-218).
static float row_dot_int4_exact(int index, const h16* x, const QW& m, int K, int pzh, int sh, int pwh);

static float row_dot_int4(int index, const h16* x, const QW& m, int K, int pzh, int sh, int pwh) {
    if (g_exact_sums) return row_dot_int4_exact(index, x, m, K, pzh, sh, pwh);
    float lane_sum[32];
    for (int lane = 0; lane < 32; lane++) {
        float sum = 0.0f;
        for (int ygq = 0; ygq * 128 + lane * 4 < pwh; ygq++) {
            uint32_t packed_q_z = m.zeros[(size_t)index * pzh + ygq];
            const uint32_t* wts = &m.weight[(size_t)index * pwh + ygq * 128 + lane * 4];
            int group_y = ygq * 8 + lane / 4;
            float q_z = (float)((packed_q_z >> (4 * (lane / 4))) & 0xFu);
            float scale = h2f(m.scales[(size_t)index * sh + group_y]);
            int y_base = ygq * 1024 + lane * 32;
            for (int qi = 0; qi < 4; qi++) {
                int ys = y_base + qi * 8;
                if (ys < K) {
                    uint32_t packed_q_w = wts[qi];
                    for (int i = 0; i < 8; i++) {
                        float q_wt = (float)(packed_q_w & 0xFu);
                        float w = (q_wt - q_z) * scale;
                        sum = fmaf(w, h2f(x[ys + i]), sum);
                        packed_q_w >>= 4;
                    }
                }
            }
        }
        lane_sum[lane] = sum;
    }
    for (int off = 16; off > 0; off >>= 1)
        for (int i = 0; i < off; i++) lane_sum[i] += lane_sum[i + off];
    return lane_sum[0];
}

// The same row with every product and sum in double precision, rounded to fp32 once: the value that any fp32
// summation order approximates.  Used only to measure how far the reference's own summation order is from it.
static float row_dot_int4_exact(int index, const h16* x, const QW& m, int K, int pzh, int sh, int pwh) {
    (void)pwh;
    double sum = 0.0;
    for (int k = 0; k < K; k++) {
        const int g = k >> 7;
        const double q = (double)((m.weight[(size_t)index * pwh + (k >> 3)] >> (4 * (k & 7))) & 0xFu);
        const double z = (double)((m.zeros[(size_t)index * pzh + (g >> 3)] >> (4 * (g & 7))) & 0xFu);
        sum += (q - z) * (double)h2f(m.scales[(size_t)index * sh + g]) * (double)h2f(x[k]);
    }
    return (float)sum;
}

// out = half(W x [+ out/gpu_count]), optionally written at out + loff + pos*N
// (gpu_kernels.h:221-248; launcher llama2_q4.cu:367-376).  Returns -1 on the
// launcher's shape guard (K or N not a multiple of 8).
int orc_matvec_int4(uint16_t* out, const uint16_t* x, const uint32_t* weight, const uint32_t* zeros, const uint16_t* scales,
                    int K, int N, int accum, int gpu_count, int loff, const int* pPos) {
    if ((K & 7) || (N & 7)) return -1;
    const int pwh = packed_weight_height(K), sh = scales_height(K), pzh = packed_zeros_height(K);
    QW m = {weight, zeros, scales};
    uint16_t* output = out;
    if (loff != -1) output += (size_t)loff + (size_t)(*pPos) * N;
#pragma omp parallel for schedule(static)
    for (int index = 0; index < N; index++) {
        float sum = row_dot_int4(index, x, m, K, pzh, sh, pwh);
        if (accum) sum += h2f(output[index]) / (float)gpu_count;
        output[index] = f2h(sum);
    }
    return 0;
}

// Three GEMVs in one call: Q -> q, K and V -> cache rows at loff + pos*N
// (gpu_kernels.h:250-262; launcher llama2_q4.cu:378-391).
int orc_qkv_matvec(uint16_t* q, uint16_t* key_cache, uint16_t* value_cache, const uint16_t* x,
                   const uint32_t* qw, const uint32_t* qz, const uint16_t* qs,
                   const uint32_t* kw, const uint32_t* kz, const uint16_t* ks,
                   const uint32_t* vw, const uint32_t* vz, const uint16_t* vs,
                   int K, int N, int loff, const int* pPos) {
    if ((K & 7) || (N & 7)) return -1;
    orc_matvec_int4(q, x, qw, qz, qs, K, N, 0, 1, -1, NULL);
    orc_matvec_int4(key_cache, x, kw, kz, ks, K, N, 0, 1, loff, pPos);
    orc_matvec_int4(value_cache, x, vw, vz, vs, K, N, 0, 1, loff, pPos);
    return 0;
}

// hb = half(silu(g) * u), g and u both kept in fp32
// (gpu_kernels.h:264-283; launcher llama2_q4.cu:393-404).
int orc_ffn_matvec_silu(uint16_t* out, const uint16_t* x,
                        const uint32_t* gw, const uint32_t* gz, const uint16_t* gs,
                        const uint32_t* uw, const uint32_t* uz, const uint16_t* us, int K, int N) {
    if ((K & 7) || (N & 7)) return -1;
    const int pwh = packed_weight_height(K), sh = scales_height(K), pzh = packed_zeros_height(K);
    QW g = {gw, gz, gs}, u = {uw, uz, us};
#pragma omp parallel for schedule(static)
    for (int index = 0; index < N; index++) {
        float g_val = row_dot_int4(index, x, g, K, pzh, sh, pwh);
        float u_val = row_dot_int4(index, x, u, K, pzh, sh, pwh);
        float val = g_val;
        val *= 1.0f / (1.0f + expf(-val));
        val *= u_val;
        out[index] = f2h(val);
    }
    return 0;
}

// ---------------------------------------------------------------- fp16 ops
// x[i] = table[tokens[*pPos]*dim + i]  (gpu_kernels.h:61-69).
void orc_embed(uint16_t* x, const uint16_t* table, int dim, const int* tokens, const int* pPos) {
    int token = tokens[*pPos];
    memcpy(x, table + (size_t)token * dim, (size_t)dim * sizeof(uint16_t));
}

// Sum of 1024 per-thread partials the way a 1024-thread block reduction does
// it: a shuffle tree inside each group of 32, then the 32 group totals added
// in order (the shape of CUB's warp-reductions block reduce; order unpinned).
static float block_sum_1024(const float* part) {
    float warp_tot[32];
    for (int w = 0; w < 32; w++) {
        float l[32];
        for (int i = 0; i < 32; i++) l[i] = part[w * 32 + i];
        for (int off = 16; off > 0; off >>= 1)
            for (int i = 0; i < off; i++) l[i] += l[i + off];
        warp_tot[w] = l[0];
    }
    float s = warp_tot[0];
    for (int w = 1; w < 32; w++) s += warp_tot[w];
    return s;
}

// o = half(x * (ss * w)), ss = 1/sqrt(mean(x^2) + 1e-5), fp32 math; in place
// allowed (gpu_kernels.h:72-105; launcher llama2_q4.cu:347-350).
void orc_rmsnorm(uint16_t* o, const uint16_t* x, const uint16_t* weight, int size) {
    float part[1024];
    int ept = div_up(size, 1024);
    for (int t = 0; t < 1024; t++) {
        float ss = 0.0f;
        for (int i = 0; i < ept; i++) {
            int idx = t + i * 1024;
            if (idx < size) {
                float v = h2f(x[idx]);
                ss = fmaf(v, v, ss);
            }
        }
        part[t] = ss;
    }
    float ss = block_sum_1024(part);
    ss /= (float)size;
    ss += 1e-5f;
    ss = 1.0f / sqrtf(ss);
    for (int i = 0; i < size; i++) {
        float val = h2f(x[i]);
        val *= ss * h2f(weight[i]);
        o[i] = f2h(val);
    }
}

// logits[r] = half(alpha * sum_j w[r*n + j] * x[j]), 32 lanes each taking 8
// consecutive halves per 256-element step, fp32, then the shuffle tree
// (gpu_kernels.h:117-147; launcher llama2_q4.cu:357-365, alpha = 1).
int orc_matvec_f16(uint16_t* out, const uint16_t* x, const uint16_t* w, int n, int d) {
    if ((n & 7) || (d & 7)) return -1;
    int serialLoads = div_up(div_up(n, 32), 8);
#pragma omp parallel for schedule(static)
    for (int index = 0; index < d; index++) {
        if (g_exact_sums) {
            double acc = 0.0;
            for (int j = 0; j < n; j++) acc += (double)h2f(w[(size_t)index * n + j]) * (double)h2f(x[j]);
            out[index] = f2h((float)acc);
            continue;
        }
        float lane_sum[32];
        for (int lane = 0; lane < 32; lane++) {
            float sum = 0.0f;
            for (int i = 0; i < serialLoads; i++) {
                int j = (i * 32 + lane) * 8;
                if (j < n)
                    for (int el = 0; el < 8; el++)
                        sum = fmaf(h2f(w[(size_t)index * n + j + el]), h2f(x[j + el]), sum);
            }
            lane_sum[lane] = sum;
        }
        for (int off = 16; off > 0; off >>= 1)
            for (int i = 0; i < off; i++) lane_sum[i] += lane_sum[i + off];
        float sum = lane_sum[0] * 1.0f;
        out[index] = f2h(sum);
    }
    return 0;
}

// Rotate-half RoPE on q (all heads) and on the K row just written to the cache
// at loff + pos*n_kv_heads*head, pairs (i, i + head/2), fp32 math, fp16 store
// (gpu_kernels.h:340-363; launcher llama2_q4.cu:406-408).
void orc_rope(uint16_t* sq, uint16_t* sk_base, int num_heads, int num_kv_heads, int head_size, const int* pPos, int loff, float rope_theta) {
    int pos = *pPos;
    for (int h = 0; h < num_heads; h++) {
        uint16_t* q = sq + (size_t)h * head_size;
        for (int i = 0; i < head_size / 2; i++) {
            int head_dim = (i * 2) % head_size;
            float freq = 1.0f / powf(rope_theta, head_dim / (float)head_size);
            float val = pos * freq;
            float fcr = cosf(val);
            float fci = sinf(val);
            float q0 = h2f(q[i]);
            float q1 = h2f(q[i + head_size / 2]);
            q[i] = f2h(q0 * fcr - q1 * fci);
            q[i + head_size / 2] = f2h(q0 * fci + q1 * fcr);
            if (h < num_kv_heads) {
                uint16_t* k = sk_base + (size_t)loff + (size_t)pos * num_kv_heads * head_size + (size_t)h * head_size;
                float k0 = h2f(k[i]);
                float k1 = h2f(k[i + head_size / 2]);
                k[i] = f2h(k0 * fcr - k1 * fci);
                k[i + head_size / 2] = f2h(k0 * fci + k1 * fcr);
            }
        }
    }
}

// Batch-1 attention over the fp16 KV cache of one layer
// (llama2_q4.cu:410-427 = mat_vec_kernel_simple gpu_kernels.h:150-176,
//  softmax_kernel :365-409, vec_mat_kernel :287-337).
// key_cache/value_cache point at the layer's (seq_len, kv_dim) block; att is
// a scratch of n_heads*(pos+1) halves with COMPACT row stride pos+1.
// Rounding points: scores -> fp16, probabilities -> fp16, output -> fp16.
void orc_attention(uint16_t* output, const uint16_t* q, const uint16_t* key_cache, const uint16_t* value_cache, uint16_t* att,
                   int num_heads, int head_size, int kv_mul, const int* pPos) {
    const int size = *pPos + 1;
    const int dim = head_size * num_heads;
    const int row_stride = dim / kv_mul;
    const float alpha = (float)(1.0 / sqrt((double)head_size));
#pragma omp parallel for schedule(dynamic, 1)
    for (int h = 0; h < num_heads; h++) {
        const uint16_t* qh = q + (size_t)h * head_size;
        const uint16_t* kh = key_cache + (size_t)(h / kv_mul) * head_size;
        const uint16_t* vh = value_cache + (size_t)(h / kv_mul) * head_size;
        uint16_t* a = att + (size_t)h * size;
        // 1. scores: lane j sums elements j, j+32, ... then the shuffle tree
        int serial = div_up(head_size, 32);
        for (int t = 0; t < size; t++) {
            float lane_sum[32];
            for (int lane = 0; lane < 32; lane++) {
                float sum = 0.0f;
                for (int i = 0; i < serial; i++) {
                    int j = i * 32 + lane;
                    if (j < head_size) sum = fmaf(h2f(kh[(size_t)t * row_stride + j]), h2f(qh[j]), sum);
                }
                lane_sum[lane] = sum;
            }
            for (int off = 16; off > 0; off >>= 1)
                for (int i = 0; i < off; i++) lane_sum[i] += lane_sum[i + off];
            a[t] = f2h(lane_sum[0] * alpha);
        }
        // 2. softmax in fp32 over fp16 scores; the kernel seeds idle lanes' max
        // with 0, so the subtracted maximum is max(true max, 0) when size < 1024
        float* e = (float*)malloc((size_t)size * sizeof(float));
        float max_val = (size < 1024) ? 0.0f : -INFINITY;
        for (int t = 0; t < size; t++) {
            float v = h2f(a[t]);
            if (v > max_val) max_val = v;
        }
        float part[1024];
        for (int t = 0; t < 1024; t++) part[t] = 0.0f;
        for (int t = 0; t < size; t++) {
            e[t] = expf(h2f(a[t]) - max_val);
            part[t & 1023] += e[t];
        }
        float sum = block_sum_1024(part);
        for (int t = 0; t < size; t++) a[t] = f2h(e[t] / sum);
        free(e);
        // 3. out[n] = sum_k att[k] * V[k][n]: lane L takes k = 32e + L, then the tree
        for (int n = 0; n < head_size; n++) {
            float lane_sum[32];
            for (int lane = 0; lane < 32; lane++) {
                float s = 0.0f;
                for (int k = lane; k < size; k += 32)
                    s = fmaf(h2f(vh[(size_t)k * row_stride + n]), h2f(a[k]), s);
                lane_sum[lane] = s;
            }
            for (int off = 16; off > 0; off >>= 1)
                for (int i = 0; i < off; i++) lane_sum[i] += lane_sum[i + off];
            output[(size_t)h * head_size + n] = f2h(lane_sum[0]);
        }
    }
}

// Greedy sampler: index of the maximum fp16 logit compared as float, LOWEST
// index on ties (the reference's tie winner is racy, gpu_kernels.h:482-487);
// then p = *pos + 1; if (write_token) tokens[p] = argmax; *pos_host = *pos_dev = p
// (gpu_kernels.h:456-501; sampler.h:77-84).  Returns the argmax.
int orc_argmax_advance(const uint16_t* logits, int size, int* tokens, int* pos_host, int* pos_dev, int write_token) {
    float best = -INFINITY;
    int best_i = 0;
    for (int i = 0; i < size; i++) {
        float v = h2f(logits[i]);
        if (v > best) { best = v; best_i = i; }
    }
    int p = *pos_host + 1;
    if (write_token) tokens[p] = best_i;
    *pos_host = p;
    if (pos_dev) *pos_dev = p;
    return best_i;
}

// ---------------------------------------------------------------- temperature / top-p sampling
// xorshift* and the [0,1) float drawn from it (sampler.h:65-74).
float orc_random_f32(unsigned long long* state) {
    *state ^= *state >> 12;
    *state ^= *state << 25;
    *state ^= *state >> 27;
    unsigned int r = (unsigned int)((*state * 0x2545F4914F6CDD1Dull) >> 32);
    return (r >> 8) / 16777216.0f;
}

// softmax_logits_kernel (gpu_kernels.h:507-557), in place: l = half(l / T); v = expf(l - max) stored as half and
// summed unrounded in fp32; p = half(float(half v) / sum).  The reference sums with cub::BlockReduce over 1024
// threads (order unpinned); the order fixed here: thread t adds elements t, t+1024, ... in index order, the 1024
// partials are then added as a balanced pairwise tree.
void orc_softmax_logits(uint16_t* logits, int size, float temperature) {
    for (int t = 0; t < size; t++) logits[t] = f2h(h2f(logits[t]) / temperature);
    float max_val = -3.402823466e+38f;
    for (int t = 0; t < size; t++) max_val = fmaxf(max_val, h2f(logits[t]));
    float part[1024];
    for (int t = 0; t < 1024; t++) part[t] = 0.0f;
    for (int t = 0; t < 1024; t++)
        for (int i = t; i < size; i += 1024) {
            float v = expf(h2f(logits[i]) - max_val);
            logits[i] = f2h(v);
            part[t] += v;
        }
    for (int n = 1024; n > 1; n >>= 1)
        for (int i = 0; i < n / 2; i++) part[i] = part[2 * i] + part[2 * i + 1];
    const float sum = part[0];
    for (int t = 0; t < size; t++) logits[t] = f2h(h2f(logits[t]) / sum);
}

// The reference's sort + inclusive prefix sum + sample_top_p_kernel (sampler.h:94-115, gpu_kernels.h:562-592),
// written out step by step: sorted != 0 orders (probability, index) pairs by descending probability, stable (the
// radix sort is); the prefix sum is exact (fp16 values are multiples of 2^-24, summed as integers) and rounded to fp16
// once, where CUB's scan adds in fp16 in an order of its own ("parity unpinned"); the answer is the index at the first
// position whose rounded prefix is >= threshold, position size-1 when none is.  Then the position advance of
// gpu_kernels.h:582-591.  Returns the token.
static uint64_t prob_units(uint16_t h) {
    const uint32_t e = h >> 10, m = h & 0x3FFu;
    return e == 0 ? (uint64_t)m : ((uint64_t)(m | 0x400u) << (e - 1));
}
int orc_sample_top_p(const uint16_t* probs, int size, float threshold, int sorted, int* tokens, int* pos_host, int* pos_dev) {
    int* idx = (int*)malloc(sizeof(int) * (size_t)size);
    for (int i = 0; i < size; i++) idx[i] = i;
    if (sorted) {
        // stable insertion-free sort: counting sort on the 16-bit key, descending, ties in index order
        int* count = (int*)calloc(65537, sizeof(int));
        for (int i = 0; i < size; i++) count[65535 - probs[i]]++;
        int run = 0;
        for (int k = 0; k < 65536; k++) { int c = count[k]; count[k] = run; run += c; }
        for (int i = 0; i < size; i++) idx[count[65535 - probs[i]]++] = i;
        free(count);
    }
    int pick = size - 1;
    uint64_t run = 0;
    for (int t = 0; t < size; t++) {
        run += prob_units(probs[idx[t]]);
        // exact value run * 2^-24 -> fp16 (one rounding, nearest even) -> float, as the kernel's (float)prefix[t]
        const double exact = (double)run * 5.9604644775390625e-08;
        const float rounded = h2f(f2h((float)exact));
        // (float)exact is itself exact here only when run has <= 24 significant bits; round from the integer instead
        float pref;
        if (run < (1ull << 24)) {
            pref = rounded;
        } else {
            const int e = 63 - __builtin_clzll(run);
            const int shift = e - 10;
            uint64_t mant = run >> shift;
            const uint64_t rem = run & ((1ull << shift) - 1ull), half_ulp = 1ull << (shift - 1);
            if (rem > half_ulp || (rem == half_ulp && (mant & 1ull))) mant++;
            pref = ldexpf((float)mant, shift - 24);
        }
        if (pref >= threshold) { pick = t; break; }
    }
    const int token = idx[pick];
    free(idx);
    int p = *pos_host + 1;
    tokens[p] = token;
    *pos_host = p;
    if (pos_dev) *pos_dev = p;
    return token;
}

// The same selection with the prefix sum ADDED IN fp16, the arithmetic cub::DeviceScan::InclusiveSum performs on half
// data (sampler.h:107-111): every partial sum is rounded to fp16, so the result depends on the order of the additions,
// which CUB chooses and the reference does not fix.  Two orders a CUB scan can take are written out, to measure how
// far the choice matters (neither is claimed to be the reference's):
//   mode 0  strictly sequential: prefix[t] = half(prefix[t-1] + p[t]);
//   mode 1  tiled, `threads` x `items` elements per tile: every thread adds up its `items` consecutive elements, the
//           thread totals are scanned across each 32-lane group in log steps (lane i takes lane i - off, off = 1, 2,
//           4, 8, 16), the group totals and the tile totals are carried forward sequentially, and each thread then
//           scans its elements again starting from the sum of everything before them.
// Returns the picked token; no position is advanced.
static inline uint16_t hadd(uint16_t a, uint16_t b) { return f2h(h2f(a) + h2f(b)); }  // fp32 holds the exact sum's rounding: innocuous
int orc_top_p_pick_fp16_scan(const uint16_t* probs, int size, float threshold, int sorted, int mode, int threads, int items) {
    int* idx = (int*)malloc(sizeof(int) * (size_t)size);
    for (int i = 0; i < size; i++) idx[i] = i;
    if (sorted) {
        int* count = (int*)calloc(65537, sizeof(int));
        for (int i = 0; i < size; i++) count[65535 - probs[i]]++;
        int run = 0;
        for (int k = 0; k < 65536; k++) { int c = count[k]; count[k] = run; run += c; }
        for (int i = 0; i < size; i++) idx[count[65535 - probs[i]]++] = i;
        free(count);
    }
    uint16_t* prefix = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)size);
    if (mode == 0) {
        uint16_t run = 0;
        for (int t = 0; t < size; t++) { run = t ? hadd(run, probs[idx[t]]) : probs[idx[t]]; prefix[t] = run; }
    } else {
        const int tile = threads * items;
        uint16_t* total = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)threads);
        uint16_t* excl = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)threads);
        char* has = (char*)malloc((size_t)threads);  // thread owns at least one element
        uint16_t carry = 0;  // sum of all earlier tiles
        bool have_carry = false;
        for (int base = 0; base < size; base += tile) {
            for (int th = 0; th < threads; th++) {
                const int b = base + th * items, e = b + items < size ? b + items : size;
                has[th] = b < size;
                uint16_t r = 0;
                for (int t = b; t < e; t++) r = t == b ? probs[idx[t]] : hadd(r, probs[idx[t]]);
                total[th] = r;
            }
            // inclusive scan of the thread totals inside each group of 32, log steps
            for (int g = 0; g < threads; g += 32) {
                const int n = threads - g < 32 ? threads - g : 32;
                for (int off = 1; off < 32; off <<= 1) {
                    uint16_t prev[32];
                    for (int l = 0; l < n; l++) prev[l] = total[g + l];
                    for (int l = off; l < n; l++)
                        if (has[g + l]) total[g + l] = hadd(prev[l - off], prev[l]);
                }
            }
            // exclusive prefix of every thread: earlier tiles + earlier groups + earlier lanes of its group
            uint16_t groups = carry;
            bool have_groups = have_carry;
            for (int g = 0; g < threads; g += 32) {
                const int n = threads - g < 32 ? threads - g : 32;
                for (int l = 0; l < n; l++) {
                    if (l == 0) excl[g] = groups;
                    else excl[g + l] = have_groups ? hadd(groups, total[g + l - 1]) : total[g + l - 1];
                }
                int last = -1;
                for (int l = 0; l < n; l++) if (has[g + l]) last = l;
                if (last >= 0) { groups = have_groups ? hadd(groups, total[g + last]) : total[g + last]; have_groups = true; }
            }
            for (int th = 0; th < threads; th++) {
                const int b = base + th * items, e = b + items < size ? b + items : size;
                const bool seeded = (th % 32 != 0) || (th >= 32) || have_carry;
                uint16_t r = excl[th];
                for (int t = b; t < e; t++) { r = (t == b && !seeded) ? probs[idx[t]] : hadd(r, probs[idx[t]]); prefix[t] = r; }
            }
            carry = groups;
            have_carry = true;
        }
        free(total); free(excl); free(has);
    }
    int pick = size - 1;
    for (int t = 0; t < size; t++)
        if (h2f(prefix[t]) >= threshold) { pick = t; break; }
    const int token = idx[pick];
    free(prefix);
    free(idx);
    return token;
}

// ---------------------------------------------------------------- model image
// Config = the 32-byte file header (common.h:15-24).
typedef struct {
    int dim, hidden_dim, n_layers, n_heads, n_kv_heads, vocab_size, seq_len;
    float rope_theta;
} OrcConfig;

typedef struct {
    QW q, k, v, o, up, gate, down;
    const h16* rms_att;
    const h16* rms_ffn;
} OrcLayer;

typedef struct {
    OrcConfig cfg;
    const h16* embed;
    const h16* wcls;
    const h16* rms_final;
    OrcLayer* layers;
    // run state (common.h:62-78)
    h16 *x, *xb, *hb, *q, *att, *logits, *key_cache, *value_cache;
    int pos;          // "device" position
    int shared_pos;   // SharedData.pos
    int* tokens;      // SharedData.tokens
} OrcModel;

static const uint8_t* take_qw(QW* w, const uint8_t* p, int K, int N) {
    // (weight, zeros, scales) back to back, sizes as in llama2_q4.cu:210-218
    size_t wb = (size_t)packed_weight_height(K) * N * 4;
    size_t zb = (size_t)packed_zeros_height(K) * N * 4;
    size_t sb = (size_t)scales_height(K) * N * 2;
    w->weight = (const uint32_t*)p; p += wb;
    w->zeros = (const uint32_t*)p; p += zb;
    w->scales = (const h16*)p; p += sb;
    return p;
}

// Byte size of a model file for a config: header, embed, lm_head, final norm,
// per layer {q,k,v,o,up,gate,down, input norm, post-attention norm}
// (llama2_q4.cu:220-246; weight_packer.cpp:256-292).
size_t orc_model_file_bytes(const OrcConfig* c) {
    int kv_dim = (c->dim * c->n_kv_heads) / c->n_heads;
    auto qw = [](int K, int N) {
        return (size_t)packed_weight_height(K) * N * 4 + (size_t)packed_zeros_height(K) * N * 4 + (size_t)scales_height(K) * N * 2;
    };
    size_t b = 32 + 2 * (size_t)c->vocab_size * c->dim * 2 + (size_t)c->dim * 2;
    size_t layer = 2 * qw(c->dim, c->dim) + 2 * qw(c->dim, kv_dim) + 2 * qw(c->dim, c->hidden_dim) + qw(c->hidden_dim, c->dim) + 2 * (size_t)c->dim * 2;
    return b + layer * c->n_layers;
}

// Map a model file image held in memory (the image must outlive the model).
void* orc_model_open(const void* image, size_t bytes) {
    if (bytes < 32) return NULL;
    OrcModel* m = (OrcModel*)calloc(1, sizeof(OrcModel));
    memcpy(&m->cfg, image, 32);
    const OrcConfig* c = &m->cfg;
    if (orc_model_file_bytes(c) > bytes) { free(m); return NULL; }
    int kv_dim = (c->dim * c->n_kv_heads) / c->n_heads;
    const uint8_t* p = (const uint8_t*)image + 32;
    m->embed = (const h16*)p; p += (size_t)c->vocab_size * c->dim * 2;
    m->wcls = (const h16*)p; p += (size_t)c->vocab_size * c->dim * 2;
    m->rms_final = (const h16*)p; p += (size_t)c->dim * 2;
    m->layers = (OrcLayer*)calloc(c->n_layers, sizeof(OrcLayer));
    for (int l = 0; l < c->n_layers; l++) {
        OrcLayer* L = &m->layers[l];
        p = take_qw(&L->q, p, c->dim, c->dim);
        p = take_qw(&L->k, p, c->dim, kv_dim);
        p = take_qw(&L->v, p, c->dim, kv_dim);
        p = take_qw(&L->o, p, c->dim, c->dim);
        p = take_qw(&L->up, p, c->dim, c->hidden_dim);
        p = take_qw(&L->gate, p, c->dim, c->hidden_dim);
        p = take_qw(&L->down, p, c->hidden_dim, c->dim);
        L->rms_att = (const h16*)p; p += (size_t)c->dim * 2;
        L->rms_ffn = (const h16*)p; p += (size_t)c->dim * 2;
    }
    // run state (llama2_q4.cu:62-74)
    m->x = (h16*)calloc(c->dim, 2);
    m->xb = (h16*)calloc(c->dim, 2);
    m->q = (h16*)calloc(c->dim, 2);
    m->hb = (h16*)calloc(c->hidden_dim, 2);
    m->att = (h16*)calloc((size_t)c->n_heads * c->seq_len, 2);
    m->logits = (h16*)calloc(c->vocab_size, 2);
    m->key_cache = (h16*)calloc((size_t)c->n_layers * c->seq_len * kv_dim, 2);
    m->value_cache = (h16*)calloc((size_t)c->n_layers * c->seq_len * kv_dim, 2);
    m->tokens = (int*)calloc((size_t)c->seq_len + 8, sizeof(int));
    return m;
}

void orc_model_close(void* mp) {
    OrcModel* m = (OrcModel*)mp;
    if (!m) return;
    free(m->layers); free(m->x); free(m->xb); free(m->q); free(m->hb); free(m->att);
    free(m->logits); free(m->key_cache); free(m->value_cache); free(m->tokens);
    free(m);
}

// Start a sequence: position 0, prompt copied into the shared token list
// (llama2_q4.cu:703-705).
void orc_model_reset(void* mp, const int* prompt, int n_prompt) {
    OrcModel* m = (OrcModel*)mp;
    m->pos = 0;
    m->shared_pos = 0;
    memcpy(m->tokens, prompt, (size_t)n_prompt * sizeof(int));
}

// Start at a later position with a caller-filled KV cache (benchmark config
// with a pre-filled context): the token consumed next is tokens[pos].
void orc_model_set_pos(void* mp, int pos, int token) {
    OrcModel* m = (OrcModel*)mp;
    m->pos = pos;
    m->shared_pos = pos;
    m->tokens[pos] = token;
}

uint16_t* orc_model_buffer(void* mp, const char* name) {
    OrcModel* m = (OrcModel*)mp;
    if (!strcmp(name, "x")) return m->x;
    if (!strcmp(name, "xb")) return m->xb;
    if (!strcmp(name, "q")) return m->q;
    if (!strcmp(name, "hb")) return m->hb;
    if (!strcmp(name, "att")) return m->att;
    if (!strcmp(name, "logits")) return m->logits;
    if (!strcmp(name, "key_cache")) return m->key_cache;
    if (!strcmp(name, "value_cache")) return m->value_cache;
    return NULL;
}
int* orc_model_tokens(void* mp) { return ((OrcModel*)mp)->tokens; }
int orc_model_pos(void* mp) { return ((OrcModel*)mp)->shared_pos; }

// One token through the network, single GPU: the reference's schedule with
// gpu_count = 1 (llama2_q4.cu:430-538), then the greedy sampler
// (llama2_q4.cu:590; sampler.h:81-84).  Returns the argmax token.
int orc_model_forward(void* mp, int gen_token) {
    OrcModel* m = (OrcModel*)mp;
    const OrcConfig* p = &m->cfg;
    const int dim = p->dim, hidden_dim = p->hidden_dim;
    const int head_size = dim / p->n_heads;
    const int kv_dim = (p->dim * p->n_kv_heads) / p->n_heads;
    const int kv_mul = p->n_heads / p->n_kv_heads;
    const int* pPos = &m->pos;

    orc_embed(m->x, m->embed, dim, m->tokens, pPos);
    for (int l = 0; l < p->n_layers; l++) {
        const OrcLayer* L = &m->layers[l];
        orc_rmsnorm(m->xb, m->x, L->rms_att, dim);
        int loff = l * p->seq_len * kv_dim;
        if (dim == kv_dim) {
            orc_qkv_matvec(m->q, m->key_cache, m->value_cache, m->xb,
                           L->q.weight, L->q.zeros, L->q.scales, L->k.weight, L->k.zeros, L->k.scales,
                           L->v.weight, L->v.zeros, L->v.scales, dim, dim, loff, pPos);
        } else {
            orc_matvec_int4(m->q, m->xb, L->q.weight, L->q.zeros, L->q.scales, dim, dim, 0, 1, -1, NULL);
            orc_matvec_int4(m->key_cache, m->xb, L->k.weight, L->k.zeros, L->k.scales, dim, kv_dim, 0, 1, loff, pPos);
            orc_matvec_int4(m->value_cache, m->xb, L->v.weight, L->v.zeros, L->v.scales, dim, kv_dim, 0, 1, loff, pPos);
        }
        orc_rope(m->q, m->key_cache, p->n_heads, p->n_kv_heads, head_size, pPos, loff, p->rope_theta);
        orc_attention(m->xb, m->q, m->key_cache + loff, m->value_cache + loff, m->att, p->n_heads, head_size, kv_mul, pPos);
        orc_matvec_int4(m->x, m->xb, L->o.weight, L->o.zeros, L->o.scales, dim, dim, 1, 1, -1, NULL);
        orc_rmsnorm(m->xb, m->x, L->rms_ffn, dim);
        orc_ffn_matvec_silu(m->hb, m->xb, L->gate.weight, L->gate.zeros, L->gate.scales,
                            L->up.weight, L->up.zeros, L->up.scales, dim, hidden_dim);
        orc_matvec_int4(m->x, m->hb, L->down.weight, L->down.zeros, L->down.scales, hidden_dim, dim, 1, 1, -1, NULL);
    }
    orc_rmsnorm(m->x, m->x, m->rms_final, dim);
    orc_matvec_f16(m->logits, m->x, m->wcls, dim, p->vocab_size);
    return orc_argmax_advance(m->logits, p->vocab_size, m->tokens, &m->shared_pos, &m->pos, gen_token);
}

// The decode loop of generate_thread (llama2_q4.cu:697-735) without printing:
// runs until `steps` positions or EOS (token 2, unless ignore_eos), returns the
// final pos.  tokens[] (prompt then generated) can be read with
// orc_model_tokens().  If logits_out != NULL it receives vocab_size halves per
// executed forward pass.
int orc_generate(void* mp, const int* prompt, int n_prompt, int steps, int ignore_eos, uint16_t* logits_out) {
    OrcModel* m = (OrcModel*)mp;
    orc_model_reset(mp, prompt, n_prompt);
    int pos = 0;
    int next;
    while (pos < steps) {
        orc_model_forward(mp, pos >= n_prompt - 1);
        if (logits_out) memcpy(logits_out + (size_t)pos * m->cfg.vocab_size, m->logits, (size_t)m->cfg.vocab_size * 2);
        // the reference reads tokens[pos] (written one iteration earlier) after
        // launching this iteration; on the CPU everything is already complete
        if (pos > 0) {
            next = m->tokens[pos];
            if (next >= m->cfg.vocab_size) next = 0;
            if (next == 2 && !ignore_eos) break;
        }
        pos++;
    }
    return pos;
}

}  // extern "C"
