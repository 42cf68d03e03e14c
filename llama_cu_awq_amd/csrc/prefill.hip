// Multi-token prefill: every projection of M prompt tokens as one int4-weight x fp16-activation GEMM on the
// fp16 matrix cores (weights dequantised into LDS), with batched RMSNorm / RoPE and causal attention around it.
//
// The reference has no such path: it feeds prompt tokens through its matrix-VECTOR kernels one at a time
// (llama2_q4.cu:716-735).  The contract here is therefore the result of that token-by-token run: after
// awq_transformer_prefill(t, M, gen) the KV cache rows, the logits of the last token, the token list and the
// position equal what M calls of awq_transformer_forward would leave (same rounding points: q/k/v, scores,
// probabilities, attention output, residual stream and hidden vector are rounded to fp16 where the reference
// kernels round them; only fp32 summation order differs).
//
// Dequantised weights are bit-exact: w16 = half_rne((q - z) * s) computed as an exact fp16 integer (q - z)
// times the fp16 scale in one rounding.
#include <string.h>

#include "common.hpp"

typedef _Float16 h16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

namespace pf {

constexpr int BM = 128;      // tokens per tile
constexpr int BN = 128;      // weight rows per tile
constexpr int BK = 32;       // K per step = one 16-byte packed chunk per weight row
constexpr int LDS_ROW = 40;  // halves per LDS tile row (32 + 8 padding)

enum Epi { EPI_STORE = 0, EPI_RESID = 1, EPI_QKV = 2, EPI_FFN = 3 };

struct GemmParams {
    const uint16_t* A;  // [M][lda] fp16 activations
    int lda, M, K;
    const uint32_t* w[3];
    const uint32_t* z[3];
    const uint16_t* s[3];
    int N[3];  // rows of each matrix
    int C, pzh, sh;
    int epi;
    uint16_t* out[3];
    long long ldo[3];       // output row stride in elements
    long long out_off[3];   // element offset of output row 0 (KV cache: loff + pos0 * kv_dim)
};

// (h0,h1)(h2,h3)(h4,h5)(h6,h7) -> (h0,h4)(h1,h5)(h2,h6)(h3,h7): the order in which one packed dword unpacks
__device__ __forceinline__ u32x4 permute8(const u32x4 v) {
    u32x4 o;
    o[0] = __builtin_amdgcn_perm(v[2], v[0], 0x05040100u);
    o[1] = __builtin_amdgcn_perm(v[2], v[0], 0x07060302u);
    o[2] = __builtin_amdgcn_perm(v[3], v[1], 0x05040100u);
    o[3] = __builtin_amdgcn_perm(v[3], v[1], 0x07060302u);
    return o;
}

// 8 nibbles of one dword -> 8 dequantised fp16 weights in the order (w0,w4)(w1,w5)(w2,w6)(w3,w7).
__device__ __forceinline__ u32x4 dequant8(uint32_t d, uint32_t z, h16x2 s2) {
    const h16x2 zlo = as_h2(0xE400E400u | (z * 0x00010001u));  // -(1024 + z)
    const h16x2 zhi = as_h2(0xD400D400u | (z * 0x00100010u));  // -(64 + z)
    const h16x2 sixteenth = {(h16_t)0.0625f, (h16_t)0.0625f};
    const uint32_t d8 = d >> 8;
    const h16x2 t0 = as_h2((d & 0x000F000Fu) | 0x64006400u) + zlo;                                      // exact q - z
    const h16x2 t1 = __builtin_elementwise_fma(as_h2((d & 0x00F000F0u) | 0x64006400u), sixteenth, zhi);  // exact
    const h16x2 t2 = as_h2((d8 & 0x000F000Fu) | 0x64006400u) + zlo;
    const h16x2 t3 = __builtin_elementwise_fma(as_h2((d8 & 0x00F000F0u) | 0x64006400u), sixteenth, zhi);
    return u32x4{as_u32(t0 * s2), as_u32(t1 * s2), as_u32(t2 * s2), as_u32(t3 * s2)};  // one rounding each
}

// Which matrix / row a tile row maps to, and where its output goes.
struct TileMap {
    int mat[2];   // matrix of tile rows [0,64) and [64,128)
    int row0[2];  // first matrix row of each half
};

__device__ __forceinline__ TileMap tile_map(const GemmParams& p, int tile) {
    TileMap t;
    if (p.epi == EPI_FFN) {  // 64 gate rows + the 64 up rows of the same indices
        t.mat[0] = 0;
        t.mat[1] = 1;
        t.row0[0] = t.row0[1] = tile * 64;
    } else {
        int m = 0, tt = tile;
        if (p.epi == EPI_QKV) {
            const int t0 = p.N[0] / BN, t1 = p.N[1] / BN;
            if (tt >= t0 + t1) {
                m = 2;
                tt -= t0 + t1;
            } else if (tt >= t0) {
                m = 1;
                tt -= t0;
            }
        }
        t.mat[0] = t.mat[1] = m;
        t.row0[0] = tt * BN;
        t.row0[1] = tt * BN + 64;
    }
    return t;
}

__global__ __launch_bounds__(256) void gemm_int4_kernel(const GemmParams p) {
    __shared__ __attribute__((aligned(16))) uint16_t As[2][BM * LDS_ROW];
    __shared__ __attribute__((aligned(16))) uint16_t Ws[2][BN * LDS_ROW];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int m0 = blockIdx.x * BM;
    const TileMap tm = tile_map(p, blockIdx.y);

    // loader role: 2 threads per tile row, 16 K elements each
    const int lrow = tid >> 1, lhalf = tid & 1;
    const int am = m0 + lrow;
    const bool a_ok = am < p.M;
    const uint16_t* a_ptr = p.A + (size_t)(a_ok ? am : 0) * p.lda + lhalf * 16;
    const int whalf = lrow >> 6;
    const int wmat = tm.mat[whalf];
    const int wrow = tm.row0[whalf] + (lrow & 63);
    const uint32_t* wbase = (wmat == 0 ? p.w[0] : (wmat == 1 ? p.w[1] : p.w[2])) + (size_t)wrow * (p.C * 4) + lhalf * 2;
    const uint32_t* zbase = (wmat == 0 ? p.z[0] : (wmat == 1 ? p.z[1] : p.z[2])) + (size_t)wrow * p.pzh;
    const uint16_t* sbase = (wmat == 0 ? p.s[0] : (wmat == 1 ? p.s[1] : p.s[2])) + (size_t)wrow * p.sh;

    f32x16 acc[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 16; j++) acc[i][j] = 0.0f;

    const int nsteps = p.K / BK;
    u32x4 ra0, ra1;
    u32x2 rw;
    uint32_t rz;
    uint16_t rs;
    auto gload = [&](int step) {
        const int k0 = step * BK;
        if (a_ok) {
            ra0 = *reinterpret_cast<const u32x4*>(a_ptr + k0);
            ra1 = *reinterpret_cast<const u32x4*>(a_ptr + k0 + 8);
        } else {
            ra0 = ra1 = u32x4{0u, 0u, 0u, 0u};
        }
        rw = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(wbase + (size_t)step * 4));
        const int g = step >> 2;
        rz = (zbase[g >> 3] >> (4 * (g & 7))) & 0xFu;
        rs = sbase[g];
    };
    auto lstore = [&](int buf) {
        u32x4* ad = reinterpret_cast<u32x4*>(&As[buf][lrow * LDS_ROW + lhalf * 16]);
        ad[0] = permute8(ra0);
        ad[1] = permute8(ra1);
        const h16_t sh = __builtin_bit_cast(h16_t, rs);
        const h16x2 s2 = {sh, sh};
        u32x4* wd = reinterpret_cast<u32x4*>(&Ws[buf][lrow * LDS_ROW + lhalf * 16]);
        wd[0] = dequant8(rw[0], rz, s2);
        wd[1] = dequant8(rw[1], rz, s2);
    };

    gload(0);
    lstore(0);
    __syncthreads();
    for (int step = 0; step < nsteps; step++) {
        const int buf = step & 1;
        if (step + 1 < nsteps) gload(step + 1);
        // wave w: token rows 32w..32w+31 against all 128 weight rows
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
            const int koff = ks * 16 + (lane >> 5) * 8;
            const h16x8 af = *reinterpret_cast<const h16x8*>(&As[buf][(wave * 32 + (lane & 31)) * LDS_ROW + koff]);
#pragma unroll
            for (int nb = 0; nb < 4; nb++) {
                const h16x8 bf = *reinterpret_cast<const h16x8*>(&Ws[buf][(nb * 32 + (lane & 31)) * LDS_ROW + koff]);
                acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf, acc[nb], 0, 0, 0);
            }
        }
        if (step + 1 < nsteps) lstore(buf ^ 1);
        __syncthreads();
    }

    // epilogue: acc[nb][j] is D[row = 8*(j/4) + 4*(lane/32) + j%4][col = lane%32] of the 32x32 block
    const int col = lane & 31;
#pragma unroll
    for (int j = 0; j < 16; j++) {
        const int m = m0 + wave * 32 + (j >> 2) * 8 + (lane >> 5) * 4 + (j & 3);
        if (m >= p.M) continue;
        if (p.epi == EPI_FFN) {
#pragma unroll
            for (int nb = 0; nb < 2; nb++) {
                float g = acc[nb][j];
                g *= 1.0f / (1.0f + expf(-g));
                const float v = g * acc[nb + 2][j];
                p.out[0][(size_t)p.out_off[0] + (size_t)m * p.ldo[0] + tm.row0[0] + nb * 32 + col] = float_to_half_bits(v);
            }
        } else {
#pragma unroll
            for (int nb = 0; nb < 4; nb++) {
                const int hsel = nb >> 1;
                const int mat = tm.mat[hsel];
                const int n = tm.row0[hsel] + (nb & 1) * 32 + col;
                uint16_t* o = (mat == 0 ? p.out[0] : (mat == 1 ? p.out[1] : p.out[2]));
                const size_t idx = (size_t)(mat == 0 ? p.out_off[0] : (mat == 1 ? p.out_off[1] : p.out_off[2])) +
                                   (size_t)m * (mat == 0 ? p.ldo[0] : (mat == 1 ? p.ldo[1] : p.ldo[2])) + n;
                float v = acc[nb][j];
                if (p.epi == EPI_RESID) v += half_bits_to_float(o[idx]);
                o[idx] = float_to_half_bits(v);
            }
        }
    }
}

// ---------------------------------------------------------------- row-wise helpers
__global__ __launch_bounds__(256) void embed_rows_kernel(uint16_t* x, const uint16_t* table, int dim, const int* tokens, int pos0) {
    const int m = blockIdx.x;
    const int token = tokens[pos0 + m];
    const u32x4* src = reinterpret_cast<const u32x4*>(table + (size_t)token * dim);
    u32x4* dst = reinterpret_cast<u32x4*>(x + (size_t)m * dim);
    for (int i = threadIdx.x; i < (dim >> 3); i += 256) dst[i] = src[i];
}

// o[m] = half(x[m] * (rsqrt(mean(x[m]^2) + 1e-5) * w))  (gpu_kernels.h:72-105, one workgroup per token row)
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(uint16_t* o, const uint16_t* x, const uint16_t* weight, int size) {
    __shared__ float red[4];
    const int tid = threadIdx.x;
    const uint16_t* xr = x + (size_t)blockIdx.x * size;
    uint16_t* orow = o + (size_t)blockIdx.x * size;
    float part = 0.0f;
    for (int i = tid; i < size; i += 256) {
        const float v = half_bits_to_float(xr[i]);
        part = fmaf(v, v, part);
    }
    part = wave_sum(part);
    if ((tid & 63) == 0) red[tid >> 6] = part;
    __syncthreads();
    float ss = (red[0] + red[1]) + (red[2] + red[3]);
    ss /= (float)size;
    ss += 1e-5f;
    ss = 1.0f / sqrtf(ss);
    for (int i = tid; i < size; i += 256) orow[i] = float_to_half_bits(half_bits_to_float(xr[i]) * (ss * half_bits_to_float(weight[i])));
}

// RoPE of q rows [M][heads*hs] and of the K cache rows pos0..pos0+M-1 (gpu_kernels.h:340-363 per position).
__global__ void rope_rows_kernel(uint16_t* q, uint16_t* kcache_layer, int num_heads, int num_kv_heads, int head_size, int pos0,
                                 float rope_theta) {
    const int m = blockIdx.y;
    const int h = blockIdx.x;
    const int i = threadIdx.x;
    const int pos = pos0 + m;
    const int half_size = head_size >> 1;
    const int head_dim = (i * 2) % head_size;
    const float freq = 1.0f / powf(rope_theta, head_dim / (float)head_size);
    const float val = pos * freq;
    const float fcr = cosf(val);
    const float fci = sinf(val);
    uint16_t* qh = q + ((size_t)m * num_heads + h) * head_size;
    const float q0 = half_bits_to_float(qh[i]);
    const float q1 = half_bits_to_float(qh[i + half_size]);
    qh[i] = float_to_half_bits(q0 * fcr - q1 * fci);
    qh[i + half_size] = float_to_half_bits(q0 * fci + q1 * fcr);
    if (h < num_kv_heads) {
        uint16_t* k = kcache_layer + ((size_t)pos * num_kv_heads + h) * head_size;
        const float k0 = half_bits_to_float(k[i]);
        const float k1 = half_bits_to_float(k[i + half_size]);
        k[i] = float_to_half_bits(k0 * fcr - k1 * fci);
        k[i + half_size] = float_to_half_bits(k0 * fci + k1 * fcr);
    }
}

// Causal attention for BQ consecutive query tokens of one head (query m attends to cache rows 0..pos0+m), with the
// reference's rounding points (llama2_q4.cu:410-427): scores -> fp16, probabilities -> fp16, output -> fp16.
constexpr int BQ = 16;

template <int LP>
__global__ __launch_bounds__(256) void attn_prefill_kernel(uint16_t* out, const uint16_t* q, const uint16_t* key_cache,
                                                           const uint16_t* value_cache, int num_heads, int head_size, int kv_mul,
                                                           int M, int pos0) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int h = blockIdx.y;
    const int mq0 = blockIdx.x * BQ;
    const int nq = min(BQ, M - mq0);
    const int nk = pos0 + mq0 + nq;  // keys visible to the last query of the block
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kv_dim = num_heads * head_size / kv_mul;
    const float alpha = (float)(1.0 / sqrt((double)head_size));
    u32x4* qs = reinterpret_cast<u32x4*>(smem);                                            // [BQ][head/8]
    uint16_t* S = reinterpret_cast<uint16_t*>(smem + BQ * head_size * 2);                    // [BQ][nk_stride] fp16 scores / probs
    const int nk_stride = (nk + 7) & ~7;
    float* stat = reinterpret_cast<float*>(smem + BQ * head_size * 2 + BQ * nk_stride * 2);  // [BQ][2]: max, sum

    constexpr int PW = 64 / LP;
    const int j = lane % LP, pr = lane / LP;
    for (int i = tid; i < nq * LP; i += 256)
        qs[i] = *reinterpret_cast<const u32x4*>(q + ((size_t)(mq0 + i / LP) * num_heads + h) * head_size + (i % LP) * 8);
    __syncthreads();

    // 1. scores
    const uint16_t* kh = key_cache + (size_t)(h / kv_mul) * head_size + j * 8;
    for (int t0 = 0; t0 < nk; t0 += 4 * PW) {
        const int t = t0 + wave * PW + pr;
        u32x4 kv = {0u, 0u, 0u, 0u};
        if (t < nk) kv = *reinterpret_cast<const u32x4*>(kh + (size_t)t * kv_dim);
        for (int qi = 0; qi < nq; qi++) {
            const u32x4 qv = qs[qi * LP + j];
            float s = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; i++) s = dot2(kv[i], qv[i], s);
            s = group_sum<LP>(s);
            if (j == 0 && t < nk) S[qi * nk_stride + t] = float_to_half_bits(s * alpha);
        }
    }
    __syncthreads();
    // 2. softmax statistics per query row (wave w takes rows w, w+4, ...)
    for (int qi = wave; qi < nq; qi += 4) {
        const int size = pos0 + mq0 + qi + 1;
        float m = (size < 1024) ? 0.0f : -INFINITY;  // the reference's idle-lane seed
        for (int t = lane; t < size; t += 64) m = fmaxf(m, half_bits_to_float(S[qi * nk_stride + t]));
        m = wave_max(m);
        float sum = 0.0f;
        for (int t = lane; t < size; t += 64) sum += expf(half_bits_to_float(S[qi * nk_stride + t]) - m);
        sum = wave_sum(sum);
        for (int t = lane; t < nk; t += 64) {
            float pv = 0.0f;
            if (t < size) pv = expf(half_bits_to_float(S[qi * nk_stride + t]) - m) / sum;
            S[qi * nk_stride + t] = float_to_half_bits(pv);  // probabilities (0 beyond the causal limit)
        }
        if (lane == 0) {
            stat[2 * qi] = m;
            stat[2 * qi + 1] = sum;
        }
    }
    __syncthreads();
    // 3. out[q][n] = sum_k P[q][k] * V[k][n]: thread = (dim pair, group of 4 queries)
    const int npairs = head_size >> 1;
    const uint16_t* vh = value_cache + (size_t)(h / kv_mul) * head_size;
    for (int item = tid; item < npairs * 4; item += 256) {
        const int np = item % npairs, qg = item / npairs;
        float acc[4][2];
#pragma unroll
        for (int a = 0; a < 4; a++) acc[a][0] = acc[a][1] = 0.0f;
        for (int t = 0; t < nk; t++) {
            const h16x2 v2 = as_h2(*reinterpret_cast<const uint32_t*>(vh + (size_t)t * kv_dim + np * 2));
            const float v0 = (float)v2[0], v1 = (float)v2[1];
#pragma unroll
            for (int a = 0; a < 4; a++) {
                const float pv = half_bits_to_float(S[(qg * 4 + a) * nk_stride + t]);
                acc[a][0] = fmaf(v0, pv, acc[a][0]);
                acc[a][1] = fmaf(v1, pv, acc[a][1]);
            }
        }
#pragma unroll
        for (int a = 0; a < 4; a++) {
            const int qi = qg * 4 + a;
            if (qi < nq) {
                uint16_t* o = out + ((size_t)(mq0 + qi) * num_heads + h) * head_size + np * 2;
                o[0] = float_to_half_bits(acc[a][0]);
                o[1] = float_to_half_bits(acc[a][1]);
            }
        }
    }
}

__global__ void set_pos_kernel(int* pos_dev, volatile int* pos_host, int value) {
    *pos_dev = value;
    *pos_host = value;
}

__global__ __launch_bounds__(256) void copy_row_kernel(uint16_t* dst, const uint16_t* src, int n8) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n8) reinterpret_cast<u32x4*>(dst)[i] = reinterpret_cast<const u32x4*>(src)[i];
}

}  // namespace pf

// ---------------------------------------------------------------- launchers (internal)
static int launch_gemm(awq_ctx* ctx, const pf::GemmParams& p, int ntiles, const char* what) {
    hipLaunchKernelGGL(pf::gemm_int4_kernel, dim3(div_up(p.M, pf::BM), ntiles), dim3(256), 0, ctx->stream, p);
    return awq_check_launch(what);
}

static void set_mat(pf::GemmParams& p, int i, const awq_qweight* w, int N, uint16_t* out, long long ldo, long long off) {
    p.w[i] = w->weight;
    p.z[i] = w->zeros;
    p.s[i] = w->scales;
    p.N[i] = N;
    p.out[i] = out;
    p.ldo[i] = ldo;
    p.out_off[i] = off;
}

static void gemm_common(pf::GemmParams& p, const uint16_t* A, int lda, int M, int K, int epi) {
    memset(&p, 0, sizeof(p));
    p.A = A;
    p.lda = lda;
    p.M = M;
    p.K = K;
    p.C = div_up(K, 32);
    p.pzh = packed_zeros_height(K);
    p.sh = scales_height(K);
    p.epi = epi;
}

int awq_launch_gemm_single(awq_ctx* ctx, uint16_t* out, long long ldo, const uint16_t* A, int lda, int M, const awq_qweight* w,
                           int K, int N, int accum) {
    pf::GemmParams p;
    gemm_common(p, A, lda, M, K, accum ? pf::EPI_RESID : pf::EPI_STORE);
    set_mat(p, 0, w, N, out, ldo, 0);
    return launch_gemm(ctx, p, N / pf::BN, "gemm_int4");
}

int awq_launch_gemm_qkv(awq_ctx* ctx, uint16_t* q, uint16_t* key_cache, uint16_t* value_cache, long long kv_row0_off,
                        const uint16_t* A, int lda, int M, const awq_qweight* qw, const awq_qweight* kw, const awq_qweight* vw,
                        int K, int Nq, int Nkv) {
    pf::GemmParams p;
    gemm_common(p, A, lda, M, K, pf::EPI_QKV);
    set_mat(p, 0, qw, Nq, q, Nq, 0);
    set_mat(p, 1, kw, Nkv, key_cache, Nkv, kv_row0_off);
    set_mat(p, 2, vw, Nkv, value_cache, Nkv, kv_row0_off);
    return launch_gemm(ctx, p, (Nq + 2 * Nkv) / pf::BN, "gemm_int4_qkv");
}

int awq_launch_gemm_ffn(awq_ctx* ctx, uint16_t* hb, const uint16_t* A, int lda, int M, const awq_qweight* gate_w,
                        const awq_qweight* up_w, int K, int N) {
    pf::GemmParams p;
    gemm_common(p, A, lda, M, K, pf::EPI_FFN);
    set_mat(p, 0, gate_w, N, hb, N, 0);
    set_mat(p, 1, up_w, N, hb, N, 0);
    return launch_gemm(ctx, p, N / 64, "gemm_int4_ffn");
}

int awq_launch_embed_rows(awq_ctx* ctx, uint16_t* x, const uint16_t* table, int dim, const int* tokens, int pos0, int M) {
    hipLaunchKernelGGL(pf::embed_rows_kernel, dim3(M), dim3(256), 0, ctx->stream, x, table, dim, tokens, pos0);
    return awq_check_launch("embed_rows");
}

int awq_launch_rmsnorm_rows(awq_ctx* ctx, uint16_t* o, const uint16_t* x, const uint16_t* w, int size, int M) {
    hipLaunchKernelGGL(pf::rmsnorm_rows_kernel, dim3(M), dim3(256), 0, ctx->stream, o, x, w, size);
    return awq_check_launch("rmsnorm_rows");
}

int awq_launch_rope_rows(awq_ctx* ctx, uint16_t* q, uint16_t* kcache_layer, int nh, int nkv, int hs, int pos0, float theta, int M) {
    hipLaunchKernelGGL(pf::rope_rows_kernel, dim3(nh, M), dim3(hs / 2), 0, ctx->stream, q, kcache_layer, nh, nkv, hs, pos0, theta);
    return awq_check_launch("rope_rows");
}

int awq_launch_attn_prefill(awq_ctx* ctx, uint16_t* out, const uint16_t* q, const uint16_t* kc, const uint16_t* vc, int nh, int hs,
                            int kv_mul, int M, int pos0) {
    const int nk_max = (pos0 + M + 7) & ~7;
    const size_t lds = (size_t)pf::BQ * hs * 2 + (size_t)pf::BQ * nk_max * 2 + pf::BQ * 8;
    if (lds > 160 * 1024) {
        awq_set_error("prefill attention: context of %d positions does not fit in LDS", pos0 + M);
        return AWQ_ERR_SHAPE;
    }
    const dim3 grid(div_up(M, pf::BQ), nh);
#define AWQ_ATTN_PF(LPV)                                                                                                  \
    do {                                                                                                                  \
        if (lds > 64 * 1024) {                                                                                            \
            hipError_t e = hipFuncSetAttribute((const void*)pf::attn_prefill_kernel<LPV>,                                 \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);                  \
            if (e != hipSuccess) {                                                                                        \
                awq_set_error("hipFuncSetAttribute(attn_prefill) failed: %s", hipGetErrorString(e));                      \
                return AWQ_ERR_HIP;                                                                                       \
            }                                                                                                             \
        }                                                                                                                 \
        hipLaunchKernelGGL((pf::attn_prefill_kernel<LPV>), grid, dim3(256), lds, ctx->stream, out, q, kc, vc, nh, hs, kv_mul, \
                           M, pos0);                                                                                      \
    } while (0)
    switch (hs) {
        case 64: AWQ_ATTN_PF(8); break;
        case 128: AWQ_ATTN_PF(16); break;
        case 256: AWQ_ATTN_PF(32); break;
        default: awq_set_error("prefill attention: head_size %d unsupported", hs); return AWQ_ERR_SHAPE;
    }
#undef AWQ_ATTN_PF
    return awq_check_launch("attn_prefill");
}

int awq_launch_set_pos(awq_ctx* ctx, int* pos_dev, volatile int* pos_host, int value) {
    hipLaunchKernelGGL(pf::set_pos_kernel, dim3(1), dim3(1), 0, ctx->stream, pos_dev, pos_host, value);
    return awq_check_launch("set_pos");
}

int awq_launch_copy_row(awq_ctx* ctx, uint16_t* dst, const uint16_t* src, int n) {
    hipLaunchKernelGGL(pf::copy_row_kernel, dim3(div_up(n >> 3, 256)), dim3(256), 0, ctx->stream, dst, src, n >> 3);
    return awq_check_launch("copy_row");
}

extern "C" {

int awq_gemm_int4(awq_ctx* ctx, uint16_t* out, int ldo, const uint16_t* a, int lda, int M, const awq_qweight* w, int K, int N,
                  int accum) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_REQUIRE(out && a && w && w->weight && w->zeros && w->scales, AWQ_ERR_ARG, "null pointer");
    if (M <= 0 || K <= 0 || N <= 0 || (K & 31) || (N & 127) || (lda & 7)) {
        awq_set_error("awq_gemm_int4: needs M > 0, K %% 32 == 0, N %% 128 == 0, lda %% 8 == 0 (got M=%d K=%d N=%d lda=%d)", M, K, N, lda);
        return AWQ_ERR_SHAPE;
    }
    return awq_launch_gemm_single(ctx, out, ldo, a, lda, M, w, K, N, accum);
}

}  // extern "C"
