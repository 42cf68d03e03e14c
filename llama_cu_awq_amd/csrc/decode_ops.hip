// The fp16 side of batch-1 decode on gfx950: embedding gather, RMSNorm, RoPE,
// KV-cache attention, the fp16 classifier matrix-vector product and the greedy
// sampler.  Arithmetic and rounding points follow the reference kernels cited
// at each entry point; launch geometry and data movement are this library's.
#include "attention.hpp"
#include "common.hpp"

namespace {


// ------------------------------------------------------------------ embed
__global__ __launch_bounds__(256) void embed_kernel(uint16_t* x, const uint16_t* table, int dim, const int* tokens,
                                                    const int* pPos) {
    const int token = tokens[*pPos];
    const u32x4* src = reinterpret_cast<const u32x4*>(table + (size_t)token * dim);
    u32x4* dst = reinterpret_cast<u32x4*>(x);
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < (dim >> 3)) dst[i] = src[i];
}

// ------------------------------------------------------------------ rmsnorm
// One workgroup of 1024 (the vector is a few KB): fp32 sum of squares,
// ss = 1/sqrt(ss/size + 1e-5), o = half(x * (ss * w)).
__global__ __launch_bounds__(1024) void rmsnorm_kernel(uint16_t* o, const uint16_t* x, const uint16_t* weight, int size) {
    __shared__ float red[16];
    __shared__ float shared_ss;
    const int tid = threadIdx.x;
    float part = 0.0f;
    for (int i = tid; i < size; i += 1024) {
        const float v = half_bits_to_float(x[i]);
        part = fmaf(v, v, part);
    }
    part = wave_sum(part);
    if ((tid & 63) == 0) red[tid >> 6] = part;
    __syncthreads();
    if (tid == 0) {
        float ss = 0.0f;
        for (int w = 0; w < 16; w++) ss += red[w];
        ss /= (float)size;
        ss += 1e-5f;
        shared_ss = 1.0f / sqrtf(ss);
    }
    __syncthreads();
    const float ss = shared_ss;
    for (int i = tid; i < size; i += 1024) {
        const float v = half_bits_to_float(x[i]);
        o[i] = float_to_half_bits(v * (ss * half_bits_to_float(weight[i])));
    }
}

// ------------------------------------------------------------------ rope
// One workgroup per head, one thread per pair (i, i + head/2).
__global__ void rope_kernel(uint16_t* sq, uint16_t* sk_base, int num_kv_heads, int head_size, const int* pPos, int loff,
                            float rope_theta) {
    const int pos = *pPos;
    const int h = blockIdx.x;
    const int i = threadIdx.x;
    const int half_size = head_size >> 1;
    const int head_dim = (i * 2) % head_size;
    const float freq = 1.0f / powf(rope_theta, head_dim / (float)head_size);
    const float val = pos * freq;
    const float fcr = cosf(val);
    const float fci = sinf(val);
    uint16_t* q = sq + (size_t)h * head_size;
    const float q0 = half_bits_to_float(q[i]);
    const float q1 = half_bits_to_float(q[i + half_size]);
    float r0, r1;
    rope_rotate(q0, q1, fcr, fci, r0, r1);
    q[i] = float_to_half_bits(r0);
    q[i + half_size] = float_to_half_bits(r1);
    if (h < num_kv_heads) {
        uint16_t* k = sk_base + (size_t)loff + (size_t)pos * num_kv_heads * head_size + (size_t)h * head_size;
        const float k0 = half_bits_to_float(k[i]);
        const float k1 = half_bits_to_float(k[i + half_size]);
        rope_rotate(k0, k1, fcr, fci, r0, r1);
        k[i] = float_to_half_bits(r0);
        k[i + half_size] = float_to_half_bits(r1);
    }
}

// ------------------------------------------------------------------ attention
// Pass 1: scores.  LP = head_size/8 lanes cover one cache row of a head
// (16 bytes each); a wave covers 64/LP positions per load and a workgroup of
// 4 waves covers 64 positions.  att[h*(pos+1) + t] = half(dot(K[t], q) / sqrt(head)).
template <int LP>
__global__ __launch_bounds__(256) void attn_scores_kernel(uint16_t* att, const uint16_t* q, const uint16_t* key_cache,
                                                          int head_size, int kv_mul, int row_stride, float alpha,
                                                          const int* pPos) {
    const int size = *pPos + 1;
    const int t0 = blockIdx.x * 64;
    if (t0 >= size) return;
    const int h = blockIdx.y;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    constexpr int PW = 64 / LP;  // positions per wave-load
    const int j = lane % LP;     // which 8 halves of the head
    const int pr = lane / LP;
    const u32x4 qv = *reinterpret_cast<const u32x4*>(q + (size_t)h * head_size + j * 8);
    const uint16_t* kh = key_cache + (size_t)(h / kv_mul) * head_size + j * 8;
    uint16_t* a = att + (size_t)h * size;
    constexpr int ITERS = 16 / PW;  // 16 positions per wave
    u32x4 kv[ITERS];
#pragma unroll
    for (int it = 0; it < ITERS; it++) {
        // (clamped, not skipped: a load inside a branch makes the compiler wait for it before the next one)
        const int t = min(t0 + wave * 16 + it * PW + pr, size - 1);
        kv[it] = *reinterpret_cast<const u32x4*>(kh + (size_t)t * row_stride);
    }
#pragma unroll
    for (int it = 0; it < ITERS; it++) {
        const int t = t0 + wave * 16 + it * PW + pr;
        float s = 0.0f;
        if (t < size) {
#pragma unroll
            for (int i = 0; i < 4; i++) s = dot2(kv[it][i], qv[i], s);
        }
        s = group_sum<LP>(s);
        if (j == 0 && t < size) a[t] = float_to_half_bits(s * alpha);
    }
}

// Pass 2: softmax and P.V.  A workgroup of 16 waves owns LR * 8 of a head's dimensions (LR lanes x 16 bytes of every
// value row) over ALL positions, so no partial sums leave the workgroup.  The 1024 / LR lane groups take positions
// g, g + 1024 / LR, ...; a lane requests R rows at once, after the scores of those positions (loads return in order
// and the softmax statistics need only the scores; each position is counted by one lane of its group).
template <int LR, int R>
__global__ __launch_bounds__(1024) void attn_pv_sliced_kernel(uint16_t* output, const uint16_t* att, const uint16_t* value_cache,
                                                              int num_heads, int head_size, int kv_mul, int row_stride,
                                                              const int* pPos) {
    constexpr int NG = 1024 / LR;  // lane groups = positions per pass
    constexpr int SW = LR * 8;     // dimensions per workgroup
    __shared__ float red[16];
    __shared__ float acc_lds[16][SW];
    const int size = *pPos + 1;
    // heads along x (the grid is padded to a multiple of 8 of them): the slices of a head share an XCD and its L2
    const int h = blockIdx.x, slice = blockIdx.y;
    if (h >= num_heads) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int pg = tid / LR, ql = tid % LR;
    const uint16_t* a = att + (size_t)h * size;
    const uint16_t* vh = value_cache + (size_t)(h / kv_mul) * head_size + slice * SW + ql * 8;
    u32x4 vv[R];
    uint16_t sv[R];
    auto request = [&](int t0) {
        // positions past the end are clamped, not skipped: a load inside a branch makes the compiler wait for it
        // before it issues the next one
#pragma unroll
        for (int k = 0; k < R; k++) sv[k] = a[min(t0 + pg + NG * k, size - 1)];
#pragma unroll
        for (int k = 0; k < R; k++)
            vv[k] = *reinterpret_cast<const u32x4*>(vh + (size_t)min(t0 + pg + NG * k, size - 1) * row_stride);
    };
    request(0);
    // statistics over all positions (gpu_kernels.h:376-400; the max seed is the reference's idle-lane 0 when its
    // 1024-thread block is not full)
    float m = (size < 1024) ? 0.0f : -INFINITY;
    if (ql == 0) {
#pragma unroll
        for (int k = 0; k < R; k++)
            if (pg + NG * k < size) m = fmaxf(m, half_bits_to_float(sv[k]));
        for (int t = pg + NG * R; t < size; t += NG) m = fmaxf(m, half_bits_to_float(a[t]));
    }
    m = wave_max(m);
    if (lane == 0) red[wave] = m;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < 16; w++) m = fmaxf(m, red[w]);
    __syncthreads();
    float sum = 0.0f;
    if (ql == 0) {
#pragma unroll
        for (int k = 0; k < R; k++)
            if (pg + NG * k < size) sum += expf(half_bits_to_float(sv[k]) - m);
        for (int t = pg + NG * R; t < size; t += NG) sum += expf(half_bits_to_float(a[t]) - m);
    }
    sum = wave_sum(sum);
    if (lane == 0) red[wave] = sum;
    __syncthreads();
    {
        float r[16];
#pragma unroll
        for (int w = 0; w < 16; w++) r[w] = red[w];
#pragma unroll
        for (int n = 16; n > 1; n >>= 1)
#pragma unroll
            for (int i = 0; i < n / 2; i++) r[i] = r[2 * i] + r[2 * i + 1];
        sum = r[0];
    }

    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = 0.0f;
    for (int t0 = 0; t0 < size; t0 += NG * R) {
        if (t0) request(t0);
#pragma unroll
        for (int k = 0; k < R; k++) {
            const int t = t0 + pg + NG * k;
            if (t < size) {
                const float e = expf(half_bits_to_float(sv[k]) - m);
                const float p = half_bits_to_float(float_to_half_bits(e / sum));  // probability rounded to fp16
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const h16x2 hv = as_h2(vv[k][i]);
                    acc[2 * i] = fmaf((float)hv[0], p, acc[2 * i]);
                    acc[2 * i + 1] = fmaf((float)hv[1], p, acc[2 * i + 1]);
                }
            }
        }
    }
    // add up the lane groups of the wave (lanes with the same lane % LR), then the 16 waves
#pragma unroll
    for (int i = 0; i < 8; i++) {
        if (LR <= 1) acc[i] += dpp_mov<0xB1>(acc[i]);   // quad_perm [1,0,3,2]
        if (LR <= 2) acc[i] += dpp_mov<0x4E>(acc[i]);   // quad_perm [2,3,0,1]
        if (LR <= 4) acc[i] += dpp_mov<0x124>(acc[i]);  // row_ror:4
        if (LR <= 8) acc[i] += dpp_mov<0x128>(acc[i]);  // row_ror:8
        acc[i] = lane_xor_sum<16>(acc[i]);
        acc[i] = lane_xor_sum<32>(acc[i]);
    }
    if (lane < LR) {
#pragma unroll
        for (int i = 0; i < 8; i++) acc_lds[wave][lane * 8 + i] = acc[i];
    }
    __syncthreads();
    if (tid < SW) {
        float r[16];
#pragma unroll
        for (int w = 0; w < 16; w++) r[w] = acc_lds[w][tid];
#pragma unroll
        for (int n = 16; n > 1; n >>= 1)
#pragma unroll
            for (int i = 0; i < n / 2; i++) r[i] = r[2 * i] + r[2 * i + 1];
        output[(size_t)h * head_size + slice * SW + tid] = float_to_half_bits(r[0]);
    }
}

// Long contexts in the fused schedule: P.V split over positions as well, so that every compute unit pulls whole
// cache lines.  A workgroup of 16 waves owns one head, one of `chunks` contiguous ranges of positions and one slice of
// 64 value dimensions (128 bytes of every row: 8 lanes x 16 bytes); it computes the softmax statistics over ALL
// positions from the fp16 scores (as every workgroup of the head does, in the same order, so they agree bit for bit),
// forms the fp16-rounded probabilities of its own positions exactly as the reference does (gpu_kernels.h:376-409) and
// writes the fp32 sum of p * v over its range to part[chunk][head * head_size + dim].  The chunks of a head are added
// up, in chunk order, by the consumer (the O projection's staging), where the sum is rounded to fp16: the rounding
// point of the reference's attention output.  No exchange between workgroups, no atomics, one launch.
constexpr int kPvPartialRows = 8;  // value rows in flight per thread

__global__ __launch_bounds__(1024) void attn_pv_partial_kernel(float* part, const uint16_t* att, const uint16_t* value_cache,
                                                              int head_size, int kv_mul, int row_stride, int chunks, int out_dim,
                                                              const int* pPos) {
    constexpr int R = kPvPartialRows;
    __shared__ float red[16];
    __shared__ float acc_lds[16][64];
    __shared__ float pl[8 * 136];  // probabilities of the positions in flight: [row of the group][row group], padded
    const int size = *pPos + 1;
    const int h = blockIdx.x, chunk = blockIdx.y, slice = blockIdx.z;
    const int per = (size + chunks - 1) / chunks;
    const int t_begin = chunk * per, t_end = min(size, t_begin + per);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int rg = tid >> 3, ql = tid & 7;  // row group (128 rows per pass), 16-byte piece of the slice
    const uint16_t* a = att + (size_t)h * size;
    const uint16_t* vh = value_cache + (size_t)(h / kv_mul) * head_size + slice * 64 + ql * 8;
    u32x4 vv[R];
    uint16_t sv[R];
    // Loads return in order: the scores that the statistics need (two per thread cover 2048 positions) are requested
    // ahead of the value rows, so that the statistics are computed while the rows are still on their way.
    uint16_t stat[2];
    // (positions past the end are clamped, not skipped: a load inside a branch makes the compiler wait for it before
    // it issues the next one)
#pragma unroll
    for (int j = 0; j < 2; j++) stat[j] = a[min(tid + 1024 * j, size - 1)];
    // rows past the range's end repeat its last row (one cache line): clamped to the end of the context instead, a
    // workgroup pulled the next range's rows as well, 1.6 times its share at three ranges of 534 positions (13B shape,
    // 1.6 K context: 415 -> 424 tokens/s)
    const int t_last = max(t_end, t_begin + 1) - 1;
    auto request = [&](int t0) {
#pragma unroll
        for (int k = 0; k < R; k++) sv[k] = a[min(t0 + rg + 128 * k, t_last)];
#pragma unroll
        for (int k = 0; k < R; k++)
            vv[k] = *reinterpret_cast<const u32x4*>(vh + (size_t)min(t0 + rg + 128 * k, t_last) * row_stride);
    };
    request(t_begin);
    // statistics over all positions (the max seed is the reference's idle-lane 0 when its 1024-thread block is not full)
    float m = (size < 1024) ? 0.0f : -INFINITY;
#pragma unroll
    for (int j = 0; j < 2; j++)
        if (tid + 1024 * j < size) m = fmaxf(m, half_bits_to_float(stat[j]));
    for (int t = tid + 2048; t < size; t += 1024) m = fmaxf(m, half_bits_to_float(a[t]));
    m = wave_max(m);
    if (lane == 0) red[wave] = m;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < 16; w++) m = fmaxf(m, red[w]);
    __syncthreads();
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < 2; j++)
        if (tid + 1024 * j < size) sum += expf(half_bits_to_float(stat[j]) - m);
    for (int t = tid + 2048; t < size; t += 1024) sum += expf(half_bits_to_float(a[t]) - m);
    sum = wave_sum(sum);
    if (lane == 0) red[wave] = sum;
    __syncthreads();
    {
        float r[16];
#pragma unroll
        for (int w = 0; w < 16; w++) r[w] = red[w];
#pragma unroll
        for (int n = 16; n > 1; n >>= 1)
#pragma unroll
            for (int i = 0; i < n / 2; i++) r[i] = r[2 * i] + r[2 * i + 1];
        sum = r[0];
    }

    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = 0.0f;
    static_assert(R == 8, "lane ql of a row group computes the probability of the group's row ql");
    for (int t0 = t_begin; t0 < t_end; t0 += 128 * R) {
        if (t0 != t_begin) {
            __syncthreads();  // the previous round's probabilities have been read
            request(t0);
        }
        // The 8 lanes of a row group need the same 8 probabilities: lane ql computes the one of row ql (exponential
        // and correctly rounded quotient once per position instead of 8 times) and the group shares them through LDS.
        {
            uint16_t sq = sv[0];
#pragma unroll
            for (int k = 1; k < R; k++) sq = ql == k ? sv[k] : sq;
            const float e = expf(half_bits_to_float(sq) - m);
            pl[ql * 136 + rg] = half_bits_to_float(float_to_half_bits(e / sum));  // probability rounded to fp16
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < R; k++) {
            const int t = t0 + rg + 128 * k;
            if (t < t_end) {
                const float p = pl[k * 136 + rg];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const h16x2 hv = as_h2(vv[k][i]);
                    acc[2 * i] = fmaf((float)hv[0], p, acc[2 * i]);
                    acc[2 * i + 1] = fmaf((float)hv[1], p, acc[2 * i + 1]);
                }
            }
        }
    }
    // the 8 row groups of a wave (lanes with the same lane % 8), then the 16 waves
#pragma unroll
    for (int i = 0; i < 8; i++) {
        acc[i] = lane_xor_sum<8>(acc[i]);
        acc[i] = lane_xor_sum<16>(acc[i]);
        acc[i] = lane_xor_sum<32>(acc[i]);
    }
    if (lane < 8) {
#pragma unroll
        for (int i = 0; i < 8; i++) acc_lds[wave][lane * 8 + i] = acc[i];
    }
    __syncthreads();
    if (tid < 64) {
        float r[16];
#pragma unroll
        for (int w = 0; w < 16; w++) r[w] = acc_lds[w][tid];
#pragma unroll
        for (int n = 16; n > 1; n >>= 1)
#pragma unroll
            for (int i = 0; i < n / 2; i++) r[i] = r[2 * i] + r[2 * i + 1];
        part[(size_t)chunk * out_dim + (size_t)h * head_size + slice * 64 + tid] = r[0];
    }
}

// Short contexts: a workgroup of 16 waves does scores, softmax and P.V of a head in a single launch (the work is a few
// hundred KB per head, so the launch count matters more than the parallelism); NS workgroups per head each take a
// slice of the value dimensions and compute the scores redundantly.  Same arithmetic and
// rounding points as the two-pass kernels above; the fp16 scores are also left in att.
template <int LP, int NS>
__global__ __launch_bounds__(1024) void attn_fused_kernel(uint16_t* output, uint16_t* att, const uint16_t* q,
                                                          const uint16_t* key_cache, const uint16_t* value_cache, int num_heads,
                                                          int head_size, int kv_mul, int row_stride, float alpha,
                                                          const int* pPos, int max_seq_len) {
    extern __shared__ float fsm[];
    // LDS was sized for max_seq_len positions by the launcher; a position beyond it (a caller that sized the launch
    // from a stale position) must not run past that
    const int size = min(*pPos + 1, max_seq_len);
    // heads along x, padded to a multiple of 8: the NS workgroups of a head (ids h, h + padded heads, ...) share an XCD
    const int h = blockIdx.x, slice = blockIdx.y;
    if (h >= num_heads) return;
    attention_head<LP, 16, NS>(output + (size_t)h * head_size, att + (size_t)h * size, q + (size_t)h * head_size,
                               key_cache + (size_t)(h / kv_mul) * head_size, value_cache + (size_t)(h / kv_mul) * head_size,
                               head_size, row_stride, alpha, size, fsm, slice);
}

// ------------------------------------------------------------------ fp16 matvec
// out[r] = half(sum_j w[r*n + j] * x[j]).  x staged in LDS in natural order;
// a lane owns the same 16-byte column slices for the R rows of its wave.
template <int R, bool NORM>
__global__ __launch_bounds__(256) void gemv_f16_kernel(uint16_t* out, const uint16_t* x, const uint16_t* w, int n, int d,
                                                       const uint16_t* norm_w, uint16_t* norm_out) {
    extern __shared__ u32x4 xs[];
    __shared__ float red[4];
    const int tid = threadIdx.x;
    const int n8 = n >> 3;
    const u32x4* xg = reinterpret_cast<const u32x4*>(x);
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int row0 = (blockIdx.x * 4 + wave) * R;
    // The first batch of the wave's rows is requested before x is staged: the rows do not depend on x, and their way
    // from memory overlaps the staging (rows past d are clamped to the last one and never stored).
    const u32x4* wrow[R];
    u32x4 a[R], b[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        wrow[r] = reinterpret_cast<const u32x4*>(w + (size_t)min(row0 + r, d - 1) * n);
        a[r] = load_nt(wrow[r] + min(lane, n8 - 1));
    }
    float ss = 0.0f;
    if (NORM) {
        float part = 0.0f;
        for (int e = tid; e < n8; e += 256) {
            const u32x4 v = xg[e];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const h16x2 hh = as_h2(v[i]);
                const float a = (float)hh[0], b = (float)hh[1];
                part = fmaf(a, a, part);
                part = fmaf(b, b, part);
            }
        }
        part = wave_sum(part);
        if ((tid & 63) == 0) red[tid >> 6] = part;
        __syncthreads();
        ss = (red[0] + red[1]) + (red[2] + red[3]);
        ss /= (float)n;
        ss += 1e-5f;
        ss = 1.0f / sqrtf(ss);
    }
    const bool store_norm = NORM && norm_out != nullptr && blockIdx.x == 0;
    for (int e = tid; e < n8; e += 256) {
        u32x4 v = xg[e];
        if (NORM) {
            const u32x4 wv = reinterpret_cast<const u32x4*>(norm_w)[e];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const h16x2 hh = as_h2(v[i]);
                const h16x2 hw = as_h2(wv[i]);
                h16x2 o;
                o[0] = (h16_t)((float)hh[0] * (ss * (float)hw[0]));
                o[1] = (h16_t)((float)hh[1] * (ss * (float)hw[1]));
                v[i] = as_u32(o);
            }
        }
        xs[e] = v;
    }
    __syncthreads();
    // norm_out must not alias x: other workgroups may still be reading x.
    if (store_norm) {
        for (int e = tid; e < n8; e += 256) reinterpret_cast<u32x4*>(norm_out)[e] = xs[e];
    }

    if (row0 >= d) return;
    float sum[R];
#pragma unroll
    for (int r = 0; r < R; r++) sum[r] = 0.0f;

    // Two batches of R x 16 bytes per lane in flight.  Every load is unconditional, pieces past the row end clamped to
    // its last one (their products are skipped): a load inside a branch is waited for, together with everything
    // requested before it, before the next one is issued.
    for (int c = lane; c < n8 + lane; c += 128) {
        const int c1 = c + 64, c2 = c + 128;
#pragma unroll
        for (int r = 0; r < R; r++) b[r] = load_nt(wrow[r] + min(c1, n8 - 1));
        if (c < n8) {
            const u32x4 xv = xs[c];
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
                for (int i = 0; i < 4; i++) sum[r] = dot2(a[r][i], xv[i], sum[r]);
        }
#pragma unroll
        for (int r = 0; r < R; r++) a[r] = load_nt(wrow[r] + min(c2, n8 - 1));
        if (c1 < n8) {
            const u32x4 xv = xs[c1];
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
                for (int i = 0; i < 4; i++) sum[r] = dot2(b[r][i], xv[i], sum[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++) sum[r] = wave_sum(sum[r]);
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < R; r++)
            if (row0 + r < d) out[row0 + r] = float_to_half_bits(sum[r]);
    }
}

// ------------------------------------------------------------------ argmax
// One workgroup of 1024: per-thread strided scan keeping the first maximum,
// then (value, index) reductions that prefer the lower index on equal values.
__global__ __launch_bounds__(1024) void argmax_kernel(const uint16_t* x, int size, int* result, volatile int* pPos,
                                                      int* pPosGpu, int write_token, int* mirror) {
    __shared__ float red_v[16];
    __shared__ int red_i[16];
    const int tid = threadIdx.x;
    // (requested with the logits, so that it has arrived when the last thread standing needs it)
    int token_pos = 0;
    if (tid == 0) token_pos = *pPosGpu;
    float best = -INFINITY;
    int best_i = 0x7FFFFFFF;
    auto take = [&](float v, int i) {
        if (v > best || (v == best && i < best_i)) {
            best = v;
            best_i = i;
        }
    };
    // 8 logits per load, 4 loads in flight per thread (x is 16-byte aligned: it is a device allocation's start)
    const int n8 = size >> 3;
    const u32x4* x8 = reinterpret_cast<const u32x4*>(x);
    for (int e0 = 0; e0 < n8; e0 += 4 * 1024) {
        u32x4 v[4];
#pragma unroll
        for (int k = 0; k < 4; k++) v[k] = x8[min(e0 + k * 1024 + tid, n8 - 1)];  // unconditional: all four in flight together
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int e = e0 + k * 1024 + tid;
            if (e < n8) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const h16x2 h = as_h2(v[k][i]);
                    take((float)h[0], e * 8 + 2 * i);
                    take((float)h[1], e * 8 + 2 * i + 1);
                }
            }
        }
    }
    for (int i = n8 * 8 + tid; i < size; i += 1024) take(half_bits_to_float(x[i]), i);
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(best, off);
        const int oi = __shfl_xor(best_i, off);
        if (ov > best || (ov == best && oi < best_i)) {
            best = ov;
            best_i = oi;
        }
    }
    if ((tid & 63) == 0) {
        red_v[tid >> 6] = best;
        red_i[tid >> 6] = best_i;
    }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < 16; w++) {
            if (red_v[w] > best || (red_v[w] == best && red_i[w] < best_i)) {
                best = red_v[w];
                best_i = red_i[w];
            }
        }
        if (best_i == 0x7FFFFFFF) best_i = 0;  // nothing compared greater than -inf (all NaN / -inf)
        token_pos++;
        if (write_token) {
            result[token_pos] = best_i;
            if (mirror) mirror[token_pos] = best_i;
        }
        *pPos = token_pos;
        *pPosGpu = token_pos;
    }
}

template <int LP>
int launch_attention(awq_ctx* ctx, uint16_t* output, const uint16_t* q, const uint16_t* key_cache,
                     const uint16_t* value_cache, uint16_t* att, int num_heads, int head_size, int kv_mul, int max_seq_len,
                     const int* pos) {
    const int row_stride = num_heads * head_size / kv_mul;
    const float alpha = (float)(1.0 / sqrt((double)head_size));
    if (max_seq_len <= kAttnFusedMaxSeq) {
        const size_t lds = (size_t)attention_head_lds_floats(max_seq_len, head_size, 16) * sizeof(float);
        // two workgroups per head (halves of the value dimensions): +0.4 .. 0.7 % tokens/s at 7B; four: no better
        awq_launch(ctx, attn_fused_kernel<LP, 2>, dim3((num_heads + 7) & ~7, 2), dim3(1024), lds, output, att, q,
                           key_cache, value_cache, num_heads, head_size, kv_mul, row_stride, alpha, pos, max_seq_len);
        return awq_check_launch("attn_fused");
    }
    awq_launch(ctx, attn_scores_kernel<LP>, dim3(div_up(max_seq_len, 64), num_heads), dim3(256), 0, att, q,
                       key_cache, head_size, kv_mul, row_stride, alpha, pos);
    if (int r = awq_check_launch("attn_scores")) return r;
    // 16 dimensions (2 lanes x 16 bytes of a row) per workgroup measured best (32: -2.5 %, 8: -4 %, 64: -12 % tokens/s
    // at the 13B shape, 1.6 K context); the head count is padded to a multiple of 8 so that the slices of a head
    // (ids h, h + padded heads, ...) share an XCD and the cache lines they split between them
    awq_launch(ctx, attn_pv_sliced_kernel<2, 4>, dim3((num_heads + 7) & ~7, LP / 2), dim3(1024), 0, output, att,
                       value_cache, num_heads, head_size, kv_mul, row_stride, pos);
    return awq_check_launch("attn_pv_sliced");
}

}  // namespace

// Internal: greedy sampler that also records the token in a device-side mirror of the token list.
int awq_launch_argmax(awq_ctx* ctx, const uint16_t* logits, int size, int* tokens, volatile int* pos_host, int* pos_dev,
                      int write_token, int* tokens_mirror) {
    awq_launch(ctx, argmax_kernel, dim3(1), dim3(1024), 0, logits, size, tokens, pos_host, pos_dev, write_token,
                       tokens_mirror);
    return awq_check_launch("argmax");
}

// Internal: into how many ranges of positions the position-split P.V divides a head's rows: about one workgroup per
// compute unit (heads x 64-dimension slices x ranges), each pulling whole cache lines.
int awq_attention_partial_chunks(const awq_ctx* ctx, int num_heads, int head_size) {
    const int slices = head_size >= 64 ? head_size / 64 : 1;
    int chunks = ctx->cus / (num_heads * slices);
    if (chunks < 1) chunks = 1;
    if (chunks > kAttnMaxChunks) chunks = kAttnMaxChunks;
    return chunks;
}

// Internal (fused schedule, launch sizes above kAttnFusedMaxSeq): scores, then P.V as fp32 partial sums over
// `*chunks_out` ranges of positions, part[chunk][num_heads * head_size]; the consumer adds the chunks up in order and
// rounds to fp16.  part must hold kAttnMaxChunks * num_heads * head_size floats.
int awq_launch_attention_partial(awq_ctx* ctx, float* part, int* chunks_out, const uint16_t* q, const uint16_t* key_cache,
                                 const uint16_t* value_cache, uint16_t* att, int num_heads, int head_size, int kv_mul,
                                 int max_seq_len, const int* pos) {
    const int row_stride = num_heads * head_size / kv_mul;
    const float alpha = (float)(1.0 / sqrt((double)head_size));
    const int slices = head_size / 64;
    const int chunks = awq_attention_partial_chunks(ctx, num_heads, head_size);
    const dim3 sgrid(div_up(max_seq_len, 64), num_heads);
    switch (head_size) {
        case 64: awq_launch(ctx, attn_scores_kernel<8>, sgrid, dim3(256), 0, att, q, key_cache, head_size, kv_mul, row_stride, alpha, pos); break;
        case 128: awq_launch(ctx, attn_scores_kernel<16>, sgrid, dim3(256), 0, att, q, key_cache, head_size, kv_mul, row_stride, alpha, pos); break;
        case 256: awq_launch(ctx, attn_scores_kernel<32>, sgrid, dim3(256), 0, att, q, key_cache, head_size, kv_mul, row_stride, alpha, pos); break;
        default: awq_set_error("attention: head_size %d unsupported (64, 128 or 256)", head_size); return AWQ_ERR_SHAPE;
    }
    if (int r = awq_check_launch("attn_scores")) return r;
    awq_launch(ctx, attn_pv_partial_kernel, dim3(num_heads, chunks, slices), dim3(1024), 0, part, att, value_cache, head_size, kv_mul,
               row_stride, chunks, num_heads * head_size, pos);
    *chunks_out = chunks;
    return awq_check_launch("attn_pv_partial");
}

// Internal: fp16 matvec with optional fused RMSNorm of x (norm_out must not alias x).
int awq_launch_matvec_f16(awq_ctx* ctx, uint16_t* out, const uint16_t* x, const uint16_t* w, int n, int d,
                          const uint16_t* norm_w, uint16_t* norm_out) {
    constexpr int R = 4;
    const dim3 grid(div_up(d, 4 * R));
    const size_t lds = (size_t)n * 2;
    if (norm_w)
        awq_launch(ctx, gemv_f16_kernel<R, true>, grid, dim3(256), lds, out, x, w, n, d, norm_w, norm_out);
    else
        awq_launch(ctx, gemv_f16_kernel<R, false>, grid, dim3(256), lds, out, x, w, n, d, norm_w, norm_out);
    return awq_check_launch("gemv_f16");
}

extern "C" {

int awq_embed(awq_ctx* ctx, uint16_t* x, const uint16_t* table, int dim, const int* tokens, const int* pos) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_REQUIRE(x && table && tokens && pos, AWQ_ERR_ARG, "null pointer");
    AWQ_REQUIRE(dim > 0 && (dim & 7) == 0, AWQ_ERR_SHAPE, "dim must be a positive multiple of 8");
    awq_launch(ctx, embed_kernel, dim3(div_up(dim >> 3, 256)), dim3(256), 0, x, table, dim, tokens, pos);
    return awq_check_launch("embed");
}

int awq_rmsnorm(awq_ctx* ctx, uint16_t* o, const uint16_t* x, const uint16_t* weight, int size) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_REQUIRE(o && x && weight, AWQ_ERR_ARG, "null pointer");
    AWQ_REQUIRE(size > 0, AWQ_ERR_SHAPE, "size must be positive");
    awq_launch(ctx, rmsnorm_kernel, dim3(1), dim3(1024), 0, o, x, weight, size);
    return awq_check_launch("rmsnorm");
}

int awq_rope(awq_ctx* ctx, uint16_t* q, uint16_t* k, int num_heads, int num_kv_heads, int head_size, const int* pos, int loff,
             float rope_theta) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_REQUIRE(q && k && pos, AWQ_ERR_ARG, "null pointer");
    AWQ_REQUIRE(num_heads > 0 && num_kv_heads >= 0 && num_kv_heads <= num_heads, AWQ_ERR_SHAPE, "bad head counts");
    AWQ_REQUIRE(head_size >= 2 && (head_size & 1) == 0 && head_size <= 2048, AWQ_ERR_SHAPE, "head_size must be even, <= 2048");
    AWQ_REQUIRE(loff >= 0, AWQ_ERR_ARG, "loff must be >= 0");
    awq_launch(ctx, rope_kernel, dim3(num_heads), dim3(head_size / 2), 0, q, k, num_kv_heads, head_size, pos,
                       loff, rope_theta);
    return awq_check_launch("rope");
}

int awq_attention(awq_ctx* ctx, uint16_t* output, const uint16_t* q, const uint16_t* key_cache, const uint16_t* value_cache,
                  uint16_t* att, int num_heads, int head_size, int kv_mul, int max_seq_len, const int* pos) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_REQUIRE(output && q && key_cache && value_cache && att && pos, AWQ_ERR_ARG, "null pointer");
    AWQ_REQUIRE(num_heads > 0 && num_heads <= kAttnMaxHeads, AWQ_ERR_SHAPE, "num_heads out of range");
    AWQ_REQUIRE(kv_mul > 0 && num_heads % kv_mul == 0, AWQ_ERR_SHAPE, "kv_mul must divide num_heads");
    AWQ_REQUIRE(max_seq_len > 0, AWQ_ERR_SHAPE, "max_seq_len must be positive");
    switch (head_size) {
        case 64:
            return launch_attention<8>(ctx, output, q, key_cache, value_cache, att, num_heads, head_size, kv_mul, max_seq_len, pos);
        case 128:
            return launch_attention<16>(ctx, output, q, key_cache, value_cache, att, num_heads, head_size, kv_mul, max_seq_len, pos);
        case 256:
            return launch_attention<32>(ctx, output, q, key_cache, value_cache, att, num_heads, head_size, kv_mul, max_seq_len, pos);
        default:
            awq_set_error("awq_attention: head_size %d unsupported (64, 128 or 256)", head_size);
            return AWQ_ERR_SHAPE;
    }
}

int awq_attention_partial(awq_ctx* ctx, float* part, int* chunks, const uint16_t* q, const uint16_t* key_cache,
                          const uint16_t* value_cache, uint16_t* att, int num_heads, int head_size, int kv_mul, int max_seq_len,
                          const int* pos) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_REQUIRE(part && chunks && q && key_cache && value_cache && att && pos, AWQ_ERR_ARG, "null pointer");
    AWQ_REQUIRE(num_heads > 0 && num_heads <= kAttnMaxHeads, AWQ_ERR_SHAPE, "num_heads out of range");
    AWQ_REQUIRE(kv_mul > 0 && num_heads % kv_mul == 0, AWQ_ERR_SHAPE, "kv_mul must divide num_heads");
    AWQ_REQUIRE(max_seq_len > 0, AWQ_ERR_SHAPE, "max_seq_len must be positive");
    static_assert(kAttnMaxChunks == AWQ_ATTENTION_MAX_CHUNKS, "header and library disagree");
    return awq_launch_attention_partial(ctx, part, chunks, q, key_cache, value_cache, att, num_heads, head_size, kv_mul, max_seq_len,
                                        pos);
}

int awq_matvec_f16(awq_ctx* ctx, uint16_t* out, const uint16_t* x, const uint16_t* w, int n, int d) {
    if (int r = awq_bind(ctx)) return r;
    if (n <= 0 || d <= 0 || (n & 7) || (d & 7)) {  // llama2_q4.cu:358
        awq_set_error("unsupported matmul size n=%d d=%d (both must be positive multiples of 8)", n, d);
        return AWQ_ERR_SHAPE;
    }
    AWQ_REQUIRE(n <= kMaxStagedK, AWQ_ERR_SHAPE, "n exceeds the activations staged in LDS");
    AWQ_REQUIRE(out && x && w, AWQ_ERR_ARG, "null pointer");
    return awq_launch_matvec_f16(ctx, out, x, w, n, d, nullptr, nullptr);
}

int awq_argmax_advance(awq_ctx* ctx, const uint16_t* logits, int size, int* tokens, volatile int* pos_host, int* pos_dev,
                       int write_token) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_REQUIRE(logits && tokens && pos_host && pos_dev, AWQ_ERR_ARG, "null pointer");
    AWQ_REQUIRE(size > 0, AWQ_ERR_SHAPE, "size must be positive");
    return awq_launch_argmax(ctx, logits, size, tokens, pos_host, pos_dev, write_token, nullptr);
}

}  // extern "C"
