// Single-workgroup attention for one head at short context (device function shared by the stand-alone kernel and
// by the QKV matrix-vector kernel, whose last-arriving workgroup of a head runs it).
//
// What it computes is MultiHeadAttention of the reference for one head (gpu_kernels.h:368-451): scores
// q.k * 1/sqrt(head_size) rounded to fp16, softmax over positions 0..pos in fp32 with the probabilities rounded to
// fp16, then the probability-weighted sum of the value rows in fp32, stored as fp16.  The fp16 scores are also left
// in att (the reference's att buffer holds them between its two phases).
#pragma once

#include "common.hpp"

// Floats of LDS the function needs for a context of at most max_seq positions.
__host__ __device__ constexpr int attention_head_lds_floats(int max_seq, int head_size, int waves) {
    return ((max_seq + 3) & ~3) + waves * head_size;
}

// LP = lanes per position (head_size / 8), NW = waves of the calling workgroup (all of them must call).
// lds: attention_head_lds_floats() floats, free for use.  k_head / v_head: the head's slice of row 0 of the layer's
// caches; rows are row_stride halves apart.
// NS > 1: NS workgroups share a head; each computes all scores but only the P.V of the value dimensions of its slice
// (lanes j with j / (LP / NS) == slice), so that a head's value rows come in through NS compute units.
template <int LP, int NW, int NS = 1>
__device__ __forceinline__ void attention_head(uint16_t* out_head, uint16_t* att_head, const uint16_t* q_head,
                                               const uint16_t* k_head, const uint16_t* v_head, int head_size,
                                               int row_stride, float alpha, int size, float* lds, int slice = 0) {
    float* sc = lds;                          // [size] scores (fp16-rounded values)
    float* acc_lds = lds + ((size + 3) & ~3);  // [NW][head_size]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    constexpr int PW = 64 / LP;
    const int j = lane % LP, pr = lane / LP;
    const int tstep = NW * PW;  // positions covered by the workgroup per round
    const int tfirst = wave * PW + pr;
    const u32x4 qv = *reinterpret_cast<const u32x4*>(q_head + j * 8);
    const uint16_t* kh = k_head + j * 8;
    const uint16_t* vh = v_head + j * 8;
    const bool mine = NS == 1 || j / (LP / NS) == slice;  // this lane's 8 value dimensions belong to the slice
    // The value rows of the first round are requested together with its key rows: at short context that is all of
    // them, and the softmax then runs while they are on their way.
    // Every load below is unconditional: positions past the end are clamped to the last one, and lanes whose value
    // dimensions belong to another slice re-read the query instead (one line for the whole wave).  A load inside a
    // branch makes the compiler wait for it before it issues the next one, which serialises the memory round trips.
    u32x4 vfirst[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int t = min(tfirst + k * tstep, size - 1);
        vfirst[k] = *reinterpret_cast<const u32x4*>(mine ? vh + (size_t)t * row_stride : q_head);
    }
    for (int t0 = tfirst; t0 - tfirst < size; t0 += 4 * tstep) {
        u32x4 kv[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int t = min(t0 + k * tstep, size - 1);
            kv[k] = *reinterpret_cast<const u32x4*>(kh + (size_t)t * row_stride);
        }
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int t = t0 + k * tstep;
            float s = 0.0f;
            if (t < size) {
#pragma unroll
                for (int i = 0; i < 4; i++) s = dot2(kv[k][i], qv[i], s);
            }
            s = group_sum<LP>(s);
            if (j == 0 && t < size) {
                const uint16_t hb = float_to_half_bits(s * alpha);
                if (NS == 1 || slice == 0) att_head[t] = hb;
                sc[t] = half_bits_to_float(hb);
            }
        }
    }
    __syncthreads();
    // Softmax statistics: every wave computes them for itself from the scores in LDS, all in the same order (lane l
    // takes positions l, l+64, ...; then the wave tree), so the values agree bit for bit and no further barrier or
    // exchange is needed.
    float m = (size < 1024) ? 0.0f : -INFINITY;  // the reference's idle-lane seed (its softmax block has 1024 threads)
    for (int t = lane; t < size; t += 64) m = fmaxf(m, sc[t]);
    m = wave_max(m);
    float sum = 0.0f;
    for (int t = lane; t < size; t += 64) sum += expf(sc[t] - m);
    sum = wave_sum(sum);

    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = 0.0f;
    for (int t0 = tfirst; t0 - tfirst < size; t0 += 4 * tstep) {
        u32x4 vv[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int t = t0 + k * tstep;
            if (t0 == tfirst)
                vv[k] = vfirst[k];
            else
                vv[k] = *reinterpret_cast<const u32x4*>(mine ? vh + (size_t)min(t, size - 1) * row_stride : q_head);
        }
        // The LP lanes of a position all need its probability.  With 16 lanes per position (one DPP row) lane k of
        // the row computes the one of round k (exponential and correctly rounded quotient once instead of four times
        // per lane) and the row takes it from there.
        float p_row = 0.0f;
        if (LP == 16) {
            const int t = t0 + min(j, 3) * tstep;
            if (j < 4 && t < size) p_row = half_bits_to_float(float_to_half_bits(expf(sc[t] - m) / sum));
        }
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int t = t0 + k * tstep;
            float pv;
            if (LP == 16)
                pv = k == 0 ? dpp_mov<0x150>(p_row) : k == 1 ? dpp_mov<0x151>(p_row) : k == 2 ? dpp_mov<0x152>(p_row) : dpp_mov<0x153>(p_row);
            if (t < size && mine) {
                if (LP != 16) pv = half_bits_to_float(float_to_half_bits(expf(sc[t] - m) / sum));
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const h16x2 hv = as_h2(vv[k][i]);
                    acc[2 * i] = fmaf((float)hv[0], pv, acc[2 * i]);
                    acc[2 * i + 1] = fmaf((float)hv[1], pv, acc[2 * i + 1]);
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 8; i++) {
        if (LP <= 8) acc[i] = lane_xor_sum<8>(acc[i]);
        if (LP <= 16) acc[i] = lane_xor_sum<16>(acc[i]);
        acc[i] = lane_xor_sum<32>(acc[i]);
    }
    if (pr == 0 && mine) {
#pragma unroll
        for (int i = 0; i < 8; i++) acc_lds[wave * head_size + j * 8 + i] = acc[i];
    }
    __syncthreads();
    const int d = NS == 1 ? tid : slice * (head_size / NS) + tid;  // output dimension of this thread
    if (tid < head_size / NS) {
        float total = 0.0f;
#pragma unroll
        for (int w = 0; w < NW; w++) total += acc_lds[w * head_size + d];
        out_head[d] = float_to_half_bits(total);
    }
}
