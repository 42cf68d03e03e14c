// Device-side building blocks of the int4 matrix-vector kernels (gemv_int4.hip): the dequantise-and-dot of one
// 32-element chunk, the register image of one 64-lane pass, and the staging of the activation vector into LDS.
#pragma once

#include "common.hpp"

namespace gemv {

// What staging needs to know about the activation vector.
struct XArgs {
    const uint16_t* x;       // K halves
    const uint16_t* norm_w;  // RMSNorm weights (NORM forms)
    uint16_t* norm_out;      // optional: workgroup (0, 0) also stores the normalised vector here
    int K;
    int C;                   // 32-element chunks = ceil(K / 32)
    const float* part;       // PARTS form: x = half(part[0][k] + part[1][k] + ...), rows K floats apart
    int parts;               // 1 .. kMaxParts
};
constexpr int kMaxParts = 4;

// 2^-20 * sum over the 32 consecutive K elements of one chunk of (q - z) * x.
//
// w: 4 dwords of 8 nibbles.  xq[qi]: the 8 activations of dword qi as fp16 pairs (x0,x4) (x1,x5) (x2,x6) (x3,x7),
// unscaled.  A nibble moved to bits 7..4 of an fp16 whose other bits are zero IS an fp16 number: the denormal
// 16 q * 2^-24 = q * 2^-20, exact, and v_dot2_f32_f16 takes denormal inputs at face value.  So a shift and a mask are
// the whole conversion, nothing has to be cancelled afterwards, and the activation enters the product as it is,
// whatever its size (the reference multiplies (q - z) * s * x in fp32, gpu_kernels.h:203-207).
//
// Why bits 7..4 and not the nibble where it lies: v_dot2_f32_f16 forms both products exactly but adds them and the
// accumulator inside a window of about 24 bits below the largest NOMINAL exponent of the three, truncating what falls
// below.  A denormal's nominal exponent is that of the smallest normal number, so a nibble in bits 3..0 sits 6 to 10
// bits below where the unit thinks it is and the accumulator loses that many bits at every step (measured at K = 4096:
// 4.6 % of the fp16 outputs rounded differently from the exact result, against 0.1 % for the reference's sequential
// fp32 sum and 0.07 % with every nibble in bits 7..4; bits 9..6 gain nothing more).  The price is two more shifts per
// dword.  The zero point comes in through the chunk's constant A = 2^-20 * sum x (computed once when x is staged): the
// accumulator starts at -z * A.  The caller multiplies the result by 2^20 * scale.
__device__ __forceinline__ float chunk_dot(const u32x4 w, const float zf, const u32x4 (&xq)[4], const float A) {
    float acc = -zf * A;
#pragma unroll
    for (int qi = 0; qi < 4; qi++) {
        const uint32_t d = w[qi];
        acc = dot2((d << 4) & 0x00F000F0u, xq[qi][0], acc);
        acc = dot2(d & 0x00F000F0u, xq[qi][1], acc);
        acc = dot2((d >> 4) & 0x00F000F0u, xq[qi][2], acc);
        acc = dot2((d >> 8) & 0x00F000F0u, xq[qi][3], acc);
    }
    return acc;
}
constexpr float kChunkDotUnscale = 1048576.0f;  // 2^20

// One 64-lane pass over the NS row streams of a wave: 16 bytes of packed weights per lane and stream, the zero-point
// dword and the scale that cover them, and (residual form) the value the result is added to.
template <int NS>
struct Stage {
    u32x4 w[NS];
    uint32_t zw[NS];
    uint16_t s[NS];
    uint16_t res[NS];
};

// Staging of x (K halves) into LDS: xs[qi*C + c] holds the 8 activations of dword qi of chunk c as pairs
// (x0,x4)(x1,x5)(x2,x6)(x3,x7), and ca[c] the chunk constant A described at chunk_dot.  Elements
// in [K, 32*C) are zero.  With NORM the vector is RMS-normalised on the way in with the reference's arithmetic
// (gpu_kernels.h:72-105): o = half(x * (rsqrt(mean(x^2) + 1e-5) * w)).
//
// Loads return in order, so the activations are requested (load_x) before the first stages of packed weights and
// staged (stage_x) while those are still on their way: XP pieces of 8 halves per thread travel in registers, the rest
// of a longer vector is fetched late by stage_x itself.
constexpr int XP = 2;
// 4-wave workgroups carry four pieces per thread, so that vectors up to 8192 elements travel in registers whole (the late
// fetch sits behind the staging barriers, one exposed round trip per 2048 elements: K = 5120 and 6656 at four waves),
// 16-wave workgroups three (K = 17920).
constexpr int pieces_for(int waves) { return waves <= 4 ? 4 : (waves >= 13 ? 3 : XP); }

template <bool NORM, int NP = XP>
struct XPieces {
    u32x4 v[NP];
    u32x4 w[NORM ? NP : 1];
};

template <int W, bool NORM>
__device__ __forceinline__ void load_x(XPieces<NORM, pieces_for(W)>& xr, const XArgs& p) {
    constexpr int XP = pieces_for(W);
    constexpr int T = W * 64;
    const int n8 = p.K >> 3;  // 8-half pieces of real data
    const u32x4* xg = reinterpret_cast<const u32x4*>(p.x);
    const u32x4* wg = reinterpret_cast<const u32x4*>(p.norm_w);
#pragma unroll
    for (int i = 0; i < XP; i++) {
        if (i > 0 && i * T >= n8) break;  // uniform: nothing left for this piece
        const int e = min(i * T + (int)threadIdx.x, n8 - 1);  // clamped, masked in stage_x
        xr.v[i] = xg[e];
        if (NORM) xr.w[i] = wg[e];
    }
}

// The PARTS form of load_x: the activation vector arrives as up to kMaxParts fp32 partial sums per element (the
// chunks of the position-split attention); their sum, added in part order and rounded to fp16 once, is x.  The loads
// are requested here, ahead of the packed weights; combine_x turns them into the pieces stage_x takes.
struct PartPieces {
    u32x4 f[XP][kMaxParts][2];  // 8 floats per piece and part
};

template <int W>
__device__ __forceinline__ void load_parts(PartPieces& pr, const XArgs& p) {
    constexpr int T = W * 64;
    const int n8 = p.K >> 3;
#pragma unroll
    for (int i = 0; i < XP; i++) {
        if (i > 0 && i * T >= n8) break;
        const int e = min(i * T + (int)threadIdx.x, n8 - 1);
#pragma unroll
        for (int s = 0; s < kMaxParts; s++) {
            if (s >= p.parts) break;  // uniform
            const u32x4* src = reinterpret_cast<const u32x4*>(p.part + (size_t)s * p.K) + 2 * e;
            pr.f[i][s][0] = src[0];
            pr.f[i][s][1] = src[1];
        }
    }
}

template <int W>
__device__ __forceinline__ void combine_x(XPieces<false, pieces_for(W)>& xr, const PartPieces& pr, const XArgs& p) {
    constexpr int T = W * 64;
    const int n8 = p.K >> 3;
#pragma unroll
    for (int i = 0; i < XP; i++) {
        if (i > 0 && i * T >= n8) break;
        // (a vector element goes through a scalar before the bit cast: cast directly, the element reference is
        // taken as the vector's storage and every lane of it reads element 0)
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t u = pr.f[i][0][j >> 2][j & 3];
            v[j] = __builtin_bit_cast(float, u);
        }
#pragma unroll
        for (int s = 1; s < kMaxParts; s++) {
            if (s >= p.parts) break;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const uint32_t u = pr.f[i][s][j >> 2][j & 3];
                v[j] += __builtin_bit_cast(float, u);
            }
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            h16x2 o;
            o[0] = (h16_t)v[2 * j];
            o[1] = (h16_t)v[2 * j + 1];
            xr.v[i][j] = as_u32(o);
        }
    }
}

// One piece of 8 halves: normalise (optional), permute, reduce the chunk constants over the 4 lanes of a chunk, store.
template <bool NORM>
__device__ __forceinline__ void stage_piece(u32x4* xs, float* ca, const XArgs& p, int e, u32x4 v, u32x4 wv, float ss,
                                            bool store_norm) {
    const int n8 = p.K >> 3;
    if (e >= n8) v = u32x4{0u, 0u, 0u, 0u};
    if (NORM) {
        // (float)h * f as fma(h, f, -0): exact, and the fp16 -> fp32 conversion rides in the multiply (v_fma_mix_f32);
        // the addend sits in a register the compiler cannot see through, or it would fold the fma away again
        float nz = -0.0f;
        asm("" : "+v"(nz));
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const h16x2 h = as_h2(v[i]);
            const h16x2 hw = as_h2(wv[i]);
            h16x2 o;
            o[0] = (h16_t)__builtin_fmaf((float)h[0], __builtin_fmaf((float)hw[0], ss, nz), nz);
            o[1] = (h16_t)__builtin_fmaf((float)h[1], __builtin_fmaf((float)hw[1], ss, nz), nz);
            v[i] = as_u32(o);
        }
        if (store_norm && e < n8) reinterpret_cast<u32x4*>(p.norm_out)[e] = v;
    }
    // v holds halves h0..h7 as (h0,h1)(h2,h3)(h4,h5)(h6,h7) -> (h0,h4)(h1,h5)(h2,h6)(h3,h7)
    const h16x2 p0 = as_h2(__builtin_amdgcn_perm(v[2], v[0], 0x05040100u));
    const h16x2 p1 = as_h2(__builtin_amdgcn_perm(v[2], v[0], 0x07060302u));
    const h16x2 p2 = as_h2(__builtin_amdgcn_perm(v[3], v[1], 0x05040100u));
    const h16x2 p3 = as_h2(__builtin_amdgcn_perm(v[3], v[1], 0x07060302u));
    // fp32 sum of the 8 halves: dot products against (1, 1)
    const uint32_t ones = 0x3C003C00u;
    float a = dot2(as_u32(p0), ones, dot2(as_u32(p1), ones, dot2(as_u32(p2), ones, dot2(as_u32(p3), ones, 0.0f))));
    // the 4 dword pieces of a chunk sit in 4 adjacent lanes
    a += dpp_mov<0xB1>(a);
    a += dpp_mov<0x4E>(a);
    if (e < p.C * 4) {
        u32x4 o = {as_u32(p0), as_u32(p1), as_u32(p2), as_u32(p3)};
        xs[(e & 3) * p.C + (e >> 2)] = o;
        if ((e & 3) == 0) ca[e >> 2] = a * (1.0f / kChunkDotUnscale);
    }
}

__device__ __forceinline__ float piece_sumsq(u32x4 v, float part) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const h16x2 h = as_h2(v[i]);
        const float a = (float)h[0], b = (float)h[1];
        part = fmaf(a, a, part);
        part = fmaf(b, b, part);
    }
    return part;
}

// red: W + 1 floats of LDS.
template <int W, bool NORM>
__device__ __forceinline__ void stage_x(u32x4* xs, float* ca, const XArgs& p, float* red, const XPieces<NORM, pieces_for(W)>& xr) {
    constexpr int XP = pieces_for(W);
    constexpr int T = W * 64;
    const int tid = threadIdx.x;
    const int n8 = p.K >> 3;
    const u32x4* xg = reinterpret_cast<const u32x4*>(p.x);
    const u32x4* wg = reinterpret_cast<const u32x4*>(p.norm_w);
    float ss = 0.0f;
    if (NORM) {
        float part = 0.0f;
#pragma unroll
        for (int i = 0; i < XP; i++)
            if (i * T + tid < n8) part = piece_sumsq(xr.v[i], part);
        for (int e = XP * T + tid; e < n8; e += T) part = piece_sumsq(xg[e], part);
        part = wave_sum(part);
        if ((tid & 63) == 0) red[tid >> 6] = part;
        __syncthreads();
        // the correctly rounded divide, square root and reciprocal are ~60 instructions on a uniform value: one wave
        // computes them for the workgroup
        if (tid < 64) {
            // pairwise tree over the waves' partial sums (wave counts that are no power of two: padded with zeros)
            constexpr int WP = W <= 4 ? 4 : (W <= 8 ? 8 : 16);
            float r[WP];
#pragma unroll
            for (int i = 0; i < WP; i++) r[i] = i < W ? red[i] : 0.0f;
#pragma unroll
            for (int n = WP; n > 1; n >>= 1)
#pragma unroll
                for (int i = 0; i < n / 2; i++) r[i] = r[2 * i] + r[2 * i + 1];
            float t = r[0];
            t /= (float)p.K;
            t += 1e-5f;
            t = 1.0f / sqrtf(t);
            if (tid == 0) red[W] = t;
        }
        __syncthreads();
        ss = red[W];
    }
    const bool store_norm = NORM && p.norm_out != nullptr && blockIdx.x == 0 && blockIdx.y == 0;
#pragma unroll
    for (int i = 0; i < XP; i++)
        if (i * T < p.C * 4)  // uniform: the quad reduction needs all lanes
            stage_piece<NORM>(xs, ca, p, i * T + tid, xr.v[i], xr.w[NORM ? i : 0], ss, store_norm);
    for (int e0 = XP * T; e0 < p.C * 4; e0 += T) {
        const int e = e0 + tid;
        const int ec = min(e, n8 - 1);
        const u32x4 v = xg[ec];
        u32x4 wv = v;
        if (NORM) wv = wg[ec];
        stage_piece<NORM>(xs, ca, p, e, v, wv, ss, store_norm);
    }
    __syncthreads();
}

}  // namespace gemv
