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

#include <mutex>

#include "common.hpp"

typedef _Float16 h16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace pf {

constexpr int BM = 128;  // tokens per tile
constexpr int BN = 128;  // weight rows per tile
constexpr int BK = 64;   // K per step: 128 bytes of fp16 per LDS tile row

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
    int mtiles, ntiles;
    int ksplit;                  // 1, or 2: two workgroups share a tile, each taking half of K
    float* part;                 // ksplit == 2: fp32 partial tiles [tile][2][128 x 128]
    unsigned int* part_counter;  // ksplit == 2: arrivals per tile, zero between launches
    // QKV with 128-wide heads: RoPE of the q and k tiles (one head each) in the epilogue, (cos, sin) from the table
    // [position][pair]; row m of the GEMM is position rope_pos0 + m.  Null: no rotation.
    const float2* rope;
    int rope_pos0;
    // FFN form: write the output with every 8 columns in the order (0,4,1,5,2,6,3,7), the order a permuted-A GEMM reads
    int out_perm;
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

// Where element j of a group of 8 sits in that order: (0,4,1,5,2,6,3,7) holds j at ((j & 3) << 1) | (j >> 2).
__device__ __forceinline__ int permuted_index(int c) { return (c & ~7) | ((c & 3) << 1) | ((c >> 2) & 1); }

// 8 nibbles of one dword -> 8 dequantised fp16 weights in the order (w0,w4)(w1,w5)(w2,w6)(w3,w7).
// magic = 0x64006400 held in a vector register: v_and_or_b32 takes no literal, and with the constant in a register
// the mask-and-merge of a nibble pair is one instruction.
__device__ __forceinline__ u32x4 dequant8(uint32_t d, uint32_t z, h16x2 s2, uint32_t magic) {
    const h16x2 zlo = as_h2(0xE400E400u | (z * 0x00010001u));  // -(1024 + z)
    const h16x2 zhi = as_h2(0xD400D400u | (z * 0x00100010u));  // -(64 + z)
    const h16x2 sixteenth = {(h16_t)0.0625f, (h16_t)0.0625f};
    const uint32_t d8 = d >> 8;
    const h16x2 t0 = as_h2((d & 0x000F000Fu) | magic) + zlo;                                      // exact q - z
    const h16x2 t1 = __builtin_elementwise_fma(as_h2((d & 0x00F000F0u) | magic), sixteenth, zhi);  // exact
    const h16x2 t2 = as_h2((d8 & 0x000F000Fu) | magic) + zlo;
    const h16x2 t3 = __builtin_elementwise_fma(as_h2((d8 & 0x00F000F0u) | magic), sixteenth, zhi);
    return u32x4{as_u32(t0 * s2), as_u32(t1 * s2), as_u32(t2 * s2), as_u32(t3 * s2)};  // one rounding each
}

// A tile's 128 columns are four blocks of 32 weight rows.  Which matrix a block belongs to and its first row:
// single / QKV: consecutive rows of one matrix; FFN: blocks alternate gate, up over the same 32 row indices, so that a
// wave (two adjacent blocks) holds a gate column and its up column in the same lane.
struct BlockMap {
    int mat, row0;
};

__device__ __forceinline__ BlockMap block_map(const GemmParams& p, int tile, int b) {
    BlockMap m;
    if (p.epi == EPI_FFN) {
        m.mat = b & 1;
        m.row0 = tile * 64 + (b >> 1) * 32;
        return m;
    }
    int mat = 0, tt = tile;
    if (p.epi == EPI_QKV) {
        const int t0 = p.N[0] / BN, t1 = p.N[1] / BN;
        if (tt >= t0 + t1) {
            mat = 2;
            tt -= t0 + t1;
        } else if (tt >= t0) {
            mat = 1;
            tt -= t0;
        }
    }
    m.mat = mat;
    m.row0 = tt * BN + b * 32;
    return m;
}

// The activation tile in LDS is [128 rows][64 halves] with the 16-byte chunk index XOR-ed with a key of the row, so
// that a wave's fragment reads (32 consecutive rows, one chunk) spread over all banks without padding.
__device__ __forceinline__ int lds_key(int row) { return (row ^ (row >> 3)) & 7; }
__device__ __forceinline__ int lds_off(int row, int chunk) { return row * BK + ((chunk ^ lds_key(row)) << 3); }

constexpr int A_STAGES = 3;                   // activation tiles in the LDS ring (2 steps ahead)
constexpr int W_STAGES = 3;                   // pairs of steps (one quantisation group) of packed weights in the LDS ring
constexpr int TILE_BYTES = BM * BK * 2;       // 16 KB
constexpr int W_WAVE_BYTES = 32 * 64 + 256 + 256;  // per wave and pair of steps: 32 rows x 64 packed bytes, zeros, scales
constexpr int W_STAGE_BYTES = 4 * W_WAVE_BYTES;
constexpr int GEMM_LDS_BYTES = A_STAGES * TILE_BYTES + W_STAGES * W_STAGE_BYTES;

// Direct global -> LDS loads: lane L's 16 (4) bytes land at lds_byte_off + 16 (4) * L.  Issued as inline assembly,
// so the compiler's wait-count bookkeeping does not see them; the kernel counts and waits for them itself.
__device__ __forceinline__ void dma16(const void* gptr, uint32_t lds_byte_off) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_byte_off), "v"(gptr) : "memory");
}
// Same with the address as a wave-uniform base plus a 32-bit byte offset per lane (no 64-bit vector arithmetic).
__device__ __forceinline__ void dma16(const void* sbase, uint32_t voff, uint32_t lds_byte_off) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_byte_off), "v"(voff), "s"(sbase) : "memory");
}
__device__ __forceinline__ void dma4(const void* gptr, uint32_t lds_byte_off) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(lds_byte_off), "v"(gptr) : "memory");
}

// inverse of permute8: (h0,h4)(h1,h5)(h2,h6)(h3,h7) -> (h0,h1)(h2,h3)(h4,h5)(h6,h7)
__device__ __forceinline__ u32x4 unpermute8(const u32x4 v) {
    u32x4 o;
    o[0] = __builtin_amdgcn_perm(v[1], v[0], 0x05040100u);
    o[1] = __builtin_amdgcn_perm(v[3], v[2], 0x05040100u);
    o[2] = __builtin_amdgcn_perm(v[1], v[0], 0x07060302u);
    o[3] = __builtin_amdgcn_perm(v[3], v[2], 0x07060302u);
    return o;
}

// C[m][n] = sum_k A[m][k] * half((q[n][k] - z) * s), tile 128 x 128, K step 64.
//  * Workgroup = 4 waves; wave w owns tile columns 32w .. 32w+31 and all 128 rows: four 32x32x16 fp16 MFMA
//    accumulators.  A lane's MFMA operand for the weights is 8 consecutive K of one weight row = one packed dword, so
//    dequantised weights never pass through LDS: lane (row l % 32, half l / 32) takes its row's 16 packed bytes of
//    the step and dequantises a dword right before the MFMAs that use it (bit-exact half((q-z)*s)).
//  * Every global load is a direct global -> LDS load.  The activation tile (16 KB, natural order, read by every
//    wave as fragments) travels two steps ahead into a ring of three tiles.  Packed weights travel per pair of steps
//    (128 K = one quantisation group: 64 contiguous bytes per row, one zero-point dword and one scale) two pairs
//    ahead into a ring that only the loading wave reads back, so they need no barrier.  LDS is the prefetch ring: no
//    register carries a load across iterations and one hand-counted s_waitcnt per step covers everything.
//  * One barrier per step.  The loop body has no conditional around its loads (steps past the end re-read the last
//    ones with zero scales), so the number of loads between a request and its use is constant.
// Workgroup ids are mapped so that the M tiles sharing a weight tile run on one XCD (ids go round-robin over the 8
// XCDs), which reads the weights from HBM once.
//
// APERM: every 16-byte chunk of A holds its 8 activations in the order (0,4,1,5,2,6,3,7), the order in which a packed
// dword dequantises.  Both MFMA operands contract over K, so any order they agree on gives the same products; with A
// already in that order the weights go into the MFMA as they come out of the dequantisation.  The prefill path writes
// its intermediate activations that way; the public entry points take A in natural order.
template <bool APERM>
__global__ __launch_bounds__(256, 2) void gemm_int4_kernel(const GemmParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_bytes[];  // [A ring][W ring]; nothing else is in LDS
    constexpr uint32_t W_RING = A_STAGES * TILE_BYTES;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int per_tile = p.mtiles * p.ksplit;
    const int tile = (slot / per_tile) * 8 + xcd;
    if (tile >= p.ntiles) return;
    const int m_index = (slot % per_tile) / p.ksplit, ks = (slot % per_tile) % p.ksplit;
    const int m0 = m_index * BM;

    // activation loader: wave w, instruction q covers tile rows (4w + q) * 8 .. + 8 (8 lanes x 16 bytes per row);
    // the lane's LDS chunk is lane & 7, so it fetches the source chunk that the swizzle maps there
    uint32_t a_off[4];  // byte offsets from p.A (a chunk of activations is far below 4 GB)
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int r = (wave * 4 + q) * 8 + (lane >> 3);
        const int c = (lane & 7) ^ lds_key(r);
        a_off[q] = (uint32_t)(((size_t)min(m0 + r, p.M - 1) * p.lda + c * 8) * 2);  // rows past M are computed, never stored
    }
    // weight loader: instruction q of a pair of steps covers the wave's rows 16q .. 16q+15, 4 lanes x 16 bytes per
    // row; 16-byte unit u of a row's 64 bytes sits at LDS unit u ^ ((row >> 1) & 3) (bank spread for the reads below)
    const BlockMap wb = block_map(p, tile, wave);
    const uint32_t* wmat = (wb.mat == 0 ? p.w[0] : (wb.mat == 1 ? p.w[1] : p.w[2]));
    const uint32_t* zmat = (wb.mat == 0 ? p.z[0] : (wb.mat == 1 ? p.z[1] : p.z[2]));
    const uint16_t* smat = (wb.mat == 0 ? p.s[0] : (wb.mat == 1 ? p.s[1] : p.s[2]));
    const uint32_t* w_src[2];
    int w_unit[2];
#pragma unroll
    for (int q = 0; q < 2; q++) {
        const int r = 16 * q + (lane >> 2);
        w_unit[q] = (lane & 3) ^ ((r >> 1) & 3);
        w_src[q] = wmat + (size_t)(wb.row0 + r) * (p.C * 4);
    }
    // consumer side: this lane's weight row and which 32-element half of a step it multiplies
    const int lrow = lane & 31, lhalf = lane >> 5;
    const uint32_t* zrow = zmat + (size_t)(wb.row0 + lrow) * p.pzh;
    const size_t s_row = (size_t)(wb.row0 + lrow) * p.sh;  // index of the row's first scale (scales travel as aligned dwords)
    const int n_groups = p.sh;

    uint32_t magic = 0x64006400u;
    asm("" : "+v"(magic));
    f32x16 acc[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 16; j++) acc[i][j] = 0.0f;

    const int nsteps = (p.K + BK - 1) / BK;
    const int k_last = (nsteps - 1) * BK;
    // split K: the halves meet at an even step, so that both start on a quantisation group
    const int s_split = (nsteps / 2) & ~1;
    const int s_begin = ks ? s_split : 0;
    const int s_end = (p.ksplit == 2 && ks == 0) ? s_split : nsteps;
    auto load_a = [&](int step) {  // 4 loads
        const int k0 = min(step * BK, k_last);
        const uint32_t dst = (uint32_t)((step % A_STAGES) * TILE_BYTES + wave * 4096);
#pragma unroll
        for (int q = 0; q < 4; q++) dma16(p.A + k0, a_off[q], dst + q * 1024);
    };
    auto load_w = [&](int pair) {  // 4 loads: K range [128 * pair, 128 * pair + 128) of the wave's 32 rows
        const uint32_t dst = W_RING + (uint32_t)((pair % W_STAGES) * W_STAGE_BYTES + wave * W_WAVE_BYTES);
#pragma unroll
        for (int q = 0; q < 2; q++) dma16(w_src[q] + (size_t)min(pair * 4 + w_unit[q], p.C - 1) * 4, dst + q * 1024);
        const int g = min(pair, n_groups - 1);
        dma4(zrow + (g >> 3), dst + 2048);
        dma4(smat + ((s_row + g) & ~(size_t)1), dst + 2304);
    };
    // K mapping of the four MFMAs of a step: MFMA j multiplies K chunk j (lanes 0-31) and chunk 4 + j (lanes 32-63),
    // i.e. dword j of each lane's 16 bytes against the matching 8 activations.
    auto compute = [&](int step) {
        const uint16_t* at = reinterpret_cast<const uint16_t*>(lds_bytes + (step % A_STAGES) * TILE_BYTES);
        const int pair = step >> 1;
        const uint8_t* ws = lds_bytes + W_RING + (pair % W_STAGES) * W_STAGE_BYTES + wave * W_WAVE_BYTES;
        const int unit = (step & 1) * 2 + lhalf;
        const u32x4 wq = *reinterpret_cast<const u32x4*>(ws + lrow * 64 + ((unit ^ ((lrow >> 1) & 3)) << 4));
        const uint32_t zw = *reinterpret_cast<const uint32_t*>(ws + 2048 + lane * 4);
        const uint32_t sw = *reinterpret_cast<const uint32_t*>(ws + 2304 + lane * 4);
        const int g = min(pair, n_groups - 1);
        const uint32_t z = (zw >> (4 * (g & 7))) & 0xFu;
        const uint16_t sbits = (uint16_t)(((s_row + g) & 1) ? (sw >> 16) : (sw & 0xFFFFu));
        const bool live = step * BK + lhalf * 32 < p.K;  // past K: zero scale, zero products
        const h16_t sh = __builtin_bit_cast(h16_t, live ? sbits : (uint16_t)0);
        const h16x2 s2 = {sh, sh};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const u32x4 dq = dequant8(wq[j], z, s2, magic);
            const h16x8 bf = __builtin_bit_cast(h16x8, APERM ? dq : unpermute8(dq));
            const int chunk = j + 4 * lhalf;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const h16x8 af = *reinterpret_cast<const h16x8*>(&at[lds_off(i * 32 + (lane & 31), chunk)]);
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf, acc[i], 0, 0, 0);
            }
        }
    };

    // Prologue: the first two activation tiles and weight pairs.
    load_a(s_begin);
    load_a(s_begin + 1);
    load_w(s_begin >> 1);
    load_w((s_begin >> 1) + 1);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    for (int step = s_begin; step < s_end; step += 2) {
        // even step: request activation tile step+2 and weight pair (step/2)+2, then multiply
        load_a(step + 2);  // into the slot that step-1 multiplied: every wave is past the barrier that ended it
        load_w((step >> 1) + 2);  // into the slot this wave finished reading at the end of the previous iteration
        compute(step);
        // needed next: activation tile step+1, requested in the previous iteration's odd half, followed by 4 + 4
        asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        __syncthreads();
        // odd step
        load_a(step + 3);
        compute(step + 1);
        // needed next: activation tile step+2 (followed by 4 + 4 loads) and weight pair (step/2)+1 (older still)
        asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        __syncthreads();
    }

    if (p.ksplit == 2) {
        // The two halves of K meet here.  Each workgroup writes its fp32 partial tile through to memory and counts
        // itself in; the first to arrive leaves, the second adds the other's partial to its own (a two-term fp32 sum
        // does not depend on which one that is) and goes on to the epilogue.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no direct-to-LDS load is still on its way
        __syncthreads();
        const size_t tile_id = (size_t)tile * p.mtiles + m_index;
        float* mine = p.part + (tile_id * 2 + ks) * (size_t)(BM * BN);
        const float* other = p.part + (tile_id * 2 + (ks ^ 1)) * (size_t)(BM * BN);
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 16; j++)
                __hip_atomic_store(&mine[((wave * 4 + i) * 16 + j) * 64 + lane], acc[i][j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        unsigned int* arrival = reinterpret_cast<unsigned int*>(lds_bytes);
        if (tid == 0) *arrival = __hip_atomic_fetch_add(&p.part_counter[tile_id], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (*arrival == 0u) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        if (tid == 0) p.part_counter[tile_id] = 0;  // ready for the next launch
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 16; j++) acc[i][j] += other[((wave * 4 + i) * 16 + j) * 64 + lane];
    }

    // ---- epilogue.  acc[i][j] is D[row = 32*i + 8*(j/4) + 4*(lane/32) + j%4][col = lane%32] of the wave's 32 columns:
    // a lane holds one column, so stored from registers every value would be a 2-byte access of its own (measured: 15 us
    // for the RoPE form, 12 for SiLU, 5 for the residual form, of a 50 us K loop).  The four waves therefore pass their
    // accumulators through the now idle LDS rings as one fp32 tile [wave][128 rows][32 columns], and every lane then
    // owns 8 consecutive columns of a row: one 16-byte store (and one 16-byte load of the old values, the rotation
    // factors or the partner columns) per 8 results.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no direct-to-LDS load is still on its way
    __syncthreads();
    float* tile_f = reinterpret_cast<float*>(lds_bytes);
    {
        float* mine = tile_f + wave * 4096 + (lane >> 5) * 128 + (lane & 31);
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 16; j++) mine[(i * 32 + (j >> 2) * 8 + (j & 3)) * 32] = acc[i][j];
    }
    __syncthreads();
    const int chunk = lane & 3, rsub = lane >> 2;  // 8 columns of row rsub, rsub + 16, ...
    auto read8 = [&](int w, int row, float (&v)[8]) {
        const f32x4* src = reinterpret_cast<const f32x4*>(tile_f + w * 4096 + row * 32 + chunk * 8);
        const f32x4 a = src[0], b = src[1];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            v[e] = a[e];
            v[4 + e] = b[e];
        }
    };
    auto pack8 = [](const float (&v)[8]) {
        u32x4 o;
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = (uint32_t)float_to_half_bits(v[2 * e]) | ((uint32_t)float_to_half_bits(v[2 * e + 1]) << 16);
        return o;
    };
    if (p.epi == EPI_FFN) {
        // waves 0, 2 hold gate columns, waves 1, 3 the up columns of the same weight rows: the two waves of a pair take
        // 64 tile rows each
        const int wg = wave & ~1;
        const int n0 = block_map(p, tile, wg).row0 + chunk * 8;
        uint16_t* o = p.out[0] + (size_t)p.out_off[0] + n0;
#pragma unroll
        for (int it = 0; it < 4; it++) {
            const int row = (wave & 1) * 64 + it * 16 + rsub;
            const int m = m0 + row;
            float g[8], u[8], v[8];
            read8(wg, row, g);
            read8(wg + 1, row, u);
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float s = g[e] * (1.0f / (1.0f + expf(-g[e])));
                v[e] = s * u[e];
            }
            if (p.out_perm) {  // (0,4,1,5,2,6,3,7): the order a permuted-A GEMM reads
                const float t[8] = {v[0], v[4], v[1], v[5], v[2], v[6], v[3], v[7]};
#pragma unroll
                for (int e = 0; e < 8; e++) v[e] = t[e];
            }
            if (m < p.M) *reinterpret_cast<u32x4*>(o + (size_t)m * p.ldo[0]) = pack8(v);
        }
        return;
    }
    const int mat = wb.mat;
    uint16_t* o = (mat == 0 ? p.out[0] : (mat == 1 ? p.out[1] : p.out[2])) +
                  (size_t)(mat == 0 ? p.out_off[0] : (mat == 1 ? p.out_off[1] : p.out_off[2])) + wb.row0 + chunk * 8;
    const size_t ld = (size_t)(mat == 0 ? p.ldo[0] : (mat == 1 ? p.ldo[1] : p.ldo[2]));
    if (p.rope && mat < 2) {
        // The tile is one head: column c < 64 rotates with column c + 64, which the wave two further on holds.  Values
        // are rounded to fp16 first and rotated in fp32, as the separate kernel does on the stored q and k
        // (gpu_kernels.h:351-361).  (cos, sin) of 8 consecutive pairs are 64 contiguous bytes of the table.
        const int pair0 = (wave & 1) * 32 + chunk * 8;  // 0 .. 63
#pragma unroll
        for (int it = 0; it < 8; it++) {
            const int row = it * 16 + rsub;
            const int m = m0 + row;
            const f32x4* cs = reinterpret_cast<const f32x4*>(p.rope + (size_t)(p.rope_pos0 + min(m, p.M - 1)) * 64 + pair0);
            const f32x4 c0 = cs[0], c1 = cs[1], c2 = cs[2], c3 = cs[3];
            const float cosv[8] = {c0[0], c0[2], c1[0], c1[2], c2[0], c2[2], c3[0], c3[2]};
            const float sinv[8] = {c0[1], c0[3], c1[1], c1[3], c2[1], c2[3], c3[1], c3[3]};
            float a[8], b[8], v[8];
            read8(wave, row, a);
            read8(wave ^ 2, row, b);
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float own = half_bits_to_float(float_to_half_bits(a[e]));
                const float other = half_bits_to_float(float_to_half_bits(b[e]));
                // columns below 64 are the first elements of their pairs, the others the second
                float r0, r1;
                if (wave < 2) rope_rotate(own, other, cosv[e], sinv[e], r0, r1);
                else rope_rotate(other, own, cosv[e], sinv[e], r0, r1);
                v[e] = wave < 2 ? r0 : r1;
            }
            if (m < p.M) *reinterpret_cast<u32x4*>(o + (size_t)m * ld) = pack8(v);
        }
        return;
    }
    // plain and residual forms; the old values of all 8 row passes are requested before the first is used
    u32x4 old[8];
    if (p.epi == EPI_RESID) {
#pragma unroll
        for (int it = 0; it < 8; it++)
            old[it] = *reinterpret_cast<const u32x4*>(o + (size_t)min(m0 + it * 16 + rsub, p.M - 1) * ld);
    }
#pragma unroll
    for (int it = 0; it < 8; it++) {
        const int row = it * 16 + rsub;
        const int m = m0 + row;
        float v[8];
        read8(wave, row, v);
        if (p.epi == EPI_RESID) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                v[2 * e] += half_bits_to_float((uint16_t)(old[it][e] & 0xFFFFu));
                v[2 * e + 1] += half_bits_to_float((uint16_t)(old[it][e] >> 16));
            }
        }
        if (m < p.M) *reinterpret_cast<u32x4*>(o + (size_t)m * ld) = pack8(v);
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

// o[m] = half(x[m] * (rsqrt(mean(x[m]^2) + 1e-5) * w))  (gpu_kernels.h:72-105, one workgroup per token row).
// 16-byte pieces; up to 4 per thread stay in registers between the two passes (rows of up to 8192), longer rows
// re-read the rest.
// perm: every 8 outputs are stored in the order (0,4,1,5,2,6,3,7) (what a permuted-A GEMM reads).
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(uint16_t* o, const uint16_t* x, const uint16_t* weight, int size, int perm) {
    __shared__ float red[4];
    constexpr int NP = 4;
    const int tid = threadIdx.x;
    const int n8 = size >> 3;
    const u32x4* xr = reinterpret_cast<const u32x4*>(x + (size_t)blockIdx.x * size);
    const u32x4* wr = reinterpret_cast<const u32x4*>(weight);
    u32x4* orow = reinterpret_cast<u32x4*>(o + (size_t)blockIdx.x * size);
    u32x4 v[NP], w[NP];
#pragma unroll
    for (int i = 0; i < NP; i++) {
        const int e = min(i * 256 + tid, n8 - 1);
        v[i] = xr[e];
        w[i] = wr[e];
    }
    auto sumsq = [](const u32x4 p, float part) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const h16x2 h = as_h2(p[k]);
            part = fmaf((float)h[0], (float)h[0], part);
            part = fmaf((float)h[1], (float)h[1], part);
        }
        return part;
    };
    auto scale = [perm](const u32x4 p, const u32x4 wv, float ss) {
        u32x4 r;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const h16x2 h = as_h2(p[k]), hw = as_h2(wv[k]);
            h16x2 q;
            q[0] = (h16_t)((float)h[0] * (ss * (float)hw[0]));
            q[1] = (h16_t)((float)h[1] * (ss * (float)hw[1]));
            r[k] = as_u32(q);
        }
        return perm ? permute8(r) : r;
    };
    float part = 0.0f;
#pragma unroll
    for (int i = 0; i < NP; i++)
        if (i * 256 + tid < n8) part = sumsq(v[i], part);
    for (int e = NP * 256 + tid; e < n8; e += 256) part = sumsq(xr[e], part);
    part = wave_sum(part);
    if ((tid & 63) == 0) red[tid >> 6] = part;
    __syncthreads();
    float ss = (red[0] + red[1]) + (red[2] + red[3]);
    ss /= (float)size;
    ss += 1e-5f;
    ss = 1.0f / sqrtf(ss);
#pragma unroll
    for (int i = 0; i < NP; i++)
        if (i * 256 + tid < n8) orow[i * 256 + tid] = scale(v[i], w[i], ss);
    for (int e = NP * 256 + tid; e < n8; e += 256) orow[e] = scale(xr[e], wr[e], ss);
}

// RoPE of q rows [M][heads*hs] and of the K cache rows pos0..pos0+M-1 (gpu_kernels.h:340-363 per position).
__global__ void rope_rows_kernel(uint16_t* q, uint16_t* kcache_layer, int num_heads, int num_kv_heads, int head_size, int pos0,
                                 float rope_theta, const float2* table) {
    const int m = blockIdx.y;
    const int h = blockIdx.x;
    const int i = threadIdx.x;
    const int pos = pos0 + m;
    const int half_size = head_size >> 1;
    float fcr, fci;
    if (table) {  // (cos, sin) per position and pair, computed once at load time with the formula below
        const float2 cs = table[(size_t)pos * half_size + i];
        fcr = cs.x;
        fci = cs.y;
    } else {
        const int head_dim = (i * 2) % head_size;
        const float freq = 1.0f / powf(rope_theta, head_dim / (float)head_size);
        const float val = pos * freq;
        fcr = cosf(val);
        fci = sinf(val);
    }
    uint16_t* qh = q + ((size_t)m * num_heads + h) * head_size;
    const float q0 = half_bits_to_float(qh[i]);
    const float q1 = half_bits_to_float(qh[i + half_size]);
    float r0, r1;
    rope_rotate(q0, q1, fcr, fci, r0, r1);
    qh[i] = float_to_half_bits(r0);
    qh[i + half_size] = float_to_half_bits(r1);
    if (h < num_kv_heads) {
        uint16_t* k = kcache_layer + ((size_t)pos * num_kv_heads + h) * head_size;
        const float k0 = half_bits_to_float(k[i]);
        const float k1 = half_bits_to_float(k[i + half_size]);
        rope_rotate(k0, k1, fcr, fci, r0, r1);
        k[i] = float_to_half_bits(r0);
        k[i + half_size] = float_to_half_bits(r1);
    }
}

// Causal attention for BQ consecutive query tokens of one head (query m attends to cache rows 0..pos0+m), with the
// reference's rounding points (llama2_q4.cu:410-427): scores -> fp16, probabilities -> fp16, output -> fp16.
constexpr int BQ = 16;

template <int LP>
__global__ __launch_bounds__(256) void attn_prefill_kernel(uint16_t* out, const uint16_t* q, const uint16_t* key_cache,
                                                           const uint16_t* value_cache, int num_heads, int head_size, int kv_mul,
                                                           int M, int pos0, int out_perm) {
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
                uint16_t* o = out + ((size_t)(mq0 + qi) * num_heads + h) * head_size;
                o[out_perm ? permuted_index(np * 2) : np * 2] = float_to_half_bits(acc[a][0]);
                o[out_perm ? permuted_index(np * 2 + 1) : np * 2 + 1] = float_to_half_bits(acc[a][1]);
            }
        }
    }
}

// Causal attention on the matrix cores for 128-wide heads: 32 consecutive query tokens of one head per workgroup.
// Same rounding points as above.
//  1. S = Q K^T: both MFMA operands are 8 consecutive head dims of a row, so q and k rows are loaded straight from
//     memory into fragments; wave w takes key blocks w, w+4, ...; scores go to LDS as fp16.
//  2. softmax per query row over its causal range, probabilities written back to LDS as fp16 (zero past the range).
//  3. O = P V: the weights operand needs 8 consecutive keys of one head dim, so value rows are transposed 8 x 8 in
//     registers on their way into LDS (64 keys per tile, next tile's rows in flight during the multiply); wave w
//     produces head dims 32w .. 32w+31.
constexpr int AQ = 32;        // queries per workgroup
constexpr int VT_STRIDE = 72; // halves per row of the transposed value tile (64 keys + 8 padding)
constexpr int KT_STRIDE = 136; // halves per row of a wave's key tile (128 dimensions + 8 padding)
static_assert(4 * 32 * KT_STRIDE <= 2 * 128 * VT_STRIDE, "the four key tiles share the value tiles' space");

// a / b correctly rounded, given rcp = 1 / b correctly rounded: the product a * rcp is within one unit of the quotient,
// and one step of a - b * q (exact in the fused multiply-add) times rcp puts it right (Markstein's correction; for
// 0 <= a <= 1 <= b no scaling is needed).  Three instructions where the division takes eleven.
__device__ __forceinline__ float quotient(float a, float b, float rcp) {
#pragma clang fp contract(off)
    const float q = a * rcp;
    const float e = __builtin_fmaf(-b, q, a);
    return __builtin_fmaf(e, rcp, q);
}

__global__ __launch_bounds__(256, 2) void attn_prefill_mfma_kernel(uint16_t* out, const uint16_t* q, const uint16_t* key_cache,
                                                                const uint16_t* value_cache, int num_heads, int kv_mul, int M,
                                                                int pos0, int s_stride, int out_perm) {
    constexpr int HS = 128;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    uint16_t* S = reinterpret_cast<uint16_t*>(smem);                          // [AQ][s_stride]
    uint16_t* Vt = reinterpret_cast<uint16_t*>(smem + AQ * s_stride * 2);     // [2][HS][VT_STRIDE]
    // Workgroup ids go round-robin over the 8 XCDs: all query blocks of a head run on one XCD, so that the head's key
    // and value rows come from memory into one L2 only (measured: with a head's blocks spread over all XCDs the score
    // phase was bound by 8 copies of every row crossing the fabric).  A head's blocks are dealt longest first; the
    // second half of an XCD's heads shortest first, so that the two workgroups of a compute unit tend to be one long
    // and one short.
    const int nqb = (M + AQ - 1) / AQ, hpx = (num_heads + 7) >> 3;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int h = xcd + 8 * (slot / nqb);
    if (h >= num_heads) return;
    const int qb = (slot / nqb) * 2 >= hpx ? slot % nqb : nqb - 1 - slot % nqb;
    const int mq0 = qb * AQ;
    const int nq = min(AQ, M - mq0);
    const int nk = pos0 + mq0 + nq;          // keys visible to the last query of the block
    const int nk_pad = (nk + 63) & ~63;      // <= s_stride - 8
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kv_dim = num_heads * HS / kv_mul;
    const float alpha = (float)(1.0 / sqrt((double)HS));
    const uint16_t* kh = key_cache + (size_t)(h / kv_mul) * HS;
    const uint16_t* vh = value_cache + (size_t)(h / kv_mul) * HS;
    const int l32 = lane & 31, lh = lane >> 5;

    // 1. scores
    h16x8 qf[8];
    {
        const uint16_t* qrow = q + ((size_t)min(mq0 + l32, M - 1) * num_heads + h) * HS + lh * 8;
#pragma unroll
        for (int f = 0; f < 8; f++) qf[f] = *reinterpret_cast<const h16x8*>(qrow + f * 16);
    }
    {
        // Each wave takes key blocks wave, wave + 4, ...; the rows of four of them are requested at once (512 keys are
        // one round trip to memory per wave).  The rows are loaded as they lie in memory, 16 lanes x 16 bytes per
        // 256-byte row, and turned into MFMA fragments through a tile of LDS private to the wave (the value tiles'
        // space, idle until phase 3): loaded straight as fragments, an instruction touches 32 rows with 32 bytes each,
        // and the address path of the compute unit takes twice as long over it (measured: 7 of the kernel's 20 us).
        // Every load is unconditional, rows past the end clamped to the last one: a load inside a branch is waited
        // for before the next one is issued.
        constexpr int KU = 4;
        uint16_t* kt = Vt + wave * (32 * KT_STRIDE);
        const int crow = lane >> 4, cpiece = lane & 15;
        for (int kb0 = wave; kb0 * 32 < nk_pad; kb0 += 4 * KU) {
            u32x4 kr[KU][8];
#pragma unroll
            for (int u = 0; u < KU; u++) {
#pragma unroll
                for (int r = 0; r < 8; r++) {
                    const int key = min((kb0 + 4 * u) * 32 + r * 4 + crow, nk - 1);
                    kr[u][r] = *reinterpret_cast<const u32x4*>(kh + (size_t)key * kv_dim + cpiece * 8);
                }
            }
            // (the compiler would otherwise move some of these loads down to their use, one wait each)
#pragma unroll
            for (int u = 0; u < KU; u++)
#pragma unroll
                for (int r = 0; r < 8; r++) asm volatile("" : "+v"(kr[u][r]));
#pragma unroll
            for (int u = 0; u < KU; u++) {
                const int kb = kb0 + 4 * u;
                if (kb * 32 < nk_pad) {
#pragma unroll
                    for (int r = 0; r < 8; r++)
                        *reinterpret_cast<u32x4*>(kt + (r * 4 + crow) * KT_STRIDE + cpiece * 8) = kr[u][r];
                    __builtin_amdgcn_wave_barrier();  // LDS serves a wave's accesses in order; this keeps the compiler from reordering them
                    h16x8 kf[8];
#pragma unroll
                    for (int f = 0; f < 8; f++) kf[f] = *reinterpret_cast<const h16x8*>(kt + l32 * KT_STRIDE + f * 16 + lh * 8);
                    __builtin_amdgcn_wave_barrier();
                    f32x16 acc;
#pragma unroll
                    for (int j = 0; j < 16; j++) acc[j] = 0.0f;
#pragma unroll
                    for (int f = 0; f < 8; f++) acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(qf[f], kf[f], acc, 0, 0, 0);
#pragma unroll
                    for (int j = 0; j < 16; j++) {
                        const int row = (j >> 2) * 8 + lh * 4 + (j & 3);
                        S[row * s_stride + kb * 32 + l32] = float_to_half_bits(acc[j] * alpha);
                    }
                }
            }
        }
    }
    // O = P V below stages the value rows through LDS, 8 keys x 8 dimensions per thread transposed in registers: the
    // waves 0-1 take the first 64 keys of a block of 128, the waves 2-3 the second.  The first two blocks are requested
    // here, so that they arrive while the softmax runs.
    const int kg = tid & 7, dc = (tid >> 3) & 15, vhalf = tid >> 7;
    u32x4 va[8], vb[8];
    auto load_v = [&](u32x4 (&vr)[8], int t0) {  // unconditional, rows past the end clamped
#pragma unroll
        for (int r = 0; r < 8; r++)
            vr[r] = *reinterpret_cast<const u32x4*>(vh + (size_t)min(t0 + vhalf * 64 + kg * 8 + r, nk - 1) * kv_dim + dc * 8);
    };
    load_v(va, 0);
    load_v(vb, 128);
    __syncthreads();
    // 2. softmax per query row; rows past nq get all-zero probabilities
    if (nk_pad <= 512) {
        // Eight lanes per row, the eight rows of a wave side by side: a lane holds up to 64 scores of its row in
        // registers (16-byte LDS accesses, one exponential per score), and the row's maximum and sum are reductions
        // over 8 lanes.  Row by row with the wave across one row, each row is a chain of dependent reductions with
        // nothing to overlap it (measured: 7 us for 32 rows of 32 scores).
        const int r8 = lane >> 3, l8 = lane & 7;
        const int qi = wave * 8 + r8;
        const int size = qi < nq ? pos0 + mq0 + qi + 1 : 0;
        uint16_t* srow = S + qi * s_stride;
        const int iters = nk_pad >> 6;  // chunks of 8 scores per lane
        float v[8][8];
        float m = (size < 1024) ? 0.0f : -INFINITY;  // the reference's idle-lane seed
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if (i < iters) {
                const int t0 = (l8 + 8 * i) * 8;
                const u32x4 raw = *reinterpret_cast<const u32x4*>(srow + t0);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const h16x2 hh = as_h2(raw[e]);
                    v[i][2 * e] = t0 + 2 * e < size ? (float)hh[0] : -INFINITY;
                    v[i][2 * e + 1] = t0 + 2 * e + 1 < size ? (float)hh[1] : -INFINITY;
                    m = fmaxf(m, fmaxf(v[i][2 * e], v[i][2 * e + 1]));
                }
            }
        }
        m = fmaxf(m, dpp_mov<0xB1>(m));
        m = fmaxf(m, dpp_mov<0x4E>(m));
        m = fmaxf(m, dpp_mov<0x141>(m));
        float sum = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if (i < iters) {
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    v[i][e] = expf(v[i][e] - m);  // exp(-inf) = 0 for the masked scores
                    sum += v[i][e];
                }
            }
        }
        sum = group_sum<8>(sum);
        if (size == 0) sum = 1.0f;  // a row past nq: all exponentials are zero, and so are the quotients
        const float rcp = 1.0f / sum;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if (i < iters) {
                const int t0 = (l8 + 8 * i) * 8;
                u32x4 o;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    h16x2 hh;
                    hh[0] = (h16_t)quotient(v[i][2 * e], sum, rcp);  // masked scores: 0 / sum
                    hh[1] = (h16_t)quotient(v[i][2 * e + 1], sum, rcp);
                    o[e] = as_u32(hh);
                }
                *reinterpret_cast<u32x4*>(srow + t0) = o;
            }
        }
    } else {
        // More than 512 keys: the same layout, with the scores read from LDS again in each of the three passes
        // (maximum, sum of exponentials, probabilities) instead of kept in registers.
        const int r8 = lane >> 3, l8 = lane & 7;
        const int qi = wave * 8 + r8;
        const int size = qi < nq ? pos0 + mq0 + qi + 1 : 0;
        uint16_t* srow = S + qi * s_stride;
        const int iters = nk_pad >> 6;
        auto scores8 = [&](int i, float (&x)[8]) {  // the lane's i-th chunk of 8 scores, masked ones as -inf
            const int t0 = (l8 + 8 * i) * 8;
            const u32x4 raw = *reinterpret_cast<const u32x4*>(srow + t0);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const h16x2 hh = as_h2(raw[e]);
                x[2 * e] = t0 + 2 * e < size ? (float)hh[0] : -INFINITY;
                x[2 * e + 1] = t0 + 2 * e + 1 < size ? (float)hh[1] : -INFINITY;
            }
        };
        float m = (size < 1024) ? 0.0f : -INFINITY;  // the reference's idle-lane seed
#pragma unroll 4
        for (int i = 0; i < iters; i++) {
            float x[8];
            scores8(i, x);
#pragma unroll
            for (int e = 0; e < 8; e++) m = fmaxf(m, x[e]);
        }
        m = fmaxf(m, dpp_mov<0xB1>(m));
        m = fmaxf(m, dpp_mov<0x4E>(m));
        m = fmaxf(m, dpp_mov<0x141>(m));
        if (size == 0) m = 0.0f;  // a row past nq (with the -inf seed of long contexts): keep exp(-inf - m) defined
        float sum = 0.0f;
#pragma unroll 2
        for (int i = 0; i < iters; i++) {
            float x[8];
            scores8(i, x);
#pragma unroll
            for (int e = 0; e < 8; e++) sum += expf(x[e] - m);
        }
        sum = group_sum<8>(sum);
        if (size == 0) sum = 1.0f;
        const float rcp = 1.0f / sum;
#pragma unroll 2
        for (int i = 0; i < iters; i++) {
            float x[8];
            scores8(i, x);
            u32x4 o;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                h16x2 hh;
                hh[0] = (h16_t)quotient(expf(x[2 * e] - m), sum, rcp);
                hh[1] = (h16_t)quotient(expf(x[2 * e + 1] - m), sum, rcp);
                o[e] = as_u32(hh);
            }
            *reinterpret_cast<u32x4*>(srow + (l8 + 8 * i) * 8) = o;
        }
    }
    // 3. O = P V, 128 keys per round: every thread transposes its 8 x 8 piece into the LDS tile of its half, then
    // every wave multiplies both tiles.  Value rows travel two rounds ahead of the multiply, in two register sets.
    auto store_v = [&](const u32x4 (&vr)[8]) {
        uint16_t* vt = Vt + vhalf * (HS * VT_STRIDE);
#pragma unroll
        for (int d = 0; d < 8; d++) {
            const uint32_t sel = (d & 1) ? 0x07060302u : 0x05040100u;
            u32x4 o;
#pragma unroll
            for (int r2 = 0; r2 < 4; r2++) o[r2] = __builtin_amdgcn_perm(vr[2 * r2 + 1][d >> 1], vr[2 * r2][d >> 1], sel);
            *reinterpret_cast<u32x4*>(&vt[(dc * 8 + d) * VT_STRIDE + kg * 8]) = o;
        }
    };
    f32x16 oacc;
#pragma unroll
    for (int j = 0; j < 16; j++) oacc[j] = 0.0f;
    auto multiply = [&](int t0, int buf) {
        const uint16_t* vt = Vt + buf * (HS * VT_STRIDE);
#pragma unroll
        for (int kc = 0; kc < 4; kc++) {
            const h16x8 pf = *reinterpret_cast<const h16x8*>(&S[l32 * s_stride + t0 + kc * 16 + lh * 8]);
            const h16x8 vf = *reinterpret_cast<const h16x8*>(&vt[(wave * 32 + l32) * VT_STRIDE + kc * 16 + lh * 8]);
            oacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(pf, vf, oacc, 0, 0, 0);
        }
    };
    for (int t0 = 0; t0 < nk_pad; t0 += 256) {
        store_v(va);
        load_v(va, t0 + 256);
        __syncthreads();  // the first one also orders the probabilities written above
        multiply(t0, 0);
        if (t0 + 64 < nk_pad) multiply(t0 + 64, 1);
        __syncthreads();  // every wave is done with the tiles before they are overwritten
        if (t0 + 128 >= nk_pad) break;
        store_v(vb);
        load_v(vb, t0 + 384);
        __syncthreads();
        multiply(t0 + 128, 0);
        if (t0 + 192 < nk_pad) multiply(t0 + 192, 1);
        __syncthreads();
    }
#pragma unroll
    for (int j = 0; j < 16; j++) {
        const int row = (j >> 2) * 8 + lh * 4 + (j & 3);
        const int d = wave * 32 + l32;
        if (row < nq) out[((size_t)(mq0 + row) * num_heads + h) * HS + (out_perm ? permuted_index(d) : d)] = float_to_half_bits(oacc[j]);
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

// ---------------------------------------------------------------- split-K workspace that needs no allocation
// awq_gemm_int4_static keeps the split-K workspace (fp32 partial tiles, then the per-tile arrival counters) in this
// file-scope device array instead of memory obtained with hipMalloc.  Every GPU the library runs on holds its own copy
// at its own address until the process ends.  In host code the array's name is only a stand-in for the symbol: the
// device address is looked up once per device with hipGetSymbolAddress and kept in g_scratch_ptr, and that pointer is
// what kernels and clears receive.
constexpr int kStaticTiles = 256;  // the split form is taken below 256 tiles only
constexpr size_t kStaticPartBytes = (size_t)kStaticTiles * 2 * pf::BM * pf::BN * sizeof(float);  // 32 MiB
constexpr size_t kStaticScratchBytes = kStaticPartBytes + kStaticTiles * sizeof(unsigned int);
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices];    // device address of `scratch` on each device, null until looked up
static bool g_gemm_lds_raised[kMaxDevices];  // the GEMM kernel's dynamic LDS limit has been raised on the device

namespace pf {
__global__ void clear_words_kernel(unsigned int* words, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) words[i] = 0u;
}
}  // namespace pf

// Once per device, with that device current: raise the GEMM kernel's LDS limit and look up the address of `scratch`.
// Called when a context is created, so that the entry points themselves do no set-up work.
int awq_gemm_device_setup(int device) {
    if (device < 0 || device >= kMaxDevices) {
        awq_set_error("device ordinal %d out of range", device);
        return AWQ_ERR_ARG;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_gemm_lds_raised[device]) {
        hipError_t e = hipFuncSetAttribute((const void*)pf::gemm_int4_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           pf::GEMM_LDS_BYTES);
        if (e == hipSuccess)
            e = hipFuncSetAttribute((const void*)pf::gemm_int4_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    pf::GEMM_LDS_BYTES);
        if (e != hipSuccess) {
            awq_set_error("hipFuncSetAttribute(gemm_int4) failed: %s", hipGetErrorString(e));
            return AWQ_ERR_HIP;
        }
        g_gemm_lds_raised[device] = true;
    }
    if (!g_scratch_ptr[device]) {
        void* ptr = nullptr;
        hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            awq_set_error("hipGetSymbolAddress(scratch) failed on device %d: %s", device, hipGetErrorString(e));
            return AWQ_ERR_HIP;
        }
        g_scratch_ptr[device] = ptr;
    }
    return AWQ_OK;
}

// ---------------------------------------------------------------- launchers (internal)
// static_ws: take the split-K workspace from the file-scope device array (no allocation) instead of the context's.
// a_perm: A holds every 8 activations in the order (0,4,1,5,2,6,3,7).
static int launch_gemm(awq_ctx* ctx, pf::GemmParams& p, int ntiles, const char* what, bool a_perm, bool static_ws = false) {
    // the kernel's 80 KB of LDS exceed the default dynamic limit; raised per device when a context is created
    // (contexts on a caller's stream included), here only for a device that was missed
    if (ctx->device < 0 || ctx->device >= kMaxDevices || !g_gemm_lds_raised[ctx->device]) {
        if (int r = awq_gemm_device_setup(ctx->device)) return r;
    }
    if ((size_t)p.M * (size_t)p.lda * 2 >= ((size_t)1 << 32)) {  // the kernel addresses A by 32-bit byte offsets
        awq_set_error("%s: activation block of %d x %d halves exceeds 4 GB", what, p.M, p.lda);
        return AWQ_ERR_SHAPE;
    }
    p.mtiles = div_up(p.M, pf::BM);
    p.ntiles = ntiles;
    p.ksplit = 1;
    // A single matrix with fewer tiles than compute units: two workgroups per tile, each half of K.
    if ((p.epi == pf::EPI_STORE || p.epi == pf::EPI_RESID) && p.mtiles * ntiles < 256 && p.K >= 8 * pf::BK) {
        const size_t tiles = (size_t)p.mtiles * ntiles;
        const size_t need = tiles * 2 * pf::BM * pf::BN * sizeof(float);
        if (static_ws) {
            if (tiles > (size_t)kStaticTiles) {
                awq_set_error("%s: %zu output tiles of 128 x 128 exceed the %d the static split-K workspace holds", what, tiles,
                              kStaticTiles);
                return AWQ_ERR_SHAPE;
            }
            unsigned char* ws = static_cast<unsigned char*>(g_scratch_ptr[ctx->device]);
            if (!ws) {
                awq_set_error("%s: the static workspace was not set up on device %d", what, ctx->device);
                return AWQ_ERR_HIP;
            }
            p.ksplit = 2;
            p.part = reinterpret_cast<float*>(ws);
            p.part_counter = reinterpret_cast<unsigned int*>(ws + kStaticPartBytes);
            // the array keeps whatever the previous call on this GPU left: the arrival counters must start at zero
            // (a fill kernel rather than a memset node, so that the call can be recorded into a graph)
            hipLaunchKernelGGL(pf::clear_words_kernel, dim3(div_up((int)tiles, 256)), dim3(256), 0, ctx->stream, p.part_counter,
                               (int)tiles);
            if (int r = awq_check_launch("clear_words")) return r;
        } else if (ctx->gemm_part_bytes < need || ctx->gemm_counter_count < tiles) {
            AWQ_HIP_TRY(hipStreamSynchronize(ctx->stream));
            if (ctx->gemm_part) (void)hipFree(ctx->gemm_part);
            if (ctx->gemm_counter) (void)hipFree(ctx->gemm_counter);
            ctx->gemm_part = nullptr;
            ctx->gemm_counter = nullptr;
            ctx->gemm_part_bytes = 0;
            ctx->gemm_counter_count = 0;
            AWQ_HIP_TRY(hipMalloc((void**)&ctx->gemm_part, need));
            AWQ_HIP_TRY(hipMalloc((void**)&ctx->gemm_counter, tiles * sizeof(unsigned int)));
            AWQ_HIP_TRY(hipMemset(ctx->gemm_counter, 0, tiles * sizeof(unsigned int)));
            ctx->gemm_part_bytes = need;
            ctx->gemm_counter_count = tiles;
        }
        if (!static_ws) {
            p.ksplit = 2;
            p.part = ctx->gemm_part;
            p.part_counter = ctx->gemm_counter;
        }
    }
    // ids go round-robin over the 8 XCDs; each XCD takes every 8th weight tile with all of its M tiles (and K halves)
    const int grid = 8 * p.mtiles * p.ksplit * div_up(ntiles, 8);
    if (a_perm)
        hipLaunchKernelGGL(pf::gemm_int4_kernel<true>, dim3(grid), dim3(256), pf::GEMM_LDS_BYTES, ctx->stream, p);
    else
        hipLaunchKernelGGL(pf::gemm_int4_kernel<false>, dim3(grid), dim3(256), pf::GEMM_LDS_BYTES, ctx->stream, p);
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
                           int K, int N, int accum, bool static_ws, bool a_perm) {
    pf::GemmParams p;
    gemm_common(p, A, lda, M, K, accum ? pf::EPI_RESID : pf::EPI_STORE);
    set_mat(p, 0, w, N, out, ldo, 0);
    return launch_gemm(ctx, p, N / pf::BN, "gemm_int4", a_perm, static_ws);
}

int awq_launch_gemm_qkv(awq_ctx* ctx, uint16_t* q, uint16_t* key_cache, uint16_t* value_cache, long long kv_row0_off,
                        const uint16_t* A, int lda, int M, const awq_qweight* qw, const awq_qweight* kw, const awq_qweight* vw,
                        int K, int Nq, int Nkv, const float2* rope128, int pos0, bool a_perm) {
    pf::GemmParams p;
    gemm_common(p, A, lda, M, K, pf::EPI_QKV);
    p.rope = rope128;  // non-null only with 128-wide heads
    p.rope_pos0 = pos0;
    set_mat(p, 0, qw, Nq, q, Nq, 0);
    set_mat(p, 1, kw, Nkv, key_cache, Nkv, kv_row0_off);
    set_mat(p, 2, vw, Nkv, value_cache, Nkv, kv_row0_off);
    return launch_gemm(ctx, p, (Nq + 2 * Nkv) / pf::BN, "gemm_int4_qkv", a_perm);
}

int awq_launch_gemm_ffn(awq_ctx* ctx, uint16_t* hb, const uint16_t* A, int lda, int M, const awq_qweight* gate_w,
                        const awq_qweight* up_w, int K, int N, bool a_perm, bool out_perm) {
    pf::GemmParams p;
    gemm_common(p, A, lda, M, K, pf::EPI_FFN);
    p.out_perm = out_perm;
    set_mat(p, 0, gate_w, N, hb, N, 0);
    set_mat(p, 1, up_w, N, hb, N, 0);
    return launch_gemm(ctx, p, N / 64, "gemm_int4_ffn", a_perm);
}

int awq_launch_embed_rows(awq_ctx* ctx, uint16_t* x, const uint16_t* table, int dim, const int* tokens, int pos0, int M) {
    hipLaunchKernelGGL(pf::embed_rows_kernel, dim3(M), dim3(256), 0, ctx->stream, x, table, dim, tokens, pos0);
    return awq_check_launch("embed_rows");
}

int awq_launch_rmsnorm_rows(awq_ctx* ctx, uint16_t* o, const uint16_t* x, const uint16_t* w, int size, int M, int perm) {
    hipLaunchKernelGGL(pf::rmsnorm_rows_kernel, dim3(M), dim3(256), 0, ctx->stream, o, x, w, size, perm);
    return awq_check_launch("rmsnorm_rows");
}

int awq_launch_rope_rows(awq_ctx* ctx, uint16_t* q, uint16_t* kcache_layer, int nh, int nkv, int hs, int pos0, float theta, int M,
                         const float2* table) {
    hipLaunchKernelGGL(pf::rope_rows_kernel, dim3(nh, M), dim3(hs / 2), 0, ctx->stream, q, kcache_layer, nh, nkv, hs, pos0, theta,
                       table);
    return awq_check_launch("rope_rows");
}

// Largest context (pos0 + M) the batched attention kernels take: they hold one fp16 score row per query in LDS.
int awq_prefill_attention_max_positions(int head_size) {
    const int lds_cap = 160 * 1024;
    if (head_size == 128) return ((lds_cap - 2 * 128 * pf::VT_STRIDE * 2) / (pf::AQ * 2) - 8) & ~63;
    return ((lds_cap - pf::BQ * head_size * 2 - pf::BQ * 8) / (pf::BQ * 2)) & ~7;
}

int awq_launch_attn_prefill(awq_ctx* ctx, uint16_t* out, const uint16_t* q, const uint16_t* kc, const uint16_t* vc, int nh, int hs,
                            int kv_mul, int M, int pos0, int out_perm) {
    if (hs == 128) {
        const int s_stride = ((pos0 + M + 63) & ~63) + 8;
        const size_t lds = (size_t)pf::AQ * s_stride * 2 + 2 * 128 * pf::VT_STRIDE * 2;
        if (lds > 160 * 1024) {
            awq_set_error("prefill attention: context of %d positions does not fit in LDS", pos0 + M);
            return AWQ_ERR_SHAPE;
        }
        if (lds > 64 * 1024) {
            hipError_t e = hipFuncSetAttribute((const void*)pf::attn_prefill_mfma_kernel,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) {
                awq_set_error("hipFuncSetAttribute(attn_prefill_mfma) failed: %s", hipGetErrorString(e));
                return AWQ_ERR_HIP;
            }
        }
        hipLaunchKernelGGL(pf::attn_prefill_mfma_kernel, dim3(8 * ((nh + 7) / 8) * div_up(M, pf::AQ)), dim3(256), lds, ctx->stream, out, q, kc, vc,
                           nh, kv_mul, M, pos0, s_stride, out_perm);
        return awq_check_launch("attn_prefill_mfma");
    }
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
                           M, pos0, out_perm);                                                                            \
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
    return awq_launch_gemm_single(ctx, out, ldo, a, lda, M, w, K, N, accum, false, false);
}

int awq_gemm_int4_static(awq_ctx* ctx, uint16_t* out, int ldo, const uint16_t* a, int lda, int M, const awq_qweight* w, int K,
                         int N, int accum) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_REQUIRE(out && a && w && w->weight && w->zeros && w->scales, AWQ_ERR_ARG, "null pointer");
    if (M <= 0 || K <= 0 || N <= 0 || (K & 31) || (N & 127) || (lda & 7)) {
        awq_set_error("awq_gemm_int4_static: needs M > 0, K %% 32 == 0, N %% 128 == 0, lda %% 8 == 0 (got M=%d K=%d N=%d lda=%d)", M, K, N,
                      lda);
        return AWQ_ERR_SHAPE;
    }
    AWQ_REQUIRE(ctx->device >= 0 && ctx->device < kMaxDevices && g_scratch_ptr[ctx->device] && g_gemm_lds_raised[ctx->device],
                AWQ_ERR_HIP, "the static workspace was not set up on this device when the context was created");
    return awq_launch_gemm_single(ctx, out, ldo, a, lda, M, w, K, N, accum, true, false);
}

}  // extern "C"
