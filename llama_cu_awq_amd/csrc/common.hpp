// Shared host/device helpers of libawq_hip (gfx950, wave64 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>
#include <stdio.h>

#include <vector>

#include "../../include/awq_hip.h"

// ---------------------------------------------------------------- host side
// While a context's `probe` is set, every kernel launched through awq_launch() carries an event pair that the
// runtime stamps with the kernel's own start and end (the launch-with-events form of the HIP extension API), tagged
// with the kind of schedule step that is current.
struct awq_launch_probe {
    std::vector<hipEvent_t> events;  // start, stop, start, stop, ...
    std::vector<int> kinds;          // one per pair
    int kind = 0;
};

struct awq_ctx {
    int device;
    int cus;  // compute units of `device` (launch geometry follows it)
    hipStream_t stream;
    bool owns_stream;
    awq_launch_probe* probe;  // null outside awq_transformer_time_launches
    // Workspace of the prefill GEMM's split-K form (allocated on first use): fp32 partial tiles and per-tile arrival
    // counters (self-resetting).
    float* gemm_part;
    size_t gemm_part_bytes;
    unsigned int* gemm_counter;
    size_t gemm_counter_count;
};

// Launch geometry of an int4 matrix-vector product as the dispatcher picks it (awq_gemv_geometry).
struct awq_gemv_geometry_t {
    int rows_per_group;  // consecutive rows (gate/up form: rows of each of the two matrices) that one workgroup takes at a time
    int groups;          // row groups in all
    int grid_x;          // workgroups along x; group g is read by workgroup g % grid_x
    int paired_rows;     // rows are dealt in rotation pairs (i, i + head/2): groups are not runs of consecutive rows
};

// What a kernel with idle workgroups may pull into the L2 caches for the launch that follows it.  L2 is per XCD and
// keeps clean lines across a kernel boundary (measured: a region of up to 32 MiB re-read by the next launch from the
// same XCDs streams at 14 TB/s with 0.28 us latency, against 7.5 TB/s and 0.93 us from HBM), and workgroup i of a
// launch runs on XCD i % 8, so a line helps only in the L2 of the XCD whose workgroup will read it.  A segment is a
// run of `nblocks` blocks of `block_bytes`; block j belongs to XCD j % 8.  nblocks == 0: the whole range
// [base, base + block_bytes) is wanted on every XCD.
struct awq_prefetch_seg {
    const char* base;
    uint32_t block_bytes;
    uint32_t nblocks;
    uint32_t lines_per_block;  // 128-byte lines a block can touch (one more than its size when it starts off a line)
    uint32_t inv_lines;        // floor(2^32 / lines_per_block) + 1: i / lines_per_block == mulhi(i, inv_lines) for i < 2^20
};
static inline awq_prefetch_seg awq_make_prefetch_seg(const void* base, size_t block_bytes, uint32_t nblocks) {
    awq_prefetch_seg sg;
    sg.base = reinterpret_cast<const char*>(base);
    sg.block_bytes = (uint32_t)block_bytes;
    sg.nblocks = nblocks;
    const uintptr_t b = reinterpret_cast<uintptr_t>(base);
    sg.lines_per_block = nblocks ? (uint32_t)((block_bytes + 127) / 128 + 1) : (uint32_t)(((b + block_bytes - 1) >> 7) - (b >> 7) + 1);
    sg.inv_lines = (uint32_t)(0x100000000ull / sg.lines_per_block) + 1;
    return sg;
}
constexpr int kPrefetchSegs = 12;
constexpr size_t kPrefetchBudgetBytes = (size_t)24 << 20;  // of the 32 MiB of L2, what one launch may ask for
struct awq_prefetch_plan {
    awq_prefetch_seg seg[kPrefetchSegs];
    int nseg;
};

constexpr int kAttnMaxHeads = 256;
constexpr int kAttnFusedMaxSeq = 256;  // up to this launch size attention runs as one workgroup per head
constexpr int kAttnMaxChunks = 4;      // ranges of positions whose partial P.V sums the O projection adds up
constexpr int kAttnSplitMinSeq = 1024;  // launch sizes from which the fused schedule splits P.V over positions

void awq_set_error(const char* fmt, ...);

#define AWQ_HIP_TRY(expr)                                                                      \
    do {                                                                                       \
        hipError_t e_ = (expr);                                                                \
        if (e_ != hipSuccess) {                                                                \
            awq_set_error("%s:%d: %s failed: %s", __FILE__, __LINE__, #expr, hipGetErrorString(e_)); \
            return AWQ_ERR_HIP;                                                                \
        }                                                                                      \
    } while (0)

#define AWQ_REQUIRE(cond, code, msg)                   \
    do {                                               \
        if (!(cond)) {                                 \
            awq_set_error("%s: %s", __func__, msg);    \
            return code;                               \
        }                                              \
    } while (0)

static inline int awq_bind(awq_ctx* ctx) {
    if (!ctx) {
        awq_set_error("null context");
        return AWQ_ERR_ARG;
    }
    AWQ_HIP_TRY(hipSetDevice(ctx->device));
    return AWQ_OK;
}

static inline int awq_check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        awq_set_error("launch of %s failed: %s", what, hipGetErrorString(e));
        return AWQ_ERR_HIP;
    }
    return AWQ_OK;
}

// Launch on the context's stream; with a probe set, through the extension launch that time-stamps the kernel itself.
template <typename... Args, typename F = void (*)(Args...)>
static inline void awq_launch(awq_ctx* ctx, F kernel, dim3 grid, dim3 block, size_t lds, Args... args) {
    if (ctx->probe) {
        hipEvent_t e0 = nullptr, e1 = nullptr;
        if (hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess) {
            hipExtLaunchKernelGGL(kernel, grid, block, (uint32_t)lds, ctx->stream, e0, e1, 0, args...);
            ctx->probe->events.push_back(e0);
            ctx->probe->events.push_back(e1);
            ctx->probe->kinds.push_back(ctx->probe->kind);
            return;
        }
        if (e0) (void)hipEventDestroy(e0);
    }
    hipLaunchKernelGGL(kernel, grid, block, lds, ctx->stream, args...);
}

static inline int div_up(int a, int b) { return (a + b - 1) / b; }
// Derived strides of a packed matrix (see awq_hip.h).
static inline int packed_weight_height(int K) { return div_up(K, 32) * 4; }
static inline int scales_height(int K) { return div_up(K, 128); }
static inline int packed_zeros_height(int K) { return div_up(scales_height(K), 8); }

// Largest reduction length the matrix-vector kernels stage in LDS (fp16
// activations, 2 bytes each, inside the 64 KB a workgroup may allocate).
constexpr int kMaxStagedK = 28672;

// ---------------------------------------------------------------- device side
#ifdef __HIPCC__

typedef _Float16 h16_t;
typedef _Float16 h16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ h16x2 as_h2(uint32_t u) { return __builtin_bit_cast(h16x2, u); }
__device__ __forceinline__ uint32_t as_u32(h16x2 h) { return __builtin_bit_cast(uint32_t, h); }
__device__ __forceinline__ float half_bits_to_float(uint16_t b) { return (float)__builtin_bit_cast(h16_t, b); }
__device__ __forceinline__ uint16_t float_to_half_bits(float f) { return __builtin_bit_cast(uint16_t, (h16_t)f); }  // RNE

// RoPE rotation of one pair, (v0, v1) -> (v0 c - v1 s, v0 s + v1 c) (gpu_kernels.h:355-361).  One fixed evaluation for
// every kernel that rotates (second product rounded on its own, first product fused with the sum), so that the
// separate kernel, the matrix-vector epilogue, the batched GEMM epilogue and the per-token kernel agree bit for bit
// whatever the compiler would have contracted in each of them.
__device__ __forceinline__ void rope_rotate(float v0, float v1, float c, float s, float& o0, float& o1) {
#pragma clang fp contract(off)
    const float t0 = v1 * s, t1 = v1 * c;
    o0 = __builtin_fmaf(v0, c, -t0);
    o1 = __builtin_fmaf(v0, s, t1);
}

// Streaming (non-temporal) loads for data that is read exactly once.
__device__ __forceinline__ u32x4 load_nt(const u32x4* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ uint32_t load_nt(const uint32_t* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ uint16_t load_nt(const uint16_t* p) { return __builtin_nontemporal_load(p); }

// fp32 += a.x*b.x + a.y*b.y (v_dot2_f32_f16)
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2(as_h2(a), as_h2(b), c, false);
}

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float read_lane(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// The row and half swaps of gfx950: v_permlane16_swap exchanges the odd rows (of 16 lanes) of its first operand with
// the even rows of the second, v_permlane32_swap the upper half of the first with the lower half of the second.  Fed
// the same value twice (in two registers) they leave the lane's own value in one and its partner's (lane ^ 16, lane ^
// 32) in the other, in the same order in both lanes.  Inline assembly: the compiler's builtin returns its first result
// twice; the s_nop cover the VALU-write -> permlane-read and permlane-write -> VALU-read hazards that the compiler
// cannot see through an asm statement.
__device__ __forceinline__ void swap16(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap32(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
// v + (v of lane ^ OFF) for OFF = 8, 16, 32 without a trip through the LDS crossbar.
template <int OFF>
__device__ __forceinline__ float lane_xor_sum(float v) {
    static_assert(OFF == 8 || OFF == 16 || OFF == 32, "unsupported distance");
    if (OFF == 8) return v + dpp_mov<0x128>(v);  // row_ror:8
    float a = v, b = v;
    if (OFF == 16) swap16(a, b); else swap32(a, b);
    return a + b;
}

// Touch the 128-byte lines of a prefetch plan that belong to XCD `xcd`, as workgroup `rank` of the `nranks` workgroups
// (of T threads) that share the job on that XCD: one dword per line.  The lines of all segments form one index space
// that the threads deal out among themselves, U to a thread per round, so that a round is one trip to memory whatever
// the mix of large and small segments.  The loads are ordinary loads whose values are folded into a word that an empty
// asm statement consumes at the end, so the compiler keeps them and does their wait-count bookkeeping itself.  (A load
// issued from inside an asm statement returns into its register long after the compiler has given that register to
// something else.)
template <int T>
__device__ __forceinline__ void prefetch_lines(const awq_prefetch_plan& plan, int xcd, int rank, int nranks) {
    constexpr int U = 2;
    auto lines_here = [&](const awq_prefetch_seg& sg) -> uint32_t {  // lines of this segment that belong to this XCD
        const uint32_t my_blocks = sg.nblocks ? (sg.nblocks + 7 - (uint32_t)xcd) >> 3 : 1u;
        return my_blocks * sg.lines_per_block;
    };
    uint32_t total = 0;
    for (int s = 0; s < plan.nseg; s++) total += lines_here(plan.seg[s]);
    if (total == 0) return;
    const uint32_t stride = (uint32_t)nranks * T, first = (uint32_t)rank * T + threadIdx.x;
    uint32_t seen = 0;
    for (uint32_t i0 = first; i0 < total; i0 += U * stride) {  // (threads past the end skip the round: nothing else needs them)
        uint32_t v[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            uint32_t i = i0 + u * stride;
            if (i >= total) i = total - 1;  // a line somebody else touches too
            int s = 0;
            uint32_t n = lines_here(plan.seg[0]);
            while (i >= n) {  // (total > i, so this ends inside the plan)
                i -= n;
                n = lines_here(plan.seg[++s]);
            }
            const awq_prefetch_seg sg = plan.seg[s];
            const uintptr_t base = reinterpret_cast<uintptr_t>(sg.base);
            const uint32_t blk = __umulhi(i, sg.inv_lines), line = i - blk * sg.lines_per_block;
            const uintptr_t span = sg.nblocks ? (uintptr_t)sg.block_bytes * sg.nblocks : (uintptr_t)sg.block_bytes;
            const uintptr_t start = sg.nblocks ? base + (uintptr_t)sg.block_bytes * ((uint32_t)xcd + 8 * blk) : base;
            uintptr_t a = (start & ~(uintptr_t)127) + (uintptr_t)line * 128;
            if (a < base) a = base;
            if (a > base + span - 4) a = base + span - 4;  // alignment slack past the end: clamped onto the last dword
            v[u] = *reinterpret_cast<const uint32_t*>(a);
        }
#pragma unroll
        for (int u = 0; u < U; u++) seen ^= v[u];
    }
    asm volatile("" ::"v"(seen));
}

// Sum within each aligned group of 16 lanes (a DPP row); every lane of the
// group ends up holding the group's sum.
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_mov<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_mov<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_mov<0x124>(v);  // row_ror:4
    v += dpp_mov<0x128>(v);  // row_ror:8
    return v;
}
// Sum over the 64 lanes of the wave; the result is wave-uniform.
__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    return (read_lane(v, 0) + read_lane(v, 16)) + (read_lane(v, 32) + read_lane(v, 48));
}
// Maximum over the 64 lanes, in every lane (DPP inside a row of 16, then the row and half swaps).
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_mov<0xB1>(v));
    v = fmaxf(v, dpp_mov<0x4E>(v));
    v = fmaxf(v, dpp_mov<0x124>(v));
    v = fmaxf(v, dpp_mov<0x128>(v));
    float a = v, b = v;
    swap16(a, b);
    a = b = fmaxf(a, b);
    swap32(a, b);
    return fmaxf(a, b);
}
// Sum within aligned groups of LP lanes (LP = 8, 16 or 32).
template <int LP>
__device__ __forceinline__ float group_sum(float v) {
    static_assert(LP == 8 || LP == 16 || LP == 32, "unsupported group width");
    v += dpp_mov<0xB1>(v);
    v += dpp_mov<0x4E>(v);
    if (LP == 8) {
        v += dpp_mov<0x141>(v);  // row_half_mirror: quads 0<->1 inside each 8 lanes
    } else {
        v += dpp_mov<0x124>(v);
        v += dpp_mov<0x128>(v);
        if (LP == 32) v = lane_xor_sum<16>(v);
    }
    return v;
}

#endif  // __HIPCC__
