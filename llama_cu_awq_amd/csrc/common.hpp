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

constexpr int kAttnMaxHeads = 256;
constexpr int kAttnFusedMaxSeq = 256;  // up to this launch size attention runs as one workgroup per head
constexpr int kAttnMaxChunks = 4;      // ranges of positions whose partial P.V sums the O projection adds up
constexpr int kAttnSplitMinSeq = 1024;  // launch sizes from which the fused schedule splits P.V over positions ...
constexpr int kAttnSplitMinRange = 320;  // ... if a range then covers at least this many positions of the launch size

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
// The int4 kernels take rows up to here (68 bytes of LDS per 32 elements: 136 KB of the compute unit's 160 KB; above
// 64 KB a kernel's limit is raised on its first such launch on a device).
constexpr int kMaxStagedKInt4 = 65536;

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
