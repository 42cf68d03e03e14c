// Temperature / top-p sampling on the GPU: the non-greedy branch of the reference's sample()
// (sampler.h:85-115) and its kernels softmax_logits_kernel / sample_top_p_kernel (gpu_kernels.h:507-592).
//
// What the reference computes: logits / temperature rounded to fp16, softmax with the probabilities rounded to fp16,
// then (top-p on) a descending stable radix sort of the fp16 probabilities with their indices, an inclusive prefix sum
// stored as fp16, and the first sorted position whose prefix reaches coin * topp (coin when top-p is off, over the
// unsorted probabilities); position n-1 when none does.
//
// How it is done here: fp16 probabilities are multiples of 2^-24, so prefix sums are exact integers and do not depend
// on the order of additions; the prefix is rounded to fp16 once (round to nearest even), which makes "prefix reaches
// the threshold" a monotone test.  The sorted order never has to be materialised: one workgroup histograms the at
// most 15361 distinct probability values in LDS, walks the bins from the largest value down to the one where the
// exact prefix crosses, works out how many equal values into that bin the crossing is, and picks that many-th
// occurrence in index order (the radix sort is stable).  One launch for softmax and selection together, no temporary
// storage, capturable in a graph.
// (CUB's scan adds in fp16 in an order of its own, so the reference's prefix is one of several roundings of the same
// sums; this one is the unambiguous member of that family.)
#include <math.h>
#include <stdint.h>

#include <mutex>
#include <new>

#include "common.hpp"

namespace {

constexpr int kProbBins = 0x3C00 + 1;  // fp16 bit patterns of 0 .. 1.0
constexpr int kSampleThreads = 1024;

// Balanced pairwise tree over the workgroup's 1024 per-thread values (fixed order: within aligned lane pairs, quads,
// ... waves, then wave pairs); every thread gets the result.
__device__ __forceinline__ float block_sum_1024(float v, float* red) {
    v = wave_sum(v);  // balanced tree over the 64 lanes
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float r[16];
#pragma unroll
    for (int i = 0; i < 16; i++) r[i] = red[i];
#pragma unroll
    for (int n = 16; n > 1; n >>= 1)
#pragma unroll
        for (int i = 0; i < n / 2; i++) r[i] = r[2 * i] + r[2 * i + 1];
    __syncthreads();
    return r[0];
}
__device__ __forceinline__ float block_max_1024(float v, float* red) {
    v = wave_max(v);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float m = red[0];
#pragma unroll
    for (int i = 1; i < 16; i++) m = fmaxf(m, red[i]);
    __syncthreads();
    return m;
}

// ---------------------------------------------------------------------------------------------------------------
// The one workgroup keeps the vocabulary in registers: thread t holds elements t, t + 1024, ... (the reference's own
// assignment of elements to threads, gpu_kernels.h:515-556), at most kMaxRows of them.  The loops over them are
// unrolled, so the loads of a pass are all in flight together and no pass waits on memory between elements; only the
// index-order selection (top-p off), which needs a contiguous run of items per thread, goes through LDS.
constexpr int kMaxRows = 64;      // 65535 elements / 1024 threads, rounded up; vocabularies up to 32768 take 32 (no spills)
__host__ __device__ constexpr int staging_dwords_for(int n) { return ((n + 7) >> 3) * 4; }
constexpr int kMaxVocab = 1 << 20;  // above 65535 entries the large-vocabulary kernels take over
constexpr int kLdsVocab = 49152;  // the index-order selection holds vocabularies up to here in LDS (96 KB of fp16 values)

__host__ __device__ inline int staging_dwords(int n) { return n <= kLdsVocab ? staging_dwords_for(n) : 0; }

template <int NR>
struct Rows {
    uint32_t bits[NR];  // fp16 bit patterns; row r is element r * 1024 + threadIdx.x
};

// Between global memory and the rows lies a transposition (a thread's 16-byte load holds 8 neighbouring elements, its
// rows are 1024 elements apart); 2-byte global accesses would do it, at 128 bytes per wave instruction.  Vocabularies
// up to kLdsVocab go through LDS instead: 16-byte global accesses on one side, 2-byte LDS accesses on the other.
__device__ __forceinline__ void copy_values(uint16_t* dst, const uint16_t* src, int n, bool vec) {
    const int tid = threadIdx.x;
    if (vec) {  // both 16-byte aligned
        const int n8 = n >> 3;
        for (int e = tid; e < n8; e += kSampleThreads) reinterpret_cast<u32x4*>(dst)[e] = reinterpret_cast<const u32x4*>(src)[e];
        for (int i = n8 * 8 + tid; i < n; i += kSampleThreads) dst[i] = src[i];
    } else {
        for (int i = tid; i < n; i += kSampleThreads) dst[i] = src[i];
    }
}
__device__ __forceinline__ bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <int NR>
__device__ __forceinline__ void rows_load(Rows<NR>& x, const uint16_t* src, int n) {
#pragma unroll
    for (int r = 0; r < NR; r++) {
        x.bits[r] = 0u;
        if (r * kSampleThreads < n) x.bits[r] = src[min(r * kSampleThreads + (int)threadIdx.x, n - 1)];  // (uniform guard; lanes past n masked later)
    }
}
template <int NR>
__device__ __forceinline__ void rows_store(uint16_t* dst, const Rows<NR>& x, int n) {
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const int i = r * kSampleThreads + (int)threadIdx.x;
        if (i < n) dst[i] = (uint16_t)x.bits[r];
    }
}

// gpu_kernels.h:507-557 on the rows: half(l / T); v = expf(l - max), rounded to half, summed unrounded in fp32 (thread
// t adds its elements in order, then the balanced tree); p = half(float(half v) / sum).
// The same through a staging area in LDS (vals: n halves, rounded up to 8); direct for larger vocabularies.
template <int NR>
__device__ __forceinline__ void rows_load_staged(Rows<NR>& x, const uint16_t* src, int n, uint16_t* vals) {
    if (n > kLdsVocab) return rows_load(x, src, n);
    copy_values(vals, src, n, aligned16(src));
    __syncthreads();
    rows_load(x, vals, n);
}
template <int NR>
__device__ __forceinline__ void rows_store_staged(uint16_t* dst, const Rows<NR>& x, int n, uint16_t* vals) {
    if (n > kLdsVocab) return rows_store(dst, x, n);
    __syncthreads();  // (everyone has its rows out of the staging area)
    rows_store(vals, x, n);
    __syncthreads();
    copy_values(dst, vals, n, aligned16(dst));
}

template <int NR>
__device__ __forceinline__ void rows_softmax(Rows<NR>& x, int n, float temperature, float* red) {
    const int tid = threadIdx.x;
    // a / b for many a and one b: with r = 1 / b correctly rounded, q = a r, then q + (a - b q) r (the remainder exact
    // in one fused multiply-add) is the correctly rounded quotient, the same bits as the division (checked on the host
    // for every fp16 a against 3000 divisors), in 3 instructions instead of about 10; operands that are not finite (or
    // an r that is not) take the division itself
    auto quotient = [](float a, float b, float r, bool r_ok) {
        const float q = a * r;
        float q1 = __builtin_fmaf(__builtin_fmaf(-b, q, a), r, q);
        if (a == 0.0f) q1 = q;  // keeps the sign of a zero
        const bool bad = !(r_ok && __builtin_isfinite(q1));
        // (a wave-uniform branch: as a per-lane select the compiler evaluates the division for every element)
        if (__builtin_expect(__ballot(bad) != 0ull, 0)) q1 = bad ? a / b : q1;
        return q1;
    };
    const float r_temp = 1.0f / temperature;
    const bool r_temp_ok = __builtin_isfinite(r_temp) && r_temp != 0.0f;
    // rows below n / 1024 are full: only the last, partial row tests the element index (the row tests are uniform)
    const int full = n / kSampleThreads;
    float max_val = -3.402823466e+38f;  // -FLT_MAX
#pragma unroll
    for (int r = 0; r < NR; r++) {
        if (r < full || r * kSampleThreads + tid < n) {
            const uint16_t h = float_to_half_bits(quotient(half_bits_to_float((uint16_t)x.bits[r]), temperature, r_temp, r_temp_ok));
            x.bits[r] = h;
            max_val = fmaxf(max_val, half_bits_to_float(h));
        }
    }
    max_val = block_max_1024(max_val, red);
    float sum = 0.0f;
#pragma unroll
    for (int r = 0; r < NR; r++) {
        if (r < full || r * kSampleThreads + tid < n) {
            const float v = expf(half_bits_to_float((uint16_t)x.bits[r]) - max_val);
            x.bits[r] = float_to_half_bits(v);
            sum += v;
        }
    }
    sum = block_sum_1024(sum, red);
    const float r_sum = 1.0f / sum;
    const bool r_sum_ok = __builtin_isfinite(r_sum) && r_sum != 0.0f;
#pragma unroll
    for (int r = 0; r < NR; r++) {
        if (r < full || r * kSampleThreads + tid < n)
            x.bits[r] = float_to_half_bits(quotient(half_bits_to_float((uint16_t)x.bits[r]), sum, r_sum, r_sum_ok));
    }
}

template <int NR>
__global__ __launch_bounds__(kSampleThreads) void softmax_logits_kernel(uint16_t* logits, int size, float temperature) {
    extern __shared__ unsigned int dyn_lds[];  // staging area
    __shared__ float red[16];
    uint16_t* vals = reinterpret_cast<uint16_t*>(dyn_lds);
    Rows<NR> x;
    rows_load_staged(x, logits, size, vals);
    rows_softmax(x, size, temperature, red);
    rows_store_staged(logits, x, size, vals);
}

// value of an fp16 bit pattern in units of 2^-24 (exact; patterns 0 .. 0x3C00)
__device__ __forceinline__ unsigned long long prob_units(uint32_t bits) {
    const uint32_t e = bits >> 10, m = bits & 0x3FFu;
    return e == 0 ? (unsigned long long)m : ((unsigned long long)(m | 0x400u) << (e - 1));
}
// an exact sum of such values (units of 2^-24), rounded to fp16 with round-to-nearest-even, as a float
__device__ __forceinline__ float units_to_half_value(unsigned long long u) {
    if (u < 1024ull) return (float)(long long)u * 5.9604644775390625e-08f;  // subnormal or zero: exact
    const int e = 63 - __builtin_clzll(u);      // u in [2^e, 2^(e+1)), e >= 10
    const int shift = e - 10;
    unsigned long long mant = u >> shift;       // 11 significant bits
    const unsigned long long rem = u & ((1ull << shift) - 1ull);
    const unsigned long long half_ulp = shift ? (1ull << (shift - 1)) : 0ull;
    if (shift && (rem > half_ulp || (rem == half_ulp && (mant & 1ull)))) mant++;  // may become 2048: still exact below
    return ldexpf((float)(long long)mant, shift - 24);
}

// Exclusive prefix sum over the workgroup's 1024 per-thread values, in thread order (integers: exact in any grouping).
__device__ __forceinline__ unsigned long long block_exclusive_scan_1024(unsigned long long v, unsigned long long* wave_totals) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    unsigned long long inc = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const unsigned long long o = __shfl_up(inc, off);
        if (lane >= off) inc += o;
    }
    if (lane == 63) wave_totals[wave] = inc;
    __syncthreads();
    unsigned long long base = 0;
    for (int w = 0; w < wave; w++) base += wave_totals[w];
    __syncthreads();
    return base + inc - v;
}

struct SampleOut {
    int* result;
    volatile int* pPos;
    int* pPosGpu;
    int* mirror;
};

// p = position + 1; tokens[p] = idx; both copies of the position = p (the tail of sample_top_p_kernel,
// gpu_kernels.h:585-590).  The position is read from its device copy: the two are equal, and the pinned one is a trip
// over the host link away; the callers request it at their start (read_position), long before it is needed.
__device__ __forceinline__ int read_position(const SampleOut& out) { return threadIdx.x == 0 ? *out.pPosGpu : 0; }
__device__ __forceinline__ void write_token(const SampleOut& out, int idx, int token_pos) {
    token_pos++;
    out.result[token_pos] = idx;
    if (out.mirror) out.mirror[token_pos] = idx;
    *out.pPos = token_pos;
    *out.pPosGpu = token_pos;
}

// sampler.h:108-113 + gpu_kernels.h:562-592, top-p off: the first index whose exact prefix sum, rounded to fp16, reaches
// the threshold; n - 1 when none does.  probs in LDS or global memory.
__device__ __forceinline__ void select_in_index_order(const uint16_t* probs, int n, float threshold, const SampleOut out) {
    __shared__ unsigned long long wave_totals[16];
    __shared__ int s_best_thread;
    __shared__ int s_index;
    const int tid = threadIdx.x;
    const int token_pos = read_position(out);
    if (tid == 0) {
        s_best_thread = kSampleThreads;
        s_index = -1;
    }
    // a contiguous run of items per thread; totals (read in a rotated order, so that the lanes of a wave fall on
    // different LDS banks), exclusive scan, and the one thread whose run holds the crossing walks it
    const int per = (n + kSampleThreads - 1) / kSampleThreads;
    const int i0 = min(tid * per, n), i1 = min(i0 + per, n);
    unsigned long long total = 0;
    for (int k = 0; k < per; k++) {
        int i = i0 + k + (tid % per);
        if (i >= i0 + per) i -= per;
        if (i < i1) total += prob_units(probs[i]);
    }
    const unsigned long long before = block_exclusive_scan_1024(total, wave_totals);  // (its barriers also publish s_best_thread)
    const bool crosses = i1 > i0 && units_to_half_value(before + total) >= threshold;  // monotone in the thread index
    if (crosses) atomicMin(&s_best_thread, tid);
    __syncthreads();
    if (crosses && s_best_thread == tid) {
        unsigned long long run = before;
        for (int i = i0; i < i1; i++) {
            run += prob_units(probs[i]);
            if (units_to_half_value(run) >= threshold) {
                s_index = i;
                break;
            }
        }
    }
    __syncthreads();
    if (tid == 0) write_token(out, s_index >= 0 ? s_index : n - 1, token_pos);
}

// sampler.h:94-107 + gpu_kernels.h:562-592, top-p: position in the descending stable order of the probabilities at
// which the exact prefix sum, rounded to fp16, first reaches the threshold; the last position when none does.
// The items come from the thread's rows (vocabularies up to 65535: counters of 16 bits, two to a dword) or, WIDE, straight
// from global memory with one 32-bit counter per value (larger vocabularies: plain loops, no staging).
struct GlobalItems {
    const uint16_t* bits;
};
template <bool WIDE, class Items>
__device__ __forceinline__ void select_in_sorted_order(const Items& x, int n, float threshold, unsigned int* hist32, const SampleOut out) {
    auto hcount = [&](int b) -> unsigned int { return WIDE ? hist32[b] : (hist32[b >> 1] >> (16 * (b & 1))) & 0xFFFFu; };
    __shared__ unsigned long long wave_totals[16];
    __shared__ unsigned int counts[kSampleThreads];
    __shared__ int s_best_thread;
    __shared__ int s_bin;
    __shared__ unsigned int s_rank;
    __shared__ int s_index;
    __shared__ int s_hi;
    __shared__ unsigned long long s_start;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int token_pos = read_position(out);
    if (tid == 0) {
        s_best_thread = kSampleThreads;
        s_index = -1;
    }
    // histogram of the probability values.  Zeros (most of a peaked distribution) are counted per thread instead of
    // through the one LDS word they would all hit.
    for (int b = tid; b < (WIDE ? kProbBins : (kProbBins + 1) / 2); b += kSampleThreads) hist32[b] = 0u;
    __syncthreads();
    unsigned int zeros = 0;
    auto count_value = [&](uint32_t bits) {
        const int b = min((int)bits, kProbBins - 1);
        if (b == 0)
            zeros++;
        else if (WIDE)
            atomicAdd(&hist32[b], 1u);
        else
            atomicAdd(&hist32[b >> 1], (b & 1) ? 0x10000u : 1u);
    };
    if constexpr (WIDE) {
        for (int i = tid; i < n; i += kSampleThreads) count_value(x.bits[i]);
    } else {
#pragma unroll
        for (int r = 0; r < (int)(sizeof(x.bits) / sizeof(x.bits[0])); r++) {
            if (r * kSampleThreads + tid < n) count_value(x.bits[r]);
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) zeros += __shfl_xor(zeros, off);
    __syncthreads();
    if (lane == 0 && zeros) atomicAdd(&hist32[0], zeros);  // bin 0 is word 0, or its low half
    __syncthreads();
    // bins in descending order, a contiguous run per thread: thread 0 owns the largest values
    constexpr int BPT = (kProbBins + kSampleThreads - 1) / kSampleThreads;
    const int hi = kProbBins - 1 - tid * BPT;              // first (largest) bin of this thread
    const int lo = max(hi - BPT + 1, 0);                   // last bin (inclusive); empty range when hi < 0
    unsigned long long total = 0;
    unsigned int present = 0;
    for (int b = hi; b >= lo && b >= 0; b--) {
        const unsigned int c = hcount(b);
        present |= c;
        total += (unsigned long long)c * prob_units((uint32_t)b);
    }
    {
        // The first bin (in descending order) that holds a value and whose rounded prefix reaches the threshold lies in
        // the first thread that holds a value and whose prefix at the end of its run does (the prefix only grows, and
        // rounding is monotone).
        const unsigned long long start = block_exclusive_scan_1024(total, wave_totals);
        const bool crosses = present != 0u && units_to_half_value(start + total) >= threshold;
        if (crosses) atomicMin(&s_best_thread, tid);
        __syncthreads();
        if (crosses && s_best_thread == tid) {
            s_hi = hi;
            s_start = start;
        }
        __syncthreads();
        if (s_best_thread < kSampleThreads && wave == 0) {
            // The first wave looks at that thread's bins side by side: lane j at bin s_hi - j.
            static_assert(BPT <= 64, "a thread's bins fit the lanes of a wave");
            const int b = s_hi - lane;
            const bool valid = lane < BPT && b >= 0;
            const unsigned int c = valid ? hcount(b) : 0u;
            const unsigned long long add = (unsigned long long)c * prob_units((uint32_t)max(b, 0));
            unsigned long long inc = add;  // inclusive prefix over the lanes (descending bins)
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const unsigned long long o = __shfl_up(inc, off);
                if (lane >= off) inc += o;
            }
            const unsigned long long hits = __ballot(c != 0u && units_to_half_value(s_start + inc) >= threshold);
            const int first = __ffsll((long long)hits) - 1;  // some lane hits: the thread's last value crosses
            const int found = s_hi - first;
            const unsigned long long before = s_start + __shfl(inc - add, first);
            const unsigned int cnt = __shfl(c, first);
            // How many equal values into the bin the prefix first reaches the threshold: the smallest a in [1, cnt] with
            // rounded(before + a val) >= threshold (monotone; true at a = cnt), found 64 candidates at a time.
            const unsigned long long val = prob_units((uint32_t)found);
            unsigned int a_lo = 1, a_hi = cnt;
            while (a_lo < a_hi) {
                const unsigned int step = (a_hi - a_lo) / 64u + 1u;
                const unsigned int mine = min(a_lo + (unsigned int)(lane + 1) * step - 1u, a_hi);  // lane 63 reaches a_hi
                const unsigned long long t = __ballot(units_to_half_value(before + (unsigned long long)mine * val) >= threshold);
                const int f = __ffsll((long long)t) - 1;
                const unsigned int upper = __shfl(mine, f);
                const unsigned int below = f == 0 ? a_lo : __shfl(mine, max(f - 1, 0)) + 1u;
                a_lo = below;
                a_hi = upper;
            }
            if (lane == 0) {
                s_bin = found;
                s_rank = a_lo;  // 1-based occurrence, in index order
            }
        }
    }
    __syncthreads();
    if (s_best_thread >= kSampleThreads) {
        // nothing crossed: position n-1 of the sorted order = the last occurrence of the smallest value present
        if (tid == 0) {
            int b = 0;
            while (b < kProbBins - 1 && hcount(b) == 0u) b++;
            s_bin = b;
            s_rank = hcount(b);
        }
        __syncthreads();
    }
    const int target_bin = s_bin;
    const unsigned int target_rank = s_rank;
    // The target_rank-th element equal to target_bin, in index order (the radix sort is stable).
    bool unique = false;
    if constexpr (!WIDE) {
        // the usual case when the crossing lies among the likely tokens: the value occurs once, and whoever holds it
        // reports its index (no counting, no scan)
        unique = hcount(target_bin) == 1u;
        if (unique) {
            constexpr int NR = (int)(sizeof(x.bits) / sizeof(x.bits[0]));
#pragma unroll
            for (int r = 0; r < NR; r++) {
                if (r * kSampleThreads + tid < n && min((int)x.bits[r], kProbBins - 1) == target_bin) s_index = r * kSampleThreads + tid;
            }
        }
    }
    if (unique) {
    } else if constexpr (WIDE) {
        // a contiguous run of items per thread: matches counted per run, the counts scanned, and the thread whose run
        // holds the wanted match walks it
        const int per = (n + kSampleThreads - 1) / kSampleThreads;
        const int i0 = min(tid * per, n), i1 = min(i0 + per, n);
        unsigned int mine = 0;
        for (int i = i0; i < i1; i++) mine += (min((int)x.bits[i], kProbBins - 1) == target_bin);
        unsigned int seen = (unsigned int)block_exclusive_scan_1024((unsigned long long)mine, wave_totals);
        if (seen < target_rank && seen + mine >= target_rank) {
            for (int i = i0; i < i1; i++) {
                if (min((int)x.bits[i], kProbBins - 1) == target_bin && ++seen == target_rank) {
                    s_index = i;
                    break;
                }
            }
        }
    } else {
        // Index order is row by row, wave by wave, lane by lane: matches are counted per (row, wave) with a ballot, the
        // counts scanned in that order, and the lane whose match has the wanted number reports its index.
        constexpr int NR = (int)(sizeof(x.bits) / sizeof(x.bits[0]));
        counts[tid] = 0u;
        __syncthreads();
#pragma unroll
        for (int r = 0; r < NR; r++) {
            if (r * kSampleThreads < n) {  // uniform
                const bool m = r * kSampleThreads + tid < n && min((int)x.bits[r], kProbBins - 1) == target_bin;
                const unsigned long long bal = __ballot(m);
                if (lane == 0) counts[r * 16 + wave] = (unsigned int)__popcll(bal);
            }
        }
        __syncthreads();
        const unsigned int before_cell = (unsigned int)block_exclusive_scan_1024((unsigned long long)counts[tid], wave_totals);
        counts[tid] = before_cell;  // (every thread rewrites the cell it read itself; the scan ended with a barrier)
        __syncthreads();
#pragma unroll
        for (int r = 0; r < NR; r++) {
            if (r * kSampleThreads < n) {
                const bool m = r * kSampleThreads + tid < n && min((int)x.bits[r], kProbBins - 1) == target_bin;
                const unsigned long long bal = __ballot(m);
                if (m) {
                    const unsigned int seen = counts[r * 16 + wave] + (unsigned int)__popcll(bal & ((1ull << lane) - 1ull));
                    if (seen + 1u == target_rank) s_index = r * kSampleThreads + tid;
                }
            }
        }
    }
    __syncthreads();
    if (tid == 0) write_token(out, s_index >= 0 ? s_index : n - 1, token_pos);
}

template <int NR>
__global__ __launch_bounds__(kSampleThreads) void sample_sorted_kernel(const uint16_t* probs, int n, float threshold, int* result,
                                                                       volatile int* pPos, int* pPosGpu, int* mirror) {
    extern __shared__ unsigned int dyn_lds[];  // staging area, then the histogram
    Rows<NR> x;
    rows_load_staged(x, probs, n, reinterpret_cast<uint16_t*>(dyn_lds));
    select_in_sorted_order<false>(x, n, threshold, dyn_lds + staging_dwords(n), SampleOut{result, pPos, pPosGpu, mirror});
}

// Vocabularies above 65535 entries (up to kMaxVocab): the same arithmetic in plain loops over global memory.
__global__ __launch_bounds__(kSampleThreads) void softmax_logits_large_kernel(uint16_t* logits, int size, float temperature) {
    __shared__ float red[16];
    const int tid = threadIdx.x;
    float max_val = -3.402823466e+38f;  // -FLT_MAX
    for (int t = tid; t < size; t += kSampleThreads) {  // (a thread re-reads only what it wrote itself)
        const uint16_t h = float_to_half_bits(half_bits_to_float(logits[t]) / temperature);
        logits[t] = h;
        max_val = fmaxf(max_val, half_bits_to_float(h));
    }
    max_val = block_max_1024(max_val, red);
    float sum = 0.0f;
    for (int t = tid; t < size; t += kSampleThreads) {
        const float v = expf(half_bits_to_float(logits[t]) - max_val);
        logits[t] = float_to_half_bits(v);
        sum += v;
    }
    sum = block_sum_1024(sum, red);
    for (int t = tid; t < size; t += kSampleThreads) logits[t] = float_to_half_bits(half_bits_to_float(logits[t]) / sum);
}

__global__ __launch_bounds__(kSampleThreads) void sample_sorted_large_kernel(const uint16_t* probs, int n, float threshold, int* result,
                                                                             volatile int* pPos, int* pPosGpu, int* mirror) {
    extern __shared__ unsigned int dyn_lds[];  // the histogram, one word per value
    select_in_sorted_order<true>(GlobalItems{probs}, n, threshold, dyn_lds, SampleOut{result, pPos, pPosGpu, mirror});
}

__global__ __launch_bounds__(kSampleThreads) void sample_plain_kernel(const uint16_t* probs, int n, float threshold, int vec,
                                                                      int* result, volatile int* pPos, int* pPosGpu, int* mirror) {
    extern __shared__ unsigned int dyn_lds[];  // the values, for vocabularies up to kLdsVocab
    const SampleOut out{result, pPos, pPosGpu, mirror};
    if (n <= kLdsVocab) {
        uint16_t* vals = reinterpret_cast<uint16_t*>(dyn_lds);
        const int tid = threadIdx.x;
        if (vec) {  // probs is 16-byte aligned
            const int n8 = n >> 3;
            for (int e = tid; e < n8; e += kSampleThreads) reinterpret_cast<u32x4*>(vals)[e] = reinterpret_cast<const u32x4*>(probs)[e];
            for (int i = n8 * 8 + tid; i < n; i += kSampleThreads) vals[i] = probs[i];
        } else {
            for (int i = tid; i < n; i += kSampleThreads) vals[i] = probs[i];
        }
        __syncthreads();
        select_in_index_order(vals, n, threshold, out);
    } else {
        select_in_index_order(probs, n, threshold, out);
    }
}

// Both steps of the non-greedy branch of sample() in one launch: the probabilities are written back to the logits, as
// the reference's in-place softmax leaves them, and selected from the registers (top-p) or from LDS (index order;
// vocabularies up to kLdsVocab).
template <bool SORTED, int NR>
__global__ __launch_bounds__(kSampleThreads) void softmax_sample_kernel(uint16_t* logits, int n, float temperature, float threshold,
                                                                        int* result, volatile int* pPos, int* pPosGpu, int* mirror) {
    extern __shared__ unsigned int dyn_lds[];
    __shared__ float red[16];
    const SampleOut out{result, pPos, pPosGpu, mirror};
    uint16_t* vals = reinterpret_cast<uint16_t*>(dyn_lds);  // staging area; behind it the histogram (top-p)
    Rows<NR> x;
    rows_load_staged(x, logits, n, vals);
    rows_softmax(x, n, temperature, red);
    rows_store_staged(logits, x, n, vals);
    if (SORTED) {
        select_in_sorted_order<false>(x, n, threshold, dyn_lds + staging_dwords(n), out);
    } else {
        // (launched for n <= kLdsVocab only: the staging area holds the probabilities)
        __syncthreads();
        select_in_index_order(vals, n, threshold, out);
    }
}

}  // namespace

// Internal: greedy sampler (decode_ops.hip)
int awq_launch_argmax(awq_ctx* ctx, const uint16_t* logits, int size, int* tokens, volatile int* pos_host, int* pos_dev,
                      int write_token, int* tokens_mirror);

struct awq_sampler {
    awq_ctx* ctx;
    int vocab_size;
    float temperature;
    float topp;
    unsigned long long rng_state;
};

// xorshift* (sampler.h:65-74)
static unsigned int random_u32(unsigned long long* state) {
    *state ^= *state >> 12;
    *state ^= *state << 25;
    *state ^= *state >> 27;
    return (unsigned int)((*state * 0x2545F4914F6CDD1Dull) >> 32);
}
static float random_f32(unsigned long long* state) { return (random_u32(state) >> 8) / 16777216.0f; }

// Dynamic LDS of the kernels above: the staging area / the values (vocabularies up to kLdsVocab) and, behind it, the
// histogram of the top-p selection.
static size_t values_lds_bytes(int size) { return (size_t)staging_dwords(size) * 4; }
static size_t hist_lds_bytes() { return (size_t)((kProbBins + 1) / 2) * sizeof(unsigned int); }
static int pointer_is_16_byte_aligned(const void* p) { return ((uintptr_t)p & 15u) == 0 ? 1 : 0; }

// The kernels may take more than the default 64 KB of dynamic LDS: raised once per device.
constexpr int kMaxSamplerDevices = 64;
static std::mutex g_sampler_mutex;
static bool g_sampler_lds_raised[kMaxSamplerDevices];
static int raise_sampler_lds(awq_ctx* ctx) {
    if (ctx->device < 0 || ctx->device >= kMaxSamplerDevices) {
        awq_set_error("device ordinal %d out of range", ctx->device);
        return AWQ_ERR_ARG;
    }
    std::lock_guard<std::mutex> lock(g_sampler_mutex);
    if (g_sampler_lds_raised[ctx->device]) return AWQ_OK;
    const int bytes = (int)(values_lds_bytes(kLdsVocab) + hist_lds_bytes());
    const void* kernels[] = {(const void*)softmax_logits_kernel<32>,        (const void*)softmax_logits_kernel<kMaxRows>,
                             (const void*)sample_sorted_kernel<32>,         (const void*)sample_sorted_kernel<kMaxRows>,
                             (const void*)sample_plain_kernel,              (const void*)softmax_sample_kernel<true, 32>,
                             (const void*)softmax_sample_kernel<true, kMaxRows>, (const void*)softmax_sample_kernel<false, 32>,
                             (const void*)softmax_sample_kernel<false, kMaxRows>};
    for (const void* k : kernels) {
        const hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        if (e != hipSuccess) {
            awq_set_error("hipFuncSetAttribute(sampler kernels) failed: %s", hipGetErrorString(e));
            return AWQ_ERR_HIP;
        }
    }
    g_sampler_lds_raised[ctx->device] = true;
    return AWQ_OK;
}

static int launch_softmax_logits(awq_ctx* ctx, uint16_t* logits, int size, float temperature) {
    if (size > 65535) {
        hipLaunchKernelGGL(softmax_logits_large_kernel, dim3(1), dim3(kSampleThreads), 0, ctx->stream, logits, size, temperature);
        return awq_check_launch("softmax_logits");
    }
    if (int r = raise_sampler_lds(ctx)) return r;
    if (size <= 32 * kSampleThreads)
        hipLaunchKernelGGL(softmax_logits_kernel<32>, dim3(1), dim3(kSampleThreads), values_lds_bytes(size), ctx->stream, logits, size,
                           temperature);
    else
        hipLaunchKernelGGL(softmax_logits_kernel<kMaxRows>, dim3(1), dim3(kSampleThreads), values_lds_bytes(size), ctx->stream, logits,
                           size, temperature);
    return awq_check_launch("softmax_logits");
}

static int launch_sample(awq_ctx* ctx, const uint16_t* probs, int size, float threshold, int sorted, int* tokens,
                         volatile int* pos_host, int* pos_dev, int* mirror) {
    if (sorted && size > 65535) {
        hipLaunchKernelGGL(sample_sorted_large_kernel, dim3(1), dim3(kSampleThreads), (size_t)kProbBins * sizeof(unsigned int),
                           ctx->stream, probs, size, threshold, tokens, pos_host, pos_dev, mirror);
        return awq_check_launch("sample_top_p");
    }
    if (int r = raise_sampler_lds(ctx)) return r;
    if (sorted) {
        const size_t lds = values_lds_bytes(size) + hist_lds_bytes();
        if (size <= 32 * kSampleThreads)
            hipLaunchKernelGGL(sample_sorted_kernel<32>, dim3(1), dim3(kSampleThreads), lds, ctx->stream, probs, size, threshold,
                               tokens, pos_host, pos_dev, mirror);
        else
            hipLaunchKernelGGL(sample_sorted_kernel<kMaxRows>, dim3(1), dim3(kSampleThreads), lds, ctx->stream, probs, size, threshold,
                               tokens, pos_host, pos_dev, mirror);
    } else {
        hipLaunchKernelGGL(sample_plain_kernel, dim3(1), dim3(kSampleThreads), values_lds_bytes(size), ctx->stream, probs, size,
                           threshold, pointer_is_16_byte_aligned(probs), tokens, pos_host, pos_dev, mirror);
    }
    return awq_check_launch("sample_top_p");
}

static int launch_softmax_sample(awq_ctx* ctx, uint16_t* logits, int size, float temperature, float threshold, int sorted,
                                 int* tokens, volatile int* pos_host, int* pos_dev, int* mirror) {
    if (int r = raise_sampler_lds(ctx)) return r;
    if (sorted) {
        const size_t lds = values_lds_bytes(size) + hist_lds_bytes();
        if (size <= 32 * kSampleThreads)
            hipLaunchKernelGGL((softmax_sample_kernel<true, 32>), dim3(1), dim3(kSampleThreads), lds, ctx->stream, logits, size,
                               temperature, threshold, tokens, pos_host, pos_dev, mirror);
        else
            hipLaunchKernelGGL((softmax_sample_kernel<true, kMaxRows>), dim3(1), dim3(kSampleThreads), lds, ctx->stream, logits, size,
                               temperature, threshold, tokens, pos_host, pos_dev, mirror);
    } else {
        if (size <= 32 * kSampleThreads)
            hipLaunchKernelGGL((softmax_sample_kernel<false, 32>), dim3(1), dim3(kSampleThreads), values_lds_bytes(size), ctx->stream,
                               logits, size, temperature, threshold, tokens, pos_host, pos_dev, mirror);
        else
            hipLaunchKernelGGL((softmax_sample_kernel<false, kMaxRows>), dim3(1), dim3(kSampleThreads), values_lds_bytes(size),
                               ctx->stream, logits, size, temperature, threshold, tokens, pos_host, pos_dev, mirror);
    }
    return awq_check_launch("softmax_sample");
}

// Internal: sample() of the reference on the given state, with an optional device mirror of the token list.
int awq_sampler_run(awq_sampler* s, uint16_t* logits, int* tokens, volatile int* pos_host, int* pos_dev, int gen_token,
                    int* mirror) {
    const float coin = random_f32(&s->rng_state);  // drawn every step, greedy or not (sampler.h:79)
    if (s->temperature == 0.0f || !gen_token)
        return awq_launch_argmax(s->ctx, logits, s->vocab_size, tokens, pos_host, pos_dev, gen_token, mirror);
    const bool nucleus = s->topp > 0.0f && s->topp < 1.0f;
    const float threshold = nucleus ? coin * s->topp : coin;
    if (nucleus ? s->vocab_size <= 65535 : s->vocab_size <= kLdsVocab)  // softmax and selection in one launch
        return launch_softmax_sample(s->ctx, logits, s->vocab_size, s->temperature, threshold, nucleus ? 1 : 0, tokens, pos_host,
                                     pos_dev, mirror);
    if (int r = launch_softmax_logits(s->ctx, logits, s->vocab_size, s->temperature)) return r;
    return launch_sample(s->ctx, logits, s->vocab_size, threshold, nucleus ? 1 : 0, tokens, pos_host, pos_dev, mirror);
}

extern "C" {

int awq_softmax_logits(awq_ctx* ctx, uint16_t* logits, int size, float temperature) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_REQUIRE(logits && size > 0, AWQ_ERR_ARG, "null pointer or empty vector");
    AWQ_REQUIRE(temperature > 0.0f, AWQ_ERR_ARG, "temperature must be positive (0 selects the greedy sampler)");
    return launch_softmax_logits(ctx, logits, size, temperature);
}

int awq_sample_top_p(awq_ctx* ctx, const uint16_t* probs, int size, float threshold, int sorted, int* tokens,
                     volatile int* pos_host, int* pos_dev) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_REQUIRE(probs && tokens && pos_host && pos_dev && size > 0, AWQ_ERR_ARG, "null pointer or empty vector");
    AWQ_REQUIRE(size <= kMaxVocab, AWQ_ERR_SHAPE, "vocabularies above 1048576 entries are not supported by the sampler");
    return launch_sample(ctx, probs, size, threshold, sorted, tokens, pos_host, pos_dev, nullptr);
}

int awq_sampler_create(awq_ctx* ctx, int vocab_size, float temperature, float topp, unsigned long long rng_seed,
                       awq_sampler** out) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_REQUIRE(out && vocab_size > 0, AWQ_ERR_ARG, "null out or empty vocabulary");
    AWQ_REQUIRE(vocab_size <= kMaxVocab, AWQ_ERR_SHAPE, "vocabularies above 1048576 entries are not supported by the sampler");
    AWQ_REQUIRE(temperature >= 0.0f, AWQ_ERR_ARG, "negative temperature");
    awq_sampler* s = new (std::nothrow) awq_sampler();
    AWQ_REQUIRE(s, AWQ_ERR_ARG, "out of host memory");
    s->ctx = ctx;
    s->vocab_size = vocab_size;
    s->temperature = temperature;
    s->topp = topp;
    s->rng_state = rng_seed;
    *out = s;
    return AWQ_OK;
}

int awq_sampler_destroy(awq_sampler* s) {
    delete s;
    return AWQ_OK;
}

int awq_sampler_sample(awq_sampler* s, uint16_t* logits, int* tokens, volatile int* pos_host, int* pos_dev, int gen_token) {
    AWQ_REQUIRE(s, AWQ_ERR_ARG, "null sampler");
    if (int r = awq_bind(s->ctx)) return r;
    AWQ_REQUIRE(logits && tokens && pos_host && pos_dev, AWQ_ERR_ARG, "null pointer");
    return awq_sampler_run(s, logits, tokens, pos_host, pos_dev, gen_token, nullptr);
}

}  // extern "C"
