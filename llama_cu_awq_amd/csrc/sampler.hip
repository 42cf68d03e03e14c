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
// occurrence in index order (the radix sort is stable).  One launch, no temporary storage, capturable in a graph.
// (CUB's scan adds in fp16 in an order of its own, so the reference's prefix is one of several roundings of the same
// sums; this one is the unambiguous member of that family.)
#include <math.h>

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

// gpu_kernels.h:507-557, in place on the logits: half(l / T); v = expf(l - max), stored as half, summed unrounded in
// fp32 (thread t adds elements t, t+1024, ... in order, then the balanced tree); p = half(float(half v) / sum).
__global__ __launch_bounds__(kSampleThreads) void softmax_logits_kernel(uint16_t* logits, int size, float temperature) {
    __shared__ float red[16];
    const int tid = threadIdx.x;
    for (int t = tid; t < size; t += kSampleThreads) logits[t] = float_to_half_bits(half_bits_to_float(logits[t]) / temperature);
    __syncthreads();
    float max_val = -3.402823466e+38f;  // -FLT_MAX
    for (int t = tid; t < size; t += kSampleThreads) max_val = fmaxf(max_val, half_bits_to_float(logits[t]));
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

// sampler.h:94-115 + gpu_kernels.h:562-592.  sorted != 0: top-p path (descending stable order); else index order.
__global__ __launch_bounds__(kSampleThreads) void sample_kernel(const uint16_t* probs, int n, float threshold, int sorted,
                                                                int* result, volatile int* pPos, int* pPosGpu, int* mirror) {
    // counts per probability value, two 16-bit counters per dword (n <= 65535 on this path), sorted path only
    extern __shared__ unsigned int hist32[];
    auto hcount = [&](int b) -> unsigned int { return (hist32[b >> 1] >> (16 * (b & 1))) & 0xFFFFu; };
    __shared__ unsigned long long scan64[kSampleThreads];
    __shared__ int s_best_thread;
    __shared__ int s_bin;
    __shared__ unsigned int s_rank;
    __shared__ int s_index;
    const int tid = threadIdx.x;
    const int per = (n + kSampleThreads - 1) / kSampleThreads;  // contiguous items per thread
    const int i0 = min(tid * per, n), i1 = min(i0 + per, n);
    if (tid == 0) {
        s_best_thread = kSampleThreads;
        s_index = -1;
    }

    if (!sorted) {
        // exact prefix in index order: thread totals, exclusive scan, then a walk over the thread's own items
        unsigned long long total = 0;
        for (int i = i0; i < i1; i++) total += prob_units(probs[i]);
        scan64[tid] = total;
        __syncthreads();
        if (tid == 0) {  // 1024 additions: not worth a parallel scan
            unsigned long long run = 0;
            for (int t = 0; t < kSampleThreads; t++) {
                const unsigned long long v = scan64[t];
                scan64[t] = run;
                run += v;
            }
        }
        __syncthreads();
        unsigned long long run = scan64[tid];
        int found = -1;
        for (int i = i0; i < i1 && found < 0; i++) {
            run += prob_units(probs[i]);
            if (units_to_half_value(run) >= threshold) found = i;
        }
        if (found >= 0) atomicMin(&s_best_thread, tid);
        __syncthreads();
        if (found >= 0 && s_best_thread == tid) s_index = found;
        __syncthreads();
        if (tid == 0) {
            const int idx = s_index >= 0 ? s_index : n - 1;
            int token_pos = *pPos;
            token_pos++;
            result[token_pos] = idx;
            if (mirror) mirror[token_pos] = idx;
            *pPos = token_pos;
            *pPosGpu = token_pos;
        }
        return;
    }

    // ---- top-p: histogram of the probability values
    for (int b = tid; b < (kProbBins + 1) / 2; b += kSampleThreads) hist32[b] = 0u;
    __syncthreads();
    for (int i = i0; i < i1; i++) {
        const int b = min((int)probs[i], kProbBins - 1);
        atomicAdd(&hist32[b >> 1], (b & 1) ? 0x10000u : 1u);
    }
    __syncthreads();
    // bins in descending order, a contiguous run per thread: thread 0 owns the largest values
    constexpr int BPT = (kProbBins + kSampleThreads - 1) / kSampleThreads;
    const int hi = kProbBins - 1 - tid * BPT;              // first (largest) bin of this thread
    const int lo = max(hi - BPT + 1, 0);                   // last bin (inclusive); empty range when hi < 0
    unsigned long long total = 0;
    for (int b = hi; b >= lo && b >= 0; b--) total += (unsigned long long)hcount(b) * prob_units((uint32_t)b);
    scan64[tid] = total;
    __syncthreads();
    if (tid == 0) {
        unsigned long long run = 0;
        for (int t = 0; t < kSampleThreads; t++) {
            const unsigned long long v = scan64[t];
            scan64[t] = run;
            run += v;
        }
    }
    __syncthreads();
    {
        unsigned long long run = scan64[tid];
        int found = -1;
        unsigned long long before = 0;
        for (int b = hi; b >= lo && b >= 0 && found < 0; b--) {
            const unsigned long long add = (unsigned long long)hcount(b) * prob_units((uint32_t)b);
            if (hcount(b) && units_to_half_value(run + add) >= threshold) {
                found = b;
                before = run;
            }
            run += add;
        }
        if (found >= 0) atomicMin(&s_best_thread, tid);
        __syncthreads();
        if (found >= 0 && s_best_thread == tid) {
            // how many equal values into the bin the prefix first reaches the threshold (monotone: binary search)
            const unsigned long long val = prob_units((uint32_t)found);
            unsigned int a = 1, c = hcount(found);
            while (a < c) {
                const unsigned int mid = (a + c) >> 1;
                if (units_to_half_value(before + (unsigned long long)mid * val) >= threshold)
                    c = mid;
                else
                    a = mid + 1;
            }
            s_bin = found;
            s_rank = a;  // 1-based occurrence, in index order
        }
    }
    __syncthreads();
    int target_bin;
    unsigned int target_rank;
    if (s_best_thread < kSampleThreads) {
        target_bin = s_bin;
        target_rank = s_rank;
    } else {
        // nothing crossed: position n-1 of the sorted order = the last occurrence of the smallest value present
        if (tid == 0) {
            int b = 0;
            while (b < kProbBins - 1 && hcount(b) == 0u) b++;
            s_bin = b;
            s_rank = hcount(b);
        }
        __syncthreads();
        target_bin = s_bin;
        target_rank = s_rank;
    }
    // the target_rank-th element equal to target_bin, in index order
    unsigned int mine = 0;
    for (int i = i0; i < i1; i++) mine += (min((int)probs[i], kProbBins - 1) == target_bin);
    __syncthreads();  // s_bin / s_rank read by everyone before scan64 is reused
    scan64[tid] = mine;
    __syncthreads();
    if (tid == 0) {
        unsigned long long run = 0;
        for (int t = 0; t < kSampleThreads; t++) {
            const unsigned long long v = scan64[t];
            scan64[t] = run;
            run += v;
        }
    }
    __syncthreads();
    {
        unsigned int seen = (unsigned int)scan64[tid];
        if (seen < target_rank && seen + mine >= target_rank) {
            for (int i = i0; i < i1; i++) {
                if (min((int)probs[i], kProbBins - 1) == target_bin && ++seen == target_rank) {
                    s_index = i;
                    break;
                }
            }
        }
    }
    __syncthreads();
    if (tid == 0) {
        const int idx = s_index >= 0 ? s_index : n - 1;
        int token_pos = *pPos;
        token_pos++;
        result[token_pos] = idx;
        if (mirror) mirror[token_pos] = idx;
        *pPos = token_pos;
        *pPosGpu = token_pos;
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

static int launch_softmax_logits(awq_ctx* ctx, uint16_t* logits, int size, float temperature) {
    hipLaunchKernelGGL(softmax_logits_kernel, dim3(1), dim3(kSampleThreads), 0, ctx->stream, logits, size, temperature);
    return awq_check_launch("softmax_logits");
}

static int launch_sample(awq_ctx* ctx, const uint16_t* probs, int size, float threshold, int sorted, int* tokens,
                         volatile int* pos_host, int* pos_dev, int* mirror) {
    const size_t lds = sorted ? (size_t)((kProbBins + 1) / 2) * sizeof(unsigned int) : 0;
    hipLaunchKernelGGL(sample_kernel, dim3(1), dim3(kSampleThreads), lds, ctx->stream, probs, size, threshold, sorted, tokens,
                       pos_host, pos_dev, mirror);
    return awq_check_launch("sample_top_p");
}

// Internal: sample() of the reference on the given state, with an optional device mirror of the token list.
int awq_sampler_run(awq_sampler* s, uint16_t* logits, int* tokens, volatile int* pos_host, int* pos_dev, int gen_token,
                    int* mirror) {
    const float coin = random_f32(&s->rng_state);  // drawn every step, greedy or not (sampler.h:79)
    if (s->temperature == 0.0f || !gen_token)
        return awq_launch_argmax(s->ctx, logits, s->vocab_size, tokens, pos_host, pos_dev, gen_token, mirror);
    if (int r = launch_softmax_logits(s->ctx, logits, s->vocab_size, s->temperature)) return r;
    const bool nucleus = s->topp > 0.0f && s->topp < 1.0f;
    const float threshold = nucleus ? coin * s->topp : coin;
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
    AWQ_REQUIRE(size <= 65535, AWQ_ERR_SHAPE, "vocabularies above 65535 entries are not supported by the sampler");
    return launch_sample(ctx, probs, size, threshold, sorted, tokens, pos_host, pos_dev, nullptr);
}

int awq_sampler_create(awq_ctx* ctx, int vocab_size, float temperature, float topp, unsigned long long rng_seed,
                       awq_sampler** out) {
    if (int r = awq_bind(ctx)) return r;
    AWQ_REQUIRE(out && vocab_size > 0, AWQ_ERR_ARG, "null out or empty vocabulary");
    AWQ_REQUIRE(vocab_size <= 65535, AWQ_ERR_SHAPE, "vocabularies above 65535 entries are not supported by the sampler");
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
