// gemv_bench: how fast does the int4 matrix-vector product of libawq_hip.so stream weights, with and without the
// fixed cost of a dependent launch?
//
// Issues awq_matvec_int4 (K x N, default 4096 x 4096) over a set of distinct matrices larger than the 256 MB
// memory-side cache, through the C-ABI only, in three ways:
//   1 stream            : launches back to back on one stream (each waits for the one before it, as in decode);
//   2 and 4 streams     : the same launches dealt round-robin to plain streams (default priority, one host thread per
//                         stream so that the host keeps up), so that the ramp of one launch overlaps the streaming of
//                         others: what the kernel sustains when launch latency is hidden.
// Prints one JSON object.  Usage: gemv_bench [K N [matrices [repetitions]]]
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <chrono>
#include <thread>
#include <vector>

#include "../../../include/awq_hip.h"

static void die_awq(int r) {
    if (r) {
        fprintf(stderr, "gemv_bench: %s\n", awq_last_error());
        exit(EXIT_FAILURE);
    }
}

static uint64_t mix(uint64_t z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

static uint16_t float_to_half(float f) {  // normal range only (scales 0.002 .. 0.02, activations of order 1)
    uint32_t u;
    memcpy(&u, &f, 4);
    const uint32_t sign = (u >> 16) & 0x8000u;
    int exp = (int)((u >> 23) & 0xFF) - 127 + 15;
    uint32_t man = (u >> 13) & 0x3FFu;
    if (exp <= 0) return (uint16_t)sign;
    if (exp >= 31) return (uint16_t)(sign | 0x7BFFu);
    return (uint16_t)(sign | ((uint32_t)exp << 10) | man);
}

int main(int argc, char** argv) {
    const int K = argc > 2 ? atoi(argv[1]) : 4096;
    const int N = argc > 2 ? atoi(argv[2]) : 4096;
    const int mats = argc > 3 ? atoi(argv[3]) : 64;
    const int reps = argc > 4 ? atoi(argv[4]) : 8;
    if (K <= 0 || N <= 0 || (K & 31) || (N & 7) || mats < 1 || reps < 1) {
        fprintf(stderr, "Usage: gemv_bench [K N [matrices [repetitions]]]  (K multiple of 32, N multiple of 8)\n");
        return EXIT_FAILURE;
    }
    const int G = (K + 127) / 128;
    const size_t wbytes = (size_t)N * (K / 8) * 4, zbytes = (size_t)N * ((G + 7) / 8) * 4, sbytes = (size_t)N * G * 2;
    const size_t mat_bytes = wbytes + zbytes + sbytes;
    const size_t algo_bytes = mat_bytes + 2 * (size_t)K + 2 * (size_t)N;

    constexpr int kMaxStreams = 4;
    awq_ctx* ctx[kMaxStreams];
    for (int i = 0; i < kMaxStreams; i++) die_awq(awq_ctx_create(0, &ctx[i]));

    // one allocation holding every matrix (weights, zeros, scales back to back, as in a model file)
    uint8_t* blob = nullptr;
    die_awq(awq_malloc(ctx[0], (void**)&blob, mat_bytes * mats));
    {
        std::vector<uint8_t> host(mat_bytes);
        for (int m = 0; m < mats; m++) {
            uint64_t* w64 = reinterpret_cast<uint64_t*>(host.data());
            for (size_t i = 0; i < (wbytes + zbytes) / 8; i++) w64[i] = mix(0x9E3779B97F4A7C15ull * (i + 1) + m);
            uint16_t* s16 = reinterpret_cast<uint16_t*>(host.data() + wbytes + zbytes);
            for (size_t i = 0; i < sbytes / 2; i++) s16[i] = float_to_half(0.002f + 0.018f * (float)(mix(i + 77 * m) >> 40) / 16777216.0f);
            die_awq(awq_memcpy_h2d(ctx[0], blob + (size_t)m * mat_bytes, host.data(), mat_bytes));
        }
    }
    uint16_t *x = nullptr, *out = nullptr;
    die_awq(awq_malloc(ctx[0], (void**)&x, 2 * (size_t)K));
    die_awq(awq_malloc(ctx[0], (void**)&out, 2 * (size_t)N * kMaxStreams));
    {
        std::vector<uint16_t> hx(K);
        for (int i = 0; i < K; i++) hx[i] = float_to_half((float)((double)(mix(i + 5) >> 11) / 9007199254740992.0 * 2.0 - 1.0) + 1e-3f);
        die_awq(awq_memcpy_h2d(ctx[0], x, hx.data(), 2 * (size_t)K));
    }
    std::vector<awq_qweight> qw(mats);
    for (int m = 0; m < mats; m++) {
        uint8_t* p = blob + (size_t)m * mat_bytes;
        qw[m].weight = reinterpret_cast<const uint32_t*>(p);
        qw[m].zeros = reinterpret_cast<const uint32_t*>(p + wbytes);
        qw[m].scales = reinterpret_cast<const uint16_t*>(p + wbytes + zbytes);
    }

    // `streams` host threads, thread s issuing matrices s, s + streams, ... on its own context, `reps` times over
    auto run = [&](int streams) {
        for (int s = 0; s < kMaxStreams; s++) die_awq(awq_stream_sync(ctx[s]));
        const auto t0 = std::chrono::steady_clock::now();
        std::vector<std::thread> th;
        for (int s = 0; s < streams; s++)
            th.emplace_back([&, s] {
                for (int r = 0; r < reps; r++)
                    for (int m = s; m < mats; m += streams)
                        die_awq(awq_matvec_int4(ctx[s], out + (size_t)s * N, x, &qw[m], K, N, 0, 1, -1, nullptr));
                die_awq(awq_stream_sync(ctx[s]));
            });
        for (auto& t : th) t.join();
        const double sec = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
        return sec * 1e6 / ((double)reps * mats);  // microseconds per product
    };
    run(1);  // warm-up: code objects, first touch
    run(4);
    double us[3];
    const int counts[3] = {1, 2, 4};
    for (int i = 0; i < 3; i++) {
        double best = 1e30;
        for (int trial = 0; trial < 3; trial++) best = fmin(best, run(counts[i]));
        us[i] = best;
    }
    printf("{\"K\": %d, \"N\": %d, \"matrices\": %d, \"distinct_bytes\": %zu, \"bytes_per_product\": %zu", K, N, mats, mat_bytes * mats,
           algo_bytes);
    for (int i = 0; i < 3; i++)
        printf(", \"streams_%d\": {\"us_per_product\": %.3f, \"gbps\": %.1f, \"frac_of_8TBps\": %.4f}", counts[i], us[i],
               algo_bytes / us[i] / 1e3, algo_bytes / us[i] / 1e3 / 8000.0);
    printf("}\n");
    die_awq(awq_free(ctx[0], blob));
    die_awq(awq_free(ctx[0], x));
    die_awq(awq_free(ctx[0], out));
    for (int i = 0; i < kMaxStreams; i++) die_awq(awq_ctx_destroy(ctx[i]));
    return 0;
}
