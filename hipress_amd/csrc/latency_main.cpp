// hipress_latency [n] [iters]: encode + decode of one tensor through the C ABI alone,
// timed with HIP events, to separate the library's launch latency from that of a
// language binding.  Prints one JSON line.
//   us_per_step_stream   mean over `iters` steps enqueued back to back between two events
//   us_per_step_wall     the same loop by the host's clock, synchronised once at the end
//   us_per_step_isolated median of steps that are each bracketed by events and waited for
#include <hip/hip_runtime.h>

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../include/hipress_amd.h"

#define CK(x)                                                                         \
    do {                                                                              \
        hipError_t e_ = (x);                                                          \
        if (e_ != hipSuccess) {                                                       \
            std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));              \
            return 1;                                                                 \
        }                                                                             \
    } while (0)
#define HP(x)                                                                         \
    do {                                                                              \
        int rc_ = (x);                                                                \
        if (rc_ != HIPRESS_OK) {                                                      \
            std::fprintf(stderr, "%s: %s\n", #x, hipress_strerror(rc_));              \
            return 1;                                                                 \
        }                                                                             \
    } while (0)

int main(int argc, char** argv) {
    const int64_t n = argc > 1 ? std::atoll(argv[1]) : 262144;
    const int iters = argc > 2 ? std::atoi(argv[2]) : 2000;
    if (n < 1 || iters < 1) return 2;
    const float tau = 0.05f;
    // N(0, 0.02) from a fixed linear congruential sequence through Box-Muller
    std::vector<float> g((size_t)n);
    uint32_t x = 12345u;
    auto uni = [&]() {
        x = 1664525u * x + 1013904223u;
        return ((x >> 8) + 0.5f) * (1.0f / 16777216.0f);
    };
    for (int64_t i = 0; i < n; ++i) g[(size_t)i] = 0.02f * std::sqrt(-2.0f * std::log(uni())) * std::cos(6.2831853f * uni());
    const int64_t pbytes = hipress_tbq_payload_bytes(n);
    float *dg, *dr, *dout;
    void* dpay;
    CK(hipMalloc((void**)&dg, 4 * n));
    CK(hipMalloc((void**)&dr, 4 * n));
    CK(hipMalloc((void**)&dout, 4 * n));
    CK(hipMalloc(&dpay, (size_t)pbytes));
    CK(hipMemcpy(dg, g.data(), 4 * n, hipMemcpyHostToDevice));
    CK(hipMemset(dr, 0, 4 * n));
    hipStream_t st;
    CK(hipStreamCreate(&st));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    auto step = [&]() -> int {
        HP(hipress_tbq_encode(dg, dr, n, dpay, pbytes, tau, st));
        HP(hipress_tbq_decode(dpay, pbytes, dout, n, st));
        return 0;
    };
    for (int i = 0; i < 50; ++i)
        if (step()) return 1;
    CK(hipStreamSynchronize(st));
    const auto t0 = std::chrono::steady_clock::now();
    CK(hipEventRecord(e0, st));
    for (int i = 0; i < iters; ++i)
        if (step()) return 1;
    CK(hipEventRecord(e1, st));
    CK(hipStreamSynchronize(st));
    const auto t1 = std::chrono::steady_clock::now();
    float ms = 0.f;
    CK(hipEventElapsedTime(&ms, e0, e1));
    const double wall_us = std::chrono::duration<double, std::micro>(t1 - t0).count() / iters;
    std::vector<float> iso;
    const int niso = std::min(iters, 200);
    for (int i = 0; i < niso; ++i) {
        CK(hipEventRecord(e0, st));
        if (step()) return 1;
        CK(hipEventRecord(e1, st));
        CK(hipStreamSynchronize(st));
        float m = 0.f;
        CK(hipEventElapsedTime(&m, e0, e1));
        iso.push_back(m * 1e3f);
    }
    std::sort(iso.begin(), iso.end());
    std::printf("{\"n\": %lld, \"iters\": %d, \"us_per_step_stream\": %.3f, \"us_per_step_wall\": %.3f, "
                "\"us_per_step_isolated\": %.3f, \"what\": \"hipress_tbq_encode + hipress_tbq_decode from a C program, no binding\"}\n",
                (long long)n, iters, ms * 1e3 / iters, wall_us, iso[iso.size() / 2]);
    (void)hipFree(dg);
    (void)hipFree(dr);
    (void)hipFree(dout);
    (void)hipFree(dpay);
    return 0;
}
