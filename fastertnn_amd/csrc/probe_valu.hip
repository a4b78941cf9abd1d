// Measures the vector-ALU issue rate the popcount GEMM is priced against: every wavefront runs a long chain of
// v_bcnt_u32_b32 (population count with accumulate) on independent registers, nothing else in the loop but the
// counter.  Prints one JSON line: lane-operations per second over all compute units, and the same figure as a
// fraction of 256 CU x 4 SIMD x 16 lanes x 2.4 GHz.  Stand-alone measurement aid; the library does not use it.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#define CHECK(x)                                                                            \
    do {                                                                                    \
        hipError_t e_ = (x);                                                                \
        if (e_ != hipSuccess) {                                                             \
            fprintf(stderr, "probe_valu: %s: %s\n", #x, hipGetErrorString(e_));             \
            return 1;                                                                       \
        }                                                                                   \
    } while (0)

constexpr int kAcc = 8;      // independent accumulators per lane
constexpr int kUnroll = 8;   // popcounts per accumulator and loop trip

__global__ __launch_bounds__(256) void k_bcnt(const uint32_t* __restrict__ in, uint32_t* __restrict__ out, int trips) {
    uint32_t x[kAcc], acc[kAcc];
#pragma unroll
    for (int i = 0; i < kAcc; i++) {
        x[i] = in[(threadIdx.x + 64 * i) & 1023];
        acc[i] = 0;
    }
    for (int t = 0; t < trips; t++) {
#pragma unroll
        for (int u = 0; u < kUnroll; u++)
#pragma unroll
            for (int i = 0; i < kAcc; i++) asm volatile("v_bcnt_u32_b32 %0, %1, %0" : "+v"(acc[i]) : "v"(x[i]));
    }
    uint32_t s = 0;
#pragma unroll
    for (int i = 0; i < kAcc; i++) s += acc[i];
    out[blockIdx.x * 256 + threadIdx.x] = s;
}

int main(int argc, char** argv) {
    const int trips = argc > 1 ? atoi(argv[1]) : 20000;
    const int reps = argc > 2 ? atoi(argv[2]) : 5;
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;
    const int blocks = cus * 8;   // 8 workgroups of 4 wavefronts per compute unit: 8 wavefronts per SIMD
    uint32_t *in, *out;
    CHECK(hipMalloc(&in, 1024 * 4));
    CHECK(hipMalloc(&out, (size_t)blocks * 256 * 4));
    uint32_t host[1024];
    for (int i = 0; i < 1024; i++) host[i] = 0x9E3779B9u * (uint32_t)(i + 1);
    CHECK(hipMemcpy(in, host, sizeof host, hipMemcpyHostToDevice));
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    hipLaunchKernelGGL(k_bcnt, dim3(blocks), dim3(256), 0, 0, in, out, trips);   // warm-up
    CHECK(hipDeviceSynchronize());
    float best = 1e30f;
    for (int r = 0; r < reps; r++) {
        CHECK(hipEventRecord(e0, 0));
        hipLaunchKernelGGL(k_bcnt, dim3(blocks), dim3(256), 0, 0, in, out, trips);
        CHECK(hipEventRecord(e1, 0));
        CHECK(hipEventSynchronize(e1));
        float ms;
        CHECK(hipEventElapsedTime(&ms, e0, e1));
        if (ms < best) best = ms;
    }
    // check one lane: acc = trips * kUnroll * popc(x) summed over the accumulators
    uint32_t got;
    CHECK(hipMemcpy(&got, out, 4, hipMemcpyDeviceToHost));
    uint32_t want = 0;
    for (int i = 0; i < kAcc; i++) want += (uint32_t)trips * kUnroll * (uint32_t)__builtin_popcount(host[(64 * i) & 1023]);
    const double lane_ops = (double)blocks * 256 * trips * kUnroll * kAcc;
    const double rate = lane_ops / (best * 1e-3);
    const double peak = (double)cus * 4 * 16 * 2.4e9;
    printf("{\"kernel\": \"v_bcnt_u32_b32 chain\", \"compute_units\": %d, \"ms\": %.4f, \"lane_ops_per_s\": %.4e, "
           "\"nominal_peak\": %.4e, \"frac_of_nominal\": %.4f, \"result_ok\": %s}\n",
           cus, best, rate, peak, rate / peak, got == want ? "true" : "false");
    CHECK(hipFree(in));
    CHECK(hipFree(out));
    return got == want ? 0 : 2;
}
