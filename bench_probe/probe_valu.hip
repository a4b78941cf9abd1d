// Measurement aid of bench.py (its own small shared library, not part of libftnn_hip.so): the vector-ALU issue
// rate the popcount GEMM is priced against, and the shader clock the chip holds while it runs.
//
//   probe_valu_run    every wavefront of a chip-filling grid runs a long chain of v_bcnt_u32_b32 (population count
//                     with accumulate) on independent registers, nothing else in the loop but the counter.  The
//                     first wavefront of every workgroup also reads the shader-clock counter (s_memtime) and the
//                     constant-rate counter (s_memrealtime) before and after its loop: their ratio is the shader
//                     clock that kernel really ran at, which is what turns "lane-ops per second" into "lane-ops
//                     per cycle".
//   probe_clock_run   a short, nearly idle kernel (one wavefront per compute unit, the same chain for a few tens
//                     of microseconds) that only reports that clock ratio: queued directly behind another kernel
//                     on the same stream it samples the clock that kernel left the chip at.
//
//   probe_copy_run    a plain copy kernel of known size (k_probe_copy: 16 bytes per thread in, 16 bytes out): the
//                     dispatch that FETCH_SIZE / WRITE_SIZE counter runs are scaled by.
//
//   probe_mfma_run    every wavefront of a chip-filling grid (one per SIMD, as the fp4 GEMM runs) issues nothing but
//                     v_mfma_f32_32x32x64_f8f6f4 on E2M1 operands holding uniformly random ternary lanes, 16
//                     accumulator tiles of 32 x 32 per wavefront, operands from registers: the matrix rate the chip
//                     sustains with no operand traffic at all, and the shader clock it holds while doing so.  The
//                     lanes are coded either as -1 / 0 / +1 (codes 0xA, 0x0, 0x2) or offset as 0 / 0.5 / 1 (codes
//                     0, 1, 2, the form the GEMM's operands travel in): the clock differs between the two.
//
//   probe_lds_run     workgroups of four wavefronts, each wavefront reading its own KiBs of LDS with 16-byte reads
//                     (ds_read_b128, lane l at byte 16 l: the layout of an MFMA operand fragment) and nothing else:
//                     the bytes per cycle and compute unit that the matrix-core tile kernels' fragment reads can
//                     reach with one workgroup per compute unit and with two.
//
// All are launched on the caller's stream and timed with HIP events recorded on that stream.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>

namespace {

constexpr int kAcc = 8;      // independent accumulators per lane
constexpr int kUnroll = 64;  // popcounts per accumulator and loop trip: 512 vector instructions per 3 scalar ones of loop control

// E2M1 codes of a lane that is -1, 0, +1, by table: 0 the plain codes, 1 the offset codes (a + 1) / 2 the GEMM's operands
// travel in; the others only show how the clock depends on the lanes' content: 2 all zero, 3 {0, +1}, 4 {0, 1, 2},
// 5 {-1.5, 0, +1.5}, 6 {-6, 0, +6}
constexpr int kForms = 7;
constexpr uint32_t kCode[kForms][3] = {{0xA, 0x0, 0x2}, {0x0, 0x1, 0x2}, {0x0, 0x0, 0x0}, {0x0, 0x0, 0x2},
                                       {0x0, 0x2, 0x4}, {0xB, 0x0, 0x3}, {0xF, 0x0, 0x7}};

struct Stamp {
    unsigned long long clk0, clk1, rt0, rt1;
};

__global__ __launch_bounds__(256) void k_bcnt(const uint32_t* __restrict__ in, uint32_t* __restrict__ out, int trips,
                                              Stamp* __restrict__ stamps) {
    uint32_t x[kAcc], acc[kAcc];
#pragma unroll
    for (int i = 0; i < kAcc; i++) {
        x[i] = in[(threadIdx.x + 64 * i) & 1023];
        acc[i] = 0;
    }
    const unsigned long long c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
    for (int t = 0; t < trips; t++) {
#pragma unroll
        for (int u = 0; u < kUnroll; u++)
#pragma unroll
            for (int i = 0; i < kAcc; i++) asm volatile("v_bcnt_u32_b32 %0, %1, %0" : "+v"(acc[i]) : "v"(x[i]));
    }
    const unsigned long long c1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
    uint32_t s = 0;
#pragma unroll
    for (int i = 0; i < kAcc; i++) s += acc[i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
    if (threadIdx.x == 0) stamps[blockIdx.x] = Stamp{c0, c1, r0, r1};
}

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void k_mfma_chain(const uint4* __restrict__ in, float* __restrict__ out, int trips,
                                                    Stamp* __restrict__ stamps) {
    const int lane = threadIdx.x & 63;
    v8i a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint4 u = in[(i * 64 + lane) & 511], w = in[((i + 4) * 64 + lane) & 511];
        a[i] = v8i{(int)u.x, (int)u.y, (int)u.z, (int)u.w, 0, 0, 0, 0};
        b[i] = v8i{(int)w.x, (int)w.y, (int)w.z, (int)w.w, 0, 0, 0, 0};
    }
    v16f acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;
    const unsigned long long c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
    for (int t = 0; t < trips; t++) {
#pragma unroll
        for (int u = 0; u < 2; u++)
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i], b[j], acc[i][j], 4, 4, 0, 0, 0, 0);
    }
    const unsigned long long c1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) s += acc[i][j][e];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
    if (threadIdx.x == 0) stamps[blockIdx.x] = Stamp{c0, c1, r0, r1};
}

__global__ __launch_bounds__(256) void k_probe_copy(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n16) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n16) dst[i] = src[i];
}

struct State {
    uint32_t *in = nullptr, *out = nullptr;
    Stamp *stamps = nullptr, *stamps_host = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int cus = 0, blocks = 0;
    double realtime_hz = 1e8;
    uint32_t host_in[1024];
    uint4* codes[kForms] = {};    // 512 x 16 bytes of E2M1 nibbles per code table (kCode)
} g;

bool ok(hipError_t e, const char* what) {
    if (e != hipSuccess) fprintf(stderr, "probe_valu: %s: %s\n", what, hipGetErrorString(e));
    return e == hipSuccess;
}

// mean shader clock in MHz over the workgroups' stamps
double mean_mhz(int blocks) {
    double sum = 0.0;
    int n = 0;
    for (int b = 0; b < blocks; b++) {
        const Stamp& s = g.stamps_host[b];
        if (s.rt1 > s.rt0) {
            sum += (double)(s.clk1 - s.clk0) / ((double)(s.rt1 - s.rt0) / g.realtime_hz) / 1e6;
            n++;
        }
    }
    return n ? sum / n : 0.0;
}

// Four wavefronts, each reading 8 fragments of 1 KiB per trip from its own 16 KiB of LDS; the addresses depend on the
// trip and the values are kept alive, so that no read is hoisted out of the loop or dropped.
__global__ __launch_bounds__(256) void k_lds_read(uint32_t* __restrict__ out, int trips, long long* __restrict__ cycles) {
    __shared__ __attribute__((aligned(16))) uint32_t lds[16384];   // 64 KiB
    for (int i = threadIdx.x; i < 16384; i += 256) lds[i] = (uint32_t)i;
    __syncthreads();
    typedef unsigned int v4u __attribute__((ext_vector_type(4)));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t acc = 0u;
    const long long t0 = clock64();
    for (int it = 0; it < trips; it++) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t* base = lds + ((wave * 4096 + (it & 1) * 2048 + j * 256) & 16383);
            const v4u v = *reinterpret_cast<const v4u*>(base + lane * 4);   // one ds_read_b128
            asm volatile("" ::"v"(v));
            acc += v.x;
        }
    }
    const long long t1 = clock64();
    out[blockIdx.x * 256 + threadIdx.x] = acc;
    if (threadIdx.x == 0 && blockIdx.x == 0) *cycles = t1 - t0;
}

}  // namespace

extern "C" {

// allocates the probe's buffers on the current device; 0 on success
__attribute__((visibility("default"))) int probe_valu_init(void) {
    if (g.in) return 0;
    hipDeviceProp_t prop;
    if (!ok(hipGetDeviceProperties(&prop, 0), "hipGetDeviceProperties")) return 1;
    g.cus = prop.multiProcessorCount;
    g.blocks = g.cus * 8;   // 8 workgroups of 4 wavefronts per compute unit: 8 wavefronts per SIMD
    int khz = 0;
    if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, 0) == hipSuccess && khz > 0) g.realtime_hz = khz * 1e3;
    if (!ok(hipMalloc(&g.in, sizeof g.host_in), "hipMalloc") ||
        !ok(hipMalloc(&g.out, (size_t)g.blocks * 256 * 4), "hipMalloc") ||
        !ok(hipMalloc(&g.stamps, (size_t)g.blocks * sizeof(Stamp)), "hipMalloc") ||
        !ok(hipHostMalloc((void**)&g.stamps_host, (size_t)g.blocks * sizeof(Stamp), hipHostMallocDefault), "hipHostMalloc"))
        return 1;
    for (int i = 0; i < 1024; i++) g.host_in[i] = 0x9E3779B9u * (uint32_t)(i + 1);
    if (!ok(hipMemcpy(g.in, g.host_in, sizeof g.host_in, hipMemcpyHostToDevice), "hipMemcpy")) return 1;
    for (int form = 0; form < kForms; form++) {
        static uint32_t codes[512 * 4];
        uint64_t x = 0x243F6A8885A308D3ull;
        for (int i = 0; i < 512 * 4; i++) {
            uint32_t w = 0;
            for (int n = 0; n < 8; n++) {
                x ^= x << 13, x ^= x >> 7, x ^= x << 17;
                w |= kCode[form][(uint32_t)(x >> 33) % 3] << (4 * n);
            }
            codes[i] = w;
        }
        if (!ok(hipMalloc(&g.codes[form], sizeof codes), "hipMalloc") ||
            !ok(hipMemcpy(g.codes[form], codes, sizeof codes, hipMemcpyHostToDevice), "hipMemcpy"))
            return 1;
    }
    if (!ok(hipEventCreate(&g.e0), "hipEventCreate") || !ok(hipEventCreate(&g.e1), "hipEventCreate")) return 1;
    return 0;
}

__attribute__((visibility("default"))) int probe_valu_compute_units(void) { return g.cus; }

// The chip-filling chain.  out[0] = kernel ms (HIP events on `stream`), out[1] = lane-ops per second,
// out[2] = mean shader clock in MHz during the kernel, out[3] = lane-ops per lane and cycle at that clock
// (1.0 = one vector instruction per cycle and SIMD), out[4] = 1 if the accumulated counts are right.
__attribute__((visibility("default"))) int probe_valu_run(int trips, void* stream, double* out) {
    if (probe_valu_init() != 0) return 1;
    hipStream_t st = (hipStream_t)stream;
    if (!ok(hipEventRecord(g.e0, st), "hipEventRecord")) return 1;
    hipLaunchKernelGGL(k_bcnt, dim3(g.blocks), dim3(256), 0, st, g.in, g.out, trips, g.stamps);
    if (!ok(hipGetLastError(), "launch") || !ok(hipEventRecord(g.e1, st), "hipEventRecord")) return 1;
    if (!ok(hipMemcpyAsync(g.stamps_host, g.stamps, (size_t)g.blocks * sizeof(Stamp), hipMemcpyDeviceToHost, st), "copy")) return 1;
    uint32_t got = 0;
    if (!ok(hipMemcpyAsync(&got, g.out, 4, hipMemcpyDeviceToHost, st), "copy") || !ok(hipStreamSynchronize(st), "sync")) return 1;
    float ms = 0.0f;
    if (!ok(hipEventElapsedTime(&ms, g.e0, g.e1), "hipEventElapsedTime")) return 1;
    uint32_t want = 0;
    for (int i = 0; i < kAcc; i++) want += (uint32_t)trips * kUnroll * (uint32_t)__builtin_popcount(g.host_in[(64 * i) & 1023]);
    const double lane_ops = (double)g.blocks * 256 * trips * kUnroll * kAcc;
    out[0] = ms;
    out[1] = lane_ops / (ms * 1e-3);
    out[2] = mean_mhz(g.blocks);
    out[3] = out[2] > 0 ? out[1] / ((double)g.cus * 4 * 16 * out[2] * 1e6) : 0.0;
    out[4] = got == want ? 1.0 : 0.0;
    return 0;
}

// The matrix-core chain: one workgroup of four wavefronts per compute unit, 32 fp4 MFMAs of 32 x 32 x 64 per trip
// and wavefront.  out[0] = kernel ms, out[1] = FLOP per second (2 x 32 x 32 x 64 per MFMA), out[2] = mean shader
// clock in MHz during the kernel, out[3] = fraction of the cycles of a SIMD at that clock in which its matrix pipe
// was busy (32 cycles per MFMA).  form: the code table of the lanes (kCode): 0 = -1 / 0 / +1, 1 = 0 / 0.5 / 1, ...
__attribute__((visibility("default"))) int probe_mfma_run(int trips, int form, void* stream, double* out) {
    if (probe_valu_init() != 0 || form < 0 || form >= kForms) return 1;
    hipStream_t st = (hipStream_t)stream;
    const int blocks = g.cus;
    if (!ok(hipEventRecord(g.e0, st), "hipEventRecord")) return 1;
    hipLaunchKernelGGL(k_mfma_chain, dim3(blocks), dim3(256), 0, st, g.codes[form], reinterpret_cast<float*>(g.out), trips, g.stamps);
    if (!ok(hipGetLastError(), "launch") || !ok(hipEventRecord(g.e1, st), "hipEventRecord")) return 1;
    if (!ok(hipMemcpyAsync(g.stamps_host, g.stamps, (size_t)blocks * sizeof(Stamp), hipMemcpyDeviceToHost, st), "copy") ||
        !ok(hipStreamSynchronize(st), "sync"))
        return 1;
    float ms = 0.0f;
    if (!ok(hipEventElapsedTime(&ms, g.e0, g.e1), "hipEventElapsedTime")) return 1;
    const double mfmas_per_simd = 32.0 * trips;
    out[0] = ms;
    out[1] = mfmas_per_simd * blocks * 4 * (2.0 * 32 * 32 * 64) / (ms * 1e-3);
    out[2] = mean_mhz(blocks);
    out[3] = out[2] > 0 ? mfmas_per_simd * 32.0 / (ms * 1e-3 * out[2] * 1e6) : 0.0;
    return 0;
}

// One wavefront per compute unit for `trips` loop trips: out[0] = kernel ms, out[1] = mean shader clock in MHz.
__attribute__((visibility("default"))) int probe_clock_run(int trips, void* stream, double* out) {
    if (probe_valu_init() != 0) return 1;
    hipStream_t st = (hipStream_t)stream;
    if (!ok(hipEventRecord(g.e0, st), "hipEventRecord")) return 1;
    hipLaunchKernelGGL(k_bcnt, dim3(g.cus), dim3(64), 0, st, g.in, g.out, trips, g.stamps);
    if (!ok(hipGetLastError(), "launch") || !ok(hipEventRecord(g.e1, st), "hipEventRecord")) return 1;
    if (!ok(hipMemcpyAsync(g.stamps_host, g.stamps, (size_t)g.cus * sizeof(Stamp), hipMemcpyDeviceToHost, st), "copy") ||
        !ok(hipStreamSynchronize(st), "sync"))
        return 1;
    float ms = 0.0f;
    if (!ok(hipEventElapsedTime(&ms, g.e0, g.e1), "hipEventElapsedTime")) return 1;
    out[0] = ms;
    out[1] = mean_mhz(g.cus);
    return 0;
}

// Copies `bytes` (a multiple of 4096) from d_src to d_dst with k_probe_copy; out[0] = kernel ms.
__attribute__((visibility("default"))) int probe_copy_run(const void* d_src, void* d_dst, size_t bytes, void* stream, double* out) {
    if (probe_valu_init() != 0 || bytes % 4096 != 0 || bytes / 4096 > 0x7fffffffull) return 1;
    hipStream_t st = (hipStream_t)stream;
    if (!ok(hipEventRecord(g.e0, st), "hipEventRecord")) return 1;
    hipLaunchKernelGGL(k_probe_copy, dim3((unsigned)(bytes / 4096)), dim3(256), 0, st, static_cast<const uint4*>(d_src),
                       static_cast<uint4*>(d_dst), bytes / 16);
    if (!ok(hipGetLastError(), "launch") || !ok(hipEventRecord(g.e1, st), "hipEventRecord") || !ok(hipStreamSynchronize(st), "sync"))
        return 1;
    float ms = 0.0f;
    if (!ok(hipEventElapsedTime(&ms, g.e0, g.e1), "hipEventElapsedTime")) return 1;
    out[0] = ms;
    return 0;
}

// `wgs_per_cu` (1 or 2) workgroups per compute unit, `trips` trips of 8 KiB per wavefront: out[0] = kernel ms, out[1] =
// bytes read per shader cycle and compute unit (cycles counted by the first workgroup itself).
__attribute__((visibility("default"))) int probe_lds_run(int wgs_per_cu, int trips, void* stream, double* out) {
    if (probe_valu_init() != 0 || wgs_per_cu < 1 || wgs_per_cu > 2 || trips < 1) return 1;
    static uint32_t* sink = nullptr;
    static long long* cyc = nullptr;
    if (!sink && (!ok(hipMalloc(&sink, (size_t)g.cus * 2 * 256 * 4), "hipMalloc") || !ok(hipMalloc(&cyc, 8), "hipMalloc"))) return 1;
    hipStream_t st = (hipStream_t)stream;
    if (!ok(hipEventRecord(g.e0, st), "hipEventRecord")) return 1;
    hipLaunchKernelGGL(k_lds_read, dim3(g.cus * wgs_per_cu), dim3(256), 0, st, sink, trips, cyc);
    long long c = 0;
    if (!ok(hipGetLastError(), "launch") || !ok(hipEventRecord(g.e1, st), "hipEventRecord") ||
        !ok(hipMemcpyAsync(&c, cyc, 8, hipMemcpyDeviceToHost, st), "copy") || !ok(hipStreamSynchronize(st), "sync"))
        return 1;
    float ms = 0.0f;
    if (!ok(hipEventElapsedTime(&ms, g.e0, g.e1), "hipEventElapsedTime") || c <= 0) return 1;
    out[0] = ms;
    out[1] = (double)trips * 8 * 4 * 1024 * wgs_per_cu / (double)c;
    return 0;
}

}  // extern "C"
