// Measurement aid of bench.py (its own small shared library, not part of libftnn_hip.so): what a grid-wide
// synchronisation costs on a chip-filling cooperative launch, against the cost of ending one kernel and starting
// the next.  It decides whether a chain of small layers is better run as one resident kernel.
//
//   probe_gridsync_run(mode, wgs_per_cu, syncs, stream, out)
//     mode 0   cooperative launch (hipLaunchCooperativeKernel: the runtime refuses it unless every workgroup is
//              resident), `syncs` times cooperative_groups::grid_group::sync() with one dependent global store and
//              load between two syncs;
//     mode 1   the same launch with a barrier of the probe's own: a counter per barrier generation in global
//              memory, one device-scope atomic add per workgroup, thread 0 polls with a bounded number of trips
//              (a wavefront that runs out of trips sets a flag and goes on, so the kernel always ends);
//     mode 2   `syncs` + 1 plain launches of a kernel that does the same store and load: the launch boundary as
//              the synchronisation.
//   out[0] = ms for the whole sequence (HIP events on `stream`), out[1] = microseconds per synchronisation,
//   out[2] = workgroups launched, out[3] = 1 if the data passed through the synchronisations is right and no
//   bounded wait ran out.
#include <hip/hip_cooperative_groups.h>
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>

namespace cg = cooperative_groups;

namespace {

constexpr int kMaxSyncs = 256;
constexpr int kSpinLimit = 1 << 22;   // trips of the bounded wait (each a few hundred ns at worst): seconds, never reached

// Between two synchronisations every workgroup writes its token and afterwards reads the token of the workgroup
// half the grid away: a missing synchronisation shows as a stale token.
__device__ __forceinline__ void exchange(uint32_t* tokens, int round, uint32_t* bad) {
    const int nb = gridDim.x;
    if (threadIdx.x == 0) {
        if (round > 0) {
            const uint32_t got = __hip_atomic_load(&tokens[(blockIdx.x + nb / 2) % nb], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (got != (uint32_t)round) atomicAdd(bad, 1u);
        }
    }
}
__device__ __forceinline__ void publish(uint32_t* tokens, int round) {
    if (threadIdx.x == 0) __hip_atomic_store(&tokens[blockIdx.x], (uint32_t)round, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Rounds alternate between two token arrays (odd rounds the first, even rounds the second): a token is overwritten two
// rounds later, and by then every reader of this round has passed the next round's synchronisation.
__device__ __forceinline__ uint32_t* round_tokens(uint32_t* tokens, int round) {
    return tokens + ((round & 1) ? 0u : gridDim.x);
}

__global__ __launch_bounds__(256) void k_sync_library(uint32_t* tokens, int syncs, uint32_t* bad) {
    cg::grid_group grid = cg::this_grid();
    for (int r = 1; r <= syncs; r++) {
        publish(round_tokens(tokens, r), r);
        grid.sync();
        exchange(round_tokens(tokens, r), r, bad);
    }
}

__global__ __launch_bounds__(256) void k_sync_own(uint32_t* tokens, int syncs, uint32_t* bad, uint32_t* counters) {
    const uint32_t nb = gridDim.x;
    for (int r = 1; r <= syncs; r++) {
        publish(round_tokens(tokens, r), r);
        // barrier generation r has a counter of its own (zeroed by the host): no reset, no sense reversal
        __syncthreads();
        if (threadIdx.x == 0) {
            __hip_atomic_fetch_add(&counters[r], 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
            int trips = 0;
            while (__hip_atomic_load(&counters[r], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) < nb) {
                if (++trips > kSpinLimit) {
                    atomicAdd(bad, 1u << 16);
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
        }
        __syncthreads();
        exchange(round_tokens(tokens, r), r, bad);
    }
}

__global__ __launch_bounds__(256) void k_sync_launch(uint32_t* tokens, int r, uint32_t* bad) {
    exchange(round_tokens(tokens, r - 1), r - 1, bad);   // the token the previous launch left in the other array
    publish(round_tokens(tokens, r), r);
}

struct State {
    uint32_t *tokens = nullptr, *bad = nullptr, *counters = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int cus = 0, max_blocks = 0;
} g;

bool ok(hipError_t e, const char* what) {
    if (e != hipSuccess) fprintf(stderr, "probe_gridsync: %s: %s\n", what, hipGetErrorString(e));
    return e == hipSuccess;
}

int init() {
    if (g.tokens) return 0;
    hipDeviceProp_t prop;
    if (!ok(hipGetDeviceProperties(&prop, 0), "hipGetDeviceProperties")) return 1;
    if (!prop.cooperativeLaunch) {
        fprintf(stderr, "probe_gridsync: the device does not support cooperative launches\n");
        return 1;
    }
    g.cus = prop.multiProcessorCount;
    g.max_blocks = g.cus * 8;
    if (!ok(hipMalloc(&g.tokens, (size_t)g.max_blocks * 2 * 4), "hipMalloc") || !ok(hipMalloc(&g.bad, 4), "hipMalloc") ||
        !ok(hipMalloc(&g.counters, (kMaxSyncs + 1) * 4), "hipMalloc") || !ok(hipEventCreate(&g.e0), "hipEventCreate") ||
        !ok(hipEventCreate(&g.e1), "hipEventCreate"))
        return 1;
    return 0;
}

}  // namespace

extern "C" {

__attribute__((visibility("default"))) int probe_gridsync_run(int mode, int wgs_per_cu, int syncs, void* stream, double* out) {
    if (init() != 0 || mode < 0 || mode > 2 || syncs < 1 || syncs > kMaxSyncs || wgs_per_cu < 1 || wgs_per_cu > 8) return 1;
    hipStream_t st = (hipStream_t)stream;
    int blocks = g.cus * wgs_per_cu;
    if (mode != 2) {
        // the grid a cooperative launch may have: what the occupancy query says fits at once
        int per_cu = 0;
        const void* k = mode == 0 ? reinterpret_cast<const void*>(&k_sync_library) : reinterpret_cast<const void*>(&k_sync_own);
        if (!ok(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, k, 256, 0), "occupancy")) return 1;
        if (per_cu < wgs_per_cu) blocks = g.cus * per_cu;
    }
    if (!ok(hipMemsetAsync(g.tokens, 0, (size_t)g.max_blocks * 2 * 4, st), "memset") || !ok(hipMemsetAsync(g.bad, 0, 4, st), "memset") ||
        !ok(hipMemsetAsync(g.counters, 0, (kMaxSyncs + 1) * 4, st), "memset"))
        return 1;
    if (!ok(hipEventRecord(g.e0, st), "hipEventRecord")) return 1;
    if (mode == 2) {
        for (int r = 1; r <= syncs + 1; r++) hipLaunchKernelGGL(k_sync_launch, dim3(blocks), dim3(256), 0, st, g.tokens, r, g.bad);
        if (!ok(hipGetLastError(), "launch")) return 1;
    } else if (mode == 0) {
        void* args[] = {&g.tokens, &syncs, &g.bad};
        if (!ok(hipLaunchCooperativeKernel(reinterpret_cast<const void*>(&k_sync_library), dim3(blocks), dim3(256), args, 0, st),
                "hipLaunchCooperativeKernel"))
            return 1;
    } else {
        void* args[] = {&g.tokens, &syncs, &g.bad, &g.counters};
        if (!ok(hipLaunchCooperativeKernel(reinterpret_cast<const void*>(&k_sync_own), dim3(blocks), dim3(256), args, 0, st),
                "hipLaunchCooperativeKernel"))
            return 1;
    }
    if (!ok(hipEventRecord(g.e1, st), "hipEventRecord")) return 1;
    uint32_t bad = 0;
    if (!ok(hipMemcpyAsync(&bad, g.bad, 4, hipMemcpyDeviceToHost, st), "copy") || !ok(hipStreamSynchronize(st), "sync")) return 1;
    float ms = 0.0f;
    if (!ok(hipEventElapsedTime(&ms, g.e0, g.e1), "hipEventElapsedTime")) return 1;
    out[0] = ms;
    out[1] = ms * 1e3 / syncs;
    out[2] = blocks;
    out[3] = bad == 0 ? 1.0 : 0.0;
    return 0;
}

}  // extern "C"
