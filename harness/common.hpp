// Shared pieces of the two timing drivers: device buffers, seeded value generation on the device, the layer
// tables, timing and the CSV files.  The drivers call the library only through include/ftnn.h.
#pragma once
#include <hip/hip_runtime.h>
#include <sys/stat.h>
#include <unistd.h>
#include <sys/time.h>
#include <time.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>
#include <string>
#include <vector>

#include "../include/ftnn.h"

namespace harness {

[[noreturn]] inline void die(const char* what, const char* detail) {
    // the reference's drivers report failure by abort() (src/timing_layers.c:156-159)
    fprintf(stderr, "%s: %s\n", what, detail);
    abort();
}

inline void hip_check(hipError_t e, const char* what) {
    if (e != hipSuccess) die(what, hipGetErrorString(e));
}

inline void ftnn_check(int rc, const char* what) {
    if (rc != FTNN_OK) die(what, ftnn_last_error());
}

// device memory that frees itself; grows on demand and never shrinks
class DeviceBuffer {
public:
    DeviceBuffer() = default;
    DeviceBuffer(const DeviceBuffer&) = delete;
    DeviceBuffer& operator=(const DeviceBuffer&) = delete;
    DeviceBuffer(DeviceBuffer&& o) noexcept : p_(o.p_), cap_(o.cap_) { o.p_ = nullptr; o.cap_ = 0; }
    ~DeviceBuffer() { if (p_) (void)hipFree(p_); }
    void* reserve(size_t bytes) {
        if (bytes > cap_) {
            if (p_) hip_check(hipFree(p_), "hipFree");
            p_ = nullptr;
            hip_check(hipMalloc(&p_, bytes ? bytes : 16), "hipMalloc");
            cap_ = bytes;
        }
        return p_;
    }
    template <typename T> T* as() const { return static_cast<T*>(p_); }

private:
    void* p_ = nullptr;
    size_t cap_ = 0;
};

// Values as the reference's generate_array draws them (src/utils.c:8-32: uniform over {-1,0,+1}, or over {-1,+1}),
// here from a counter-based generator on the device, so that a gigabyte of weights takes microseconds and a run is
// reproducible from its seed alone.
__device__ inline uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

__global__ void k_fill_values(float* out, size_t n, uint64_t seed, int ternary) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const uint64_t r = splitmix64(seed * 0x100000001B3ull + i) >> 11;
    out[i] = ternary ? (float)((int)(r % 3) - 1) : (float)(2 * (int)(r % 2) - 1);
}

inline void fill_values(float* d, size_t n, uint64_t seed, bool ternary, hipStream_t st) {
    if (n == 0) return;
    hipLaunchKernelGGL(k_fill_values, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, d, n, seed, ternary ? 1 : 0);
    hip_check(hipGetLastError(), "k_fill_values");
}

inline void fill_const(float* d, size_t n, float v, hipStream_t st) {
    std::vector<float> h(n, v);
    hip_check(hipMemcpyAsync(d, h.data(), n * sizeof(float), hipMemcpyHostToDevice, st), "hipMemcpyAsync");
    hip_check(hipStreamSynchronize(st), "hipStreamSynchronize");
}

// one row of a layer table: C IH IW KN KW KH pad stride (the reference's order, include/timing/shapes_e2e.h:2:
// the fifth entry is the kernel WIDTH, the sixth its height, src/timing_layers.c:29-40)
struct Row {
    int c, ih, iw, kn, kw, kh, pad, stride;
    int oh() const { return ftnn_out_dim(ih, pad, kh, stride); }
    int ow() const { return ftnn_out_dim(iw, pad, kw, stride); }
    double macs(int batch) const { return (double)batch * oh() * ow() * kn * c * kh * kw; }
};

struct Table {
    std::string name;
    std::vector<Row> rows;
};

// the tables of `mode` ("e2e", "layer", "test") from the plain-text file fastertnn_amd/data/reference_shape_tables.txt
inline std::vector<Table> read_tables(const std::string& path, const std::string& mode) {
    std::ifstream f(path);
    if (!f) die("cannot open the shape tables", path.c_str());
    std::vector<Table> out;
    std::string line;
    bool mine = false;
    while (std::getline(f, line)) {
        if (line.empty() || line[0] == '#') continue;
        if (line[0] == '[') {
            std::istringstream s(line.substr(1, line.size() - 2));
            std::string m, n;
            s >> m >> n;
            mine = m == mode;
            if (mine) out.push_back(Table{n, {}});
            continue;
        }
        if (!mine) continue;
        std::istringstream s(line);
        Row r;
        if (!(s >> r.c >> r.ih >> r.iw >> r.kn >> r.kw >> r.kh >> r.pad >> r.stride)) die("bad row in the shape tables", line.c_str());
        out.back().rows.push_back(r);
    }
    if (out.empty()) die("no tables of this mode in", path.c_str());
    return out;
}

// the tables lie beside the library: <dir of this executable>/../fastertnn_amd/data/, or $FTNN_SHAPE_TABLES
inline std::string tables_path(const char* argv0) {
    if (const char* e = getenv("FTNN_SHAPE_TABLES")) return e;
    char buf[4096];
    ssize_t n = readlink("/proc/self/exe", buf, sizeof(buf) - 1);
    std::string exe = n > 0 ? std::string(buf, (size_t)n) : std::string(argv0);
    const size_t slash = exe.rfind('/');
    const std::string dir = slash == std::string::npos ? "." : exe.substr(0, slash);
    return dir + "/../fastertnn_amd/data/reference_shape_tables.txt";
}

inline double now_seconds() {
    struct timeval tv;
    gettimeofday(&tv, nullptr);
    return (double)tv.tv_sec + (double)tv.tv_usec / 1e6;
}

// out/measurements[/gemm]/measurement_<tm fields>.csv below the working directory, the reference's naming
// (src/timing_layers.c:83-88, src/timing_gemm.c:69-74); unlike the reference the directories are created
inline FILE* open_measurement(const char* subdir, std::string* path_out) {
    std::string dir = "out";
    mkdir(dir.c_str(), 0777);
    dir += "/measurements";
    mkdir(dir.c_str(), 0777);
    if (subdir && *subdir) {
        dir += std::string("/") + subdir;
        mkdir(dir.c_str(), 0777);
    }
    time_t raw = time(nullptr);
    struct tm* t = localtime(&raw);
    char name[300];
    snprintf(name, sizeof name, "%s/measurement_%d_%d_%d_%d_%d_%d.csv", dir.c_str(), t->tm_year, t->tm_mon, t->tm_mday,
             t->tm_hour, t->tm_min, t->tm_sec);
    FILE* f = fopen(name, "w");
    if (!f) {
        fprintf(stderr, "failed to open measurement output file:\n");
        perror(name);
        return nullptr;
    }
    *path_out = name;
    return f;
}

// `runs` repetitions of fn() after `warmup` untimed ones: mean wall-clock seconds of a repetition as the host sees
// it (launch to completion: the stream is synchronised inside the timed region, as a host caller of a synchronous
// entry point would experience it) and mean device milliseconds from HIP events around the launches
template <typename Fn>
void time_runs(Fn&& fn, int warmup, int runs, hipStream_t st, double* wall_seconds, double* device_ms) {
    hipEvent_t e0, e1;
    hip_check(hipEventCreate(&e0), "hipEventCreate");
    hip_check(hipEventCreate(&e1), "hipEventCreate");
    for (int r = 0; r < warmup; r++) fn();
    hip_check(hipStreamSynchronize(st), "hipStreamSynchronize");
    double wall = 0.0, dev = 0.0;
    for (int r = 0; r < runs; r++) {
        const double t0 = now_seconds();
        hip_check(hipEventRecord(e0, st), "hipEventRecord");
        fn();
        hip_check(hipEventRecord(e1, st), "hipEventRecord");
        hip_check(hipStreamSynchronize(st), "hipStreamSynchronize");
        wall += now_seconds() - t0;
        float ms = 0.0f;
        hip_check(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime");
        dev += ms;
    }
    *wall_seconds = wall / runs;
    *device_ms = dev / runs;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
}

// published peaks the roofline column is quoted against
constexpr double kFp4PeakFlops = 10.1e15;                      // dense fp4 MFMA
constexpr double kInt8PeakOps = 5.0e15;                        // dense int8 MFMA
constexpr double kValuPeakLaneOps = 256.0 * 4 * 16 * 2.4e9;    // int32 vector-ALU lane operations

inline const char* engine_name(int engine) {
    switch (engine) {
        case FTNN_ENGINE_VALU: return "valu";
        case FTNN_ENGINE_MFMA_I8: return "mfma_i8";
        case FTNN_ENGINE_MFMA_F4: return "mfma_f4";
        default: return "auto";
    }
}

// fraction of the engine's roofline that `macs` lane multiply-accumulates in `seconds` come to: matrix-core engines
// against their dense peak (2 operations per MAC); the vector ALU against 4 (TNN) or 2 (other types) lane
// operations per 32 lanes, counted on the padded row length `row_lanes` per output
inline double roofline_fraction(int engine, int type, double macs, double padded_lane_macs, double seconds) {
    if (seconds <= 0) return 0.0;
    if (engine == FTNN_ENGINE_MFMA_F4) return 2.0 * macs / seconds / kFp4PeakFlops;
    if (engine == FTNN_ENGINE_MFMA_I8) return 2.0 * macs / seconds / kInt8PeakOps;
    const double ops_per_32 = type == TNN ? 4.0 : 2.0;
    return padded_lane_macs / 32.0 * ops_per_32 / seconds / kValuPeakLaneOps;
}

}  // namespace harness
