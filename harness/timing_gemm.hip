// ftnn_timing_gemm <version>
//
// The GEMM driver of the reference (src/timing_gemm.c) for the MI355X library: the same command line (:127-134),
// sweep (m = n in 32 .. 4096, p = 8 m: :90-97), run counts (10 warm-up, 30 measured: :25-30) and CSV file
// (out/measurements/gemm/measurement_<time>.csv, header and first five columns as :73-81), with the operands
// resident on the device: values drawn on the device, packed by ftnn_pack_gemm_operand (bitpacking2), and a run is one
// ftnn_mm_engine call on the engine the library picks, with slope 1 as tnns_gemm fixes it
// (src/tnns/tnns_cpu_mm_p2.c:123).  Unlike the reference's shipped driver (its check is switched off, :132) the first
// result of every size is compared with a plain fp32 product of the unpacked operands; a mismatch aborts.
// Columns added after the reference's five: device time from HIP events, GMAC/s by device time, engine, fraction of
// that engine's roofline.
#include "common.hpp"

using namespace harness;

namespace {

// y[i][j] = sum_k x[i][k] * w[j][k]: what direct_mmm computes (src/utils.c:161-176); exact in fp32 for +-1 / 0 values
__global__ void k_direct_mmm(const float* __restrict__ x, const float* __restrict__ w, float* __restrict__ y, int m, int n, int p) {
    const int j = blockIdx.x * blockDim.x + threadIdx.x, i = blockIdx.y;
    if (j >= n) return;
    float acc = 0.0f;
    for (int k = 0; k < p; k++) acc += x[(size_t)i * p + k] * w[(size_t)j * p + k];
    y[(size_t)i * n + j] = acc;
}

int run(const char* version) {
    std::string csv_path;
    FILE* csv = open_measurement("gemm", &csv_path);
    if (!csv) return EXIT_FAILURE;
    fprintf(csv, "m,n,p,Runtime,Type,Device-ms,GMAC/s,Engine,Roofline-frac\n");
    hipStream_t st;
    hip_check(hipStreamCreate(&st), "hipStreamCreate");
    DeviceBuffer x, w, xp, wp, y, y_ref, scratch;
    for (int k = 32; k <= 4096; k *= 2) {
        const int m = k, n = k, p = 8 * k, p_packed = p / 64;
        const size_t elems = (size_t)m * p;
        fill_values(static_cast<float*>(x.reserve(elems * sizeof(float))), elems, 11 + k, true, st);
        fill_values(static_cast<float*>(w.reserve(elems * sizeof(float))), elems, 12 + k, true, st);
        ftnn_check(ftnn_pack_gemm_operand(x.as<float>(), m, p, static_cast<int64_t*>(xp.reserve(elems / 4)), st), "ftnn_pack_gemm_operand");
        ftnn_check(ftnn_pack_gemm_operand(w.as<float>(), n, p, static_cast<int64_t*>(wp.reserve(elems / 4)), st), "ftnn_pack_gemm_operand");
        const int engine = ftnn_select_engine(TNN, m, 1, 1, n, p_packed);
        const int64_t sb = ftnn_mm_scratch_bytes(FTNN_ENGINE_AUTO, TNN, m, 1, 1, n, p_packed);
        void* d_scr = scratch.reserve((size_t)(sb > 0 ? sb : 16));
        float* out = static_cast<float*>(y.reserve((size_t)m * n * sizeof(float)));
        auto call = [&] {
            ftnn_check(ftnn_mm_engine(FTNN_ENGINE_AUTO, TNN, xp.as<int64_t>(), wp.as<int64_t>(), m, 1, 1, n, p_packed, 0, 1.0f, out,
                                      d_scr, sb, st),
                       "ftnn_mm_engine");
        };
        call();
        hipLaunchKernelGGL(k_direct_mmm, dim3((unsigned)((n + 255) / 256), (unsigned)m), dim3(256), 0, st, x.as<float>(), w.as<float>(),
                           static_cast<float*>(y_ref.reserve((size_t)m * n * sizeof(float))), m, n, p);
        hip_check(hipGetLastError(), "k_direct_mmm");
        std::vector<float> a((size_t)m * n), b((size_t)m * n);
        hip_check(hipMemcpyAsync(a.data(), out, a.size() * sizeof(float), hipMemcpyDeviceToHost, st), "copy");
        hip_check(hipMemcpyAsync(b.data(), y_ref.as<float>(), b.size() * sizeof(float), hipMemcpyDeviceToHost, st), "copy");
        hip_check(hipStreamSynchronize(st), "hipStreamSynchronize");
        if (memcmp(a.data(), b.data(), a.size() * sizeof(float)) != 0) {
            fprintf(stderr, "Function did not return the correct result! (m = n = %d, p = %d)\n", m, p);
            fprintf(csv, "error\n");
            abort();
        }
        double wall = 0.0, dev_ms = 0.0;
        time_runs(call, 10, 30, st, &wall, &dev_ms);   // src/timing_gemm.c:25-30
        const double macs = (double)m * n * p;
        fprintf(csv, "%d,%d,%d,%lf,%s,%.4f,%.1f,%s,%.4f\n", m, n, p, wall, version, dev_ms, macs / (dev_ms * 1e-3) / 1e9,
                engine_name(engine), roofline_fraction(engine, TNN, macs, macs, dev_ms * 1e-3));
        fflush(csv);
        printf("m = n = %d, p = %d: %.4f ms on %s\n", m, p, dev_ms, engine_name(engine));
        fflush(stdout);
    }
    fclose(csv);
    hip_check(hipStreamDestroy(st), "hipStreamDestroy");
    printf("measurements: %s\n", csv_path.c_str());
    return EXIT_SUCCESS;
}

}  // namespace

int main(int argc, char** argv) {
    if (argc != 2) {
        printf("Usage: %s version", argv[0]);
        return EXIT_FAILURE;
    }
    return run(argv[1]);
}
