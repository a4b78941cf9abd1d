// ftnn_timing_layers <version> <tnn|tbn|btn|bnn> <layer|e2e|test>
//
// The layer driver of the reference (src/timing_layers.c) for the MI355X library, with the same command line
// (:226-261), constants (batch 8, 5 warm-up and 10 measured runs, PReLU slope 0.5, thresholds by type: :46-48,
// :100-107,121) and CSV file (out/measurements/measurement_<time>.csv, header and first five columns as :83-94,209),
// but with the tensors resident on the device:
//   layer  the 17 single layers: weights packed and prepared once per layer (ftnn_pack_weights,
//          ftnn_conv_prepare_weights), a run is one ftnn_conv_prepared call;
//   e2e    the seven networks: one ftnn_net_* chain per network, a run is one ftnn_net_run (activations stay on the
//          device between layers; tables that leave out their pooling layers run with FTNN_NET_REREAD_PREFIX, which is
//          what the reference's driver does with them, :187-200);
//   test   the 12 self-test shapes: ftnn_conv against an fp32 direct convolution of the padded input computed here by
//          a plain kernel (pad value 0, or +1 for binary activations, :150), tolerance 0.01 (:142-165); a mismatch
//          aborts.  The shapes are then timed like the single layers.
// Columns added after the reference's five: device time from HIP events, GMAC of a run, GMAC/s by device time, the
// engine the library picked, and the fraction of that engine's roofline.
#include "common.hpp"

using namespace harness;

namespace {

constexpr int kBatch = 8, kWarmupRuns = 5, kMeasurementRuns = 10;   // src/timing_layers.c:46-48
constexpr float kAlpha = 0.5f;                                       // :121

const char* type_name(int t) {   // include/tnns/common.h:18-26
    switch (t) {
        case TNN: return "TNN";
        case TBN: return "TBN";
        case BTN: return "BTN";
        case BNN: return "BNN";
        default: return "UNKNOWN";
    }
}

bool act_ternary(int t) { return t == TNN || t == TBN; }
bool weight_ternary(int t) { return t == TNN || t == BTN; }

// fp32 direct convolution + PReLU of values that are already in {-1,0,+1}: one thread per output, taps outside the
// image contribute pad_value.  Exact in fp32 (sums of +-1 far below 2^24).
__global__ void k_direct_conv(const float* __restrict__ x, const float* __restrict__ w, float* __restrict__ y, int N, int C,
                              int H, int W, int KN, int KH, int KW, int pad, int stride, int OH, int OW, float pad_value,
                              float alpha) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t total = (size_t)N * KN * OH * OW;
    if (idx >= total) return;
    const int ow = (int)(idx % OW), oh = (int)(idx / OW % OH), kn = (int)(idx / ((size_t)OW * OH) % KN);
    const int n = (int)(idx / ((size_t)OW * OH * KN));
    float acc = 0.0f;
    for (int c = 0; c < C; c++)
        for (int kh = 0; kh < KH; kh++)
            for (int kw = 0; kw < KW; kw++) {
                const int ih = oh * stride + kh - pad, iw = ow * stride + kw - pad;
                const float v = (ih >= 0 && ih < H && iw >= 0 && iw < W) ? x[(((size_t)n * C + c) * H + ih) * W + iw] : pad_value;
                acc += v * w[(((size_t)kn * C + c) * KH + kh) * KW + kw];
            }
    y[idx] = acc >= 0.0f ? acc : alpha * acc;
}

struct PreparedLayer {
    Row row;
    DeviceBuffer packed, prepared;
};

// fp32 weights of one layer (seeded by its position), packed into Packing-2 rows on the device
void make_weights(int type, const Row& r, uint64_t seed, DeviceBuffer& w_f32, DeviceBuffer& thr, DeviceBuffer& packed,
                  hipStream_t st) {
    const size_t elems = (size_t)r.kn * r.c * r.kh * r.kw;
    const bool wt = weight_ternary(type);
    fill_values(static_cast<float*>(w_f32.reserve(elems * sizeof(float))), elems, seed, wt, st);
    // weight thresholds: 0.5 for ternary weights, 0.0 for binary ones (src/timing_layers.c:105-107)
    fill_const(static_cast<float*>(thr.reserve((size_t)r.kn * sizeof(float))), (size_t)r.kn, wt ? 0.5f : 0.0f, st);
    const size_t words = (size_t)r.kn * (size_t)ftnn_row_words(r.c, r.kh, r.kw, wt);
    ftnn_check(ftnn_pack_weights(wt, w_f32.as<float>(), thr.as<float>(), r.kn, r.c, r.kh, r.kw,
                                 static_cast<int64_t*>(packed.reserve(words * sizeof(int64_t))), st),
               "ftnn_pack_weights");
}

void self_test(int type, const Row& r, const float* d_x, const float* d_thr, const float* d_w, const int64_t* d_qw,
               DeviceBuffer& scratch, DeviceBuffer& y, DeviceBuffer& y_ref, hipStream_t st) {
    const size_t out = (size_t)kBatch * r.kn * r.oh() * r.ow();
    const int64_t sb = ftnn_conv_scratch_bytes(type, kBatch, r.c, r.ih, r.iw, r.kn, r.kh, r.kw, r.pad, r.pad, r.stride, r.stride);
    ftnn_check(ftnn_conv(type, d_x, d_thr, d_qw, kBatch, r.c, r.ih, r.iw, r.kn, r.kh, r.kw, r.pad, r.pad, r.stride, r.stride,
                         kAlpha, scratch.reserve((size_t)sb), static_cast<float*>(y.reserve(out * sizeof(float))), st),
               "ftnn_conv");
    const float pad_value = act_ternary(type) ? 0.0f : 1.0f;   // src/timing_layers.c:150
    hipLaunchKernelGGL(k_direct_conv, dim3((unsigned)((out + 255) / 256)), dim3(256), 0, st, d_x, d_w,
                       static_cast<float*>(y_ref.reserve(out * sizeof(float))), kBatch, r.c, r.ih, r.iw, r.kn, r.kh, r.kw, r.pad,
                       r.stride, r.oh(), r.ow(), pad_value, kAlpha);
    hip_check(hipGetLastError(), "k_direct_conv");
    std::vector<float> a(out), b(out);
    hip_check(hipMemcpyAsync(a.data(), y.as<float>(), out * sizeof(float), hipMemcpyDeviceToHost, st), "copy");
    hip_check(hipMemcpyAsync(b.data(), y_ref.as<float>(), out * sizeof(float), hipMemcpyDeviceToHost, st), "copy");
    hip_check(hipStreamSynchronize(st), "hipStreamSynchronize");
    for (size_t i = 0; i < out; i++) {
        const float d = a[i] - b[i];
        if (!(d <= 0.01f && d >= -0.01f)) {   // the reference's tolerance (src/utils.c:37-55)
            fprintf(stderr, "Function did not return the correct result! element %zu: %f, direct convolution: %f\n", i, a[i], b[i]);
            abort();
        }
    }
}

int run(const char* version, int type, const std::string& mode, const char* argv0) {
    const std::vector<Table> tables = read_tables(tables_path(argv0), mode == "test" ? "test" : mode);
    std::string csv_path;
    FILE* csv = open_measurement("", &csv_path);
    if (!csv) return EXIT_FAILURE;
    fprintf(csv, "TNNs-type, Version, Shape-type, Shape, Runtime, Device-ms, GMAC, GMAC/s, Engine, Roofline-frac\n");
    const char* mode_name = mode == "layer" ? "LAYER" : (mode == "e2e" ? "E2E" : "TEST");   // src/timing_layers.c:51-58

    hipStream_t st;
    hip_check(hipStreamCreate(&st), "hipStreamCreate");
    DeviceBuffer x, thr, w_f32, w_thr, scratch, y, y_ref;
    // activation thresholds: 0.5 for ternary activations, 0.0 for binary ones (src/timing_layers.c:102-104)
    fill_const(static_cast<float*>(thr.reserve(kBatch * sizeof(float))), kBatch, act_ternary(type) ? 0.5f : 0.0f, st);

    for (size_t shape = 0; shape < tables.size(); shape++) {
        const Table& tb = tables[shape];
        printf("SHAPE %zu\n", shape);
        fflush(stdout);
        const Row& first = tb.rows.front();
        const size_t in_elems = (size_t)kBatch * first.c * first.ih * first.iw;
        fill_values(static_cast<float*>(x.reserve(in_elems * sizeof(float))), in_elems, 1000 + shape, act_ternary(type), st);

        std::vector<PreparedLayer> layers(tb.rows.size());
        double macs = 0.0;
        for (size_t i = 0; i < tb.rows.size(); i++) {
            layers[i].row = tb.rows[i];
            make_weights(type, tb.rows[i], 7000 + 100 * shape + i, w_f32, w_thr, layers[i].packed, st);
            macs += tb.rows[i].macs(kBatch);
        }
        double wall = 0.0, dev_ms = 0.0, frac = 0.0;
        int engine = FTNN_ENGINE_AUTO;
        if (mode == "e2e") {
            std::vector<ftnn_layer_t> desc(layers.size());
            bool chains = true;
            int c = first.c, h = first.ih, w = first.iw;
            for (size_t i = 0; i < layers.size(); i++) {
                const Row& r = layers[i].row;
                chains = chains && r.c == c && r.ih == h && r.iw == w;
                c = r.kn, h = r.oh(), w = r.ow();
                desc[i] = ftnn_layer_t{type, r.c, r.ih, r.iw, r.kn, r.kh, r.kw, r.pad, r.stride, act_ternary(type) ? 0.5f : 0.0f,
                                       kAlpha, layers[i].packed.as<int64_t>()};
            }
            ftnn_net_t* net = ftnn_net_create_ex(kBatch, (int)desc.size(), desc.data(), chains ? 0 : FTNN_NET_REREAD_PREFIX);
            if (!net) die("ftnn_net_create", ftnn_last_error());
            float* out = static_cast<float*>(y.reserve((size_t)ftnn_net_output_elems(net) * sizeof(float)));
            time_runs([&] { ftnn_check(ftnn_net_run(net, x.as<float>(), out, 0, st), "ftnn_net_run"); }, kWarmupRuns,
                      kMeasurementRuns, st, &wall, &dev_ms);
            ftnn_net_destroy(net);
            // a chain mixes engines; its fraction is quoted against the fp4 matrix-core peak, the engine of all but
            // few-channel first layers
            engine = FTNN_ENGINE_MFMA_F4;
            frac = roofline_fraction(engine, type, macs, 0.0, dev_ms * 1e-3);
        } else {
            // single layers (and the self-test shapes): the driver's chain has one link
            for (PreparedLayer& L : layers) {
                const Row& r = L.row;
                if (mode == "test")
                    self_test(type, r, x.as<float>(), thr.as<float>(), w_f32.as<float>(), L.packed.as<int64_t>(), scratch, y, y_ref, st);
                ftnn_check(ftnn_conv_prepare_weights(type, L.packed.as<int64_t>(), r.c, r.kn, r.kh, r.kw,
                                                     L.prepared.reserve((size_t)ftnn_conv_weights_bytes(type, r.c, r.kn, r.kh, r.kw)), st),
                           "ftnn_conv_prepare_weights");
                const int64_t sb = ftnn_conv_scratch_bytes(type, kBatch, r.c, r.ih, r.iw, r.kn, r.kh, r.kw, r.pad, r.pad, r.stride, r.stride);
                void* d_scr = scratch.reserve((size_t)sb);
                float* out = static_cast<float*>(y.reserve((size_t)kBatch * r.kn * r.oh() * r.ow() * sizeof(float)));
                time_runs([&] {
                    ftnn_check(ftnn_conv_prepared(type, x.as<float>(), thr.as<float>(), L.prepared.as<void>(), kBatch, r.c, r.ih, r.iw,
                                                  r.kn, r.kh, r.kw, r.pad, r.pad, r.stride, r.stride, kAlpha, d_scr, out, st),
                               "ftnn_conv_prepared");
                }, kWarmupRuns, kMeasurementRuns, st, &wall, &dev_ms);
                engine = ftnn_select_conv_engine(type, kBatch, r.c, r.ih, r.iw, r.kn, r.kh, r.kw, r.pad, r.pad, r.stride, r.stride);
                const double padded = (double)kBatch * r.oh() * r.ow() * r.kn * 64.0 *
                                      (double)(ftnn_row_words(r.c, r.kh, r.kw, 0));
                frac = roofline_fraction(engine, type, macs, padded, dev_ms * 1e-3);
            }
        }
        fprintf(csv, "%s, %s, %s, %zu, %lf, %.4f, %.3f, %.1f, %s, %.4f\n", type_name(type), version, mode_name, shape, wall, dev_ms,
                macs / 1e9, macs / (dev_ms * 1e-3) / 1e9, engine_name(engine), frac);
        fflush(csv);
    }
    fclose(csv);
    hip_check(hipStreamDestroy(st), "hipStreamDestroy");
    printf("measurements: %s\n", csv_path.c_str());
    return EXIT_SUCCESS;
}

}  // namespace

int main(int argc, char** argv) {
    if (argc != 4) {
        printf("Usage: %s version tnns_type shape_type", argv[0]);
        return EXIT_FAILURE;
    }
    int type;
    if (strcmp(argv[2], "tnn") == 0) type = TNN;
    else if (strcmp(argv[2], "tbn") == 0) type = TBN;
    else if (strcmp(argv[2], "btn") == 0) type = BTN;
    else if (strcmp(argv[2], "bnn") == 0) type = BNN;
    else {
        printf("Invalid tnns_type %s", argv[2]);
        return EXIT_FAILURE;
    }
    const std::string mode = argv[3];
    if (mode != "layer" && mode != "e2e" && mode != "test") {
        printf("Invalid shape_type %s", argv[3]);
        return EXIT_FAILURE;
    }
    return run(argv[1], type, mode, argv[0]);
}
