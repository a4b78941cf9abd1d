// Chain of conv layers with device-resident activations (the reference's e2e mode,
// src/timing_layers.c:182-207, without the per-layer host round trip).
#include <new>
#include <vector>

#include "../../include/ftnn.h"
#include "ftnn_internal.h"

struct ftnn_net {
    int batch = 0;
    std::vector<ftnn_layer_t> layers;
    std::vector<int> OH, OW;
    std::vector<float*> d_thr;       // per layer: batch copies of its threshold
    std::vector<void*> d_wf;         // per layer on the fp4 engine: its weights as matrix-core fragments
    float* d_act[2] = {nullptr, nullptr};
    void* d_scratch = nullptr;
    int64_t out_elems = 0;
    // recorded graph and what it was recorded for
    hipGraphExec_t exec = nullptr;
    const float* g_x = nullptr;
    float* g_y = nullptr;
    hipStream_t g_stream = nullptr;
};

namespace {

using namespace ftnn;

int enqueue_layers(ftnn_net* net, const float* d_x, float* d_y, hipStream_t st) {
    const int n = (int)net->layers.size();
    const float* in = d_x;
    for (int i = 0; i < n; i++) {
        const ftnn_layer_t& L = net->layers[i];
        float* out = (i == n - 1) ? d_y : net->d_act[i & 1];
        int rc;
        if (net->d_wf[i])
            rc = conv_f4_expanded(L.type, in, net->d_thr[i], net->d_wf[i], net->batch, L.C, L.H, L.W, L.KN, L.KH,
                                  L.KW, L.pad, L.pad, L.stride, L.stride, L.prelu_alpha, net->d_scratch, out, st);
        else
            rc = ftnn_conv_engine(FTNN_ENGINE_VALU, L.type, in, net->d_thr[i], L.d_qw, net->batch, L.C, L.H, L.W,
                                  L.KN, L.KH, L.KW, L.pad, L.pad, L.stride, L.stride, L.prelu_alpha,
                                  net->d_scratch, out, st);
        if (rc != FTNN_OK) return rc;
        in = out;
    }
    return FTNN_OK;
}

void drop_graph(ftnn_net* net) {
    if (net->exec) (void)hipGraphExecDestroy(net->exec);
    net->exec = nullptr;
}

}  // namespace

extern "C" {

ftnn_net_t* ftnn_net_create(int batch, int n_layers, const ftnn_layer_t* layers) {
    if (batch <= 0 || batch > 65535 || n_layers <= 0 || !layers) {
        fail(FTNN_EINVAL, "bad batch or layer count");
        return nullptr;
    }
    ftnn_net* net = new (std::nothrow) ftnn_net;
    if (!net) {
        fail(FTNN_ENOMEM, "host allocation failed");
        return nullptr;
    }
    net->batch = batch;
    int64_t max_act = 0, max_scratch = 0;
    for (int i = 0; i < n_layers; i++) {
        const ftnn_layer_t& L = layers[i];
        const bool ok = L.type >= kTNN && L.type <= kBNN && L.C > 0 && L.H > 0 && L.W > 0 && L.KN > 0 &&
                        L.KH > 0 && L.KW > 0 && L.pad >= 0 && L.stride > 0 && L.H + 2 * L.pad >= L.KH &&
                        L.W + 2 * L.pad >= L.KW && L.d_qw;
        if (!ok) {
            fail(FTNN_EINVAL, "layer %d: bad description", i);
            ftnn_net_destroy(net);
            return nullptr;
        }
        if (i > 0) {
            const ftnn_layer_t& P = layers[i - 1];
            if (L.C != P.KN || L.H != net->OH[i - 1] || L.W != net->OW[i - 1]) {
                fail(FTNN_EINVAL, "layer %d: input %dx%dx%d is not the output %dx%dx%d of layer %d", i, L.C, L.H,
                     L.W, P.KN, net->OH[i - 1], net->OW[i - 1], i - 1);
                ftnn_net_destroy(net);
                return nullptr;
            }
        }
        net->layers.push_back(L);
        net->OH.push_back(out_dim(L.H, L.pad, L.KH, L.stride));
        net->OW.push_back(out_dim(L.W, L.pad, L.KW, L.stride));
        const int64_t out = (int64_t)batch * L.KN * net->OH[i] * net->OW[i];
        if (i < n_layers - 1 && out > max_act) max_act = out;
        const int64_t scr = ftnn_conv_scratch_bytes(L.type, batch, L.C, L.H, L.W, L.KN, L.KH, L.KW, L.pad, L.pad,
                                                    L.stride, L.stride);
        if (scr > max_scratch) max_scratch = scr;
        net->out_elems = out;
    }
    bool good = hipMalloc(&net->d_scratch, (size_t)max_scratch) == hipSuccess;
    for (int b = 0; b < 2 && good && max_act > 0; b++)
        good = hipMalloc((void**)&net->d_act[b], (size_t)max_act * sizeof(float)) == hipSuccess;
    std::vector<float> host((size_t)batch);
    for (int i = 0; i < n_layers && good; i++) {
        float* d = nullptr;
        good = hipMalloc((void**)&d, (size_t)batch * sizeof(float)) == hipSuccess;
        if (!good) break;
        net->d_thr.push_back(d);
        for (int b = 0; b < batch; b++) host[(size_t)b] = layers[i].threshold;
        good = hipMemcpy(d, host.data(), (size_t)batch * sizeof(float), hipMemcpyHostToDevice) == hipSuccess;
    }
    // layers that run on the fp4 matrix cores get their weights expanded once, here
    net->d_wf.assign((size_t)n_layers, nullptr);
    for (int i = 0; i < n_layers && good; i++) {
        const ftnn_layer_t& L = layers[i];
        if (ftnn_select_conv_engine(L.type, batch, L.C, L.H, L.W, L.KN, L.KH, L.KW, L.pad, L.pad, L.stride,
                                    L.stride) != FTNN_ENGINE_MFMA_F4)
            continue;
        const int Kw = round4(cpack_of(L.C) * L.KH * L.KW);
        good = hipMalloc(&net->d_wf[i], (size_t)mfma_fragment_bytes(true, L.KN, Kw)) == hipSuccess;
        if (!good) break;
        good = launch_mfma_expand(true, L.type == kTNN || L.type == kBTN, L.d_qw, L.KN, Kw, net->d_wf[i], nullptr) ==
                   hipSuccess &&
               hipStreamSynchronize(nullptr) == hipSuccess;
    }
    if (!good) {
        fail(FTNN_ENOMEM, "device allocation for the layer chain failed");
        ftnn_net_destroy(net);
        return nullptr;
    }
    return net;
}

void ftnn_net_destroy(ftnn_net_t* net) {
    if (!net) return;
    drop_graph(net);
    for (float* p : net->d_thr) (void)hipFree(p);
    for (void* p : net->d_wf)
        if (p) (void)hipFree(p);
    for (int b = 0; b < 2; b++)
        if (net->d_act[b]) (void)hipFree(net->d_act[b]);
    if (net->d_scratch) (void)hipFree(net->d_scratch);
    delete net;
}

int64_t ftnn_net_output_elems(const ftnn_net_t* net) { return net ? net->out_elems : 0; }

int ftnn_net_run(ftnn_net_t* net, const float* d_x, float* d_y, int use_graph, void* stream) {
    if (!net || !d_x || !d_y) return fail(FTNN_EINVAL, "null argument");
    hipStream_t st = (hipStream_t)stream;
    if (!use_graph) return enqueue_layers(net, d_x, d_y, st);
    if (!st) return fail(FTNN_EINVAL, "graph replay needs an explicit (non-null) stream");
    if (!net->exec || net->g_x != d_x || net->g_y != d_y || net->g_stream != st) {
        drop_graph(net);
        hipError_t e = hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal);
        if (e != hipSuccess) return fail(FTNN_EHIP, "hipStreamBeginCapture: %s", hipGetErrorString(e));
        const int rc = enqueue_layers(net, d_x, d_y, st);
        hipGraph_t graph = nullptr;
        e = hipStreamEndCapture(st, &graph);
        if (rc != FTNN_OK) {
            if (graph) (void)hipGraphDestroy(graph);
            return rc;
        }
        if (e != hipSuccess) return fail(FTNN_EHIP, "hipStreamEndCapture: %s", hipGetErrorString(e));
        e = hipGraphInstantiate(&net->exec, graph, nullptr, nullptr, 0);
        (void)hipGraphDestroy(graph);
        if (e != hipSuccess) {
            net->exec = nullptr;
            return fail(FTNN_EHIP, "hipGraphInstantiate: %s", hipGetErrorString(e));
        }
        net->g_x = d_x;
        net->g_y = d_y;
        net->g_stream = st;
    }
    hipError_t e = hipGraphLaunch(net->exec, st);
    return e == hipSuccess ? FTNN_OK : fail(FTNN_EHIP, "hipGraphLaunch: %s", hipGetErrorString(e));
}

}  // extern "C"
