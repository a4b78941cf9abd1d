// Chain of conv layers with device-resident activations (the reference's e2e mode,
// src/timing_layers.c:182-207, without the per-layer host round trip).
//
// Between two layers the reference holds fp32 activations (its tnns_conv returns them and the next
// call quantises them again).  Here a layer that feeds a layer on the fp4 matrix-core engine
// quantises its own results in its epilogue, with the next layer's thresholds, and writes that
// layer's operand (P4) directly: the fp32 tensor in between (e.g. 103 MB after a batch-32 stem)
// is neither written nor read, and the next layer needs no quantise launch.  The values compared
// against the thresholds are the same fp32 numbers, so the chain's output is unchanged.
#include <algorithm>
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
    float* d_act[2] = {nullptr, nullptr};   // fp32 activations between layers that need them
    void* d_p4[2] = {nullptr, nullptr};     // quantised input of the fp4 layers, by layer parity
    void* d_scratch = nullptr;              // work space of the vector-ALU layers
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
    const float* in = d_x;    // fp32 input of layer i (unused when p4_ready)
    bool p4_ready = false;    // d_p4[i & 1] already holds layer i's quantised input
    for (int i = 0; i < n; i++) {
        const ftnn_layer_t& L = net->layers[i];
        // the next layer takes a quantised hand-over if it is an fp4 layer that reads P4 (not a few-channel one)
        const bool next_f4 = i + 1 < n && net->d_wf[i + 1] &&
                             !dense_f4_applies(net->layers[i + 1].C, net->layers[i + 1].KH, net->layers[i + 1].KW);
        QuantOut qo;
        if (next_f4) {
            const int nt = net->layers[i + 1].type;
            qo.p4 = net->d_p4[(i + 1) & 1];
            qo.thr = net->d_thr[i + 1];
            qo.mode = (nt == kTNN || nt == kTBN) ? 1 : 2;
        }
        float* out = next_f4 ? nullptr : ((i == n - 1) ? d_y : net->d_act[i & 1]);
        int rc;
        if (net->d_wf[i])
            rc = conv_f4_expanded(L.type, p4_ready ? nullptr : in, net->d_thr[i], net->d_wf[i], net->batch, L.C, L.H,
                                  L.W, L.KN, L.KH, L.KW, L.pad, L.pad, L.stride, L.stride, L.prelu_alpha,
                                  net->d_p4[i & 1], out, st, qo);
        else
            rc = conv_valu(L.type, in, net->d_thr[i], L.d_qw, net->batch, L.C, L.H, L.W, L.KN, L.KH, L.KW, L.pad,
                           L.pad, L.stride, L.stride, L.prelu_alpha, net->d_scratch, out, st, qo, false);
        if (rc != FTNN_OK) return rc;
        p4_ready = next_f4;
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
    for (int i = 0; i < n_layers; i++) {
        const ftnn_layer_t& L = layers[i];
        int oh = 0, ow = 0;
        if (L.type < kTNN || L.type > kBNN || L.KN <= 0 || !L.d_qw) {
            fail(FTNN_EINVAL, "layer %d: bad description", i);
            ftnn_net_destroy(net);
            return nullptr;
        }
        // the same shape rules and size limits as a single layer call (the failure text is the check's)
        if (check_conv_shape(batch, L.C, L.H, L.W, L.pad, L.pad, L.KH, L.KW, L.stride, L.stride, &oh, &ow) != FTNN_OK ||
            ((int64_t)batch * oh * ow > 0x7fffff00LL &&
             fail(FTNN_EINVAL, "layer %d: more than 2^31 output rows", i) != FTNN_OK)) {
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
        net->OH.push_back(oh);
        net->OW.push_back(ow);
        net->out_elems = (int64_t)batch * L.KN * net->OH[i] * net->OW[i];
    }
    // engine of every layer, then the buffers the chain needs between them
    std::vector<char> f4((size_t)n_layers, 0);
    int64_t max_act = 0, max_scratch = 256, max_p4 = 0;
    for (int i = 0; i < n_layers; i++) {
        const ftnn_layer_t& L = layers[i];
        f4[i] = ftnn_select_conv_engine(L.type, batch, L.C, L.H, L.W, L.KN, L.KH, L.KW, L.pad, L.pad, L.stride,
                                        L.stride) == FTNN_ENGINE_MFMA_F4;
        if (f4[i] && ((int64_t)batch * L.H * L.W * cpack_of(L.C) > 0x7fffffffLL ||
                      (int64_t)batch * net->OH[i] * net->OW[i] * conv_f4_weight_words(L.C, L.KH, L.KW) > 0x7fffffffLL))
            f4[i] = 0;   // beyond the 32-bit pixel indices of the fp4 layer kernel: the vector-ALU layer takes it
        if (f4[i]) {
            max_p4 = std::max(max_p4, conv_f4_operand_bytes(batch, L.C, L.H, L.W, L.KH, L.KW, net->OH[i], net->OW[i], L.KN));
            if (i > 0 && dense_f4_applies(L.C, L.KH, L.KW))   // its input arrives as fp32
                max_act = std::max(max_act, (int64_t)batch * L.C * L.H * L.W);
        } else {
            max_scratch = std::max(max_scratch, ftnn_conv_scratch_bytes(L.type, batch, L.C, L.H, L.W, L.KN, L.KH, L.KW,
                                                                        L.pad, L.pad, L.stride, L.stride));
            if (i > 0)   // its input arrives as fp32
                max_act = std::max(max_act, (int64_t)batch * L.C * L.H * L.W);
        }
    }
    bool good = hipMalloc(&net->d_scratch, (size_t)max_scratch) == hipSuccess;
    for (int b = 0; b < 2 && good && max_act > 0; b++)
        good = hipMalloc((void**)&net->d_act[b], (size_t)max_act * sizeof(float)) == hipSuccess;
    for (int b = 0; b < 2 && good && max_p4 > 0; b++)
        good = hipMalloc(&net->d_p4[b], (size_t)max_p4) == hipSuccess;
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
        if (!f4[i]) continue;
        const int Kw = conv_f4_weight_words(L.C, L.KH, L.KW);
        const bool wt = L.type == kTNN || L.type == kBTN;
        good = hipMalloc(&net->d_wf[i], (size_t)mfma_fragment_bytes(true, L.KN, Kw)) == hipSuccess;
        if (!good) break;
        const int64_t* rows = L.d_qw;
        void* d_wd = nullptr;
        if (dense_f4_applies(L.C, L.KH, L.KW)) {   // few channels: the weights take the dense re-packing first
            good = hipMalloc(&d_wd, (size_t)L.KN * Kw * (wt ? 16 : 8)) == hipSuccess &&
                   launch_dense_weights(wt, L.d_qw, L.KN, L.C, L.KH, L.KW, static_cast<int64_t*>(d_wd), nullptr) ==
                       hipSuccess;
            rows = static_cast<const int64_t*>(d_wd);
        }
        good = good && launch_mfma_expand(true, wt, rows, L.KN, Kw, net->d_wf[i], nullptr) == hipSuccess &&
               hipStreamSynchronize(nullptr) == hipSuccess;
        if (d_wd) (void)hipFree(d_wd);
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
    for (int b = 0; b < 2; b++)
        if (net->d_p4[b]) (void)hipFree(net->d_p4[b]);
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
