// Chain of conv layers with device-resident activations (the reference's e2e mode,
// src/timing_layers.c:182-207, without the per-layer host round trip).
//
// Between two layers the reference holds fp32 activations (its tnns_conv returns them and the next
// call quantises them again).  Here a layer that feeds a layer on the fp4 matrix-core engine
// quantises its own results in its epilogue, with the next layer's thresholds, and writes that
// layer's operand (P4) directly: the fp32 tensor in between (e.g. 103 MB after a batch-32 stem)
// is neither written nor read, and the next layer needs no quantise launch.  The values compared
// against the thresholds are the same fp32 numbers, so the chain's output is unchanged.
#include <stdlib.h>

#include <algorithm>
#include <new>
#include <vector>

#include "../../include/ftnn.h"
#include "ftnn_internal.h"

// One share of the batch: a contiguous run of images with buffers of its own.  The images of a batch never meet
// (every row of the GEMM belongs to one image), so a batch can run as two chains side by side on two streams: the
// per-launch latency of one chain (a layer kernel here is a few microseconds long, a good part of it dispatch and
// drain) then overlaps with the other chain's work.
struct NetPart {
    int first = 0, batch = 0;               // images [first, first + batch)
    float* d_act[2] = {nullptr, nullptr};   // fp32 activations between layers that need them
    void* d_p4[2] = {nullptr, nullptr};     // quantised input of the fp4 layers, by layer parity
    void* d_scratch = nullptr;              // work space of the vector-ALU layers
};

struct ftnn_net {
    int batch = 0;
    std::vector<ftnn_layer_t> layers;
    std::vector<int> OH, OW;
    std::vector<float*> d_thr;       // per layer: batch copies of its threshold
    std::vector<void*> d_wf;         // per layer on the fp4 engine: its weights as matrix-core fragments
    std::vector<char> rereads;       // per layer: its input is the leading part of the previous layer's fp32 output
    std::vector<NetPart> parts;      // one, or two that run concurrently
    hipStream_t side = nullptr;      // stream of the second part
    hipEvent_t fork = nullptr, join = nullptr;
    int64_t in_elems_per_image = 0, out_elems_per_image = 0;
    int64_t out_elems = 0;
    // recorded graph and what it was recorded for
    hipGraphExec_t exec = nullptr;
    const float* g_x = nullptr;
    float* g_y = nullptr;
    hipStream_t g_stream = nullptr;
};

namespace {

using namespace ftnn;

// layer i of one part; `in` / `p4_ready` carry the part's state from layer to layer
int enqueue_layer(ftnn_net* net, const NetPart& part, int i, const float*& in, bool& p4_ready, float* d_y,
                  hipStream_t st) {
    const int n = (int)net->layers.size();
    const ftnn_layer_t& L = net->layers[i];
    // the next layer takes a quantised hand-over if it is an fp4 layer that reads P4 (not a few-channel one)
    const bool next_f4 = i + 1 < n && net->d_wf[i + 1] && !net->rereads[i + 1] &&
                         !dense_f4_applies(net->layers[i + 1].C, net->layers[i + 1].KH, net->layers[i + 1].KW);
    QuantOut qo;
    if (next_f4) {
        const int nt = net->layers[i + 1].type;
        qo.p4 = part.d_p4[(i + 1) & 1];
        qo.thr = net->d_thr[i + 1];   // every entry holds the layer's threshold: any run of `batch` entries serves
        qo.mode = (nt == kTNN || nt == kTBN) ? 1 : 2;
    }
    float* out = next_f4 ? nullptr : ((i == n - 1) ? d_y : part.d_act[i & 1]);
    int rc;
    if (net->d_wf[i])
        rc = conv_f4_expanded(L.type, p4_ready ? nullptr : in, net->d_thr[i], net->d_wf[i], part.batch, L.C, L.H, L.W,
                              L.KN, L.KH, L.KW, L.pad, L.pad, L.stride, L.stride, L.prelu_alpha, part.d_p4[i & 1], out,
                              st, qo);
    else
        rc = conv_valu(L.type, in, net->d_thr[i], L.d_qw, part.batch, L.C, L.H, L.W, L.KN, L.KH, L.KW, L.pad, L.pad,
                       L.stride, L.stride, L.prelu_alpha, part.d_scratch, out, st, qo, false);
    p4_ready = next_f4;
    in = out;
    return rc;
}

// The whole batch: one chain on `st`, or two side by side (the second on the net's own stream, forked from and
// joined back into `st` with events, which also holds under stream capture).  The launches of the two chains
// alternate, so that both streams have work from the start.
int enqueue_layers(ftnn_net* net, const float* d_x, float* d_y, hipStream_t st) {
    const int n = (int)net->layers.size();
    const size_t np = net->parts.size();
    hipError_t e = hipSuccess;
    if (np > 1) {
        e = hipEventRecord(net->fork, st);
        if (e == hipSuccess) e = hipStreamWaitEvent(net->side, net->fork, 0);
        if (e != hipSuccess) return fail(FTNN_EHIP, "fork of the second chain: %s", hipGetErrorString(e));
    }
    const float* in[2];
    float* y[2];
    bool p4_ready[2] = {false, false};
    for (size_t p = 0; p < np; p++) {
        in[p] = d_x + (size_t)net->parts[p].first * net->in_elems_per_image;
        y[p] = d_y + (size_t)net->parts[p].first * net->out_elems_per_image;
    }
    int rc = FTNN_OK;
    for (int i = 0; i < n && rc == FTNN_OK; i++)
        for (size_t p = 0; p < np && rc == FTNN_OK; p++)
            rc = enqueue_layer(net, net->parts[p], i, in[p], p4_ready[p], y[p], p == 0 ? st : net->side);
    if (np > 1) {
        // join even after a failure: a capture in progress must see the side stream return
        e = hipEventRecord(net->join, net->side);
        if (e == hipSuccess) e = hipStreamWaitEvent(st, net->join, 0);
        if (rc == FTNN_OK && e != hipSuccess) rc = fail(FTNN_EHIP, "join of the second chain: %s", hipGetErrorString(e));
    }
    return rc;
}

void drop_graph(ftnn_net* net) {
    if (net->exec) (void)hipGraphExecDestroy(net->exec);
    net->exec = nullptr;
}

}  // namespace

extern "C" {

ftnn_net_t* ftnn_net_create(int batch, int n_layers, const ftnn_layer_t* layers) {
    return ftnn_net_create_ex(batch, n_layers, layers, 0);
}

ftnn_net_t* ftnn_net_create_ex(int batch, int n_layers, const ftnn_layer_t* layers, int flags) {
    if (flags & ~FTNN_NET_REREAD_PREFIX) {
        fail(FTNN_EINVAL, "unknown flags 0x%x", flags);
        return nullptr;
    }
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
        char reread = 0;
        if (i > 0) {
            const ftnn_layer_t& P = layers[i - 1];
            if (L.C != P.KN || L.H != net->OH[i - 1] || L.W != net->OW[i - 1]) {
                // the reference's e2e driver hands the previous output buffer on whatever the next table row says
                // (src/timing_layers.c:187-200): the next layer then reads the buffer's leading floats as its NCHW input
                const int64_t have = (int64_t)P.KN * net->OH[i - 1] * net->OW[i - 1], want = (int64_t)L.C * L.H * L.W;
                if (!(flags & FTNN_NET_REREAD_PREFIX) || want > have) {
                    fail(FTNN_EINVAL, "layer %d: input %dx%dx%d is not the output %dx%dx%d of layer %d", i, L.C, L.H,
                         L.W, P.KN, net->OH[i - 1], net->OW[i - 1], i - 1);
                    ftnn_net_destroy(net);
                    return nullptr;
                }
                reread = 1;
            }
        }
        net->rereads.push_back(reread);
        net->layers.push_back(L);
        net->OH.push_back(oh);
        net->OW.push_back(ow);
        net->out_elems = (int64_t)batch * L.KN * net->OH[i] * net->OW[i];
    }
    net->in_elems_per_image = (int64_t)layers[0].C * layers[0].H * layers[0].W;
    net->out_elems_per_image = net->out_elems / batch;
    // Two chains side by side from batch 48 on.  Measured on MI355X on a 19-layer ResNet-18-like stack (one chain /
    // two): batch 48 0.218 / 0.195 ms, 64 0.240 / 0.214, 128 0.364 / 0.311, 256 0.609 / 0.519; at batch 32 the two
    // chains' 38 launches take the host longer (0.19 ms) than the device needs for one chain (0.16 ms).
    // FTNN_NET_PARTS = 1 / 2 overrides (tuning aid).
    int nparts = batch >= 48 ? 2 : 1;
    if (const char* env = getenv("FTNN_NET_PARTS")) nparts = atoi(env) >= 2 ? 2 : 1;
    if (nparts > batch) nparts = 1;
    for (char r : net->rereads)
        if (r) nparts = 1;   // such a layer's input runs across the images of the previous output
    net->parts.resize((size_t)nparts);
    for (int p = 0, first = 0; p < nparts; p++) {
        net->parts[(size_t)p].first = first;
        net->parts[(size_t)p].batch = (batch - first + (nparts - p) - 1) / (nparts - p);
        first += net->parts[(size_t)p].batch;
    }
    // engine of every layer (by the larger part: both parts must agree), then the buffers each part needs
    const int pb = net->parts[0].batch;
    std::vector<char> f4((size_t)n_layers, 0);
    int64_t max_act = 0, max_scratch = 256, max_p4 = 0;
    for (int i = 0; i < n_layers; i++) {
        const ftnn_layer_t& L = layers[i];
        f4[i] = ftnn_select_conv_engine(L.type, pb, L.C, L.H, L.W, L.KN, L.KH, L.KW, L.pad, L.pad, L.stride,
                                        L.stride) == FTNN_ENGINE_MFMA_F4;
        if (f4[i] && ((int64_t)pb * L.H * L.W * cpack_of(L.C) > 0x7fffffffLL ||
                      (int64_t)pb * net->OH[i] * net->OW[i] * conv_f4_weight_words(L.C, L.KH, L.KW) > 0x7fffffffLL))
            f4[i] = 0;   // beyond the 32-bit pixel indices of the fp4 layer kernel: the vector-ALU layer takes it
        // sized for the larger part; a very large layer's operand region depends on the batch in steps (the
        // im2row + GEMM form), so the smaller part is asked too
        for (const NetPart& part : net->parts) {
            if (f4[i])
                max_p4 = std::max(max_p4, conv_f4_operand_bytes(part.batch, L.C, L.H, L.W, L.KH, L.KW, net->OH[i],
                                                                net->OW[i], L.KN, L.stride));
            else
                max_scratch = std::max(max_scratch, ftnn_conv_scratch_bytes(L.type, part.batch, L.C, L.H, L.W, L.KN, L.KH,
                                                                            L.KW, L.pad, L.pad, L.stride, L.stride));
        }
        // its input arrives as fp32 unless it is an fp4 layer that reads the previous layer's hand-over
        if (i > 0 && (!f4[i] || dense_f4_applies(L.C, L.KH, L.KW)))
            max_act = std::max(max_act, (int64_t)pb * L.C * L.H * L.W);
        if (i > 0 && net->rereads[i])   // the previous layer writes its whole fp32 output, this one reads the start of it
            max_act = std::max(max_act, (int64_t)pb * layers[i - 1].KN * net->OH[i - 1] * net->OW[i - 1]);
    }
    bool good = true;
    for (NetPart& part : net->parts) {
        good = good && hipMalloc(&part.d_scratch, (size_t)max_scratch) == hipSuccess;
        for (int b = 0; b < 2 && good && max_act > 0; b++)
            good = hipMalloc((void**)&part.d_act[b], (size_t)max_act * sizeof(float)) == hipSuccess;
        for (int b = 0; b < 2 && good && max_p4 > 0; b++)
            good = hipMalloc(&part.d_p4[b], (size_t)max_p4) == hipSuccess;
    }
    if (good && nparts > 1)
        good = hipStreamCreateWithFlags(&net->side, hipStreamNonBlocking) == hipSuccess &&
               hipEventCreateWithFlags(&net->fork, hipEventDisableTiming) == hipSuccess &&
               hipEventCreateWithFlags(&net->join, hipEventDisableTiming) == hipSuccess;
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
    for (NetPart& part : net->parts) {
        for (int b = 0; b < 2; b++) {
            if (part.d_act[b]) (void)hipFree(part.d_act[b]);
            if (part.d_p4[b]) (void)hipFree(part.d_p4[b]);
        }
        if (part.d_scratch) (void)hipFree(part.d_scratch);
    }
    if (net->fork) (void)hipEventDestroy(net->fork);
    if (net->join) (void)hipEventDestroy(net->join);
    if (net->side) (void)hipStreamDestroy(net->side);
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
