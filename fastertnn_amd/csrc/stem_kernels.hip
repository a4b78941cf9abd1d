// First layers on the fp4 matrix cores: few input channels (C <= 8), fp32 input, one kernel.
//
// A layer with C <= 8 would waste most of a 64-lane word on one tap, so T = 64 / C taps share a word
// (lane (tap % T) * C + c of word tap / T: the layout launch_dense_weights gives the weights).  The
// activation side of that layout has no stored form here: a workgroup loads the fp32 input patch of its
// 16 x 16 output pixels once, quantises it into LDS (one dword of nibbles per input pixel), and every
// lane strings the nibbles of its taps together from there, straight into the registers of the MFMA B
// operand.  The input is read once from memory and nothing but the layer's result is written: neither the
// quantised image nor the per-pixel rows (38 MB for a batch-32 7x7 stem) exist.
//
// Arithmetic and result are those of the reference's layer (src/tnns/tnns_cpu_mm_p2.c:6-80): strict
// compares against thr[n] (src/tnns/ternarize2row_avx2.c:443-449, src/tnns/binarize2row_avx2.c:19-21),
// padding 0 for ternary and +1 for binary activations, the PReLU forms of mm_p2_final_{tnn,tbn}_avx2.c.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include <stdlib.h>

#include "ftnn_internal.h"

namespace ftnn {

namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kTile = 16;   // output pixels per workgroup: kTile wide, 4 rows per wavefront (16 rows with four wavefronts)

struct StemGeom {
    int C, H, W, OH, OW, KW, taps, Kd;
    int H_pad, W_pad, H_stride, W_stride;
    int PH, PW;          // input patch of a tile: ((kTile - 1) * stride + K) per direction
    int tiles_x;
    FastDiv dPW, dKW, dTX;
};

// ABIN / FORM0 / QMODE as in k_conv_f4; C is compile-time so that every shift below is a constant.
template <bool ABIN, bool FORM0, int QMODE, int C>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 8))) void k_stem_f4(
    const float* __restrict__ x, const float* __restrict__ thr, const uint4* __restrict__ Wf, float* __restrict__ Y,
    int KN, int KB, int bias, float alpha, StemGeom g, QuantOut qo) {
    constexpr int T = 64 / C;                    // taps per word
    constexpr int J1 = 32 / C;                   // first tap that reaches into the upper half of a word
    constexpr int NI0 = (32 + C - 1) / C;        // taps that touch the lower half
    constexpr int NI = NI0 > T - J1 ? NI0 : T - J1;   // taps a lane strings together per word
    constexpr int TT = J1 + NI;                  // table entries per word (the upper half may run past T)
    constexpr int SR = 4 * (32 - C * J1);        // bits of tap J1 that belong to the lower half
    constexpr uint32_t padv = ABIN ? 0x22222222u : 0u;
    constexpr uint32_t cmask = C >= 8 ? 0xffffffffu : ((1u << (4 * (C & 7))) - 1u);
    static_assert(4 * C * NI <= 160, "five dwords hold the taps of one half");

    extern __shared__ __align__(16) uint32_t lds[];
    const int PP = g.PH * g.PW;
    uint32_t* patch = lds;                 // [0, PP): the quantised patch; [PP, 2 PP): padding nibbles
    uint32_t* toff = lds + 2 * PP;         // [Kd][TT]: byte offset of a tap in the patch (or into the padding)
    // [Kd][2] weight fragments of this kernel tile, 16-byte aligned behind the table
    uint4* wl = reinterpret_cast<uint4*>(lds + (2 * PP + g.Kd * TT + 3) / 4 * 4);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = lane >> 5, lr = lane & 31;
    const int n = blockIdx.z, kn0 = blockIdx.y * 64;
    const int ty = (int)fastdiv(blockIdx.x, g.dTX), tx = (int)blockIdx.x - ty * g.tiles_x;
    const int NT = blockDim.x;   // 64 per wavefront: a tile is 4 rows of kTile pixels per wavefront
    const int oh0 = ty * (int)(blockDim.x >> 4), ow0 = tx * kTile;
    const int HW = g.H * g.W;

    // ---- the patch: quantise on the way into LDS ----
    {
        // the weight fragments of the tile travel to LDS beside the patch (their loads leave first): a load per
        // word inside the loop below would put a memory latency into every step
        const int rbm = (KN + 31) / 32 - 1;
        const int nwf = g.Kd * 2 * 64;
        constexpr int kWR = 2;   // rounds of 256 sixteen-byte pieces in flight at once (Kd <= 4 in one go)
        const float t = thr[n];
        const int ihb = oh0 * g.H_stride - g.H_pad, iwb = ow0 * g.W_stride - g.W_pad;
        const float* xn = x + (size_t)n * C * HW;
        uint4 wreg[kWR];
#pragma unroll
        for (int k = 0; k < kWR; k++) {
            const int i = min(tid + NT * k, nwf - 1);
            const int d = i >> 7, a = (i >> 6) & 1, l = i & 63;
            wreg[k] = Wf[((size_t)min(kn0 / 32 + a, rbm) * KB + d) * 64 + l];
        }
        // kCH patch pixels per thread and round, all their loads issued before the first is used: the fill is a
        // chain of memory latencies otherwise (one round covers the 37 x 37 patch of a stride-2 7x7 layer)
        constexpr int kCH = 6;
        for (int base = 0; base < PP; base += NT * kCH) {
            float v[kCH][C];
            bool in[kCH];
#pragma unroll
            for (int k = 0; k < kCH; k++) {
                in[k] = false;
                if (base + NT * k < PP) {   // wave-uniform up to the last 256 pixels
                    const int idx = min(base + NT * k + tid, PP - 1);
                    const int py = (int)fastdiv((uint32_t)idx, g.dPW), px = idx - py * g.PW;
                    const int ih = ihb + py, iw = iwb + px;
                    in[k] = (unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W;
                    const float* xp = xn + (in[k] ? (size_t)ih * g.W + iw : (size_t)0);
#pragma unroll
                    for (int c = 0; c < C; c++) v[k][c] = xp[(size_t)c * HW];
                }
            }
#pragma unroll
            for (int k = 0; k < kCH; k++) {
                const int idx = base + NT * k + tid;
                if (idx < PP) {
                    uint32_t dw = 0u;
#pragma unroll
                    for (int c = 0; c < C; c++) {
                        uint32_t nib;
                        if (ABIN) nib = v[k][c] < t ? 0xAu : 0x2u;
                        else nib = v[k][c] < -t ? 0xAu : (v[k][c] > t ? 0x2u : 0x0u);
                        dw |= nib << (4 * c);
                    }
                    patch[idx] = in[k] ? dw : (padv & cmask);
                    patch[PP + idx] = padv & cmask;
                }
            }
        }
#pragma unroll
        for (int k = 0; k < kWR; k++)
            if (tid + NT * k < nwf) wl[tid + NT * k] = wreg[k];
        for (int i = tid + NT * kWR; i < nwf; i += NT) {   // more than 4 words: the rest, one by one
            const int d = i >> 7, a = (i >> 6) & 1, l = i & 63;
            wl[i] = Wf[((size_t)min(kn0 / 32 + a, rbm) * KB + d) * 64 + l];
        }
        for (int idx = tid; idx < g.Kd * TT; idx += NT) {
            const int d = idx / TT, j = idx - d * TT;
            const int tap = d * T + j;
            uint32_t off = (uint32_t)PP;   // a tap that does not exist reads the padding region
            if (j < T && tap < g.taps) {
                const int kh = (int)fastdiv((uint32_t)tap, g.dKW), kw = tap - kh * g.KW;
                off = (uint32_t)(kh * g.PW + kw);
            }
            toff[idx] = off * 4u;
        }
    }
    __syncthreads();

    // ---- this wavefront's 64 pixels: block b, lane lr -> row 4 wave + 2 b + lr / 16, column lr % 16 ----
    uint32_t po[2];   // byte offset of the pixel's window origin in the patch
    int oh[2], ow[2];
#pragma unroll
    for (int b = 0; b < 2; b++) {
        const int row = 4 * wave + 2 * b + (lr >> 4), col = lr & 15;
        oh[b] = oh0 + row;
        ow[b] = ow0 + col;
        po[b] = (uint32_t)((row * g.H_stride) * g.PW + col * g.W_stride) * 4u;
    }
    v16f acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[a][b][e] = 0.0f;

    const unsigned char* patch_b = reinterpret_cast<const unsigned char*>(patch);
    const uint32_t* toff_h = toff + h * J1;   // the upper half starts at tap J1 of each word
    for (int d = 0; d < g.Kd; d++) {
        uint4 wv[2];
#pragma unroll
        for (int a = 0; a < 2; a++) wv[a] = wl[(d * 2 + a) * 64 + lane];
        v8i xv[2];
#pragma unroll
        for (int b = 0; b < 2; b++) {
            // taps J .. J + NI - 1 of word d (J = 0 or J1) side by side from bit 0 on
            uint32_t o[6] = {0u, 0u, 0u, 0u, 0u, 0u};
#pragma unroll
            for (int i = 0; i < NI; i++) {
                const uint32_t off = toff_h[d * TT + i];
                const uint32_t v = *reinterpret_cast<const uint32_t*>(patch_b + po[b] + off);
                const int bit = 4 * C * i, lo = bit >> 5, sh = bit & 31;
                o[lo] |= v << sh;
                if (sh + 4 * C > 32) o[lo + 1] |= v >> (32 - sh);
            }
            // past the last tap: padding lanes
            constexpr int used = 4 * C * NI;
#pragma unroll
            for (int k = 0; k < 5; k++) {
                if (32 * k >= used) o[k] |= padv;
                else if (32 * (k + 1) > used) o[k] |= padv & ~((1u << (used - 32 * k)) - 1u);
            }
            // the upper half begins SR bits into tap J1
            const uint32_t sr = h ? (uint32_t)SR : 0u;
#pragma unroll
            for (int k = 0; k < 4; k++) xv[b][k] = (int)__builtin_amdgcn_alignbit(o[k + 1], o[k], sr);
#pragma unroll
            for (int k = 4; k < 8; k++) xv[b][k] = 0;
        }
#pragma unroll
        for (int a = 0; a < 2; a++) {
            const v8i av = {(int)wv[a].x, (int)wv[a].y, (int)wv[a].z, (int)wv[a].w, 0, 0, 0, 0};
#pragma unroll
            for (int b = 0; b < 2; b++)
                // cbsz = blgp = 4: both operands E2M1, unscaled
                acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, xv[b], acc[a][b], 4, 4, 0, 0, 0, 0);
        }
    }

    // ---- epilogue: accumulator e of block (a, b): kernel = 32 a + 8 (e / 4) + 4 h + e % 4, pixel = lane's ----
    const int OHW = g.OH * g.OW;
    const float fbias = (float)bias;
    float qthr = 0.0f;
    if constexpr (QMODE != 0) qthr = qo.thr[n];
    const DirectQuant dq = direct_quant<QMODE>(alpha, qthr);   // whether the hand-over may take its compare-free form
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++) {
            const bool live = oh[b] < g.OH && ow[b] < g.OW;
            const int pix = live ? oh[b] * g.OW + ow[b] : 0;
            float r[16];
#pragma unroll
            for (int e = 0; e < 16; e++) r[e] = FORM0 ? acc[a][b][e] : acc[a][b][e] - fbias;   // only BNN has a bias
            if constexpr (QMODE == 0) {
                float* yq = Y + ((size_t)n * KN + kn0 + 32 * a + 4 * h) * OHW + pix;
                if (live) {
                    if (kn0 + 32 * a + 32 <= KN) {   // uniform: whole block inside
#pragma unroll
                        for (int e = 0; e < 16; e++)
                            yq[(size_t)(8 * (e >> 2) + (e & 3)) * OHW] = prelu_ref<FORM0>(r[e], alpha);
                    } else {
#pragma unroll
                        for (int e = 0; e < 16; e++) {
                            const int p = kn0 + 32 * a + 8 * (e >> 2) + 4 * h + (e & 3);
                            if (p < KN) yq[(size_t)(8 * (e >> 2) + (e & 3)) * OHW] = prelu_ref<FORM0>(r[e], alpha);
                        }
                    }
                }
            } else {
                // as in k_conv_f4: lane half h ends up with bytes 16 a + 8 h .. + 8 of the pixel's 64-channel word
                const uint2 out = hand_over_block<FORM0, QMODE>(r, alpha, qthr, dq, kn0 + 32 * a, h, KN);
                const size_t word = ((size_t)n * gridDim.y + blockIdx.y) * OHW + pix;
                if (live)
                    *reinterpret_cast<uint2*>(static_cast<unsigned char*>(qo.p4) + word * 32 + 16 * a + 8 * h) = out;
            }
        }
}

}  // namespace

// LDS the kernel needs for this layer, or 0 where the fused first-layer kernel does not apply (more than 8
// channels, or an input patch beyond the 64 KiB a workgroup gets without opting in)
static int64_t stem_lds_bytes_for(int C, int KH, int KW, int H_stride, int W_stride, int waves) {
    if (C < 1 || C > 8) return 0;
    const int T = 64 / C, J1 = 32 / C, NI0 = (32 + C - 1) / C, NI = NI0 > T - J1 ? NI0 : T - J1;
    const int64_t PH = (int64_t)(4 * waves - 1) * H_stride + KH, PW = (int64_t)(kTile - 1) * W_stride + KW;
    const int64_t Kd = ((int64_t)KH * KW + T - 1) / T;
    // patch and padding, tap table (rounded up to 16 bytes), weight fragments of one kernel tile
    const int64_t bytes = ((2 * PH * PW + Kd * (J1 + NI) + 3) / 4 * 4) * 4 + Kd * 2 * 1024;
    return bytes <= 64 * 1024 ? bytes : 0;
}

// the layer runs in the fused kernel if its patch fits with the smaller tile (two wavefronts, 8 rows)
int64_t stem_f4_lds_bytes(int C, int KH, int KW, int H_stride, int W_stride) {
    return stem_lds_bytes_for(C, KH, KW, H_stride, W_stride, 2);
}

hipError_t launch_stem_f4(int type, const float* d_x, const float* d_thr, const void* d_wf, int N, int C, int H,
                          int W, int KN, int KH, int KW, int H_pad, int W_pad, int H_stride, int W_stride,
                          float alpha, float* d_y, hipStream_t st, const QuantOut& qo) {
    const int OH = out_dim(H, H_pad, KH, H_stride), OW = out_dim(W, W_pad, KW, W_stride);
    // wavefronts per workgroup = tile height / 4 (tuning aid: FTNN_STEM_WAVES)
    static const int forced = getenv("FTNN_STEM_WAVES") ? atoi(getenv("FTNN_STEM_WAVES")) : 0;
    int waves = 4;
    if (forced == 2 || forced == 4) waves = forced;
    if (stem_lds_bytes_for(C, KH, KW, H_stride, W_stride, waves) == 0) waves = 2;
    const int64_t lds_bytes = stem_lds_bytes_for(C, KH, KW, H_stride, W_stride, waves);
    if (lds_bytes == 0) return hipErrorInvalidValue;
    const int tile_h = 4 * waves;
    const int T = 64 / C, taps = KH * KW, Kd = (taps + T - 1) / T;
    StemGeom g;
    g.C = C; g.H = H; g.W = W; g.OH = OH; g.OW = OW; g.KW = KW; g.taps = taps; g.Kd = Kd;
    g.H_pad = H_pad; g.W_pad = W_pad; g.H_stride = H_stride; g.W_stride = W_stride;
    g.PH = (tile_h - 1) * H_stride + KH;
    g.PW = (kTile - 1) * W_stride + KW;
    g.tiles_x = (OW + kTile - 1) / kTile;
    const int tiles_y = (OH + tile_h - 1) / tile_h;
    g.dPW = make_fastdiv((uint32_t)g.PW);
    g.dKW = make_fastdiv((uint32_t)KW);
    g.dTX = make_fastdiv((uint32_t)g.tiles_x);
    const int64_t tiles = (int64_t)g.tiles_x * tiles_y;
    const int kn_tiles = (KN + 63) / 64;
    if (tiles > 0x7fffffffLL || kn_tiles > 65535 || N > 65535) return hipErrorInvalidValue;
    dim3 grid((unsigned)tiles, (unsigned)kn_tiles, (unsigned)N);
    const uint4* Wf = static_cast<const uint4*>(d_wf);
    const int KB = round4(Kd);
    // BNN: every lane of the Kd words that is not a real (tap, channel) is +1 in both operands
    const int bias = type == kBNN ? 64 * Kd - C * taps : 0;
    auto by_c = [&](auto abin, auto form0, auto qmode) -> hipError_t {
        constexpr bool A = decltype(abin)::value, F = decltype(form0)::value;
        constexpr int Q = decltype(qmode)::value;
#define FTNN_STEM(C_)                                                                                         \
    case C_:                                                                                                  \
        hipLaunchKernelGGL((k_stem_f4<A, F, Q, C_>), grid, dim3(64 * waves), (size_t)lds_bytes, st, d_x, d_thr, Wf, d_y, KN, \
                           KB, bias, alpha, g, qo);                                                           \
        break;
        switch (C) {
            FTNN_STEM(1) FTNN_STEM(2) FTNN_STEM(3) FTNN_STEM(4) FTNN_STEM(5) FTNN_STEM(6) FTNN_STEM(7) FTNN_STEM(8)
            default: return hipErrorInvalidValue;
        }
#undef FTNN_STEM
        return hipGetLastError();
    };
    auto by_mode = [&](auto abin, auto form0) -> hipError_t {
        if (qo.mode == 0) return by_c(abin, form0, std::integral_constant<int, 0>{});
        if (qo.mode == 1) return by_c(abin, form0, std::integral_constant<int, 1>{});
        if (qo.mode == 2) return by_c(abin, form0, std::integral_constant<int, 2>{});
        return hipErrorInvalidValue;
    };
    if (type == kTNN) return by_mode(std::false_type{}, std::true_type{});
    if (type == kTBN) return by_mode(std::false_type{}, std::false_type{});
    return by_mode(std::true_type{}, std::false_type{});   // BTN, BNN
}

}  // namespace ftnn
