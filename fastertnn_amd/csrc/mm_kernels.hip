// Bit-packed popcount GEMM + PReLU on the vector ALU (gfx950).
//
// Semantics: src/tnns/mm_p2_final_{tnn,tbn,btn,bnn}_avx2.c with the output index
// of include/tnns/mm.h:30.  Layout of the operands:
//   ternary rows: groups of 16 dwords = 4 sign words (8 dwords) then their 4 zero
//                 words (8 dwords); row stride 4*Kw dwords
//   binary rows : plain words, row stride 2*Kw dwords; "group" = 4 words = 8 dwords
//
// Design.  The work is integer VALU work: per pair of 32-lane dwords TNN needs
// four vector ops (v_or, v_bitop3, two v_bcnt with free accumulate) and
// TBN/BTN/BNN two.  To keep the vector ALU on nothing else:
//   * lanes run along the rows of A (= output pixels, the contiguous direction
//     of the NCHW result); each lane owns TM rows and TN columns of accumulators;
//   * the B operand (weights) of a wavefront is wave-uniform, so it is read with
//     scalar loads into SGPRs and enters every vector op as its one scalar
//     source: no LDS traffic, no VGPRs and no vector instructions for B;
//   * A tiles are copied global -> LDS with coalesced 16-byte loads, then each
//     lane reads its own rows back with 128-bit LDS reads; the row stride is
//     padded by 4 dwords so that the 8 lanes of a 128-byte LDS beat hit distinct
//     banks.
// A workgroup is 4 wavefronts sharing one A tile of 64*TM rows; wavefront w
// computes columns [w*TN, (w+1)*TN) of the workgroup's 4*TN columns.
#include "ftnn_internal.h"

namespace ftnn {

namespace {

// acc += popcount(x): one v_bcnt_u32_b32 (popcount with accumulate)
__device__ __forceinline__ void bcnt_acc(uint32_t& acc, uint32_t x) {
    asm("v_bcnt_u32_b32 %0, %1, %0" : "+v"(acc) : "v"(x));
}

template <int MODE>
struct Traits {
    static constexpr bool kATern = (MODE == kTNN || MODE == kTBN);
    static constexpr bool kBTern = (MODE == kTNN || MODE == kBTN);
    static constexpr int kAGroup = kATern ? 16 : 8;  // dwords of A per group of 4 words
    static constexpr int kBGroup = kBTern ? 16 : 8;
};

template <int MODE, int TM, int TN, int GC>
__global__ __launch_bounds__(256) void k_mm(const uint32_t* __restrict__ A,
                                            const uint32_t* __restrict__ B,
                                            float* __restrict__ Y, int M, int KN, int OHW, int G,
                                            int K_unpack, float alpha) {
    using T = Traits<MODE>;
    constexpr int BM = 64 * TM;
    constexpr int AG = T::kAGroup, BG = T::kBGroup;
    constexpr int QPG = AG / 4;          // 16-byte quads of A per group
    constexpr int LDW = GC * AG + 4;     // LDS row stride in dwords (padded)
    __shared__ uint32_t lds[BM * LDW];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t row0 = (int64_t)blockIdx.x * BM;
    const int col0 = (blockIdx.y * 4 + wave) * TN;
    const size_t RDA = (size_t)G * AG, RDB = (size_t)G * BG;

    uint32_t cn[TM][TN];                 // popcount of "negative product" lanes
    uint32_t cz[TM][TN];                 // TNN only: popcount of "zero product" lanes
    uint32_t rowz[TM];                   // TBN only: popcount of za per row
    uint32_t colz[TN];                   // BTN only: popcount of zb per column (uniform)
#pragma unroll
    for (int a = 0; a < TM; a++) {
        rowz[a] = 0;
#pragma unroll
        for (int b = 0; b < TN; b++) {
            cn[a][b] = 0;
            cz[a][b] = 0;
        }
    }
#pragma unroll
    for (int b = 0; b < TN; b++) colz[b] = 0;

    for (int g0 = 0; g0 < G; g0 += GC) {
        const int gc = min(GC, G - g0);
        __syncthreads();
        for (int e = tid; e < BM * GC * QPG; e += 256) {
            const int r = e / (GC * QPG), q = e % (GC * QPG);
            if (q < gc * QPG) {
                const int64_t gr = min(row0 + r, (int64_t)M - 1);
                const uint4 v = *reinterpret_cast<const uint4*>(A + gr * RDA + (size_t)g0 * AG + q * 4);
                *reinterpret_cast<uint4*>(lds + r * LDW + q * 4) = v;
            }
        }
        __syncthreads();
        for (int g = 0; g < gc; g++) {
#pragma unroll
            for (int h = 0; h < 2; h++) {
                uint4 sa[TM], za[TM];
#pragma unroll
                for (int a = 0; a < TM; a++) {
                    const uint32_t* lp = lds + (lane + 64 * a) * LDW + g * AG + h * 4;
                    sa[a] = *reinterpret_cast<const uint4*>(lp);
                    if (T::kATern) za[a] = *reinterpret_cast<const uint4*>(lp + 8);
                }
                if (MODE == kTBN) {
#pragma unroll
                    for (int a = 0; a < TM; a++) {
                        bcnt_acc(rowz[a], za[a].x);
                        bcnt_acc(rowz[a], za[a].y);
                        bcnt_acc(rowz[a], za[a].z);
                        bcnt_acc(rowz[a], za[a].w);
                    }
                }
#pragma unroll
                for (int b = 0; b < TN; b++) {
                    const int col = min(col0 + b, KN - 1);
                    const uint32_t* bp = B + (size_t)col * RDB + (size_t)(g0 + g) * BG + h * 4;
                    const uint4 sb = *reinterpret_cast<const uint4*>(bp);
                    uint4 zb = make_uint4(0, 0, 0, 0);
                    if (T::kBTern) zb = *reinterpret_cast<const uint4*>(bp + 8);
                    if (MODE == kBTN) colz[b] += __popc(zb.x) + __popc(zb.y) + __popc(zb.z) + __popc(zb.w);
#pragma unroll
                    for (int a = 0; a < TM; a++) {
#define FTNN_STEP(c)                                                            \
    if (MODE == kTNN) {                                                         \
        const uint32_t z = za[a].c | zb.c;                                      \
        const uint32_t n = (sa[a].c ^ sb.c) & ~z;                               \
        bcnt_acc(cz[a][b], z);                                                  \
        bcnt_acc(cn[a][b], n);                                                  \
    } else if (MODE == kTBN) {                                                  \
        bcnt_acc(cn[a][b], (sa[a].c ^ sb.c) & ~za[a].c);                        \
    } else if (MODE == kBTN) {                                                  \
        bcnt_acc(cn[a][b], (sa[a].c ^ sb.c) & ~zb.c);                           \
    } else {                                                                    \
        bcnt_acc(cn[a][b], sa[a].c ^ sb.c);                                     \
    }
                        FTNN_STEP(x)
                        FTNN_STEP(y)
                        FTNN_STEP(z)
                        FTNN_STEP(w)
#undef FTNN_STEP
                    }
                }
            }
        }
    }

    const int lanes_total = G * 4 * 64;  // 64 * Kw
#pragma unroll
    for (int a = 0; a < TM; a++) {
        const int64_t i = row0 + lane + 64 * a;
        if (i < M) {
            const int64_t img = i / OHW;
            const int pix = (int)(i - img * OHW);
#pragma unroll
            for (int b = 0; b < TN; b++) {
                const int j = col0 + b;
                if (j < KN) {
                    float f;
                    if (MODE == kTNN) {
                        // src/tnns/mm_p2_final_tnn_avx2.c:178,204-208
                        const int acc = lanes_total - (int)(cz[a][b] + 2u * cn[a][b]);
                        f = (float)acc;
                        if (f <= 0) f *= alpha;
                    } else {
                        int r;
                        if (MODE == kTBN) r = lanes_total - (int)rowz[a] - 2 * (int)cn[a][b];
                        else if (MODE == kBTN) r = lanes_total - (int)colz[b] - 2 * (int)cn[a][b];
                        else r = K_unpack - 2 * (int)cn[a][b];
                        // src/tnns/mm_p2_final_tbn_avx2.c:72-73
                        f = r >= 0 ? (float)r : alpha * r;
                    }
                    Y[((size_t)img * KN + j) * OHW + pix] = f;
                }
            }
        }
    }
}

template <int MODE, int TM, int TN, int GC>
hipError_t launch_cfg(const uint32_t* A, const uint32_t* B, float* Y, int64_t M, int KN, int OHW,
                      int G, int K_unpack, float alpha, hipStream_t st) {
    const int64_t gx = (M + 64 * TM - 1) / (64 * TM);
    const int64_t gy = (KN + 4 * TN - 1) / (4 * TN);
    if (gx > 0x7fffffffLL || gy > 65535) return hipErrorInvalidValue;
    hipLaunchKernelGGL((k_mm<MODE, TM, TN, GC>), dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, st,
                       A, B, Y, (int)M, KN, OHW, G, K_unpack, alpha);
    return hipGetLastError();
}

template <int MODE>
hipError_t launch_mode(const uint32_t* A, const uint32_t* B, float* Y, int64_t M, int KN, int OHW,
                       int G, int K_unpack, float alpha, hipStream_t st) {
    // pick the largest row tile that still gives the 256 CUs a few workgroups each
    auto wgs = [&](int tm, int tn) {
        return ((M + 64 * tm - 1) / (64 * tm)) * ((KN + 4 * tn - 1) / (4 * tn));
    };
    if (wgs(4, 8) >= 1024) return launch_cfg<MODE, 4, 8, 2>(A, B, Y, M, KN, OHW, G, K_unpack, alpha, st);
    if (wgs(2, 8) >= 512) return launch_cfg<MODE, 2, 8, 2>(A, B, Y, M, KN, OHW, G, K_unpack, alpha, st);
    if (wgs(1, 8) >= 256) return launch_cfg<MODE, 1, 8, 2>(A, B, Y, M, KN, OHW, G, K_unpack, alpha, st);
    return launch_cfg<MODE, 1, 4, 2>(A, B, Y, M, KN, OHW, G, K_unpack, alpha, st);
}

}  // namespace

hipError_t launch_mm(int type, const int64_t* d_a, const int64_t* d_b, int64_t M, int OHW, int KN,
                     int Kw, int K_unpack, float alpha, float* d_y, hipStream_t st) {
    const uint32_t* A = reinterpret_cast<const uint32_t*>(d_a);
    const uint32_t* B = reinterpret_cast<const uint32_t*>(d_b);
    const int G = Kw / 4;
    switch (type) {
        case kTNN: return launch_mode<kTNN>(A, B, d_y, M, KN, OHW, G, K_unpack, alpha, st);
        case kTBN: return launch_mode<kTBN>(A, B, d_y, M, KN, OHW, G, K_unpack, alpha, st);
        case kBTN: return launch_mode<kBTN>(A, B, d_y, M, KN, OHW, G, K_unpack, alpha, st);
        case kBNN: return launch_mode<kBNN>(A, B, d_y, M, KN, OHW, G, K_unpack, alpha, st);
    }
    return hipErrorInvalidValue;
}

}  // namespace ftnn
