// Quantise / bit-pack / im2row kernels (gfx950).
//
// Activations (t2r_p2_opt, src/tnns/ternarize2row_avx2.c:715-803; b2r,
// src/tnns/binarize2row_avx2.c:131-199) are produced in two HBM-bound steps:
//
//   1. quantise: fp32 NCHW -> channel-packed pixels P[n][pixel][ic], one 64-bit
//      word per plane for 64 channels.  The input is read exactly once.  Two
//      forms: lanes along pixels (coalesced reads of each channel plane, every
//      lane assembles its own word), and, for 1x1 spatial inputs and row-major
//      GEMM operands where 64 consecutive floats ARE one word, one wavefront
//      ballot per word.
//   2. im2row: a gather of 64-bit words from P into the Packing-2 row layout,
//      one work-item per output word, with the fill rules of the reference for
//      everything not backed by a real (pixel, channel).
//
// Weights (ternarize_opt_avx2 / binarize_opt_avx2, src/utils.c:468-521,634-675)
// and GEMM operands (bitpacking2, src/utils.c:257-291) are packed by their own
// ballot kernels (k_pack_weights, k_pack_gemm_operand): offline work in the
// reference, HBM-bound here (a wavefront per output word group, several coalesced
// loads in flight per lane).
#include "ftnn_internal.h"

namespace ftnn {

namespace {

// position of word idx of plane `plane` in a Packing-2 row
// (src/tnns/ternarize2row_avx2.c:464-469)
__device__ __forceinline__ int64_t p2_pos(int64_t idx, int plane) {
    return (idx >> 2) * 8 + (idx & 3) + (plane ? 4 : 0);
}

// ---------------------------------------------------------------- quantise
// Block = 32 consecutive pixels x 8 channel octets of one 64-channel word.  The 32 lanes
// of an octet read 128 contiguous bytes of one channel plane (coalesced); every thread
// thresholds 8 channels into one byte per plane, the bytes meet in LDS and 32 threads
// write the finished words.  grid (ceil(HW/32), C_pack, N).
template <bool TERN>
__global__ __launch_bounds__(256) void k_quantize_pixels(const float* __restrict__ x,
                                                         const float* __restrict__ thr, int C,
                                                         int HW, int CP,
                                                         unsigned long long* __restrict__ P) {
    __shared__ unsigned long long s_neg[32], s_nz[32];
    const int px = threadIdx.x & 31, oct = threadIdx.x >> 5;
    const int p = blockIdx.x * 32 + px;
    const int ic = blockIdx.y, n = blockIdx.z;
    const float t = thr[n];
    const int c0 = ic * 64 + oct * 8;
    uint32_t neg = 0u, nz = 0u;
    if (p < HW) {
        const float* xp = x + ((size_t)n * C + c0) * HW + p;
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = (c0 + j < C) ? xp[(size_t)j * HW] : 0.0f;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            if (c0 + j < C) {
                if (TERN) {
                    // strict compares, src/tnns/ternarize2row_avx2.c:443-449
                    const bool isneg = v[j] < -t;
                    const bool ispos = v[j] > t;
                    neg |= (isneg ? 1u : 0u) << j;
                    nz |= ((isneg || ispos) ? 1u : 0u) << j;
                } else {
                    // src/tnns/binarize2row_avx2.c:19-21
                    neg |= (v[j] < t ? 1u : 0u) << j;
                }
            }
        }
    }
    reinterpret_cast<unsigned char*>(s_neg)[px * 8 + oct] = (unsigned char)neg;
    if (TERN) reinterpret_cast<unsigned char*>(s_nz)[px * 8 + oct] = (unsigned char)nz;
    __syncthreads();
    if (threadIdx.x < 32 && p < HW) {
        const size_t o = ((size_t)n * HW + p) * CP + ic;
        if (TERN) reinterpret_cast<ulonglong2*>(P)[o] = make_ulonglong2(s_neg[px], ~s_nz[px]);
        else P[o] = s_neg[px];
    }
}

// Quantise straight into the operand form of the fp4 matrix-core layer kernel: one E2M1 nibble
// per channel (0x2 = +1, 0x0 = 0, 0xA = -1; low nibble = even channel), 32 bytes per pixel and
// 64 channels, in planes of 64 channels: P4[n][C_pack][pixel][32 bytes], so that the 32
// consecutive pixels of a matrix-core fragment are (for stride 1) one contiguous KiB.  Channels past C read as the reference's padding
// lanes: zero for ternary inputs (src/tnns/ternarize2row_avx2.c:440-441), +1 for binary ones
// (cleared bits, src/tnns/binarize2row_avx2.c:151).  Same block shape and loads as
// k_quantize_pixels; a thread's 8 channels are one dword, transposed through LDS so that a
// pixel's 32 bytes leave contiguously.
// TILED: the operand of the tile kernel with implicit im2row instead (k_mfma, IMPL): the two 16-byte halves of a record in
// planes of their own, and the columns of an image row sorted by column % stride_w, T4[n][C_pack][half][row][column %
// s][column / s][16 bytes] with ceil(W / s) slots per class: the 32 lanes of a fragment half -- consecutive output
// pixels, i.e. input columns s apart -- then read consecutive 16-byte pieces within an output row, whatever the stride.
template <bool TERN, bool TILED = false>
__global__ __launch_bounds__(256) void k_quantize_f4(const float* __restrict__ x,
                                                     const float* __restrict__ thr, int C, int HW,
                                                     int CP, uint32_t* __restrict__ P4, int W = 0, int SW = 1, int Ws = 0,
                                                     FastDiv dW = FastDiv(), FastDiv dSW = FastDiv()) {
    __shared__ uint32_t s_dw[32 * 9];
    const int px = threadIdx.x & 31, oct = threadIdx.x >> 5;
    const int p = blockIdx.x * 32 + px;
    const int ic = blockIdx.y, n = blockIdx.z;
    const float t = thr[n];
    const int c0 = ic * 64 + oct * 8;
    uint32_t dw = TERN ? 0u : 0x22222222u;
    if (p < HW) {
        const float* xp = x + ((size_t)n * C + c0) * HW + p;
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = (c0 + j < C) ? xp[(size_t)j * HW] : 0.0f;
        dw = 0u;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            uint32_t nib;
            if (TERN) {
                // strict compares, src/tnns/ternarize2row_avx2.c:443-449
                nib = v[j] < -t ? 0xAu : (v[j] > t ? 0x2u : 0x0u);
                if (c0 + j >= C) nib = 0x0u;
            } else {
                // src/tnns/binarize2row_avx2.c:19-21
                nib = v[j] < t ? 0xAu : 0x2u;
                if (c0 + j >= C) nib = 0x2u;
            }
            dw |= nib << (4 * j);
        }
    }
    s_dw[px * 9 + oct] = dw;
    __syncthreads();
    if constexpr (TILED) {
        // thread (pixel, half) stores the half record's 16 bytes
        if (threadIdx.x < 64) {
            const int wp = threadIdx.x & 31, half = threadIdx.x >> 5;
            const int q = blockIdx.x * 32 + wp;
            if (q < HW) {
                const uint32_t ih = fastdiv((uint32_t)q, dW), iw = (uint32_t)q - ih * (uint32_t)W;
                const uint32_t cls_q = fastdiv(iw, dSW), cls = iw - cls_q * (uint32_t)SW;
                const int H = HW / W;
                const size_t piece = ((((size_t)n * CP + ic) * 2 + half) * H + ih) * ((size_t)SW * Ws) + (size_t)cls * Ws + cls_q;
                const uint32_t* d = s_dw + wp * 9 + half * 4;
                reinterpret_cast<uint4*>(P4)[piece] = make_uint4(d[0], d[1], d[2], d[3]);
            }
        }
        // the fill piece right behind the planes: what a tap outside the image contributes (0, or +1 for binary inputs)
        if (threadIdx.x == 64 && blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0) {
            const uint32_t f = TERN ? 0u : 0x22222222u;
            const int H = HW / W;
            reinterpret_cast<uint4*>(P4)[(size_t)gridDim.z * CP * 2 * H * ((size_t)SW * Ws)] = make_uint4(f, f, f, f);
        }
    } else {
        const int wp = threadIdx.x >> 3, wo = threadIdx.x & 7;
        const int q = blockIdx.x * 32 + wp;
        if (q < HW) P4[(((size_t)n * CP + ic) * HW + q) * 8 + wo] = s_dw[wp * 9 + wo];
    }
}

// One wavefront ballot per 64-bit word: rows of J consecutive floats.
// MODE 0: ternary thresholds, 1: binary threshold, 2: exact values {-1,0,+1}
// (bitpacking2).  P2ROW: write straight into Packing-2 rows of 2*J/64 words
// instead of the (sign, zero) pair array.  grid (R, ceil(words/4)), block 256.
template <int MODE, bool P2ROW>
__global__ __launch_bounds__(256) void k_quantize_ballot(const float* __restrict__ x,
                                                         const float* __restrict__ thr, int J,
                                                         int words,
                                                         unsigned long long* __restrict__ out) {
    const int lane = threadIdx.x & 63;
    const int wd = blockIdx.y * 4 + (threadIdx.x >> 6);
    const int r = blockIdx.x;
    if (wd >= words) return;  // uniform per wavefront
    const int j = wd * 64 + lane;
    const bool in = j < J;
    const float v = in ? x[(size_t)r * J + j] : 0.0f;
    bool isneg, isnz;
    if (MODE == 0) {
        const float t = thr[r];
        isneg = in && v < -t;
        isnz = in && (isneg || v > t);
    } else if (MODE == 1) {
        isneg = in && v < thr[r];
        isnz = true;
    } else {
        isneg = v == -1.0f;
        isnz = !(v == 0.0f);
    }
    const unsigned long long s = __ballot(isneg);
    const unsigned long long z = ~__ballot(isnz);
    if (lane == 0) {
        if (P2ROW) {
            unsigned long long* row = out + (size_t)r * 2 * words;
            row[p2_pos(wd, 0)] = s;
            row[p2_pos(wd, 1)] = z;
        } else if (MODE == 1) {
            out[(size_t)r * words + wd] = s;
        } else {
            reinterpret_cast<ulonglong2*>(out)[(size_t)r * words + wd] = make_ulonglong2(s, z);
        }
    }
}

// ------------------------------------------------------------------ im2row
// One work-item per 16 bytes of output: two consecutive words of one plane of one group of 4 words of
// one output row (ternary group = 4 sign words then 4 zero words, 64 bytes; binary group = 4 words, 32
// bytes).  It gathers its two (tap, channel word) sources from P, or takes the fill
// (src/tnns/ternarize2row_avx2.c:440-441,748-755; src/tnns/binarize2row_avx2.c:151).  Neighbouring
// work-items write neighbouring 16 bytes, so every store instruction covers one contiguous KiB.
template <bool TERN>
__global__ __launch_bounds__(256) void k_im2row(const unsigned long long* __restrict__ P, int H,
                                                int W, int CP, int OHW, int OW, int KW, int K,
                                                int Kw, int H_pad, int W_pad, int H_stride,
                                                int W_stride, int64_t total, FastDiv dPR, FastDiv dOHW,
                                                FastDiv dOW, FastDiv dCP, FastDiv dKW,
                                                ulonglong2* __restrict__ out) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;   // < 2^32, checked by the host
    if (e >= total) return;
    constexpr int PPG = TERN ? 4 : 2;             // 16-byte pieces per group
    const int PR = (Kw / 4) * PPG;                // pieces per row
    const uint32_t r = fastdiv((uint32_t)e, dPR);
    const int pr = (int)((uint32_t)e - r * (uint32_t)PR);
    const int g = pr / PPG, piece = pr % PPG;
    const bool zero_plane = TERN && piece >= 2;
    const int idx0 = 4 * g + 2 * (piece & 1);     // first of the two words
    const uint32_t n = fastdiv(r, dOHW), pix = r - n * (uint32_t)OHW;
    const int oh = (int)fastdiv(pix, dOW), ow = (int)pix - oh * OW;
    const int ih0 = oh * H_stride - H_pad, iw0 = ow * W_stride - W_pad;
    const size_t img = (size_t)n * H * W;
    unsigned long long v[2];
#pragma unroll
    for (int q = 0; q < 2; q++) {
        const int idx = idx0 + q;
        v[q] = zero_plane ? ~0ull : 0ull;
        if (idx < K) {
            const int tap = (int)fastdiv((uint32_t)idx, dCP), ic = idx - tap * CP;
            const int kh = (int)fastdiv((uint32_t)tap, dKW), kw = tap - kh * KW;
            const int ih = ih0 + kh, iw = iw0 + kw;
            if ((unsigned)ih < (unsigned)H && (unsigned)iw < (unsigned)W) {
                const size_t o = (img + (size_t)ih * W + iw) * CP + ic;
                v[q] = TERN ? P[2 * o + (zero_plane ? 1 : 0)] : P[o];
            }
        }
    }
    out[e] = make_ulonglong2(v[0], v[1]);
}

// ------------------------------------------------------------- weight packers
// w is fp32 (KN, C, KH, KW).  A wavefront packs the words of one (kernel n, channel word ic): lane = channel within
// the word, one ballot per tap and plane.  The taps of a channel are neighbours in memory, so a wavefront meets the
// same cache lines again from tap to tap, and four taps' loads leave before the first is used.  The wavefront of
// ic = 0 also writes the padding words that round a row up to a multiple of 4.
// grid ceil(KN * CP / 4), block 256.
template <bool TERN>
__global__ __launch_bounds__(256) void k_pack_weights(const float* __restrict__ w,
                                                      const float* __restrict__ thr, int C,
                                                      int taps, int CP, int K, int Kw,
                                                      int64_t pairs,
                                                      unsigned long long* __restrict__ out) {
    const int lane = threadIdx.x & 63;
    const int64_t e = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);   // (n, ic), uniform per wavefront
    if (e >= pairs) return;
    const int64_t n = e / CP;
    const int ic = (int)(e - n * CP);
    const int c = ic * 64 + lane;
    const bool real = c < C;
    const float t = thr[n];
    const float* src = w + ((size_t)n * C + (real ? c : 0)) * taps;
    unsigned long long* row = out + (size_t)n * (TERN ? 2 : 1) * Kw;
    for (int tap0 = 0; tap0 < taps; tap0 += 4) {
        float v[4];
#pragma unroll
        for (int k = 0; k < 4; k++) v[k] = (real && tap0 + k < taps) ? src[tap0 + k] : 0.0f;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            if (tap0 + k >= taps) break;   // uniform
            const int idx = (tap0 + k) * CP + ic;
            if (TERN) {
                // channels past C read as 0.0 and take the same compares, positive side first (src/utils.c:498-509)
                const bool pos = v[k] > t;
                const bool neg = !pos && v[k] < -t;
                const unsigned long long s = __ballot(neg), z = __ballot(!pos && !neg);
                if (lane == 0) {
                    row[p2_pos(idx, 0)] = s;
                    row[p2_pos(idx, 1)] = z;
                }
            } else {
                const unsigned long long s = __ballot(real && v[k] < t);   // src/utils.c:654-660
                if (lane == 0) row[idx] = s;
            }
        }
    }
    // padding words: (sign 0, zero all ones) for ternary rows (src/utils.c:483-490), 0 for binary ones (:643-647)
    if (ic == 0 && lane < Kw - K) {
        const int idx = K + lane;
        if (TERN) {
            row[p2_pos(idx, 0)] = 0ull;
            row[p2_pos(idx, 1)] = ~0ull;
        } else {
            row[idx] = 0ull;
        }
    }
}

// ------------------------------------------------------- dense rows for small C
// With C <= 32 a Packing-2 word carries C live lanes out of 64 (C = 3 in an RGB stem: 3 of 64).
// The GEMM result only depends on the multiset of (activation lane, weight lane) pairs, so both
// operands may be re-packed with T = 64 / C taps per word: lane (tap t, channel c) -> word t / T,
// bit (t % T) * C + c.  Unused lanes are (sign 0, zero 1) / 0 exactly like the reference's fill, and
// the existing GEMM kernels run unchanged on Kd = ceil(KH*KW / T) words instead of KH*KW.

// activations: one work-item per (row, dense word); gathers T taps from P (C_pack = 1)
template <bool TERN>
__global__ __launch_bounds__(256) void k_dense_rows(const unsigned long long* __restrict__ P, int C, int T,
                                                    int H, int W, int OH, int OW, int KW, int taps, int Kd,
                                                    int Kdw, int H_pad, int W_pad, int H_stride,
                                                    int W_stride, int64_t total,
                                                    unsigned long long* __restrict__ out) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= total) return;
    const int64_t r = e / Kdw;
    const int d = (int)(e - r * Kdw);
    unsigned long long s = 0ull, z = ~0ull;
    if (d < Kd) {
        const int ow = (int)(r % OW);
        const int64_t t2 = r / OW;
        const int oh = (int)(t2 % OH);
        const int64_t n = t2 / OH;
        const unsigned long long cmask = (1ull << C) - 1ull;
        for (int j = 0; j < T; j++) {
            const int tap = d * T + j;
            if (tap >= taps) break;
            const int kh = tap / KW, kw = tap - kh * KW;
            const int ih = oh * H_stride + kh - H_pad, iw = ow * W_stride + kw - W_pad;
            if (ih >= 0 && ih < H && iw >= 0 && iw < W) {
                const size_t o = (size_t)n * H * W + (size_t)ih * W + iw;
                if (TERN) {
                    const ulonglong2 v = reinterpret_cast<const ulonglong2*>(P)[o];
                    s |= (v.x & cmask) << (j * C);
                    z &= ~((~v.y & cmask) << (j * C));
                } else {
                    s |= (P[o] & cmask) << (j * C);
                }
            }
        }
    }
    if (!TERN && d >= Kd) s = 0ull;
    if (TERN) {
        unsigned long long* row = out + (size_t)r * 2 * Kdw;
        row[p2_pos(d, 0)] = s;
        row[p2_pos(d, 1)] = z;
    } else {
        out[(size_t)r * Kdw + d] = s;
    }
}

// ---- the same re-packing for the fp4 matrix-core layer kernel (C <= 8) ----
// k_quantize_nib: one dword per pixel, nibble c = channel c as E2M1 (0x2 / 0x0 / 0xA), channels past C
// as the padding lane of the type (ternary 0, binary +1).
template <bool TERN>
__global__ __launch_bounds__(256) void k_quantize_nib(const float* __restrict__ x, const float* __restrict__ thr,
                                                      int C, int HW, uint32_t* __restrict__ Pq) {
    const int p = blockIdx.x * 256 + threadIdx.x, n = blockIdx.y;
    if (p >= HW) return;
    const float t = thr[n];
    const float* xp = x + (size_t)n * C * HW + p;
    uint32_t dw = 0u;
#pragma unroll
    for (int c = 0; c < 8; c++) {
        const float v = c < C ? xp[(size_t)c * HW] : 0.0f;
        uint32_t nib;
        if (TERN) nib = c < C ? (v < -t ? 0xAu : (v > t ? 0x2u : 0x0u)) : 0x0u;
        else nib = c < C ? (v < t ? 0xAu : 0x2u) : 0x2u;
        dw |= nib << (4 * c);
    }
    Pq[(size_t)n * HW + p] = dw;
}

// k_dense_rows_f4: one work-item per output pixel walks the KH*KW taps once and strings their C
// nibbles together, T = 64 / C taps per 64-lane word (lane (tap % T)*C + c, as in k_dense_rows), the
// lanes left over holding the padding lane of the type like taps outside the image.  C is a template
// parameter: every shift and every position in the word's eight dwords is then a constant, the word
// is assembled in registers and leaves as two 16-byte stores (32 contiguous bytes per pixel,
// neighbouring pixels next to each other).
// Output = the fp4 layer kernel's operand for a 1x1 layer over the output pixels with Kd words per
// pixel: A4[n][d][pixel][32 bytes].
template <bool TERN, int C>
__global__ __launch_bounds__(256) void k_dense_rows_f4(const uint32_t* __restrict__ Pq, int H, int W, int OHW,
                                                       int OW, int KW, int taps, int Kd, int H_pad, int W_pad,
                                                       int H_stride, int W_stride, FastDiv dOW,
                                                       uint4* __restrict__ A4) {
    constexpr int T = 64 / C;
    constexpr uint32_t padv = TERN ? 0u : 0x22222222u;
    constexpr uint32_t cmask = C >= 8 ? 0xffffffffu : ((1u << (4 * (C & 7))) - 1u);
    const int pix = blockIdx.x * 256 + threadIdx.x, n = blockIdx.y;
    if (pix >= OHW) return;
    const int oh = (int)fastdiv((uint32_t)pix, dOW), ow = pix - oh * OW;
    const int ih0 = oh * H_stride - H_pad, iw0 = ow * W_stride - W_pad;
    const uint32_t* img = Pq + (size_t)n * H * W;
    int kh = 0, kw = 0, tap = 0;
    for (int d = 0; d < Kd; d++) {
        uint32_t o[8];
#pragma unroll
        for (int i = 0; i < 8; i++) o[i] = padv;   // left-over lanes and missing taps stay padding
#pragma unroll
        for (int j = 0; j < T; j++) {
            const int ih = ih0 + kh, iw = iw0 + kw;
            const bool in = tap < taps && (unsigned)ih < (unsigned)H && (unsigned)iw < (unsigned)W;
            // the load is unconditional (pixel 0 stands in for a tap outside the image) so that all T loads
            // of a word can be in flight together
            const uint32_t raw = img[in ? ih * W + iw : 0];
            const uint32_t v = (in ? raw : padv) & cmask;
            if (++kw == KW) {
                kw = 0;
                kh++;
            }
            tap++;
            // lanes [j*C, j*C + C) of the word: bits [4*j*C, 4*j*C + 4*C) of its eight dwords
            const int bit = 4 * j * C, lo = bit >> 5, sh = bit & 31;
            o[lo] = (o[lo] & ~(cmask << sh)) | (v << sh);
            if (sh + 4 * C > 32) {   // compile-time after unrolling: the tap straddles two dwords
                const int rest = 32 - sh;
                o[lo + 1] = (o[lo + 1] & ~(cmask >> rest)) | (v >> rest);
            }
        }
        uint4* dst = A4 + (((size_t)n * Kd + d) * OHW + pix) * 2;
        dst[0] = make_uint4(o[0], o[1], o[2], o[3]);
        dst[1] = make_uint4(o[4], o[5], o[6], o[7]);
    }
}

// The same with the kernel window known at compile time (the 3x3 and 7x7 windows of first layers): the tap of
// every word position is then a constant, so the row and column of a tap are looked up in per-thread tables
// filled once (clamped index, validity), its address is one add, and it enters the word with one or two
// shift-or instructions.
template <bool TERN, int C, int KH, int KW>
__global__ __launch_bounds__(256) void k_dense_rows_f4_win(const uint32_t* __restrict__ Pq, int H, int W, int OHW,
                                                           int OW, int H_pad, int W_pad, int H_stride, int W_stride,
                                                           FastDiv dOW, uint4* __restrict__ A4) {
    constexpr int T = 64 / C, taps = KH * KW, Kd = (taps + T - 1) / T;
    constexpr uint32_t padv = TERN ? 0u : 0x22222222u;
    constexpr uint32_t cmask = C >= 8 ? 0xffffffffu : ((1u << (4 * (C & 7))) - 1u);
    const int pix = blockIdx.x * 256 + threadIdx.x, n = blockIdx.y;
    if (pix >= OHW) return;
    const int oh = (int)fastdiv((uint32_t)pix, dOW), ow = pix - oh * OW;
    const int ih0 = oh * H_stride - H_pad, iw0 = ow * W_stride - W_pad;
    const uint32_t* img = Pq + (size_t)n * H * W;
    int rowoff[KH], col[KW];
    bool rowok[KH], colok[KW];
#pragma unroll
    for (int kh = 0; kh < KH; kh++) {
        const int ih = ih0 + kh;
        rowok[kh] = (unsigned)ih < (unsigned)H;
        rowoff[kh] = (rowok[kh] ? ih : 0) * W;
    }
#pragma unroll
    for (int kw = 0; kw < KW; kw++) {
        const int iw = iw0 + kw;
        colok[kw] = (unsigned)iw < (unsigned)W;
        col[kw] = colok[kw] ? iw : 0;
    }
#pragma unroll
    for (int d = 0; d < Kd; d++) {
        uint32_t o[8];
#pragma unroll
        for (int i = 0; i < 8; i++) o[i] = 0u;
#pragma unroll
        for (int j = 0; j < T; j++) {
            const int tap = d * T + j;
            const int bit = 4 * j * C, lo = bit >> 5, sh = bit & 31;
            uint32_t v;
            if (tap < taps) {   // compile-time after unrolling
                const int kh = tap / KW, kw = tap % KW;
                const uint32_t raw = img[rowoff[kh] + col[kw]];
                v = ((rowok[kh] && colok[kw]) ? raw : padv) & cmask;
            } else {
                v = padv & cmask;
            }
            o[lo] |= v << sh;
            if (sh + 4 * C > 32) o[lo + 1] |= v >> (32 - sh);
        }
        // lanes past T * C hold the padding lane of the type
        constexpr int used = 4 * T * C;   // bits
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if (32 * i >= used) o[i] |= padv;
            else if (32 * (i + 1) > used) o[i] |= padv & ~((1u << (used - 32 * i)) - 1u);
        }
        uint4* dst = A4 + (((size_t)n * Kd + d) * OHW + pix) * 2;
        dst[0] = make_uint4(o[0], o[1], o[2], o[3]);
        dst[1] = make_uint4(o[4], o[5], o[6], o[7]);
    }
}

// weights: one work-item per (kernel, dense word); source rows are the reference's packed rows
// with C_pack = 1 (word index = tap)
template <bool TERN>
__global__ __launch_bounds__(256) void k_dense_weights(const unsigned long long* __restrict__ Q, int C, int T,
                                                       int taps, int Kw, int Kd, int Kdw, int64_t total,
                                                       unsigned long long* __restrict__ out) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= total) return;
    const int64_t n = e / Kdw;
    const int d = (int)(e - n * Kdw);
    unsigned long long s = 0ull, z = TERN ? ~0ull : 0ull;
    if (d < Kd) {
        const unsigned long long cmask = (1ull << C) - 1ull;
        for (int j = 0; j < T; j++) {
            const int tap = d * T + j;
            if (tap >= taps) break;
            if (TERN) {
                const unsigned long long* row = Q + (size_t)n * 2 * Kw;
                s |= (row[p2_pos(tap, 0)] & cmask) << (j * C);
                z &= ~((~row[p2_pos(tap, 1)] & cmask) << (j * C));
            } else {
                s |= (Q[(size_t)n * Kw + tap] & cmask) << (j * C);
            }
        }
    }
    if (TERN) {
        unsigned long long* row = out + (size_t)n * 2 * Kdw;
        row[p2_pos(d, 0)] = s;
        row[p2_pos(d, 1)] = z;
    } else {
        out[(size_t)n * Kdw + d] = s;
    }
}

}  // namespace

bool dense_applies(int C, int KH, int KW, int* T_out, int* Kd_out) {
    if (C > 32) return false;
    const int T = 64 / C, taps = KH * KW;
    const int Kd = (taps + T - 1) / T;
    if (T_out) *T_out = T;
    if (Kd_out) *Kd_out = Kd;
    return round4(taps) >= 2 * round4(Kd);   // at least halves the GEMM work
}

hipError_t launch_dense_rows(bool ternary, const void* d_p, int N, int C, int H, int W, int H_pad, int W_pad,
                             int kH, int kW, int H_stride, int W_stride, int64_t* d_out, hipStream_t st) {
    int T, Kd;
    dense_applies(C, kH, kW, &T, &Kd);
    const int OH = out_dim(H, H_pad, kH, H_stride), OW = out_dim(W, W_pad, kW, W_stride);
    const int Kdw = round4(Kd);
    const int64_t total = (int64_t)N * OH * OW * Kdw;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    const unsigned long long* P = static_cast<const unsigned long long*>(d_p);
    unsigned long long* out = reinterpret_cast<unsigned long long*>(d_out);
    if (ternary)
        hipLaunchKernelGGL((k_dense_rows<true>), dim3(blocks), dim3(256), 0, st, P, C, T, H, W, OH, OW, kW,
                           kH * kW, Kd, Kdw, H_pad, W_pad, H_stride, W_stride, total, out);
    else
        hipLaunchKernelGGL((k_dense_rows<false>), dim3(blocks), dim3(256), 0, st, P, C, T, H, W, OH, OW, kW,
                           kH * kW, Kd, Kdw, H_pad, W_pad, H_stride, W_stride, total, out);
    return hipGetLastError();
}

bool dense_f4_applies(int C, int KH, int KW) { return C <= 8 && dense_applies(C, KH, KW, nullptr, nullptr); }

int64_t dense_f4_pq_bytes(int N, int H, int W) { return ((int64_t)N * H * W * 4 + 255) / 256 * 256; }

hipError_t launch_dense_rows_f4(bool ternary, const float* d_x, const float* d_thr, int N, int C, int H, int W,
                                int H_pad, int W_pad, int kH, int kW, int H_stride, int W_stride, void* d_pq,
                                void* d_a4, hipStream_t st) {
    int T, Kd;
    dense_applies(C, kH, kW, &T, &Kd);
    const int OH = out_dim(H, H_pad, kH, H_stride), OW = out_dim(W, W_pad, kW, W_stride);
    const int HW = H * W, OHW = OH * OW;
    if (N > 65535 || Kd > 65535) return hipErrorInvalidValue;
    uint32_t* Pq = static_cast<uint32_t*>(d_pq);
    uint4* A4 = static_cast<uint4*>(d_a4);
    dim3 gq((HW + 255) / 256, N), gr((OHW + 255) / 256, N);
    const FastDiv dOW = make_fastdiv((uint32_t)OW);
    (void)T;
    if (ternary) hipLaunchKernelGGL((k_quantize_nib<true>), gq, dim3(256), 0, st, d_x, d_thr, C, HW, Pq);
    else hipLaunchKernelGGL((k_quantize_nib<false>), gq, dim3(256), 0, st, d_x, d_thr, C, HW, Pq);
#define FTNN_DENSE_WIN(TERN_, C_, K_)                                                                             \
    hipLaunchKernelGGL((k_dense_rows_f4_win<TERN_, C_, K_, K_>), gr, dim3(256), 0, st, Pq, H, W, OHW, OW, H_pad, W_pad, \
                       H_stride, W_stride, dOW, A4)
#define FTNN_DENSE_T(TERN_, C_)                                                                                     \
    if (kH == 3 && kW == 3) FTNN_DENSE_WIN(TERN_, C_, 3);                                                           \
    else if (kH == 7 && kW == 7) FTNN_DENSE_WIN(TERN_, C_, 7);                                                      \
    else hipLaunchKernelGGL((k_dense_rows_f4<TERN_, C_>), gr, dim3(256), 0, st, Pq, H, W, OHW, OW, kW, kH * kW, Kd,    \
                            H_pad, W_pad, H_stride, W_stride, dOW, A4)
#define FTNN_DENSE(C_)                                                                                              \
    case C_:                                                                                                        \
        if (ternary) { FTNN_DENSE_T(true, C_); }                                                                    \
        else { FTNN_DENSE_T(false, C_); }                                                                           \
        break;
    switch (C) {
        FTNN_DENSE(1) FTNN_DENSE(2) FTNN_DENSE(3) FTNN_DENSE(4) FTNN_DENSE(5) FTNN_DENSE(6) FTNN_DENSE(7) FTNN_DENSE(8)
        default: return hipErrorInvalidValue;
    }
#undef FTNN_DENSE
#undef FTNN_DENSE_T
#undef FTNN_DENSE_WIN
    return hipGetLastError();
}

hipError_t launch_dense_weights(bool ternary, const int64_t* d_qw, int KN, int C, int kH, int kW,
                                int64_t* d_out, hipStream_t st) {
    int T, Kd;
    dense_applies(C, kH, kW, &T, &Kd);
    const int Kw = round4(kH * kW), Kdw = round4(Kd);
    const int64_t total = (int64_t)KN * Kdw;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    const unsigned long long* Q = reinterpret_cast<const unsigned long long*>(d_qw);
    unsigned long long* out = reinterpret_cast<unsigned long long*>(d_out);
    if (ternary)
        hipLaunchKernelGGL((k_dense_weights<true>), dim3(blocks), dim3(256), 0, st, Q, C, T, kH * kW, Kw, Kd, Kdw,
                           total, out);
    else
        hipLaunchKernelGGL((k_dense_weights<false>), dim3(blocks), dim3(256), 0, st, Q, C, T, kH * kW, Kw, Kd,
                           Kdw, total, out);
    return hipGetLastError();
}

hipError_t launch_quantize(bool ternary, const float* d_x, const float* d_thr, int N, int C, int H, int W,
                           void* d_p, hipStream_t st) {
    const int CP = cpack_of(C), HW = H * W;
    unsigned long long* P = static_cast<unsigned long long*>(d_p);
    if (HW == 1) {
        // 64 consecutive floats are one word: wavefront ballot
        dim3 grid(N, (CP + 3) / 4);
        if (ternary)
            hipLaunchKernelGGL((k_quantize_ballot<0, false>), grid, dim3(256), 0, st, d_x, d_thr, C,
                               CP, P);
        else
            hipLaunchKernelGGL((k_quantize_ballot<1, false>), grid, dim3(256), 0, st, d_x, d_thr, C,
                               CP, P);
    } else {
        dim3 grid((HW + 31) / 32, CP, N);
        if (ternary)
            hipLaunchKernelGGL((k_quantize_pixels<true>), grid, dim3(256), 0, st, d_x, d_thr, C, HW,
                               CP, P);
        else
            hipLaunchKernelGGL((k_quantize_pixels<false>), grid, dim3(256), 0, st, d_x, d_thr, C,
                               HW, CP, P);
    }
    return hipGetLastError();
}

hipError_t launch_quantize_f4(bool ternary, const float* d_x, const float* d_thr, int N, int C, int H, int W,
                              void* d_p4, hipStream_t st) {
    const int CP = cpack_of(C), HW = H * W;
    dim3 grid((HW + 31) / 32, CP, N);
    uint32_t* P4 = static_cast<uint32_t*>(d_p4);
    if (ternary) hipLaunchKernelGGL((k_quantize_f4<true>), grid, dim3(256), 0, st, d_x, d_thr, C, HW, CP, P4, 0, 1, 0, FastDiv(), FastDiv());
    else hipLaunchKernelGGL((k_quantize_f4<false>), grid, dim3(256), 0, st, d_x, d_thr, C, HW, CP, P4, 0, 1, 0, FastDiv(), FastDiv());
    return hipGetLastError();
}

// bytes of T4 (k_quantize_f4 with TILED) for this input and column stride
int64_t quantize_f4_tiled_bytes(int N, int C, int H, int W, int W_stride) {
    return (int64_t)N * cpack_of(C) * 2 * H * W_stride * ((W + W_stride - 1) / W_stride) * 16 + 16;   // + the fill piece
}

hipError_t launch_quantize_f4_tiled(bool ternary, const float* d_x, const float* d_thr, int N, int C, int H, int W,
                                    int W_stride, void* d_t4, hipStream_t st) {
    const int CP = cpack_of(C), HW = H * W, Ws = (W + W_stride - 1) / W_stride;
    dim3 grid((HW + 31) / 32, CP, N);
    uint32_t* T4 = static_cast<uint32_t*>(d_t4);
    const FastDiv dW = make_fastdiv((uint32_t)W), dSW = make_fastdiv((uint32_t)W_stride);
    // slots of a class past its last column (W % s != 0) are never read: the gather reads real columns only
    if (ternary) hipLaunchKernelGGL((k_quantize_f4<true, true>), grid, dim3(256), 0, st, d_x, d_thr, C, HW, CP, T4, W, W_stride, Ws, dW, dSW);
    else hipLaunchKernelGGL((k_quantize_f4<false, true>), grid, dim3(256), 0, st, d_x, d_thr, C, HW, CP, T4, W, W_stride, Ws, dW, dSW);
    return hipGetLastError();
}

hipError_t launch_quantize_im2row(bool ternary, const float* d_x, const float* d_thr, int N, int C,
                                  int H, int W, int H_pad, int W_pad, int kH, int kW, int H_stride,
                                  int W_stride, int64_t* d_out, void* d_scratch, hipStream_t st) {
    const int CP = cpack_of(C);
    const int OH = out_dim(H, H_pad, kH, H_stride), OW = out_dim(W, W_pad, kW, W_stride);
    const int K = CP * kH * kW, Kw = round4(K);
    unsigned long long* P = static_cast<unsigned long long*>(d_scratch);
    hipError_t e = launch_quantize(ternary, d_x, d_thr, N, C, H, W, d_scratch, st);
    if (e != hipSuccess) return e;
    const int pieces_per_row = (Kw / 4) * (ternary ? 4 : 2);   // 16-byte pieces
    const int64_t total = (int64_t)N * OH * OW * pieces_per_row;
    if (total > 0xffffffffLL) return hipErrorInvalidValue;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    ulonglong2* out = reinterpret_cast<ulonglong2*>(d_out);
    const FastDiv dPR = make_fastdiv((uint32_t)pieces_per_row), dOHW = make_fastdiv((uint32_t)(OH * OW)),
                  dOW = make_fastdiv((uint32_t)OW), dCP = make_fastdiv((uint32_t)CP), dKW = make_fastdiv((uint32_t)kW);
    if (ternary)
        hipLaunchKernelGGL((k_im2row<true>), dim3(blocks), dim3(256), 0, st, P, H, W, CP, OH * OW, OW, kW,
                           K, Kw, H_pad, W_pad, H_stride, W_stride, total, dPR, dOHW, dOW, dCP, dKW, out);
    else
        hipLaunchKernelGGL((k_im2row<false>), dim3(blocks), dim3(256), 0, st, P, H, W, CP, OH * OW, OW,
                           kW, K, Kw, H_pad, W_pad, H_stride, W_stride, total, dPR, dOHW, dOW, dCP, dKW, out);
    return hipGetLastError();
}

hipError_t launch_pack_weights(bool ternary, const float* d_w, const float* d_thr, int KN, int C,
                               int KH, int KW, int64_t* d_out, hipStream_t st) {
    const int CP = cpack_of(C), K = CP * KH * KW, Kw = round4(K);
    const int64_t pairs = (int64_t)KN * CP;   // (kernel, channel word)
    if ((pairs + 3) / 4 > 0x7fffffffLL) return hipErrorInvalidValue;
    const unsigned blocks = (unsigned)((pairs + 3) / 4);
    unsigned long long* out = reinterpret_cast<unsigned long long*>(d_out);
    if (ternary)
        hipLaunchKernelGGL((k_pack_weights<true>), dim3(blocks), dim3(256), 0, st, d_w, d_thr, C,
                           KH * KW, CP, K, Kw, pairs, out);
    else
        hipLaunchKernelGGL((k_pack_weights<false>), dim3(blocks), dim3(256), 0, st, d_w, d_thr, C,
                           KH * KW, CP, K, Kw, pairs, out);
    return hipGetLastError();
}

// bitpacking2 (src/utils.c:257-291) of rows of J = 256 * groups floats in {-1, 0, +1}.  A wavefront packs one group
// of 256 values into its 4 sign and 4 zero words: lane l loads values l, 64 + l, 128 + l, 192 + l (four coalesced
// loads in flight per lane), one ballot per load and plane is one word, and lanes 0..7 store the group's 64 bytes.
// grid (rows, ceil(groups / 4)), block 256.
__global__ __launch_bounds__(256) void k_pack_gemm_operand(const float* __restrict__ x, int J, int groups,
                                                           unsigned long long* __restrict__ out) {
    const int lane = threadIdx.x & 63;
    const int g = blockIdx.y * 4 + (threadIdx.x >> 6);
    const size_t r = blockIdx.x;
    if (g >= groups) return;   // uniform per wavefront
    const float* src = x + r * (size_t)J + (size_t)g * 256 + lane;
    float v[4];
#pragma unroll
    for (int c = 0; c < 4; c++) v[c] = src[64 * c];
    unsigned long long mine = 0;
#pragma unroll
    for (int c = 0; c < 4; c++) {
        const unsigned long long s = __ballot(v[c] == -1.0f);
        const unsigned long long z = ~__ballot(!(v[c] == 0.0f));
        if (lane == c) mine = s;
        if (lane == 4 + c) mine = z;
    }
    if (lane < 8) out[(r * (size_t)groups + (size_t)g) * 8 + lane] = mine;
}

hipError_t launch_pack_gemm_operand(const float* d_x, int I, int J, int64_t* d_out, hipStream_t st) {
    const int groups = J / 256;   // the caller has checked J % 256 == 0
    dim3 grid(I, (groups + 3) / 4);
    hipLaunchKernelGGL(k_pack_gemm_operand, grid, dim3(256), 0, st, d_x, J, groups,
                       reinterpret_cast<unsigned long long*>(d_out));
    return hipGetLastError();
}

}  // namespace ftnn
