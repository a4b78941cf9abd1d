// Matrix-core formulation of the same GEMMs (gfx950): the comparison path to the
// vector-ALU popcount kernel of mm_kernels.hip, selected where it measures faster.
//
// Semantics are unchanged (src/tnns/mm_p2_final_{tnn,tbn,btn,bnn}_avx2.c): every
// accumulator is the integer dot product of the decoded {-1,0,+1} / {-1,+1} lanes,
// which is what the popcount formulas compute, so results stay bit-exact:
//   * MFMA int8  (v_mfma_i32_32x32x32_i8): lanes become bytes 0x01 / 0x00 / 0xFF, int32
//     accumulate;
//   * MFMA fp4   (v_mfma_f32_32x32x64_f8f6f4, E2M1): lanes become nibbles 0x2 / 0x0 / 0xA
//     (+1.0 / 0 / -1.0), fp32 accumulate -- exact while 64*Kw < 2^24, which the host
//     checks.  Twice the matrix rate of int8 and half the operand bytes.  This is the form
//     of the conv layer kernels and their prepared weights; the fp4 GEMM engine itself
//     (k_pack4, k_mfma_p4 further down) codes a lane a as (a + 1) / 2 at two bits per lane.
//
// The kernels of the int8 engine and of the layers' GEMM route:
//   k_expand  Packing-2 (or single-plane binary) rows -> "fragments": 1 KiB blocks
//             holding 32 rows x 32 (int8) or 64 (fp4) lanes in exactly the register
//             layout of an MFMA operand (lane l = (k half l/32, row l%32), 16 bytes).
//             HBM-bound, one pass per operand.
//   k_mfma    256 x 256 output tile per workgroup (4 wavefronts, 128 x 128 each, 256
//             accumulator registers per lane).  Fragments travel global -> LDS with
//             LDS-direct loads (no VGPRs, and a fragment lands contiguously, so the
//             later 128-bit LDS reads are conflict-free without padding), through a
//             4-stage ring; one barrier per step.  LDS reads of the next fragment and
//             the DMA issue are interleaved with the MFMAs of the current one.
#include <type_traits>

#include "ftnn_internal.h"

namespace ftnn {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));

// Ring of NS LDS buffers, each holding KF fragments (K words for fp4) per row-block: one barrier per KF fragments.
// A workgroup of 2 x 2 wavefronts computes (64 WTP) x (64 WTQ) results, a wavefront WTP x WTQ blocks of 32 x 32:
// 4 x 4 for problems with enough 256 x 256 tiles to fill the chip, 2 x 2 (128 x 128) below that, 4 x 2 (256 kernels x
// 128 pixels) for conv layers on the tile kernel, whose kernel side is the cheaper one to stage.
template <int WTP, int WTQ, int KF, int NS>
struct Tile {
    static constexpr int RBP = 2 * WTP, RBQ = 2 * WTQ;   // row-blocks per operand side
    static constexpr int FR = (RBP + RBQ) * KF;          // fragments per step: the P row-blocks' first, then the Q ones'
    static constexpr int FW = FR / 4;                    // fragments staged by one wavefront per step
    static constexpr int NL = WTP + WTQ;                 // LDS reads per wavefront and k fragment
    static constexpr int NM = WTP * WTQ;                 // multiplies per wavefront and k fragment
    static constexpr int DPI = FW / NL;                  // fragments a wavefront stages per LDS read of the last fragment
    static constexpr size_t lds_bytes = (size_t)NS * FR * 1024;
    static_assert(FR % 4 == 0 && FW % NL == 0, "whole staged fragments per wavefront and per LDS read");
    static_assert(NS >= 2 && KF % 2 == 0, "register sets alternate per fragment");
};

// ------------------------------------------------------------------ expansion
// grid (row-blocks, groups / 4), block 256: thread = (row r = t%32, dword pair dq = t/32).
// A group is 4 words (256 lanes) of a packed row: 16 dwords (8 sign, 8 zero) for ternary
// rows, 8 dwords for binary rows.  Rows past `rows` expand to zeros.
template <bool F4, bool TERN>
__device__ __forceinline__ void expand_block(const uint32_t* __restrict__ P, int rows, int G, uint4* __restrict__ out, int rb,
                                             int gy, uint32_t* stage) {
    // A workgroup expands kGPB adjacent groups of its 32 rows: 256 contiguous bytes of each ternary row (128 of a
    // binary one).  They are fetched row-wise, 16 bytes per thread with neighbouring threads on neighbouring bytes,
    // and turned through LDS into the (row, dword) order the expansion works in: fetched in that order directly,
    // every load instruction would touch 32 cache lines for 256 bytes.
    constexpr int kGPB = 4;
    constexpr int DPG = TERN ? 16 : 8;        // dwords per group and row
    constexpr int RD = kGPB * DPG;            // dwords per row in the block: 64 / 32
    constexpr int RS = RD + 1;                // LDS row stride: odd, the 32 rows of a read hit 32 banks
    const int g0 = gy * kGPB, t = threadIdx.x;
    {
        constexpr int PPR = RD / 4;           // 16-byte pieces per row: 16 / 8
        const int gmax = min(kGPB, G - g0) * (DPG / 4);   // pieces of a row that exist
#pragma unroll
        for (int k = 0; k < (32 * PPR) / 256; k++) {
            const int idx = t + 256 * k, rr = idx / PPR, pc = idx - rr * PPR;
            const int srow = min(rb * 32 + rr, rows - 1);
            uint4 v = make_uint4(0u, 0u, 0u, 0u);
            if (pc < gmax) v = *reinterpret_cast<const uint4*>(P + ((size_t)srow * G + g0) * DPG + pc * 4);
            uint32_t* d = stage + rr * RS + pc * 4;
            d[0] = v.x;
            d[1] = v.y;
            d[2] = v.z;
            d[3] = v.w;
        }
    }
    __syncthreads();
    const int r = t & 31, dq = t >> 5;
    const bool live = rb * 32 + r < rows;
    uint32_t sv[kGPB], zv[kGPB];
#pragma unroll
    for (int i = 0; i < kGPB; i++) {
        sv[i] = stage[r * RS + i * DPG + dq];
        zv[i] = TERN ? stage[r * RS + i * DPG + 8 + dq] : 0u;
    }
#pragma unroll
    for (int i = 0; i < kGPB; i++) {
        const int g = g0 + i;
        if (g >= G) break;
        const uint32_t nz = live ? ~zv[i] : 0u;
        const uint32_t s = sv[i] & nz;   // a lane flagged zero is zero whatever its sign bit says
        if (F4) {
            // fragment = one 64-lane word: dword dq&1 is its k half; nibble = sign<<3 | nonzero<<1
            uint4* frag = out + ((size_t)rb * (G * 4) + (g * 4 + (dq >> 1))) * 64;
            uint32_t o[4];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                uint32_t a = (s >> (8 * q)) & 0xffu, b = (nz >> (8 * q)) & 0xffu;
                a = (a | (a << 12)) & 0x000F000Fu;
                a = (a | (a << 6)) & 0x03030303u;
                a = (a | (a << 3)) & 0x11111111u;
                b = (b | (b << 12)) & 0x000F000Fu;
                b = (b | (b << 6)) & 0x03030303u;
                b = (b | (b << 3)) & 0x11111111u;
                o[q] = (a << 3) | (b << 1);
            }
            frag[(dq & 1) * 32 + r] = make_uint4(o[0], o[1], o[2], o[3]);
        } else {
            // fragment = one 32-lane dword: its two 16-lane halves are the k halves
            uint4* frag = out + ((size_t)rb * (G * 8) + (g * 8 + dq)) * 64;
#pragma unroll
            for (int half = 0; half < 2; half++) {
                const uint32_t sh = (s >> (16 * half)) & 0xffffu, nh = (nz >> (16 * half)) & 0xffffu;
                uint32_t o[4];
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    // 4 bits -> 4 byte LSBs: bit i lands on bit 8i, no carries
                    const uint32_t sb = (((sh >> (4 * q)) & 15u) * 0x204081u) & 0x01010101u;
                    const uint32_t nb = (((nh >> (4 * q)) & 15u) * 0x204081u) & 0x01010101u;
                    o[q] = nb | (sb * 0xffu);
                }
                frag[half * 32 + r] = make_uint4(o[0], o[1], o[2], o[3]);
            }
        }
    }
}

template <bool F4, bool TERN>
__global__ __launch_bounds__(256) void k_expand(const uint32_t* __restrict__ P, int rows, int G, uint4* __restrict__ out) {
    __shared__ uint32_t stage[32 * 65];
    expand_block<F4, TERN>(P, rows, G, out, blockIdx.x, blockIdx.y, stage);
}

// both operands of a GEMM in one launch (the same K): the first ceil(rows_a / 32) workgroup columns expand A, the others B
template <bool F4, bool TA, bool TB>
__global__ __launch_bounds__(256) void k_expand2(const uint32_t* __restrict__ Pa, int rows_a, uint4* __restrict__ out_a,
                                                 const uint32_t* __restrict__ Pb, int rows_b, uint4* __restrict__ out_b, int G) {
    __shared__ uint32_t stage[32 * 65];
    const int rba = (rows_a + 31) / 32;
    if ((int)blockIdx.x < rba) expand_block<F4, TA>(Pa, rows_a, G, out_a, blockIdx.x, blockIdx.y, stage);
    else expand_block<F4, TB>(Pb, rows_b, G, out_b, (int)blockIdx.x - rba, blockIdx.y, stage);
}

// ----------------------------------------------------------------------- GEMM
template <bool F4>
struct Acc {
    typedef v16i type;
};
template <>
struct Acc<true> {
    typedef v16f type;
};

template <bool F4>
__device__ __forceinline__ void mfma(typename Acc<F4>::type& c, const uint4& a, const uint4& b) {
    if constexpr (F4) {
        const v8i va = {(int)a.x, (int)a.y, (int)a.z, (int)a.w, 0, 0, 0, 0};
        const v8i vb = {(int)b.x, (int)b.y, (int)b.z, (int)b.w, 0, 0, 0, 0};
        // cbsz = blgp = 4: both operands E2M1; scale operands 0 select the unscaled instruction
        c = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(va, vb, c, 4, 4, 0, 0, 0, 0);
    } else {
        const v4i va = {(int)a.x, (int)a.y, (int)a.z, (int)a.w};
        const v4i vb = {(int)b.x, (int)b.y, (int)b.z, (int)b.w};
        c = __builtin_amdgcn_mfma_i32_32x32x32_i8(va, vb, c, 0, 0, 0);
    }
}

// LDS-direct load of 16 bytes per lane: the 64 lanes land contiguously at lds_byte_addr.
// Issued through inline asm so that the compiler does not order its own LDS reads against
// it; the kernel waits for it by hand (s_waitcnt vmcnt before the barrier that publishes
// the buffer).  M0 carries the LDS address; one wait state is required after writing M0.
__device__ __forceinline__ void dma16(const uint4* gsrc, uint32_t lds_byte_addr) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gsrc), "s"(lds_byte_addr)
                 : "memory");
}

// Epilogue of the GEMM kernels: r = acc - bias, then PReLU in the reference's form for the type (form 0 "f = r; if
// (f <= 0) f *= alpha", mm_p2_final_tnn_avx2.c:204-208; form 1 "r >= 0 ? r : alpha * r", mm_p2_final_tbn_avx2.c:73), stored
// row-major (SWAP = false, OHW == 1) or in NCHW order.  Accumulator e of block (a, b): P row = 32 * (prb + a) + 8 * (e / 4)
// + 4 * (lane / 32) + e % 4, Q row = 32 * (qrb + b) + lane % 32.
template <bool F4, bool SWAP, int WTP, int WTQ>
__device__ __forceinline__ void store_tile(const typename Acc<F4>::type (&acc)[WTP][WTQ], float* __restrict__ Y, int M, int KN,
                                           int OHW, int prb, int qrb, int lane, int bias, int form, float alpha) {
    const bool le_form = form == 0;
#pragma unroll
    for (int a = 0; a < WTP; a++)
#pragma unroll
        for (int b = 0; b < WTQ; b++) {
            const int q = (qrb + b) * 32 + (lane & 31);
            const int pbase = (prb + a) * 32 + 4 * (lane >> 5);
            size_t qoff;
            if (SWAP) {   // q = i is fixed per block: split it into (image, pixel) once
                const int img = q / OHW;
                qoff = (size_t)img * KN * OHW + (q - img * OHW);
            } else {
                qoff = (size_t)q;
            }
            const bool qok = q < (SWAP ? M : KN);
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int p = pbase + 8 * (e >> 2) + (e & 3);
                const int r = (int)acc[a][b][e] - bias;
                const float fr = (float)r;
                // form 0: scale when f <= 0 (a zero becomes 0 * alpha); form 1: scale when r < 0
                const bool scale = le_form ? (fr <= 0.0f) : (r < 0);
                const float f = scale ? fr * alpha : fr;
                const size_t o = SWAP ? qoff + (size_t)p * OHW : (size_t)p * KN + qoff;
                if (qok && p < (SWAP ? KN : M)) __builtin_nontemporal_store(f, &Y[o]);
            }
        }
}

// P operand = MFMA A side (its rows index the accumulator registers), Q operand = MFMA B
// side (its rows run along the lanes).  SWAP = false: P = activation rows i, Q = weight
// rows j (lanes along j: contiguous for a row-major m x n result).  SWAP = true: P =
// weights, Q = activations (lanes along i: contiguous for an NCHW result with OHW > 1).
// The epilogue computes r = acc - bias, then PReLU in the reference's form for the type:
// form 0 "f = r; if (f <= 0) f *= alpha" (mm_p2_final_tnn_avx2.c:204-208), form 1
// "r >= 0 ? r : alpha * r" (mm_p2_final_tbn_avx2.c:73).
// IMPL (fp4, SWAP): a conv layer with implicit im2row.  Qf is then not a fragment array but the layer's quantised input
// in the form T4[n][C_pack][half][row][column % s][column / s][16 bytes] (k_quantize_f4 with TILED): the two wavefronts
// that stage the Q side compute, per fragment, each lane's own source address -- lane (pixel, K half) of the fragment of
// K word w = (kh KW + kw) C_pack + ic reads its 16 bytes at input pixel (oh s + kh - p, ow s + kw - p) of plane ic, or a
// the fill piece behind the planes (16 bytes of zeros, or of +1 nibbles for binary activations: the reference's
// fill, src/tnns/ternarize2row_avx2.c:748-755, src/tnns/binarize2row_avx2.c:151) where that pixel lies outside the image or w is a padding word -- and the LDS-direct load drops the 64
// lanes contiguously into the ring exactly as it drops a stored fragment.  In T4 the 32 pixels of a fragment half are
// consecutive 16-byte pieces within an output row whatever the stride (records of 32 bytes gathered at the stride
// took the load unit four times as many requests: 50 against 32 us on a 1024-channel 28 x 28 stride-2 layer).  The im2row rows and their expansion are never written (for a 1024-channel 56 x 56 layer:
// 116 + 231 MB less traffic and two launches less), and everything behind the ring is the GEMM kernel unchanged.
template <bool F4, bool SWAP, int WTP, int WTQ, int kKF, int kNS, bool IMPL = false, bool BAL = false>
__global__ __launch_bounds__(256) void k_mfma(const uint4* __restrict__ Pf, const uint4* __restrict__ Qf,
                                              float* __restrict__ Y, int M, int KN, int OHW, int KB,
                                              int bias, int form, float alpha, ConvGeom cg = ConvGeom(),
                                              FastDiv dOHW = FastDiv(), int Ws = 0, FastDiv dSW = FastDiv()) {
    static_assert(!IMPL || (F4 && SWAP), "implicit im2row: fp4 layer with the pixels along the lanes");
    static_assert(!BAL || IMPL, "the balanced assignment of fragments is for the gathering kernel");
    extern __shared__ uint4 lds[];   // kNS buffers of kFR KiB
    typedef typename Acc<F4>::type acc_t;
    typedef Tile<WTP, WTQ, kKF, kNS> TL;
    constexpr int RBP = TL::RBP, RBQ = TL::RBQ, kFR = TL::FR, kFW = TL::FW, NL = TL::NL, NM = TL::NM, DPI = TL::DPI;
    constexpr int kPF = RBP * kKF;   // fragments of the P side per step
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wy = wave >> 1, wx = wave & 1;
    const int prow = SWAP ? KN : M, qrow = SWAP ? M : KN;
    // Tile of this workgroup.  Under IMPL the kernel tiles of one pixel tile read the same part of T4; workgroups are dealt
    // to the eight XCDs round-robin by their linear number, so the tiles are renumbered to keep those on one XCD (its L2
    // then fetches that part once, not once per kernel tile): XCD x takes the pixel tiles x, x + 8, ...; the pixel
    // tiles beyond the last multiple of eight keep the plain order.
    uint32_t bx = blockIdx.x, by = blockIdx.y;
    if constexpr (IMPL) {
        const uint32_t kt = gridDim.x, pt8 = gridDim.y / 8 * 8, lin = bx + kt * by;
        if (lin < kt * pt8) {
            const uint32_t xcd = lin & 7u, slot = lin >> 3;
            by = xcd + 8u * (slot / kt);
            bx = slot % kt;
        }
    }
    const int prb0 = bx * RBP, qrb0 = by * RBQ;
    const int prbmax = (prow + 31) / 32 - 1, qrbmax = (qrow + 31) / 32 - 1;
    acc_t acc[WTP][WTQ];
#pragma unroll
    for (int a = 0; a < WTP; a++)
#pragma unroll
        for (int b = 0; b < WTQ; b++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[a][b][e] = 0;

    // fragment f of a step: the P side's kPF fragments first (row-block f / kKF, k fragment f % kKF), then the Q
    // side's; row-blocks past the operand are clamped (their results are never stored)
    // Which fragments a wavefront stages: in order (wavefront w the fragments w kFW .. w kFW + kFW - 1), or, BAL, a
    // quarter of each side (PW fragments of the P side, then QW of the Q side), so that under IMPL every wavefront
    // gathers the same number of fragments and none of them holds the others up at the step's barrier.
    constexpr int PW = BAL ? kPF / 4 : 0, QW = BAL ? kFW - PW : 0;
    static_assert(!BAL || (kPF % 4 == 0 && (QW % kKF == 0 || (QW == 1 && kKF == 2))), "a quarter of each side per wavefront");
    auto frag_of = [&](int i) -> int {   // fragment number (its place in a stage of the ring) of the wavefront's slot i
        if constexpr (BAL) return i < PW ? wave * PW + i : kPF + wave * QW + (i - PW);
        else return wave * kFW + i;
    };
    const uint4* src[kFW];
#pragma unroll
    for (int i = 0; i < kFW; i++) {
        const int f = frag_of(i);
        const bool qside = f >= kPF;
        const int g = qside ? f - kPF : f, rbi = g / kKF, kbi = g % kKF;
        const uint4* base = !qside ? Pf + ((size_t)min(prb0 + rbi, prbmax) * KB + kbi) * 64
                                   : Qf + ((size_t)min(qrb0 + rbi, qrbmax) * KB + kbi) * 64;
        src[i] = base + lane;
    }
    // IMPL: the Q side's fragments are gathered.  They are the last RBQ * kKF fragments of a step, staged by wavefront
    // 3 and, where the tile is not square, by the tail of wavefront 2; a wavefront's Q fragments cover whole row blocks
    // of 32 pixels, at most QMAX of them, from row block qfirst on.  A wavefront issues one instruction every few
    // cycles, so what the gather adds per fragment must stay a handful of instructions:
    //   * a table behind the ring, one entry per K word w = (kh KW + kw) C_pack + ic, holds what does not depend on
    //     the lane: the bit of the word's tap (0 for a padding word), and the word's part of the piece index (plane,
    //     tap row, column class and slot offset);
    //   * per row block a lane keeps the mask of the taps that fall inside the image for its pixel, and its pixel's
    //     part of the piece index;
    // a fragment's source is then one AND, one add, one select and the address.
    static_assert(!IMPL || kKF == 2, "two table entries per read");
    static_assert(!IMPL || BAL || (kPF % kKF == 0 && kFW % kKF == 0 && kPF >= 2 * kFW), "Q fragments in whole row blocks, on wavefronts 2 and 3 only");
    constexpr int QMAX = BAL ? (QW + kKF - 1) / kKF : kFW / kKF;
    const bool gathers = IMPL && (BAL || (wave + 1) * kFW > kPF);   // wave-uniform: this wavefront stages Q fragments
    const int qfirst = BAL ? (wave * QW) / kKF : max(0, wave * kFW - kPF) / kKF;
    uint32_t tapmask[IMPL ? QMAX : 1], pbase[IMPL ? QMAX : 1];
    const uint32_t row16 = (uint32_t)(cg.W_stride * Ws);          // pieces per input row
    const uint32_t half16 = (uint32_t)cg.H * row16;               // per half plane
    const uint32_t fill_piece = (uint32_t)(cg.CP * 2) * half16 * (uint32_t)((M - 1) / OHW + 1);   // right behind the planes
    uint2* const wtab = reinterpret_cast<uint2*>(lds + (size_t)kNS * kFR * 64);
    if constexpr (IMPL) {
        for (int w = tid; w < KB; w += 256) {
            const int tap = (int)fastdiv((uint32_t)w, cg.dCP), ic = w - tap * cg.CP;
            const int kh = (int)fastdiv((uint32_t)tap, cg.dKW), kw = tap - kh * cg.KW;
            // column ow s + d with d = kw - pad: class d mod s, slot ow + floor(d / s) (d made non-negative by a
            // multiple of s first: the host keeps the padding below 4096 s)
            const uint32_t dd = (uint32_t)(kw - cg.W_pad + 4096 * cg.W_stride);
            const uint32_t dq = fastdiv(dd, dSW), cls = dd - dq * (uint32_t)cg.W_stride;
            wtab[w] = make_uint2(w < cg.K ? 1u << tap : 0u,
                                 (uint32_t)ic * 2u * half16 + (uint32_t)kh * row16 + cls * (uint32_t)Ws + dq - 4096u);
        }
#pragma unroll
        for (int j = 0; j < QMAX; j++) {
            const int rb = min(qfirst + j, RBQ - 1);
            const uint32_t q = (uint32_t)min((qrb0 + rb) * 32 + (lane & 31), M - 1);
            const uint32_t img = fastdiv(q, dOHW);
            const uint32_t pix = q - img * (uint32_t)OHW;
            const int oh = (int)fastdiv(pix, cg.dOW), ow = (int)pix - oh * cg.OW;
            const int ih0 = oh * cg.H_stride - cg.H_pad, iw0 = ow * cg.W_stride - cg.W_pad;
            // (image, plane 0, this lane's half, row ih0, class 0, slot ow): wraps for a negative ih0, and the
            // word's part brings it back whenever the tap is inside
            pbase[j] = (img * (uint32_t)cg.CP * 2u + (uint32_t)(lane >> 5)) * half16 + (uint32_t)ih0 * row16 + (uint32_t)ow;
            uint32_t m = 0u;
            for (int kh = 0, tap = 0; kh < cg.K / (cg.CP * cg.KW); kh++)
                for (int kw = 0; kw < cg.KW; kw++, tap++)
                    m |= ((unsigned)(ih0 + kh) < (unsigned)cg.H && (unsigned)(iw0 + kw) < (unsigned)cg.W ? 1u : 0u) << tap;
            tapmask[j] = m;
        }
        __syncthreads();   // the table is complete before the first stage is issued
    }
    // the table entries of the kKF words of the stage about to be issued (stages are issued strictly in order), read
    // from LDS one stage ahead of their use (the table has two entries to spare behind its last word)
    int g_w = kKF;
    uint4 wt = make_uint4(0u, 0u, 0u, 0u), wt_ahead = make_uint4(0u, 0u, 0u, 0u);
    if constexpr (IMPL) {
        if (gathers) wt_ahead = *reinterpret_cast<const uint4*>(wtab);
    }
    auto next_words = [&]() {
        wt = wt_ahead;
        wt_ahead = *reinterpret_cast<const uint4*>(wtab + min(g_w, KB));
        g_w += kKF;
    };
    // the gathered source of fragment i of wavefront W (both compile-time): its row block's slot in tapmask / pbase is
    // then a constant
    auto gathered = [&](auto wtag, int i) -> const uint4* {
        constexpr int W = decltype(wtag)::value;
        int j;
        bool even;   // the fragment's K word within the stage
        if constexpr (BAL) {
            // slot i holds Q fragment w QW + (i - PW): with whole row blocks per wavefront both are compile-time; with one
            // fragment per wavefront (QW == 1) the K word is the wavefront's parity
            j = QW % kKF == 0 ? (i - PW) / kKF : 0;
            even = QW % kKF == 0 ? ((i - PW) % kKF) == 0 : (wave & 1) == 0;
        } else {
            constexpr int first = (W * kFW > kPF ? W * kFW - kPF : 0) / kKF;
            j = (W * kFW + i - kPF) / kKF - first;
            even = (i % kKF) == 0;
        }
        const uint32_t bit = even ? wt.x : wt.z, off = even ? wt.y : wt.w;
        const uint32_t piece = pbase[j] + off;
        return Qf + ((tapmask[j] & bit) != 0u ? piece : fill_piece);   // a select on the index: no branch
    };
    const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)lds);
    const int nstep = KB / kKF;
    uint4 fa[2][WTP], fb[2][WTQ];
    // one LDS read of fragment k of buffer `buf` into register set `set`, in the order the MFMAs
    // consume them: i = 0: fa0, 1..WTQ: fb0..fb(WTQ-1), then fa1..fa(WTP-1)
    auto ldone = [&](int buf, int k, int set, int i) {
        const uint4* L = lds + (size_t)buf * kFR * 64;
        if (i == 0) fa[set][0] = L[((wy * WTP + 0) * kKF + k) * 64 + lane];
        else if (i <= WTQ) fb[set][i - 1] = L[((RBP + wx * WTQ + (i - 1)) * kKF + k) * 64 + lane];
        else fa[set][i - WTQ] = L[((wy * WTP + (i - WTQ)) * kKF + k) * 64 + lane];
    };
    // the multiplies that go with LDS read i: the NM of a k fragment spread evenly over its NL reads (WT / 2 each on a
    // square tile), in the order (a, b) = (m / WTQ, m % WTQ)
    auto mfma2 = [&](int set, int i) {
#pragma unroll
        for (int m = i * NM / NL; m < (i + 1) * NM / NL; m++) mfma<F4>(acc[m / WTQ][m % WTQ], fa[set][m / WTQ], fb[set][m % WTQ]);
    };

    // The pipeline, instantiated per role of the wavefront so that no fragment's source is chosen at run time: role 0
    // stages stored fragments only (every wavefront without IMPL; wavefronts 0 and 1 with it), roles 2 and 3 are
    // wavefronts 2 and 3 under IMPL, whose Q fragments are gathered.  Every role passes the same barriers.
    auto pipeline = [&](auto role_tag) {
        constexpr int ROLE = decltype(role_tag)::value;
        // source of the wavefront's fragment i for K step `step` (gathered: of the stage next_words() was last called for)
        auto source = [&](int i, int step) -> const uint4* {
            if constexpr (BAL) {
                if (i >= PW) return gathered(role_tag, i);
            } else if constexpr (ROLE != 0) {
                if (ROLE * kFW + i >= kPF) return gathered(role_tag, i);
            }
            return src[i] + (size_t)step * kKF * 64;
        };
        auto stage = [&](int step) {
            const uint32_t dst = lds0 + (uint32_t)(step % kNS) * (kFR * 1024);
            if constexpr (ROLE != 0) next_words();
#pragma unroll
            for (int i = 0; i < kFW; i++) dma16(source(i, step), dst + (uint32_t)frag_of(i) * 1024);
        };
        // prologue: the first kNS stages in flight, wait for stage 0 only
#pragma unroll
        for (int p = 0; p < kNS; p++)
            if (p < nstep) stage(p);
        if (nstep >= kNS) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kFW * (kNS - 1)) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
#pragma unroll
        for (int i = 0; i < NL; i++) ldone(0, 0, 0, i);

        auto step_body = [&](int s, auto full_tag) {
            constexpr bool FULL = decltype(full_tag)::value;   // FULL: s + kNS < nstep
#pragma unroll
            for (int k = 0; k < kKF; k++) {
                const int set = k & 1;
                if (k + 1 < kKF) {
#pragma unroll
                    for (int i = 0; i < NL; i++) {
                        ldone(s % kNS, k + 1, set ^ 1, i);
                        mfma2(set, i);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                } else {
                    // Last fragment of the step: all of this step is in registers.  Stage s+1 must
                    // have landed (stages s+2 .. s+kNS-1 may still be in flight); after the barrier
                    // buffer s % kNS is free for stage s+kNS.
                    if (FULL || s + kNS - 1 < nstep) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kFW * (kNS - 2)) : "memory");
                    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    __syncthreads();
                    const bool do_ld = FULL || s + 1 < nstep;
                    const uint32_t dst = lds0 + (uint32_t)(s % kNS) * (kFR * 1024);
                    if constexpr (FULL && ROLE != 0) next_words();
#pragma unroll
                    for (int i = 0; i < NL; i++) {
                        if (FULL) {
#pragma unroll
                            for (int j = 0; j < DPI; j++) dma16(source(i * DPI + j, s + kNS), dst + (uint32_t)frag_of(i * DPI + j) * 1024);
                        }
                        if (do_ld) ldone((s + 1) % kNS, 0, set ^ 1, i);
                        mfma2(set, i);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        };
        int s = 0;
        for (; s + kNS < nstep; s++) step_body(s, std::true_type{});
        for (; s < nstep; s++) step_body(s, std::false_type{});
    };
    if constexpr (BAL) {
        pipeline(std::integral_constant<int, 1>{});   // every wavefront stages and gathers alike
    } else if constexpr (IMPL) {
        if (wave == 3) pipeline(std::integral_constant<int, 3>{});
        else if (wave == 2) pipeline(std::integral_constant<int, 2>{});
        else pipeline(std::integral_constant<int, 0>{});
    } else {
        pipeline(std::integral_constant<int, 0>{});
    }

    store_tile<F4, SWAP, WTP, WTQ>(acc, Y, M, KN, OHW, prb0 + wy * WTP, qrb0 + wx * WTQ, lane, bias, form, alpha);
}

// ------------------------------------------------- fp4 operands at two bits per lane, offset codes
// The fp4 GEMM above is bound by power, not by its schedule.  The same instruction stream runs a quarter faster on
// operands that are all zero, and a chain of nothing but these MFMAs on registers holds 2.39 GHz on zeros, 2.25 GHz on
// lanes of {0, 0.5, 1} and 1.97 GHz on lanes of {-1, 0, +1}: it is the mixed signs in the adder trees and the operand
// bytes on the move (L2 -> LDS -> registers) that hold the clock down.  The GEMM's own operand form answers both:
//
//   offset codes   a lane a in {-1, 0, +1} travels as a' = (a + 1) / 2 in {0, 0.5, 1}, E2M1 codes 0, 1, 2: no negative
//                  product anywhere.  With S = sum a' b' over all L = 64 Kw lanes of a row pair (padding lanes are
//                  a = b = 0 or +-1 like any other and enter the sums below the same way)
//                      sum a b = 4 S - sum a - sum b - L,
//                  exact in fp32 while 4 L <= 2^24 (S is a multiple of 1/4 below L).  The row sums are counted when
//                  the operand is packed and sit behind its blocks; the epilogue undoes the offset.
//   two bits       codes 0, 1, 2 use bits 0 and 1 of a nibble, so two dwords of nibbles D0, D1 share one dword,
//                  P = D0 | D1 << 2, and come apart with D0 = P & 0x33333333, D1 = (P >> 2) & 0x33333333: 1.5 vector
//                  instructions per dword, issued beside the MFMAs.  Half the bytes in HBM, through L2 -> LDS and
//                  through the LDS reads.
//
// Layout ("packed4"): 1 KiB blocks [row block of 32][pair of K words][lane l = (k half l / 32, row l % 32)][16 bytes], the
// 16 bytes of a lane being (P0, P1) of the even K word and (P0, P1) of the odd one, P0 = D0 | D1 << 2, P1 = D2 | D3 << 2
// with D0..D3 the lane's 16 bytes of the plain fragment layout above in offset codes.  One LDS-direct load of 16 bytes
// per lane moves a row block's two K words.  Behind the blocks: one int32 per row (rows rounded up to 32), sum of the
// row's lanes.

// zeroes p[0 .. n) and q[0 .. m) (m may be 0)
__global__ void k_zero_i32(int* __restrict__ p, int n, int* __restrict__ q, int m) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
    else if (i - n < m) q[i - n] = 0;
}

// grid (row blocks, groups / 4), block 256: as k_expand<true, TERN>, writing the packed4 layout (Kw words per row) and
// adding the lanes of its rows into sums (zeroed before the launch)
template <bool TERN>
__device__ __forceinline__ void pack4_block(const uint32_t* __restrict__ P, int rows, int G, uint2* __restrict__ out,
                                            int* __restrict__ sums, int rb, int gy, uint32_t* stage, int* rowsum) {
    constexpr int kGPB = 4;
    constexpr int DPG = TERN ? 16 : 8;        // dwords per group and row
    constexpr int RD = kGPB * DPG;            // dwords per row in the block
    constexpr int RS = RD + 1;                // LDS row stride: odd, the 32 rows of a read hit 32 banks
    const int g0 = gy * kGPB, t = threadIdx.x;
    if (t < 32) rowsum[t] = 0;
    {
        constexpr int PPR = RD / 4;           // 16-byte pieces per row
        const int gmax = min(kGPB, G - g0) * (DPG / 4);
#pragma unroll
        for (int k = 0; k < (32 * PPR) / 256; k++) {
            const int idx = t + 256 * k, rr = idx / PPR, pc = idx - rr * PPR;
            const int srow = min(rb * 32 + rr, rows - 1);
            uint4 v = make_uint4(0u, 0u, 0u, 0u);
            if (pc < gmax) v = *reinterpret_cast<const uint4*>(P + ((size_t)srow * G + g0) * DPG + pc * 4);
            uint32_t* d = stage + rr * RS + pc * 4;
            d[0] = v.x;
            d[1] = v.y;
            d[2] = v.z;
            d[3] = v.w;
        }
    }
    __syncthreads();
    const int r = t & 31, dq = t >> 5;        // dq: dword of the group = (K word dq / 2, k half dq % 2)
    int lanesum = 0;
#pragma unroll
    for (int i = 0; i < kGPB; i++) {
        const int g = g0 + i;
        if (g >= G) break;
        const uint32_t sv = stage[r * RS + i * DPG + dq];
        const uint32_t zero = TERN ? stage[r * RS + i * DPG + 8 + dq] : 0u;
        const uint32_t plus = ~(sv | zero), minus = sv & ~zero;
        lanesum += __popc(plus) - __popc(minus);
        uint32_t o[4];
#pragma unroll
        for (int q = 0; q < 4; q++) {   // 8 lanes -> 8 nibbles: bit i lands on bit 4 i
            uint32_t a = (plus >> (8 * q)) & 0xffu, b = (zero >> (8 * q)) & 0xffu;
            a = (a | (a << 12)) & 0x000F000Fu;
            a = (a | (a << 6)) & 0x03030303u;
            a = (a | (a << 3)) & 0x11111111u;
            b = (b | (b << 12)) & 0x000F000Fu;
            b = (b | (b << 6)) & 0x03030303u;
            b = (b | (b << 3)) & 0x11111111u;
            o[q] = (a << 1) | b;        // +1 -> 2 (1.0), 0 -> 1 (0.5), -1 -> 0
        }
        const int w = g * 4 + (dq >> 1), h = dq & 1;   // K word and k half of this thread's 32 lanes
        const size_t block = (size_t)rb * (G * 2) + (w >> 1);
        out[(block * 64 + h * 32 + r) * 2 + (w & 1)] = make_uint2(o[0] | (o[1] << 2), o[2] | (o[3] << 2));
    }
    atomicAdd(&rowsum[r], lanesum);
    __syncthreads();
    if (t < 32 && rb * 32 + t < rows) atomicAdd(&sums[rb * 32 + t], rowsum[t]);
}

template <bool TERN>
__global__ __launch_bounds__(256) void k_pack4(const uint32_t* __restrict__ P, int rows, int G, uint2* __restrict__ out,
                                               int* __restrict__ sums) {
    __shared__ uint32_t stage[32 * 65];
    __shared__ int rowsum[32];
    pack4_block<TERN>(P, rows, G, out, sums, blockIdx.x, blockIdx.y, stage, rowsum);
}

// both operands of a GEMM in one launch, as k_expand2
template <bool TA, bool TB>
__global__ __launch_bounds__(256) void k_pack4_2(const uint32_t* __restrict__ Pa, int rows_a, uint2* __restrict__ out_a,
                                                 int* __restrict__ sums_a, const uint32_t* __restrict__ Pb, int rows_b,
                                                 uint2* __restrict__ out_b, int* __restrict__ sums_b, int G) {
    __shared__ uint32_t stage[32 * 65];
    __shared__ int rowsum[32];
    const int rba = (rows_a + 31) / 32;
    if ((int)blockIdx.x < rba) pack4_block<TA>(Pa, rows_a, G, out_a, sums_a, blockIdx.x, blockIdx.y, stage, rowsum);
    else pack4_block<TB>(Pb, rows_b, G, out_b, sums_b, (int)blockIdx.x - rba, blockIdx.y, stage, rowsum);
}

// (P0, P1) of one K word -> the lane's 16 bytes of nibbles
__device__ __forceinline__ uint4 unpack4(uint32_t p0, uint32_t p1) {
    constexpr uint32_t m = 0x33333333u;
    return make_uint4(p0 & m, (p0 >> 2) & m, p1 & m, (p1 >> 2) & m);
}

// The epilogue of the offset form: dot = 4 acc - sum of the P row - sum of the Q row - lanes, then as store_tile
// (off = lanes + the BNN bias).  sums: the tile's row sums in LDS, RB * 32 of the P side, then RB * 32 of the Q side
// (zero for rows past the operand, which store nothing).
template <bool SWAP, int WT>
__device__ __forceinline__ void store_tile_offset(const Acc<true>::type (&acc)[WT][WT], float* __restrict__ Y, int M, int KN, int OHW,
                                                  int prb, int qrb, int lane, const int* sums, int wy, int wx, int off, int form,
                                                  float alpha) {
    constexpr int RB = 2 * WT;
    const bool le_form = form == 0;
    const int prow = SWAP ? KN : M, qrow = SWAP ? M : KN;
#pragma unroll
    for (int a = 0; a < WT; a++) {
        int4 sp[4];   // the lane's 16 P rows of this block: rows 4 * (lane / 32) + 8 * j + (0..3)
#pragma unroll
        for (int j = 0; j < 4; j++) sp[j] = *reinterpret_cast<const int4*>(sums + (wy * WT + a) * 32 + 4 * (lane >> 5) + 8 * j);
        const int pbase = (prb + a) * 32 + 4 * (lane >> 5);
#pragma unroll
        for (int b = 0; b < WT; b++) {
            const int q = (qrb + b) * 32 + (lane & 31);
            const bool qok = q < qrow;
            const int sq = sums[RB * 32 + (wx * WT + b) * 32 + (lane & 31)] + off;
            size_t qoff;
            if (SWAP) {   // q = i is fixed per block: split it into (image, pixel) once
                const int img = q / OHW;
                qoff = (size_t)img * KN * OHW + (q - img * OHW);
            } else {
                qoff = (size_t)q;
            }
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int p = pbase + 8 * (e >> 2) + (e & 3);
                const int4& s4 = sp[e >> 2];
                const int spv = (e & 3) == 0 ? s4.x : (e & 3) == 1 ? s4.y : (e & 3) == 2 ? s4.z : s4.w;
                const int r = (int)(acc[a][b][e] * 4.0f) - spv - sq;
                const float fr = (float)r;
                const bool scale = le_form ? (fr <= 0.0f) : (r < 0);
                const float f = scale ? fr * alpha : fr;
                const size_t o = SWAP ? qoff + (size_t)p * OHW : (size_t)p * KN + qoff;
                if (qok && p < prow) __builtin_nontemporal_store(f, &Y[o]);
            }
        }
    }
}

// The fp4 GEMM on packed4 operands.  Same tiling as k_mfma<true, ...> (2 x 2 wavefronts, WT x WT blocks of 32 x 32 each,
// steps of two K words, ring of kNS stages filled by LDS-direct loads that the kernel counts by hand), with one 1 KiB block
// per row block and step.  A step: the first K word's 16 multiplies run while the second one's operands are unpacked;
// then the barrier; the second K word's multiplies run beside the loads of stage s + kNS and the LDS reads of stage
// s + 1, one read per slot of two multiplies (a 16-byte LDS read holds the wavefront's issue for 16 cycles), each block
// unpacked LAG slots after its read -- the last LAG blocks in the first slots of the next step.
template <bool SWAP, int WT, int kNS>
__global__ __launch_bounds__(256) void k_mfma_p4(const uint4* __restrict__ Pc, const uint4* __restrict__ Qc, float* __restrict__ Y,
                                                 int M, int KN, int OHW, int KP, const int* __restrict__ sP,
                                                 const int* __restrict__ sQ, int off, int form, float alpha) {
    extern __shared__ uint4 lds[];   // kNS stages of kFR KiB
    typedef typename Acc<true>::type acc_t;
    constexpr int RB = 2 * WT, kFR = 2 * RB, kFW = kFR / 4, NL = 2 * WT;   // kFW = WT blocks staged per wavefront and step
    static_assert(NL % kFW == 0 && (NL / 2) % 2 == 0, "loads and reads spread evenly over the slots");
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wy = wave >> 1, wx = wave & 1;
    const int prow = SWAP ? KN : M, qrow = SWAP ? M : KN;
    const int prb0 = blockIdx.x * RB, qrb0 = blockIdx.y * RB;
    const int prbmax = (prow + 31) / 32 - 1, qrbmax = (qrow + 31) / 32 - 1;
    acc_t acc[WT][WT];
#pragma unroll
    for (int a = 0; a < WT; a++)
#pragma unroll
        for (int b = 0; b < WT; b++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[a][b][e] = 0;

    // block f of a stage: side f / RB (0 = P, 1 = Q), row block f % RB; row blocks past the operand are clamped
    const uint4* src[kFW];
#pragma unroll
    for (int i = 0; i < kFW; i++) {
        const int f = wave * kFW + i;
        const int side = f / RB, rbi = f % RB;
        const uint4* base = side == 0 ? Pc + (size_t)min(prb0 + rbi, prbmax) * KP * 64 : Qc + (size_t)min(qrb0 + rbi, qrbmax) * KP * 64;
        src[i] = base + lane;
    }
    const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)lds);
    const int nstep = KP;
    auto stage = [&](int step) {
        const uint32_t dst = lds0 + (uint32_t)(step % kNS) * (kFR * 1024) + wave * (kFW * 1024);
#pragma unroll
        for (int i = 0; i < kFW; i++) dma16(src[i] + (size_t)step * 64, dst + i * 1024);
    };
    // raw: the packed blocks of the stage being consumed; e[k]: the unpacked operands of its K word k.  Slots in the
    // order the multiplies take them: 0: P block 0, 1..WT: Q blocks, then P blocks 1..WT-1.
    uint4 ra[WT], rq[WT], ea[2][WT], eq[2][WT];
    auto read_raw = [&](int buf, int i) {
        const uint4* L = lds + (size_t)buf * kFR * 64;
        if (i == 0) ra[0] = L[(wy * WT + 0) * 64 + lane];
        else if (i <= WT) rq[i - 1] = L[(RB + wx * WT + (i - 1)) * 64 + lane];
        else ra[i - WT] = L[(wy * WT + (i - WT)) * 64 + lane];
    };
    auto unpack = [&](int k, int i) {
        const uint4& r = i == 0 ? ra[0] : (i <= WT ? rq[i - 1] : ra[i - WT]);
        const uint4 v = k == 0 ? unpack4(r.x, r.y) : unpack4(r.z, r.w);
        if (i == 0) ea[k][0] = v;
        else if (i <= WT) eq[k][i - 1] = v;
        else ea[k][i - WT] = v;
    };
    auto mfma2 = [&](int k, int i) {
#pragma unroll
        for (int j = 0; j < WT / 2; j++) {
            const int m = (WT / 2) * i + j;
            mfma<true>(acc[m / WT][m % WT], ea[k][m / WT], eq[k][m % WT]);
        }
    };

    // prologue: the first kNS stages in flight, wait for stage 0 only
#pragma unroll
    for (int p = 0; p < kNS; p++)
        if (p < nstep) stage(p);
    if (nstep >= kNS) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kFW * (kNS - 1)) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NL; i++) read_raw(0, i);
#pragma unroll
    for (int i = 0; i < NL; i++) unpack(0, i);

    // slots between the LDS read of a block and its unpacking: far enough for the read to have landed, near enough for
    // every block to be unpacked by the slot that multiplies it first (block b: slot 0 for P block 0, (b - 1) / (WT / 2)
    // for Q block b - 1, 2 (b - WT) for P block b - WT)
    constexpr int LAG = WT >= 4 ? 4 : 3;
    static_assert(LAG <= NL - 1 && LAG <= NL - WT + (WT - 1) / (WT / 2) && LAG <= WT + 1, "a block is unpacked before its first multiply");
    auto step_body = [&](int s, auto full_tag) {
        constexpr bool FULL = decltype(full_tag)::value;   // FULL: s + kNS < nstep
        // first K word: multiply, and unpack the second one's operands (their packed blocks arrived a phase ago); the
        // first LAG slots also unpack the last LAG blocks of this stage's first K word, read at the end of the step before
#pragma unroll
        for (int i = 0; i < NL; i++) {
            if (i < LAG && s > 0) unpack(0, NL - LAG + i);
            unpack(1, i);
            mfma2(0, i);
            __builtin_amdgcn_sched_barrier(0);
        }
        // Everything of this stage is in registers.  Stage s + 1 must have landed (stages s + 2 .. s + kNS - 1 may
        // still be in flight); after the barrier buffer s % kNS is free for stage s + kNS.
        if (FULL || s + kNS - 1 < nstep) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kFW * (kNS - 2)) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        const bool do_ld = FULL || s + 1 < nstep;
        const uint32_t dst = lds0 + (uint32_t)(s % kNS) * (kFR * 1024) + wave * (kFW * 1024);
        // second K word: every slot issues one LDS read of the next stage and unpacks the block read LAG slots before;
        // the first kFW slots also issue the loads of stage s + kNS
#pragma unroll
        for (int i = 0; i < NL; i++) {
            if (do_ld) read_raw((s + 1) % kNS, i);
            if (FULL && i < kFW) dma16(src[i] + (size_t)(s + kNS) * 64, dst + i * 1024);
            if (do_ld && i >= LAG) unpack(0, i - LAG);
            mfma2(1, i);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    int s = 0;
    for (; s + kNS < nstep; s++) step_body(s, std::true_type{});
    for (; s < nstep; s++) step_body(s, std::false_type{});

    // the tile's row sums through LDS (every load of the ring has landed and been read: the last steps wait for all)
    __syncthreads();
    int* sums = reinterpret_cast<int*>(lds);
    if (tid < RB * 32) {
        const int pr = prb0 * 32 + tid, qr = qrb0 * 32 + tid;
        sums[tid] = pr < prow ? sP[pr] : 0;
        sums[RB * 32 + tid] = qr < qrow ? sQ[qr] : 0;
    }
    __syncthreads();
    store_tile_offset<SWAP, WT>(acc, Y, M, KN, OHW, prb0 + wy * WT, qrb0 + wx * WT, lane, sums, wy, wx, off, form, alpha);
}

// ------------------------------------------------------------ conv layer (fp4)
// Layer-sized problems (a few GMAC, 10^3..10^5 output pixels) are latency-, not throughput-bound,
// and their im2row operand does not exist in memory.  This kernel therefore works on small tiles
// with many wavefronts in flight and gathers its activation fragments itself:
//   * a wavefront owns 64 kernels x 64 output pixels (2 x 2 MFMA blocks, 64 accumulator
//     registers).  A workgroup is 4 wavefronts: S of them split the K loop of one tile (word w of
//     the reference's K order (kh*KW + kw)*C_pack + ic goes to wavefront w % S of the tile), so
//     it covers 4/S pixel tiles.  S = 1 for layers with 600 tiles or more (no exchange at all), 2 or
//     4 where the tiles alone would leave most of the chip idle; the partial tiles then meet in
//     LDS and each wavefront finishes 4/S of the tile's four blocks;
//   * weights are the MFMA A side (rows = accumulator registers), pixels the B side (rows =
//     lanes), so a store instruction writes 32 consecutive pixels of one NCHW plane;
//   * an activation fragment is 32 pixels x 64 channels of one kernel tap: lane (pixel, half)
//     loads its 16 bytes straight from P4 (k_quantize_f4's output) at the tap's input pixel,
//     or takes the padding value: zeros for ternary inputs, +1 nibbles for binary ones (the
//     reference's fill, src/tnns/ternarize2row_avx2.c:748-755, src/tnns/binarize2row_avx2.c:151);
//   * the padding words that round K up to a multiple of 4 are skipped: their products are zero
//     except for BNN, whose epilogue constant counts the real words only.
struct ConvFrag {
    v4i w[2], x[2];
    bool in[2];   // x[b] holds a real input pixel (else the padding value replaces it)
};

// ABIN: binary activations (padding value +1).  FORM0: the TNN form of PReLU, "f <= 0 -> f *= alpha"
// (mm_p2_final_tnn_avx2.c:204-208), else "r >= 0 ? r : alpha * r" (mm_p2_final_tbn_avx2.c:73).
// QMODE: 0 = fp32 NCHW result, 1 / 2 = ternary / binary hand-over to the next layer (QuantOut).
// All three are compile-time so that the per-element epilogue carries no selects for them.
// The unsplit hand-over variants are the ones launched with several thousand wavefronts (stems,
// first stages): they are asked to fit three wavefronts per SIMD, which they do without scratch.
// BUF: fragments arrive through buffer loads.  Their offsets are 32-bit, the weight fragment of a word is addressed
// by a scalar offset alone, and for ternary activations an offset beyond the buffer returns zeros, which is what a
// tap outside the image must contribute: no select on the loaded data, a third of the K loop's vector instructions
// gone (binary activations pad with +1 and keep the select).  Needs both operands below 4 GiB (p4_bytes, wf_bytes: the sizes the descriptors announce).
template <bool ABIN, bool FORM0, int QMODE, int S, int NB, bool BUF>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu((S == 1 && QMODE != 0) ? 3 : 1, 8))) void k_conv_f4(const uint4* __restrict__ P4, const uint4* __restrict__ Wf,
                                                 float* __restrict__ Y, int M, int KN, int OHW, int KB,
                                                 int bias, float alpha, FastDiv dOHW, ConvGeom cg, QuantOut qo,
                                                 uint32_t p4_bytes, uint32_t wf_bytes) {
    // NB register sets of fragments: NB - 1 steps of loads in flight
    constexpr int WPB = 4;                // wavefronts per workgroup (single-wavefront workgroups for S = 1
                                          // measured slower: neighbours no longer share weight fragments in L1)
    constexpr int PUB = 4 - 4 / S;        // blocks a wavefront hands to the others of its tile
    __shared__ float4 red[S > 1 ? 4 * PUB * 4 * 64 : 1];   // [wavefront][slot][e / 4][lane]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ks = wave % S, pt = wave / S;   // K share and pixel tile of this wavefront
    const int h = lane >> 5, lr = lane & 31;
    const int px0 = (blockIdx.x * (WPB / S) + pt) * 64, kn0 = blockIdx.y * 64;

    int ih0[2], iw0[2];
    uint32_t pb[2];
#pragma unroll
    for (int b = 0; b < 2; b++) {
        const uint32_t q = (uint32_t)min(px0 + 32 * b + lr, M - 1);
        const uint32_t n = fastdiv(q, dOHW);
        const uint32_t pix = q - n * (uint32_t)OHW;
        const int oh = (int)fastdiv(pix, cg.dOW), ow = (int)pix - oh * cg.OW;
        ih0[b] = oh * cg.H_stride - cg.H_pad;
        iw0[b] = ow * cg.W_stride - cg.W_pad;
        pb[b] = n * (uint32_t)(cg.CP * cg.H * cg.W);   // image n of P4[n][C_pack][pixel]
    }
    // threshold of each pixel block's image for the hand-over, fetched now, in front of the K loop's loads
    float qthr[2] = {0.0f, 0.0f};
    if constexpr (QMODE != 0) {
#pragma unroll
        for (int b = 0; b < 2; b++)
            qthr[b] = qo.thr[fastdiv((uint32_t)min(px0 + 32 * b + lr, M - 1), dOHW)];
    }
    const int HWin = cg.H * cg.W;
    const int rbmax = (KN + 31) / 32 - 1;
    const uint4* wb[2];
#pragma unroll
    for (int a = 0; a < 2; a++) wb[a] = Wf + (size_t)min(kn0 / 32 + a, rbmax) * KB * 64 + lane;

    v16f acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[a][b][e] = 0.0f;

    const uint32_t fillv = ABIN ? 0x22222222u : 0u;
    // All four loads of a step are unconditional (a tap outside the image reads pixel 0 of its image and is replaced
    // by the padding value before use) and are issued two steps ahead of the step being multiplied.  They are ordinary
    // loads (plain, or buffer-load builtins), so the compiler owns the dependency between a load and the use of its
    // registers and places every s_waitcnt vmcnt itself; what keeps a load where the code issues it -- and not next to
    // its use, where the scheduler would sink it -- is the scheduling fence after each step's loads (fence_loads).
    auto ld16 = [](v4i& dst, const uint4* src) { dst = *reinterpret_cast<const v4i*>(src); };
    // buffer descriptors (base; stride 0; bytes; raw 32-bit data format) and this lane's fixed offsets
    __amdgpu_buffer_rsrc_t brs_x = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint4*>(P4), 0, (int)p4_bytes, 0x00020000);
    __amdgpu_buffer_rsrc_t brs_w = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint4*>(Wf), 0, (int)wf_bytes, 0x00020000);
    uint32_t wofs[2] = {0u, 0u}, xofs[2] = {0u, 0u};
    if constexpr (BUF) {
#pragma unroll
        for (int a = 0; a < 2; a++) wofs[a] = ((uint32_t)min(kn0 / 32 + a, rbmax) * (uint32_t)KB * 64u + (uint32_t)lane) * 16u;
#pragma unroll
        for (int b = 0; b < 2; b++)
            xofs[b] = ((pb[b] + (uint32_t)(ih0[b] * cg.W + iw0[b])) * 2u + (uint32_t)h) * 16u;
    }
    auto ldbuf = [&](v4i& dst, uint32_t voff, uint32_t soff, bool weights) {
        const v4u v = __builtin_amdgcn_raw_buffer_load_b128(weights ? brs_w : brs_x, (int)voff, (int)soff, 0);
        dst = v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
    };
    auto load = [&](int w, ConvFrag& f) {   // w is wave-uniform
        const int tap = (int)fastdiv((uint32_t)w, cg.dCP), ic = w - tap * cg.CP;
        const int kh = (int)fastdiv((uint32_t)tap, cg.dKW), kw = tap - kh * cg.KW;
        if constexpr (BUF) {
            const uint32_t wsoff = (uint32_t)__builtin_amdgcn_readfirstlane(w) * 1024u;
#pragma unroll
            for (int a = 0; a < 2; a++) ldbuf(f.w[a], wofs[a], wsoff, true);
            // byte offset of the record = this lane's part (xofs, fixed) + the word's part (scalar); the sum wraps
            // to the right value whenever the tap lies inside the image
            const uint32_t tapoff = (uint32_t)__builtin_amdgcn_readfirstlane((ic * HWin + kh * cg.W + kw) * 32);
#pragma unroll
            for (int b = 0; b < 2; b++) {
                const int ih = ih0[b] + kh, iw = iw0[b] + kw;
                const bool in = (unsigned)ih < (unsigned)cg.H && (unsigned)iw < (unsigned)cg.W;
                // ternary activations: an offset beyond p4_bytes returns the zeros that padding is; binary ones pad
                // with +1, read record 0 instead and take the select in compute()
                ldbuf(f.x[b], in ? xofs[b] + tapoff : (ABIN ? 0u : 0xffffff00u), 0u, false);
                f.in[b] = ABIN ? in : true;
            }
        } else {
#pragma unroll
            for (int a = 0; a < 2; a++) ld16(f.w[a], wb[a] + (size_t)w * 64);
#pragma unroll
            for (int b = 0; b < 2; b++) {
                const int ih = ih0[b] + kh, iw = iw0[b] + kw;
                const bool in = (unsigned)ih < (unsigned)cg.H && (unsigned)iw < (unsigned)cg.W;
                const size_t o = (size_t)(pb[b] + (uint32_t)(ic * HWin + (in ? ih * cg.W + iw : 0))) * 2 + h;
                ld16(f.x[b], P4 + o);
                f.in[b] = in;
            }
        }
    };
    auto fence_loads = []() { __builtin_amdgcn_sched_barrier(0); };   // the loads issued so far stay in front of this point
    auto compute = [&](const ConvFrag& f) {
        v8i x[2], wv[2];
#pragma unroll
        for (int b = 0; b < 2; b++) {
#pragma unroll
            for (int i = 0; i < 4; i++) x[b][i] = ((BUF && !ABIN) || f.in[b]) ? f.x[b][i] : (int)fillv;
#pragma unroll
            for (int i = 4; i < 8; i++) x[b][i] = 0;
        }
#pragma unroll
        for (int a = 0; a < 2; a++) wv[a] = v8i{f.w[a][0], f.w[a][1], f.w[a][2], f.w[a][3], 0, 0, 0, 0};
        // cbsz = blgp = 4: both operands E2M1, unscaled (see mfma<true>)
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
            for (int b = 0; b < 2; b++)
                acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wv[a], x[b], acc[a][b], 4, 4, 0, 0, 0, 0);
    };

    // The register sets rotate by name (the loop is unrolled by NB); loads past the last word
    // re-read it and are not multiplied (whole rounds of NB steps).
    const int K = cg.K;
    ConvFrag f[NB];
    int w = ks;
#pragma unroll
    for (int j = 0; j < NB - 1; j++) load(min(w + S * j, K - 1), f[j]);
    for (; w < K; w += S * NB) {
#pragma unroll
        for (int j = 0; j < NB; j++) {
            load(min(w + S * (j + NB - 1), K - 1), f[(j + NB - 1) % NB]);
            fence_loads();
            if (j == 0 || w + S * j < K) compute(f[j]);
        }
    }

    // hand-over: whether every lane of a pixel block may take the compare-free form
    DirectQuant direct_q[2] = {{false, false}, {false, false}};
    if constexpr (QMODE != 0) {
#pragma unroll
        for (int b = 0; b < 2; b++) direct_q[b] = direct_quant<QMODE>(alpha, qthr[b]);
    }
    // Block id = 2*a + b; wavefront ks of a tile finishes the blocks with id % S == ks and hands
    // the others over through LDS.  Every copy below names its accumulator registers statically,
    // under a wave-uniform branch, so that no register array is indexed at run time.
    auto for_blocks = [&](auto&& fn) {
        fn(std::integral_constant<int, 0>{});
        fn(std::integral_constant<int, 1>{});
        fn(std::integral_constant<int, 2>{});
        fn(std::integral_constant<int, 3>{});
    };
    if constexpr (S > 1) {
        for_blocks([&](auto blk_tag) {
            constexpr int BLK = decltype(blk_tag)::value;
            if (BLK % S != ks) {
                // slot of BLK among the blocks wavefront ks does not own
                const int slot = S == 4 ? (BLK < ks ? BLK : BLK - 1) : BLK / 2;
                float4* dst = red + (size_t)((wave * PUB + slot) * 4) * 64 + lane;
                const v16f& c = acc[BLK >> 1][BLK & 1];
#pragma unroll
                for (int e4 = 0; e4 < 4; e4++)
                    dst[e4 * 64] = make_float4(c[4 * e4], c[4 * e4 + 1], c[4 * e4 + 2], c[4 * e4 + 3]);
            }
        });
        __syncthreads();
    }
    for_blocks([&](auto blk_tag) {
        constexpr int BLK = decltype(blk_tag)::value;
        if (BLK % S == ks) {
            v16f mine = acc[BLK >> 1][BLK & 1];
            if constexpr (S > 1) {
#pragma unroll
                for (int v = 0; v < S; v++) {
                    if (v != BLK % S) {   // source wavefront pt*S + v holds BLK in the slot computed as above
                        const int slot = S == 4 ? (BLK < v ? BLK : BLK - 1) : BLK / 2;
                        const float4* src = red + (size_t)(((pt * S + v) * PUB + slot) * 4) * 64 + lane;
#pragma unroll
                        for (int e4 = 0; e4 < 4; e4++) {
                            const float4 t = src[e4 * 64];
                            mine[4 * e4] += t.x;
                            mine[4 * e4 + 1] += t.y;
                            mine[4 * e4 + 2] += t.z;
                            mine[4 * e4 + 3] += t.w;
                        }
                    }
                }
            }
            // accumulator e: kernel = 32*a + 8*(e/4) + 4*(lane/32) + e%4, pixel = 32*b + lane%32
            constexpr int a = BLK >> 1, b = BLK & 1;
            const int q = px0 + 32 * b + lr;
            const uint32_t qc = (uint32_t)min(q, M - 1);
            const uint32_t img = fastdiv(qc, dOHW);
            const uint32_t pix = qc - img * (uint32_t)OHW;
            // r = acc - bias: both are integers below 2^24 in fp32, and so is their difference (only BNN has a bias)
            const float fbias = (float)bias;
            float r[16];
#pragma unroll
            for (int e = 0; e < 16; e++) r[e] = FORM0 ? mine[e] : mine[e] - fbias;
            if constexpr (QMODE == 0) {
                float* yq = Y + ((size_t)img * KN + kn0 + 32 * a + 4 * h) * OHW + pix;
                if (q < M) {
                    if (kn0 + 32 * a + 32 <= KN) {   // whole block inside: no per-kernel checks
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
                // Hand-over to an fp4 layer.  Registers 4g .. 4g+3 of this lane are kernels 8g + 4h + {0..3} of the
                // block: half of nibble dword g of the pixel, the other half sits in lane ^ 32.  Lane half h ends up
                // with bytes 16a + 8h .. + 8 of the pixel's 64-channel word.
                const uint2 out = hand_over_block<FORM0, QMODE>(r, alpha, qthr[b], direct_q[b], kn0 + 32 * a, h, KN);
                const size_t word = ((size_t)img * gridDim.y + blockIdx.y) * OHW + pix;
                if (q < M) *reinterpret_cast<uint2*>(static_cast<unsigned char*>(qo.p4) + word * 32 + 16 * a + 8 * h) = out;
            }
        }
    });
}

// The same layer on tiles of 32 kernels x 32 pixels, for layers with few tiles of 64 x 64: a wavefront moves a
// bounded number of bytes per cycle from a cold L2 whatever its prefetch depth (600-700 cycles per K word of a
// 64 x 64 tile, measured), so a small layer gets faster only with more wavefronts, on more compute units.  A
// workgroup is one tile; its four wavefronts split the K loop four ways (word w to wavefront w % 4, one weight and
// one activation fragment per word), wavefronts 1..3 hand their partial block over through LDS and wavefront 0
// finishes it.  Kernel tiles come in pairs under the hand-over (a pixel's 64-channel word is written by two
// workgroups, 16 bytes each; a tile past KN writes padding lanes).
// BUF: fragments through buffer loads, as in k_conv_f4.
template <bool ABIN, bool FORM0, int QMODE, bool BUF>
__global__ __launch_bounds__(256) void k_conv_f4_small(const uint4* __restrict__ P4, const uint4* __restrict__ Wf,
                                                       float* __restrict__ Y, int M, int KN, int OHW, int KB, int bias,
                                                       float alpha, FastDiv dOHW, ConvGeom cg, QuantOut qo,
                                                       uint32_t p4_bytes, uint32_t wf_bytes) {
    constexpr int S = 4, NB = 3;
    __shared__ float4 red[3 * 4 * 64];   // [wavefront - 1][e / 4][lane]
    const int tid = threadIdx.x, lane = tid & 63;
    const int ks = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = lane >> 5, lr = lane & 31;
    const int px0 = blockIdx.x * 32, kn0 = blockIdx.y * 32;

    const int q = px0 + lr;
    const uint32_t qc = (uint32_t)min(q, M - 1);
    const uint32_t img = fastdiv(qc, dOHW);
    const uint32_t pix = qc - img * (uint32_t)OHW;
    const int oh = (int)fastdiv(pix, cg.dOW), ow = (int)pix - oh * cg.OW;
    const int ih0 = oh * cg.H_stride - cg.H_pad, iw0 = ow * cg.W_stride - cg.W_pad;
    const uint32_t pb = img * (uint32_t)(cg.CP * cg.H * cg.W);   // image of P4[n][C_pack][pixel]
    float qthr = 0.0f;
    if constexpr (QMODE != 0) qthr = qo.thr[img];   // fetched in front of the K loop's loads (see k_conv_f4)
    const int HWin = cg.H * cg.W;
    const int rbmax = (KN + 31) / 32 - 1;
    const uint4* wb = Wf + (size_t)min(kn0 / 32, rbmax) * KB * 64 + lane;

    v16f acc;
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] = 0.0f;
    const uint32_t fillv = ABIN ? 0x22222222u : 0u;

    struct Frag {
        v4i w, x;
        bool in;
    };
    auto ld16 = [](v4i& dst, const uint4* src) { dst = *reinterpret_cast<const v4i*>(src); };   // loads as in k_conv_f4
    __amdgpu_buffer_rsrc_t brs_x = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint4*>(P4), 0, (int)p4_bytes, 0x00020000);
    __amdgpu_buffer_rsrc_t brs_w = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint4*>(Wf), 0, (int)wf_bytes, 0x00020000);
    uint32_t wofs = 0u, xofs = 0u;
    if constexpr (BUF) {
        wofs = ((uint32_t)min(kn0 / 32, rbmax) * (uint32_t)KB * 64u + (uint32_t)lane) * 16u;
        xofs = ((pb + (uint32_t)(ih0 * cg.W + iw0)) * 2u + (uint32_t)h) * 16u;
    }
    auto ldbuf = [&](v4i& dst, uint32_t voff, uint32_t soff, bool weights) {
        const v4u v = __builtin_amdgcn_raw_buffer_load_b128(weights ? brs_w : brs_x, (int)voff, (int)soff, 0);
        dst = v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
    };
    auto load = [&](int w, Frag& f) {   // w is wave-uniform
        const int tap = (int)fastdiv((uint32_t)w, cg.dCP), ic = w - tap * cg.CP;
        const int kh = (int)fastdiv((uint32_t)tap, cg.dKW), kw = tap - kh * cg.KW;
        const int ih = ih0 + kh, iw = iw0 + kw;
        if constexpr (BUF) {
            ldbuf(f.w, wofs, (uint32_t)__builtin_amdgcn_readfirstlane(w) * 1024u, true);
            const bool in = (unsigned)ih < (unsigned)cg.H && (unsigned)iw < (unsigned)cg.W;
            const uint32_t tapoff = (uint32_t)__builtin_amdgcn_readfirstlane((ic * HWin + kh * cg.W + kw) * 32);
            ldbuf(f.x, in ? xofs + tapoff : (ABIN ? 0u : 0xffffff00u), 0u, false);   // as in k_conv_f4
            f.in = ABIN ? in : true;
        } else {
            ld16(f.w, wb + (size_t)w * 64);
            f.in = (unsigned)ih < (unsigned)cg.H && (unsigned)iw < (unsigned)cg.W;
            const size_t o = (size_t)(pb + (uint32_t)(ic * HWin + (f.in ? ih * cg.W + iw : 0))) * 2 + h;
            ld16(f.x, P4 + o);
        }
    };
    auto fence_loads = []() { __builtin_amdgcn_sched_barrier(0); };
    auto compute = [&](const Frag& f) {
        v8i x, wv;
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] = ((BUF && !ABIN) || f.in) ? f.x[i] : (int)fillv;
#pragma unroll
        for (int i = 4; i < 8; i++) x[i] = 0;
        wv = v8i{f.w[0], f.w[1], f.w[2], f.w[3], 0, 0, 0, 0};
        acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wv, x, acc, 4, 4, 0, 0, 0, 0);
    };

    // as in k_conv_f4: register sets rotate by name, loads past the last word re-read it and are not multiplied
    const int K = cg.K;
    Frag f[NB];
    int w = ks;
#pragma unroll
    for (int j = 0; j < NB - 1; j++) load(min(w + S * j, K - 1), f[j]);
    for (; w < K; w += S * NB) {
#pragma unroll
        for (int j = 0; j < NB; j++) {
            load(min(w + S * (j + NB - 1), K - 1), f[(j + NB - 1) % NB]);
            fence_loads();
            if (j == 0 || w + S * j < K) compute(f[j]);
        }
    }

    if (ks != 0) {
        float4* dst = red + (size_t)((ks - 1) * 4) * 64 + lane;
#pragma unroll
        for (int e4 = 0; e4 < 4; e4++)
            dst[e4 * 64] = make_float4(acc[4 * e4], acc[4 * e4 + 1], acc[4 * e4 + 2], acc[4 * e4 + 3]);
    }
    __syncthreads();
    if (ks != 0) return;
#pragma unroll
    for (int v = 0; v < 3; v++) {
        const float4* src = red + (size_t)(v * 4) * 64 + lane;
#pragma unroll
        for (int e4 = 0; e4 < 4; e4++) {
            const float4 t = src[e4 * 64];
            acc[4 * e4] += t.x;
            acc[4 * e4 + 1] += t.y;
            acc[4 * e4 + 2] += t.z;
            acc[4 * e4 + 3] += t.w;
        }
    }

    // accumulator e: kernel = kn0 + 8*(e/4) + 4*h + e%4, pixel = px0 + lr
    const float fbias = (float)bias;
    float r[16];
#pragma unroll
    for (int e = 0; e < 16; e++) r[e] = FORM0 ? acc[e] : acc[e] - fbias;   // only BNN has a bias
    if constexpr (QMODE == 0) {
        float* yq = Y + ((size_t)img * KN + kn0 + 4 * h) * OHW + pix;
        if (q < M) {
            if (kn0 + 32 <= KN) {   // uniform: whole block inside
#pragma unroll
                for (int e = 0; e < 16; e++) yq[(size_t)(8 * (e >> 2) + (e & 3)) * OHW] = prelu_ref<FORM0>(r[e], alpha);
            } else {
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    const int p = kn0 + 8 * (e >> 2) + 4 * h + (e & 3);
                    if (p < KN) yq[(size_t)(8 * (e >> 2) + (e & 3)) * OHW] = prelu_ref<FORM0>(r[e], alpha);
                }
            }
        }
    } else {
        const uint2 out = hand_over_block<FORM0, QMODE>(r, alpha, qthr, direct_quant<QMODE>(alpha, qthr), kn0, h, KN);
        // this tile is half a 64-channel word: bytes 16 * (tile parity) of the pixel's 32
        const size_t word = ((size_t)img * (gridDim.y >> 1) + (blockIdx.y >> 1)) * OHW + pix;
        if (q < M)
            *reinterpret_cast<uint2*>(static_cast<unsigned char*>(qo.p4) + word * 32 + 16 * (blockIdx.y & 1) + 8 * h) = out;
    }
}

// tiles of 256 x 256 below which the 128 x 128 kernel is used (FTNN_MFMA_SMALL_BELOW: tuning aid)
inline int64_t mfma_small_tile_below() {
    static const int64_t v = []() {
        const char* e = getenv("FTNN_MFMA_SMALL_BELOW");
        return e ? (int64_t)atoll(e) : (int64_t)160;
    }();
    return v;
}

template <bool F4, bool SWAP, int WTP, int WTQ, int KF, int NS>
hipError_t launch_gemm_tile(const uint4* Pf, const uint4* Qf, float* Y, int M, int KN, int OHW, int KB,
                            int bias, int form, float alpha, hipStream_t st) {
    auto kern = k_mfma<F4, SWAP, WTP, WTQ, KF, NS>;
    constexpr size_t lds_bytes = Tile<WTP, WTQ, KF, NS>::lds_bytes;
    // the opt-in to more than 64 KiB of dynamic LDS is per kernel; done once, thread-safe
    // The kernel counts its LDS-direct loads by hand (s_waitcnt vmcnt(N)); a scratch access would be one more
    // vector-memory operation inside those windows, so a build of it that spills is refused (once per variant).
    static const hipError_t configured = []() {
        const void* kern = reinterpret_cast<const void*>(&k_mfma<F4, SWAP, WTP, WTQ, KF, NS>);
        hipFuncAttributes attr;
        hipError_t e = hipFuncGetAttributes(&attr, kern);
        if (e == hipSuccess && attr.localSizeBytes != 0) e = hipErrorLaunchFailure;
        if (e != hipSuccess) return e;
        return hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)Tile<WTP, WTQ, KF, NS>::lds_bytes);
    }();
    if (configured != hipSuccess) return configured;
    const int prow = SWAP ? KN : M, qrow = SWAP ? M : KN;
    dim3 grid((prow + 64 * WTP - 1) / (64 * WTP), (qrow + 64 * WTQ - 1) / (64 * WTQ));
    if (grid.y > 65535) return hipErrorInvalidValue;
    hipLaunchKernelGGL(kern, grid, dim3(256), lds_bytes, st, Pf, Qf, Y, M, KN, OHW, KB, bias, form, alpha, ConvGeom(), FastDiv(), 0,
                       FastDiv());
    return hipGetLastError();
}

template <bool F4, bool SWAP>
hipError_t launch_gemm(const uint4* Pf, const uint4* Qf, float* Y, int M, int KN, int OHW, int KB,
                       int bias, int form, float alpha, hipStream_t st) {
    // 256 x 256 tiles re-read the operands least, but a problem must have enough of them for the chip's
    // 256 compute units; below that, 128 x 128 tiles (two workgroups fit a compute unit)
    const int64_t big = (((int64_t)M + 255) / 256) * ((KN + 255) / 256);
    bool small = big < mfma_small_tile_below();
    // two fragments per step and a ring of four: four fragments per step with a ring of two (the same LDS, half
    // the barriers) measured 0.87 against 0.76 ms on 8192 x 8192 x 32768 -- the ring then no longer covers the loads
    // Fewer than 112 tiles of 128 x 128 leave most compute units idle: tiles of 64 x 64 then, four K words per step
    // (1024 x 1024 x 8192 as a whole call: 25.7 -> 19.0 us, 768: 21.2 -> 15.7, 1280 (100 tiles): 29.6 -> 27.2; from 144
    // tiles on the larger tile is faster, 33.6 against 39.6 us at 1536; tiles of 128 x 64 lose everywhere).
    // FTNN_MFMA_TINY_BELOW = n moves the threshold (tuning aid).
    static const int tiny_below = getenv("FTNN_MFMA_TINY_BELOW") ? atoi(getenv("FTNN_MFMA_TINY_BELOW")) : 112;
    const int64_t mid = (((int64_t)M + 127) / 128) * ((KN + 127) / 128);
    if (small && mid < tiny_below) return launch_gemm_tile<F4, SWAP, 1, 1, 4, 4>(Pf, Qf, Y, M, KN, OHW, KB, bias, form, alpha, st);
    return small ? launch_gemm_tile<F4, SWAP, 2, 2, 2, 4>(Pf, Qf, Y, M, KN, OHW, KB, bias, form, alpha, st)
                 : launch_gemm_tile<F4, SWAP, 4, 4, 2, 4>(Pf, Qf, Y, M, KN, OHW, KB, bias, form, alpha, st);
}

template <bool F4>
hipError_t launch_expand(bool tern, const uint32_t* rows_ptr, int rows, int G, uint4* out, hipStream_t st) {
    dim3 grid((rows + 31) / 32, (G + 3) / 4);   // 4 groups per workgroup (kGPB in the kernel)
    if (grid.y > 65535) return hipErrorInvalidValue;
    if (tern) hipLaunchKernelGGL((k_expand<F4, true>), grid, dim3(256), 0, st, rows_ptr, rows, G, out);
    else hipLaunchKernelGGL((k_expand<F4, false>), grid, dim3(256), 0, st, rows_ptr, rows, G, out);
    return hipGetLastError();
}

template <bool SWAP, int WT, int NS>
hipError_t launch_gemm_p4_tile(const uint4* Pc, const uint4* Qc, float* Y, int M, int KN, int OHW, int KP, const int* sP,
                               const int* sQ, int off, int form, float alpha, hipStream_t st) {
    auto kern = k_mfma_p4<SWAP, WT, NS>;
    constexpr size_t lds_bytes = (size_t)NS * 4 * WT * 1024;
    // hand-counted LDS-direct loads: no scratch (see launch_gemm_tile); the opt-in to more than 64 KiB of LDS is per kernel
    static const hipError_t configured = []() {
        const void* k = reinterpret_cast<const void*>(&k_mfma_p4<SWAP, WT, NS>);
        hipFuncAttributes attr;
        hipError_t e = hipFuncGetAttributes(&attr, k);
        if (e == hipSuccess && attr.localSizeBytes != 0) e = hipErrorLaunchFailure;
        if (e != hipSuccess) return e;
        return hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)((size_t)NS * 4 * WT * 1024));
    }();
    if (configured != hipSuccess) return configured;
    const int prow = SWAP ? KN : M, qrow = SWAP ? M : KN, edge = 64 * WT;
    dim3 grid((prow + edge - 1) / edge, (qrow + edge - 1) / edge);
    if (grid.y > 65535) return hipErrorInvalidValue;
    hipLaunchKernelGGL(kern, grid, dim3(256), lds_bytes, st, Pc, Qc, Y, M, KN, OHW, KP, sP, sQ, off, form, alpha);
    return hipGetLastError();
}

template <bool SWAP>
hipError_t launch_gemm_p4(const uint4* Pc, const uint4* Qc, float* Y, int M, int KN, int OHW, int KP, const int* sP, const int* sQ,
                          int off, int form, float alpha, hipStream_t st) {
    const int64_t big = (((int64_t)M + 255) / 256) * ((KN + 255) / 256);
    return big < mfma_small_tile_below() ? launch_gemm_p4_tile<SWAP, 2, 4>(Pc, Qc, Y, M, KN, OHW, KP, sP, sQ, off, form, alpha, st)
                                         : launch_gemm_p4_tile<SWAP, 4, 4>(Pc, Qc, Y, M, KN, OHW, KP, sP, sQ, off, form, alpha, st);
}

}  // namespace

int64_t mfma_fragment_bytes(bool f4, int64_t rows, int Kw) {
    // 1 KiB fragments: 32 rows x one word (fp4) or half a word (int8)
    return ((rows + 31) / 32) * (int64_t)(f4 ? Kw : 2 * Kw) * 1024;
}

hipError_t launch_mfma_expand(bool f4, bool ternary, const int64_t* d_rows, int rows, int Kw, void* d_out,
                              hipStream_t st) {
    const uint32_t* R = reinterpret_cast<const uint32_t*>(d_rows);
    uint4* out = static_cast<uint4*>(d_out);
    return f4 ? launch_expand<true>(ternary, R, rows, Kw / 4, out, st)
              : launch_expand<false>(ternary, R, rows, Kw / 4, out, st);
}

hipError_t launch_mfma_gemm(bool f4, int type, const void* d_af, const void* d_bf, int64_t M, int OHW, int KN,
                            int Kw, int K_unpack, float alpha, float* d_y, hipStream_t st) {
    const int KB = f4 ? Kw : 2 * Kw;
    const uint4* Af = static_cast<const uint4*>(d_af);
    const uint4* Bf = static_cast<const uint4*>(d_bf);
    // BNN: the lanes past K_unpack are +1 in both operands and add 64*Kw - K_unpack to the dot
    // product; the reference's K_unpack - 2*popc(a^b) leaves them out (mm_p2_final_bnn_avx2.c:55-58)
    const int bias = type == kBNN ? 64 * Kw - K_unpack : 0;
    const int form = type == kTNN ? 0 : 1;
    const bool swap = OHW > 1;
    if (f4) {
        return swap ? launch_gemm<true, true>(Bf, Af, d_y, (int)M, KN, OHW, KB, bias, form, alpha, st)
                    : launch_gemm<true, false>(Af, Bf, d_y, (int)M, KN, OHW, KB, bias, form, alpha, st);
    }
    return swap ? launch_gemm<false, true>(Bf, Af, d_y, (int)M, KN, OHW, KB, bias, form, alpha, st)
                : launch_gemm<false, false>(Af, Bf, d_y, (int)M, KN, OHW, KB, bias, form, alpha, st);
}

// ---- packed4: the fp4 GEMM's operands at two bits per lane in offset codes (Kw a multiple of 4, as everywhere) ----
namespace {
inline int64_t packed4_block_bytes(int64_t rows, int Kw) { return ((rows + 31) / 32) * (int64_t)(Kw / 2) * 1024; }
}  // namespace

// the blocks, then one int32 per row of the row blocks (a multiple of 128 bytes)
int64_t mfma_packed4_bytes(int64_t rows, int Kw) { return packed4_block_bytes(rows, Kw) + ((rows + 31) / 32) * 128; }

namespace {
inline int* packed4_sums(void* d_out, int64_t rows, int Kw) {
    return reinterpret_cast<int*>(static_cast<char*>(d_out) + packed4_block_bytes(rows, Kw));
}

// zero_sums = false: the caller has zeroed the row sums on the stream already
hipError_t launch_pack4(bool ternary, const int64_t* d_rows, int rows, int Kw, void* d_out, bool zero_sums, hipStream_t st) {
    dim3 grid((rows + 31) / 32, (Kw / 4 + 3) / 4);   // 4 groups of 4 words per workgroup
    if (grid.y > 65535) return hipErrorInvalidValue;
    const uint32_t* R = reinterpret_cast<const uint32_t*>(d_rows);
    int* sums = packed4_sums(d_out, rows, Kw);
    if (grid.x > 0x7fffff00u / 32) return hipErrorInvalidValue;
    const int nsum = (int)grid.x * 32;
    if (zero_sums) hipLaunchKernelGGL(k_zero_i32, dim3((nsum + 255) / 256), dim3(256), 0, st, sums, nsum, nullptr, 0);
    if (ternary) hipLaunchKernelGGL((k_pack4<true>), grid, dim3(256), 0, st, R, rows, Kw / 4, static_cast<uint2*>(d_out), sums);
    else hipLaunchKernelGGL((k_pack4<false>), grid, dim3(256), 0, st, R, rows, Kw / 4, static_cast<uint2*>(d_out), sums);
    return hipGetLastError();
}
}  // namespace

hipError_t launch_mfma_pack4(bool ternary, const int64_t* d_rows, int rows, int Kw, void* d_out, hipStream_t st) {
    return launch_pack4(ternary, d_rows, rows, Kw, d_out, true, st);
}

hipError_t launch_mfma_gemm_packed4(int type, const void* d_ac, const void* d_bc, int64_t M, int OHW, int KN, int Kw, int K_unpack,
                                    float alpha, float* d_y, hipStream_t st) {
    const uint4* Ac = static_cast<const uint4*>(d_ac);
    const uint4* Bc = static_cast<const uint4*>(d_bc);
    const int* sA = reinterpret_cast<const int*>(static_cast<const char*>(d_ac) + packed4_block_bytes(M, Kw));
    const int* sB = reinterpret_cast<const int*>(static_cast<const char*>(d_bc) + packed4_block_bytes(KN, Kw));
    const int bias = type == kBNN ? 64 * Kw - K_unpack : 0;   // as launch_mfma_gemm
    const int off = 64 * Kw + bias;                           // the lanes of a row pair, padding included
    const int form = type == kTNN ? 0 : 1;
    return OHW > 1 ? launch_gemm_p4<true>(Bc, Ac, d_y, (int)M, KN, OHW, Kw / 2, sB, sA, off, form, alpha, st)
                   : launch_gemm_p4<false>(Ac, Bc, d_y, (int)M, KN, OHW, Kw / 2, sA, sB, off, form, alpha, st);
}

namespace {
constexpr int kMaxTileRouteWords = 2040;   // K words per row the tile kernel keeps a table entry for (16 KiB of LDS with the two spare ones)
template <int WTP, int WTQ, int NS, bool BAL>
hipError_t launch_conv_tiles_wt(const uint4* Wf, const uint4* P4, float* Y, int M, int KN, int OHW, int KB, int bias, int form,
                                float alpha, const ConvGeom& cg, hipStream_t st) {
    auto kern = k_mfma<true, true, WTP, WTQ, 2, NS, true, BAL>;
    typedef Tile<WTP, WTQ, 2, NS> TL;
    constexpr size_t kLdsMax = 160u << 10;   // LDS of a compute unit
    const size_t lds_bytes = TL::lds_bytes + (size_t)(KB + 2) * 8;   // the ring, then the table of K words (+ 2 read ahead)
    if (KB > kMaxTileRouteWords || lds_bytes > kLdsMax) return hipErrorInvalidValue;
    // as launch_gemm_tile: hand-counted LDS-direct loads, so no scratch; the LDS opt-in is per kernel
    static const hipError_t configured = []() {
        const void* k = reinterpret_cast<const void*>(&k_mfma<true, true, WTP, WTQ, 2, NS, true, BAL>);
        hipFuncAttributes attr;
        hipError_t e = hipFuncGetAttributes(&attr, k);
        if (e == hipSuccess && attr.localSizeBytes != 0) e = hipErrorLaunchFailure;
        if (e != hipSuccess) return e;
        return hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsMax);
    }();
    if (configured != hipSuccess) return configured;
    dim3 grid((KN + 64 * WTP - 1) / (64 * WTP), (M + 64 * WTQ - 1) / (64 * WTQ));   // P = weights, Q = pixels
    if (grid.y > 65535) return hipErrorInvalidValue;
    hipLaunchKernelGGL(kern, grid, dim3(256), lds_bytes, st, Wf, P4, Y, M, KN, OHW, KB, bias, form, alpha, cg,
                       make_fastdiv((uint32_t)OHW), (cg.W + cg.W_stride - 1) / cg.W_stride, make_fastdiv((uint32_t)cg.W_stride));
    return hipGetLastError();
}
}  // namespace

// A layer goes to the tile kernel with implicit im2row from 90 tiles of 128 x 128 on, if its rows have at least 16
// words and it has at least 512 output pixels.  Measured on MI355X, the reference's batch-8 stride-2 layers, quantiser
// included: 512 channels at 56 x 56 (196 tiles) 38.6 -> 28.6 us, 1024 channels at 56 x 56 (392 tiles) 77.6 -> 60.4 us
// (80 us as quantise + im2row + expansion + GEMM); with 98 and 104 tiles (256 channels at 56 x 56, 1024 at 28 x 28) the
// layer kernel is as fast or faster than tiles of 128 x 128 (17.7 against 18.7, 31.8 against 33.1 us) and tiles of
// 64 x 64 are faster than both (16.5 and 28.4 us); with 52 tiles (512 channels at 28 x 28) a tie, below that the layer
// kernels win.  FTNN_CONV_TILES_FROM = n: tuning aid; it sets the tile count and drops the conditions on words and pixels.
namespace {
// the tile kernel's limits: a tap mask of 32 bits per pixel, a table entry per K word, 32-bit piece indices into T4,
// pixel indices below 2^31 and its way of keeping kw - pad non-negative
bool conv_tiles_within_limits(int64_t M, int CP, int taps, int64_t t4_bytes, int W_pad, int W_stride) {
    const int64_t K = (int64_t)CP * taps;
    return taps <= 32 && (K + 3) / 4 * 4 <= kMaxTileRouteWords && M <= 0x7fffff00LL && t4_bytes / 16 <= 0x7fffffffLL &&
           W_pad < 4096 * (int64_t)W_stride;
}
}  // namespace

bool conv_f4_tile_route(int64_t M, int KN, int CP, int taps, int64_t t4_bytes, int W_pad, int W_stride) {
    static const char* tune = getenv("FTNN_CONV_TILES_FROM");
    static const int64_t from = tune ? atoll(tune) : 90;
    const int64_t tiles = ((M + 127) / 128) * ((KN + 127) / 128);
    const int64_t K = (int64_t)CP * taps;
    return tiles >= from && (tune || (K >= 16 && M >= 512)) && conv_tiles_within_limits(M, CP, taps, t4_bytes, W_pad, W_stride);
}

// A large conv layer as workgroup tiles staged through LDS, the activation fragments gathered from T4
// (launch_quantize_f4_tiled; k_mfma with IMPL): fp32 NCHW result only.  d_wf: the weights as fp4 fragments
// (KB = round4(cg.K) words per row).
hipError_t launch_conv_f4_tiles(int type, const void* d_p4, const void* d_wf, const ConvGeom& cg, int N, int KN, int K_unpack,
                                float alpha, float* d_y, hipStream_t st) {
    const int OHW = cg.OH * cg.OW;
    const int64_t M = (int64_t)N * OHW;
    const int KB = round4(cg.K);
    if (!conv_tiles_within_limits(M, cg.CP, cg.K / cg.CP, quantize_f4_tiled_bytes(N, cg.CP * 64, cg.H, cg.W, cg.W_stride), cg.W_pad, cg.W_stride))
        return hipErrorInvalidValue;
    // BNN: every lane that is no real (channel, tap) is +1 x +1 in both operands, padding words included
    const int bias = type == kBNN ? 64 * KB - K_unpack : 0;
    const int form = type == kTNN ? 0 : 1;
    const uint4* Wf = static_cast<const uint4*>(d_wf);
    const uint4* P4 = static_cast<const uint4*>(d_p4);
    // tile shape (kernels x pixels): FTNN_CONV_TILE_SHAPE = 11 | 22 | 42 | 44 forces one (tuning aid)
    static const int tune = getenv("FTNN_CONV_TILE_SHAPE") ? atoi(getenv("FTNN_CONV_TILE_SHAPE")) : 0;
    // 256 x 256 tiles once they fill the chip; 256 kernels x 128 pixels where those fill most of it in one round (the
    // 1024-channel 56 x 56 layer at batch 8: 196 workgroups, 60.4 against 63.8 us on 392 tiles of 128 x 128); else
    // 128 x 128, and 64 x 64 below 150 of those
    const int64_t big = ((M + 255) / 256) * ((KN + 255) / 256), mid = ((M + 127) / 128) * ((KN + 255) / 256);
    const int64_t sq = ((M + 127) / 128) * ((KN + 127) / 128);
    int shape = big >= mfma_small_tile_below() ? 44 : (mid >= 180 ? 42 : (sq >= 150 ? 22 : 11));
    if (tune == 11 || tune == 22 || tune == 42 || tune == 44) shape = tune;
    // 128 x 128 and 256 x 128 tiles: every wavefront gathers a quarter of the activation fragments (1024 channels at
    // 56 x 56, batch 8: 60.2 -> 57.4 us; 512 channels: 27.3 -> 26.8); on 64 x 64 tiles the two gathering wavefronts of the
    // plain order are faster (28.3 against 29.0 us), and 256 x 256 tiles have no registers to spare for four gatherers
    if (shape == 44) return launch_conv_tiles_wt<4, 4, 4, false>(Wf, P4, d_y, (int)M, KN, OHW, KB, bias, form, alpha, cg, st);
    if (shape == 42) return launch_conv_tiles_wt<4, 2, 4, true>(Wf, P4, d_y, (int)M, KN, OHW, KB, bias, form, alpha, cg, st);
    if (shape == 11) return launch_conv_tiles_wt<1, 1, 4, false>(Wf, P4, d_y, (int)M, KN, OHW, KB, bias, form, alpha, cg, st);
    return launch_conv_tiles_wt<2, 2, 4, true>(Wf, P4, d_y, (int)M, KN, OHW, KB, bias, form, alpha, cg, st);
}

hipError_t launch_conv_f4(int type, const void* d_p4, const void* d_wf, const ConvGeom& cg, int N, int KN,
                          int K_unpack, float alpha, float* d_y, hipStream_t st, const QuantOut& qo) {
    const int OHW = cg.OH * cg.OW;
    const int64_t M = (int64_t)N * OHW;
    const int KB = round4(cg.K);
    // BNN: the channel lanes past C are +1 in both operands (see launch_mfma_gemm); padding words are skipped
    const int bias = type == kBNN ? 64 * cg.K - K_unpack : 0;
    // K split: enough wavefronts to occupy the chip's 1024 SIMDs, but no exchange where the tiles
    // alone do that (a tile = 64 kernels x 64 pixels)
    const int64_t tiles = ((M + 63) / 64) * ((KN + 63) / 64);
    int split = tiles >= 600 ? 1 : (tiles >= 450 ? 2 : 4);   // measured on MI355X (1024 SIMDs)
    static const int tune = []() {   // tuning aid: force the K split (1, 2 or 4; anything else is ignored)
        const char* e = getenv("FTNN_CONV_SPLIT");
        const int v = e ? atoi(e) : 0;
        return (v == 1 || v == 2 || v == 4) ? v : 0;
    }();
    if (tune) split = tune;
    while (split > 1 && cg.K < split) split /= 2;   // no wavefront without K words of its own, forced or not
    const int wpb = 4, tpb = wpb / split;   // wavefronts and pixel tiles per workgroup (see the kernel)
    // few 64 x 64 tiles: tiles of 32 x 32, four times the workgroups (k_conv_f4_small)
    static const int small_below = getenv("FTNN_CONV_SMALL_BELOW") ? atoi(getenv("FTNN_CONV_SMALL_BELOW")) : 150;
    const bool small = tiles < small_below;
    dim3 grid((unsigned)(((M + 63) / 64 + tpb - 1) / tpb), (unsigned)((KN + 63) / 64));
    if (small) grid = dim3((unsigned)((M + 31) / 32), (unsigned)(qo.mode != 0 ? 2 * ((KN + 63) / 64) : (KN + 31) / 32));
    if (M > 0x7fffff00LL || grid.y > 65535) return hipErrorInvalidValue;   // pixel indices stay below 2^31
    const uint4* P4 = static_cast<const uint4*>(d_p4);
    const uint4* Wf = static_cast<const uint4*>(d_wf);
    const FastDiv dOHW = make_fastdiv((uint32_t)OHW);
    // operand sizes: the buffer-load variants announce them in their descriptors
    const int64_t p4_bytes = (int64_t)N * cg.CP * cg.H * cg.W * 32, wf_bytes = (int64_t)((KN + 31) / 32) * KB * 1024;
    static const bool no_buf = getenv("FTNN_CONV_NO_BUFFER_LOADS") != nullptr;   // tuning aid
    const bool buf = !no_buf && p4_bytes <= 0xf0000000LL && wf_bytes <= 0xf0000000LL;
    auto launch64 = [&](auto variant) -> hipError_t {
        constexpr auto kern = decltype(variant)::value;
        hipLaunchKernelGGL(kern, grid, dim3(64 * wpb), 0, st, P4, Wf, d_y, (int)M, KN, OHW, KB, bias, alpha, dOHW, cg, qo,
                           (uint32_t)std::min<int64_t>(p4_bytes, 0xffffffffLL), (uint32_t)std::min<int64_t>(wf_bytes, 0xffffffffLL));
        return hipGetLastError();
    };
    auto by_buf = [&](auto abin, auto form0, auto qmode, auto sp) -> hipError_t {
        constexpr bool A = decltype(abin)::value, F = decltype(form0)::value;
        constexpr int Q = decltype(qmode)::value, SP = decltype(sp)::value;
        if (buf) return launch64(std::integral_constant<decltype(&k_conv_f4<A, F, Q, SP, 3, true>), &k_conv_f4<A, F, Q, SP, 3, true>>{});
        return launch64(std::integral_constant<decltype(&k_conv_f4<A, F, Q, SP, 3, false>), &k_conv_f4<A, F, Q, SP, 3, false>>{});
    };
    // kernel variant: activation kind and PReLU form follow the type, then hand-over mode and split
    auto by_split = [&](auto abin, auto form0, auto qmode) -> hipError_t {
        constexpr bool A = decltype(abin)::value, F = decltype(form0)::value;
        constexpr int Q = decltype(qmode)::value;
        if (small) {
            if (buf) return launch64(std::integral_constant<decltype(&k_conv_f4_small<A, F, Q, true>), &k_conv_f4_small<A, F, Q, true>>{});
            return launch64(std::integral_constant<decltype(&k_conv_f4_small<A, F, Q, false>), &k_conv_f4_small<A, F, Q, false>>{});
        }
        // three register sets: deeper prefetch measured no faster at any layer size
        if (split == 1) return by_buf(abin, form0, qmode, std::integral_constant<int, 1>{});
        if (split == 2) return by_buf(abin, form0, qmode, std::integral_constant<int, 2>{});
        if (split == 4) return by_buf(abin, form0, qmode, std::integral_constant<int, 4>{});
        return hipErrorInvalidValue;
    };
    auto by_mode = [&](auto abin, auto form0) -> hipError_t {
        if (qo.mode == 0) return by_split(abin, form0, std::integral_constant<int, 0>{});
        if (qo.mode == 1) return by_split(abin, form0, std::integral_constant<int, 1>{});
        if (qo.mode == 2) return by_split(abin, form0, std::integral_constant<int, 2>{});
        return hipErrorInvalidValue;
    };
    if (type == kTNN) return by_mode(std::false_type{}, std::true_type{});
    if (type == kTBN) return by_mode(std::false_type{}, std::false_type{});
    return by_mode(std::true_type{}, std::false_type{});   // BTN, BNN
}

// A whole call from packed rows expands both operands itself, so it may pick the operand form by shape: problems on
// 128 x 128 tiles (few tiles; one workgroup per compute unit, nothing to hide the read -> unpack -> multiply chain of the
// packed4 kernel's short steps) run faster on plain fp4 fragments (2048 x 2048 x 16384: 54 against 62 us, 1024 x 1024 x
// 8192: 30 against 36), the large ones on packed4 in offset codes.
static bool f4_whole_call_plain(int64_t M, int KN) {
    return ((M + 255) / 256) * ((KN + 255) / 256) < mfma_small_tile_below();
}

int64_t mfma_f4_mm_scratch_bytes(int64_t M, int KN, int Kw) {
    return f4_whole_call_plain(M, KN) ? mfma_fragment_bytes(true, M, Kw) + mfma_fragment_bytes(true, KN, Kw)
                                      : mfma_packed4_bytes(M, Kw) + mfma_packed4_bytes(KN, Kw);
}

hipError_t launch_mm_mfma(bool f4, int type, const int64_t* d_a, const int64_t* d_b, int64_t M, int OHW,
                          int KN, int Kw, int K_unpack, float alpha, float* d_y, void* d_scratch,
                          hipStream_t st) {
    const bool a_tern = (type == kTNN || type == kTBN), b_tern = (type == kTNN || type == kBTN);
    if (f4 && !f4_whole_call_plain(M, KN)) {   // the fp4 GEMM takes its operands at two bits per lane
        void* Ac = d_scratch;
        void* Bc = static_cast<char*>(d_scratch) + mfma_packed4_bytes(M, Kw);
        const int64_t na64 = (M + 31) / 32 * 32, nb64 = ((int64_t)KN + 31) / 32 * 32;
        if (na64 + nb64 > 0x7fffff00LL) return hipErrorInvalidValue;
        const int na = (int)na64, nb = (int)nb64;   // one launch zeroes both operands' row sums
        hipLaunchKernelGGL(k_zero_i32, dim3((na + nb + 255) / 256), dim3(256), 0, st, packed4_sums(Ac, M, Kw), na,
                           packed4_sums(Bc, KN, Kw), nb);
        // both operands packed by one launch
        const dim3 grid((unsigned)(na / 32 + nb / 32), (unsigned)((Kw / 4 + 3) / 4));
        if (grid.y > 65535) return hipErrorInvalidValue;
        const uint32_t *Ra = reinterpret_cast<const uint32_t*>(d_a), *Rb = reinterpret_cast<const uint32_t*>(d_b);
        uint2 *Oa = static_cast<uint2*>(Ac), *Ob = static_cast<uint2*>(Bc);
        int *Sa = packed4_sums(Ac, M, Kw), *Sb = packed4_sums(Bc, KN, Kw);
#define FTNN_PACK2(TA_, TB_) hipLaunchKernelGGL((k_pack4_2<TA_, TB_>), grid, dim3(256), 0, st, Ra, (int)M, Oa, Sa, Rb, KN, Ob, Sb, Kw / 4)
        if (a_tern && b_tern) FTNN_PACK2(true, true);
        else if (a_tern) FTNN_PACK2(true, false);
        else if (b_tern) FTNN_PACK2(false, true);
        else FTNN_PACK2(false, false);
#undef FTNN_PACK2
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        return launch_mfma_gemm_packed4(type, Ac, Bc, M, OHW, KN, Kw, K_unpack, alpha, d_y, st);
    }
    void* Af = d_scratch;
    void* Bf = static_cast<char*>(d_scratch) + mfma_fragment_bytes(f4, M, Kw);
    {   // both operands expanded by one launch
        const dim3 grid((unsigned)((M + 31) / 32 + (KN + 31) / 32), (unsigned)((Kw / 4 + 3) / 4));
        if (grid.y > 65535) return hipErrorInvalidValue;
        const uint32_t *Ra = reinterpret_cast<const uint32_t*>(d_a), *Rb = reinterpret_cast<const uint32_t*>(d_b);
        uint4 *Oa = static_cast<uint4*>(Af), *Ob = static_cast<uint4*>(Bf);
#define FTNN_EXP2(F4_, TA_, TB_) hipLaunchKernelGGL((k_expand2<F4_, TA_, TB_>), grid, dim3(256), 0, st, Ra, (int)M, Oa, Rb, KN, Ob, Kw / 4)
#define FTNN_EXP2T(F4_)                          \
    if (a_tern && b_tern) FTNN_EXP2(F4_, true, true);  \
    else if (a_tern) FTNN_EXP2(F4_, true, false);      \
    else if (b_tern) FTNN_EXP2(F4_, false, true);      \
    else FTNN_EXP2(F4_, false, false)
        if (f4) { FTNN_EXP2T(true); } else { FTNN_EXP2T(false); }
#undef FTNN_EXP2T
#undef FTNN_EXP2
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return launch_mfma_gemm(f4, type, Af, Bf, M, OHW, KN, Kw, K_unpack, alpha, d_y, st);
}

}  // namespace ftnn
