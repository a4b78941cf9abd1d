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
//     scalar loads (one s_load_dwordx16 per column and group) into SGPRs and
//     enters every vector op as its one scalar source: no LDS traffic, no VGPRs
//     and no vector instructions for B.  The load of column b+1 is issued before
//     the arithmetic of column b;
//   * A tiles are copied global -> registers -> LDS with coalesced 16-byte loads
//     (the loads of chunk c+1 are issued before the arithmetic of chunk c and
//     land in the other half of a double-buffered LDS tile: one barrier per
//     chunk); each lane reads its own rows back with 128-bit LDS reads; the row
//     stride is padded by 4 dwords so that the 8 lanes of a 128-byte LDS beat hit
//     distinct banks.
// A workgroup is 4 wavefronts sharing one A tile of 64*TM rows; wavefront w
// computes columns [w*TN, (w+1)*TN) of the workgroup's 4*TN columns.
#include <stdio.h>
#include <stdlib.h>

#include "ftnn_internal.h"

namespace ftnn {

namespace {

// acc += popcount(x): one v_bcnt_u32_b32 (popcount with accumulate).  Inline asm keeps
// the compiler from splitting the accumulation chain into partial sums plus adds.
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

// one group of a B row: 8 sign dwords (s0, s1) and, for ternary B, 8 zero dwords (z0, z1)
struct BGroup {
    uint4 s0, s1, z0, z1;
};

template <bool TERN>
__device__ __forceinline__ BGroup load_b(const uint32_t* bp) {
    const uint4* q = reinterpret_cast<const uint4*>(bp);
    BGroup r;
    r.s0 = q[0];
    r.s1 = q[1];
    if (TERN) {
        r.z0 = q[2];
        r.z1 = q[3];
    } else {
        r.z0 = r.z1 = make_uint4(0, 0, 0, 0);
    }
    return r;
}

// the arithmetic of one dword pair; SA/ZA are per-lane (VGPR), SB/ZB wave-uniform (SGPR)
template <int MODE>
__device__ __forceinline__ void step(uint32_t sa, uint32_t za, uint32_t sb, uint32_t zb, uint32_t& cz,
                                     uint32_t& cn) {
    if (MODE == kTNN) {
        const uint32_t z = za | zb;
        bcnt_acc(cz, z);
        bcnt_acc(cn, (sa ^ sb) & ~z);
    } else if (MODE == kTBN) {
        bcnt_acc(cn, (sa ^ sb) & ~za);
    } else if (MODE == kBTN) {
        bcnt_acc(cn, (sa ^ sb) & ~zb);
    } else {
        bcnt_acc(cn, sa ^ sb);
    }
}

template <int MODE>
__device__ __forceinline__ void step4(const uint4& sa, const uint4& za, const uint4& sb, const uint4& zb,
                                      uint32_t& cz, uint32_t& cn) {
    step<MODE>(sa.x, za.x, sb.x, zb.x, cz, cn);
    step<MODE>(sa.y, za.y, sb.y, zb.y, cz, cn);
    step<MODE>(sa.z, za.z, sb.z, zb.z, cz, cn);
    step<MODE>(sa.w, za.w, sb.w, zb.w, cz, cn);
}

__device__ __forceinline__ uint32_t popc4(const uint4& v) {
    return __popc(v.x) + __popc(v.y) + __popc(v.z) + __popc(v.w);
}

// IMPL = true: implicit im2row.  A is then not a matrix of packed rows but the channel-packed
// input P[n][pixel][ic] (one (sign, zero) pair of words, or one word for binary inputs, per
// pixel and 64 channels); the staging step gathers word idx = (kh*KW + kw)*C_pack + ic of row
// (n, oh, ow) from pixel (oh*s + kh - p, ow*s + kw - p) and applies the reference's fill rules
// (src/tnns/ternarize2row_avx2.c:438-472, :748-755; src/tnns/binarize2row_avx2.c:151), so the
// im2row matrix is never written to memory.
// TR = true stores the result transposed, Y[column * M + row] (row-major GEMM results only): the
// launcher uses it to run a BTN GEMM as a TBN GEMM with the operands exchanged, see launch_mm.
// KS = 4 or 8 splits K over the KS wavefronts of a workgroup, for problems whose tiles alone leave most of the chip
// idle (the reference's CPU-sized GEMM, 256 x 256 x 4096, is 128 workgroups of the smallest tile on 256 compute
// units): a chunk is GC = KS groups, wavefront w takes group w of every chunk for all TN columns of the workgroup
// (four times the workgroups of KS / 4 times the wavefronts, 1 / KS of the K loop each), and the partial counts meet
// in LDS at the end, where wavefront 0 finishes the tile.  Integer counts: any order of the sum is exact.
template <int MODE, int TM, int TN, int GC, bool IMPL, bool TR = false, int KS = 0>
__global__ __launch_bounds__(KS ? 64 * KS : 256) void k_mm(const uint32_t* __restrict__ A,
                                            const uint32_t* __restrict__ B,
                                            float* __restrict__ Y, int M, int KN, int OHW, int G,
                                            int K_unpack, float alpha, FastDiv dOHW, ConvGeom cg, QuantOut qo,
                                            int panel) {
    using T = Traits<MODE>;
    constexpr int BM = 64 * TM;
    constexpr int AG = T::kAGroup, BG = T::kBGroup;
    constexpr int LDW = GC * AG + 4;           // LDS row stride in dwords (padded)
    constexpr int QPR = GC * AG / 4;           // 16-byte quads per row and chunk
    constexpr int QUADS = BM * QPR;            // quads per chunk
    constexpr int NW = KS ? KS : 4, NT = 64 * NW;   // wavefronts and threads of a workgroup
    constexpr int IT = (QUADS + NT - 1) / NT;  // staging passes per thread
    constexpr int RPI = NT / QPR;              // rows covered by one staging pass
    static_assert(NT % QPR == 0, "a staging pass must cover whole rows");
    static_assert(!KS || (GC == KS && !IMPL), "the K split hands one group of a chunk to each wavefront");
    // counts a wavefront hands over under the K split: cn, and what the type has of cz, rowz, colz
    constexpr int NV = TM * TN * (MODE == kTNN ? 2 : 1) + (MODE == kTBN ? TM : 0) + (MODE == kBTN ? TN : 0);
    static_assert(!KS || (NW - 1) * NV * 64 <= 2 * BM * LDW, "the partial counts fit the operand buffers");
    __shared__ uint32_t lds[2][BM * LDW];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Tile of this workgroup.  Large grids are walked in panels of `panel` row tiles: workgroups are dealt to the
    // eight XCDs round-robin by their linear number, so within a panel an XCD keeps meeting the same panel / 8 row
    // tiles of A while the column tiles of B stream past -- its private L2 then fetches each A tile once per
    // round of resident workgroups instead of once per column tile.
    uint32_t bx = blockIdx.x, by = blockIdx.y;
    if (panel > 0) {
        const uint32_t gx = gridDim.x, gy = gridDim.y;
        const uint32_t lin = bx + gx * by, per = (uint32_t)panel * gy;
        const uint32_t p = lin / per, within = lin - p * per;
        const uint32_t pw = min((uint32_t)panel, gx - p * (uint32_t)panel);   // the last panel may be narrower
        by = within / pw;
        bx = p * (uint32_t)panel + (within - by * pw);
    }
    const int64_t row0 = (int64_t)bx * BM;
    const int col0 = KS ? (int)by * TN : (int)(by * 4 + wave) * TN;
    const size_t RDA = (size_t)G * AG, RDB = (size_t)G * BG;

    uint32_t cn[TM][TN];  // popcount of "negative product" lanes
    uint32_t cz[TM][TN];  // TNN only: popcount of "zero product" lanes
    uint32_t rowz[TM];    // TBN only: popcount of za per row
    uint32_t colz[TN];    // BTN only: popcount of zb per column (wave-uniform, scalar ALU)
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

    // columns past KN and rows past M are clamped for the loads and skipped at the store
    const uint32_t* bcol[TN];
#pragma unroll
    for (int b = 0; b < TN; b++) bcol[b] = B + (size_t)min(col0 + b, KN - 1) * RDB;

    // staging map (explicit rows): pass `it` of this thread moves quad sq of tile row sr + it*RPI
    const int sq = IMPL ? (tid & 3) : tid % QPR, sr = IMPL ? (tid >> 2) : tid / QPR;
    const bool stager = IMPL || (QUADS % NT == 0) || (tid < QUADS);
    const uint32_t* ap[IT];
    uint32_t* const lw = &lds[0][0] + sr * LDW + sq * (IMPL ? 2 : 4);
    uint4 stage[IT];
    // staging map (implicit im2row): thread = (word sq of the group, tile row sr + it*64)
    constexpr int ITI = IMPL ? TM : 1;
    int ih0[ITI], iw0[ITI];
    size_t pix0[ITI];
    ulonglong2 istage[ITI];
    static_assert(!IMPL || GC == 1, "implicit im2row stages one group per chunk");
    if (IMPL) {
#pragma unroll
        for (int it = 0; it < ITI; it++) {
            const uint32_t r = (uint32_t)min(row0 + sr + it * 64, (int64_t)M - 1);
            const uint32_t n = fastdiv(r, dOHW);
            const uint32_t pix = r - n * (uint32_t)OHW;
            const int oh = (int)fastdiv(pix, cg.dOW), ow = (int)pix - oh * cg.OW;
            ih0[it] = oh * cg.H_stride - cg.H_pad;
            iw0[it] = ow * cg.W_stride - cg.W_pad;
            pix0[it] = (size_t)n * cg.H * cg.W;
        }
    } else {
#pragma unroll
        for (int it = 0; it < IT; it++)
            ap[it] = A + (size_t)min(row0 + sr + it * RPI, (int64_t)M - 1) * RDA + sq * 4;
    }
    // word idx = 4*g + sq of the group being fetched, kept as (kh, kw, ic) and advanced by 4 words per
    // chunk without divisions (chunks are fetched in order, one group each)
    int f_ic = 0, f_kh = 0, f_kw = 0;
    if (IMPL) {
        const int tap = (int)fastdiv((uint32_t)sq, cg.dCP);
        f_ic = sq - tap * cg.CP;
        f_kh = (int)fastdiv((uint32_t)tap, cg.dKW);
        f_kw = tap - f_kh * cg.KW;
    }
    // issue the global loads of group-chunk starting at group g0 into the staging registers
    auto fetch = [&](int g0) {
        if (IMPL) {
            const bool valid = g0 * 4 + sq < cg.K;
            const int ic = f_ic, kh = f_kh, kw = f_kw;
            f_ic += 4;
            const int wraps = cg.CP >= 4 ? 1 : 4;   // uniform: one wrap suffices when C_pack >= 4
#pragma unroll
            for (int w = 0; w < 4; w++) {
                if (w < wraps && f_ic >= cg.CP) {
                    f_ic -= cg.CP;
                    if (++f_kw == cg.KW) {
                        f_kw = 0;
                        f_kh++;
                    }
                }
            }
#pragma unroll
            for (int it = 0; it < ITI; it++) {
                const int ih = ih0[it] + kh, iw = iw0[it] + kw;
                const bool in = valid && ih >= 0 && ih < cg.H && iw >= 0 && iw < cg.W;
                const size_t o = (pix0[it] + (size_t)(in ? ih * cg.W + iw : 0)) * cg.CP + (in ? ic : 0);
                if (T::kATern) {
                    istage[it] = in ? reinterpret_cast<const ulonglong2*>(A)[o] : make_ulonglong2(0ull, ~0ull);
                } else {
                    istage[it].x = in ? reinterpret_cast<const unsigned long long*>(A)[o] : 0ull;
                }
            }
        } else {
            const bool on = stager && sq < min(GC, G - g0) * (AG / 4);
#pragma unroll
            for (int it = 0; it < IT; it++)
                stage[it] = on ? *reinterpret_cast<const uint4*>(ap[it] + (size_t)g0 * AG) : make_uint4(0, 0, 0, 0);
        }
    };
    // write the staging registers into LDS buffer `buf`
    auto commit = [&](int buf) {
        uint32_t* l = lw + buf * (BM * LDW);
        if (IMPL) {
#pragma unroll
            for (int it = 0; it < ITI; it++) {
                *reinterpret_cast<unsigned long long*>(l + it * 64 * LDW) = istage[it].x;
                if (T::kATern) *reinterpret_cast<unsigned long long*>(l + it * 64 * LDW + 8) = istage[it].y;
            }
        } else if (stager) {
#pragma unroll
            for (int it = 0; it < IT; it++) *reinterpret_cast<uint4*>(l + it * RPI * LDW) = stage[it];
        }
    };

    const int nchunk = (G + GC - 1) / GC;
    fetch(0);
    commit(0);
    __syncthreads();

    for (int c = 0; c < nchunk; c++) {
        const int g0 = c * GC;
        const int gc = min(GC, G - g0);
        const bool more = c + 1 < nchunk;
        if (more) fetch(g0 + GC);  // the loads of the next chunk land after the arithmetic
        const uint32_t* lr = &lds[c & 1][0];
        // K split: this wavefront's group of the chunk, if the chunk has it (only the last chunk can be short)
        for (int g = KS ? wave : 0; g < (KS ? min(gc, wave + 1) : gc); g++) {
            uint4 sa0[TM], sa1[TM], za0[TM], za1[TM];
#pragma unroll
            for (int a = 0; a < TM; a++) {
                const uint4* lp = reinterpret_cast<const uint4*>(lr + (lane + 64 * a) * LDW + g * AG);
                sa0[a] = lp[0];
                sa1[a] = lp[1];
                if (T::kATern) {
                    za0[a] = lp[2];
                    za1[a] = lp[3];
                } else {
                    za0[a] = za1[a] = make_uint4(0, 0, 0, 0);
                }
            }
            // per-row zero count, src/tnns/mm_p2_final_tbn_avx2.c:44-52.  It depends on the row alone and the four
            // wavefronts of a workgroup hold the same rows: each counts every fourth group, the sums meet after the loop
            // (under the K split a wavefront's groups are its own anyway)
            if (MODE == kTBN && (KS || ((g0 + g) & 3) == wave)) {
#pragma unroll
                for (int a = 0; a < TM; a++) {
                    bcnt_acc(rowz[a], za0[a].x);
                    bcnt_acc(rowz[a], za0[a].y);
                    bcnt_acc(rowz[a], za0[a].z);
                    bcnt_acc(rowz[a], za0[a].w);
                    bcnt_acc(rowz[a], za1[a].x);
                    bcnt_acc(rowz[a], za1[a].y);
                    bcnt_acc(rowz[a], za1[a].z);
                    bcnt_acc(rowz[a], za1[a].w);
                }
            }
            const size_t goff = (size_t)(g0 + g) * BG;
            BGroup cur = load_b<T::kBTern>(bcol[0] + goff);
#pragma unroll
            for (int b = 0; b < TN; b++) {
                BGroup nxt = cur;
                if (b + 1 < TN) nxt = load_b<T::kBTern>(bcol[b + 1] + goff);
                // per-column zero count, src/tnns/mm_p2_final_btn_avx2.c:42-50
                if (MODE == kBTN) colz[b] += popc4(cur.z0) + popc4(cur.z1);
#pragma unroll
                for (int a = 0; a < TM; a++) {
                    step4<MODE>(sa0[a], za0[a], cur.s0, cur.z0, cz[a][b], cn[a][b]);
                    step4<MODE>(sa1[a], za1[a], cur.s1, cur.z1, cz[a][b], cn[a][b]);
                }
                cur = nxt;
            }
        }
        if (more) commit((c + 1) & 1);
        __syncthreads();
    }

    if constexpr (MODE == kTBN && !KS) {
        // the loop's last barrier has passed: the operand buffers are free for the four partial zero counts of each row
        static_assert(4 * BM <= 2 * BM * LDW, "the partial zero counts fit the operand buffers");
        uint32_t* red = &lds[0][0];
#pragma unroll
        for (int a = 0; a < TM; a++) red[wave * BM + lane + 64 * a] = rowz[a];
        __syncthreads();
#pragma unroll
        for (int a = 0; a < TM; a++) {
            rowz[a] = 0;
#pragma unroll
            for (int w = 0; w < 4; w++) rowz[a] += red[w * BM + lane + 64 * a];
        }
    }
    if constexpr (KS) {
        // the loop's last barrier has passed: the operand buffers are free for the partial counts [wavefront - 1][count][lane]
        uint32_t* red = &lds[0][0];
        auto each = [&](auto&& fn) {
            int v = 0;
#pragma unroll
            for (int a = 0; a < TM; a++)
#pragma unroll
                for (int b = 0; b < TN; b++) {
                    fn(cn[a][b], v++);
                    if (MODE == kTNN) fn(cz[a][b], v++);
                }
            if (MODE == kTBN) {
#pragma unroll
                for (int a = 0; a < TM; a++) fn(rowz[a], v++);
            }
            if (MODE == kBTN) {
#pragma unroll
                for (int b = 0; b < TN; b++) fn(colz[b], v++);
            }
        };
        if (wave != 0) each([&](uint32_t& c, int v) { red[((wave - 1) * NV + v) * 64 + lane] = c; });
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int w = 0; w < NW - 1; w++) each([&](uint32_t& c, int v) { c += red[(w * NV + v) * 64 + lane]; });
    }
    const int lanes_total = G * 4 * 64;  // 64 * Kw
    // PReLU in the reference's form for the type, from the integer accumulators of (row a, column b)
    auto finish = [&](int a, int b) -> float {
        if (MODE == kTNN) {
            // src/tnns/mm_p2_final_tnn_avx2.c:178,204-208
            const int acc = lanes_total - (int)(cz[a][b] + 2u * cn[a][b]);
            float f = (float)acc;
            if (f <= 0) f *= alpha;
            return f;
        }
        int r;
        if (MODE == kTBN) r = lanes_total - (int)rowz[a] - 2 * (int)cn[a][b];
        else if (MODE == kBTN) r = lanes_total - (int)colz[b] - 2 * (int)cn[a][b];
        else r = K_unpack - 2 * (int)cn[a][b];
        // src/tnns/mm_p2_final_tbn_avx2.c:72-73
        return r >= 0 ? (float)r : alpha * r;
    };
    // Row-major result (OHW == 1, the GEMM entry points): a lane's TN columns are contiguous, so they
    // leave as 16-byte stores (full 32-byte sectors) instead of TN scattered dwords.
    const bool vec = TN % 4 == 0 && OHW == 1 && (KN & 3) == 0 && col0 + TN <= KN &&
                     (reinterpret_cast<uintptr_t>(Y) & 15u) == 0;
#pragma unroll
    for (int a = 0; a < TM; a++) {
        const int64_t i = row0 + lane + 64 * a;
        if (i < M) {
            if (!TR && qo.mode != 0) {
                // hand-over to an fp4 layer: this lane's TN kernels are TN consecutive nibbles of one pixel
                const uint32_t img = fastdiv((uint32_t)i, dOHW);
                const uint32_t pix = (uint32_t)i - img * (uint32_t)OHW;
                const float t = qo.thr[img];
                uint32_t dw = 0u;
                const bool tern = qo.mode == 1;
                if (col0 + TN <= KN) {   // uniform: all of this wavefront's columns are real kernels
#pragma unroll
                    for (int b = 0; b < TN; b++) dw |= quant_nibble(finish(a, b), t, tern, true) << (4 * b);
                } else {
#pragma unroll
                    for (int b = 0; b < TN; b++) dw |= quant_nibble(finish(a, b), t, tern, col0 + b < KN) << (4 * b);
                }
                const size_t word = ((size_t)img * ((KN + 63) / 64) + (col0 >> 6)) * OHW + pix;
                unsigned char* dst = static_cast<unsigned char*>(qo.p4) + word * 32 + ((col0 & 63) >> 1);
                if (TN == 8) *reinterpret_cast<uint32_t*>(dst) = dw;
                else if (TN == 4) *reinterpret_cast<unsigned short*>(dst) = (unsigned short)dw;
                else *dst = (unsigned char)dw;
            } else if (TR) {   // consecutive lanes write consecutive floats of one output row
#pragma unroll
                for (int b = 0; b < TN; b++) {
                    const int j = col0 + b;
                    if (j < KN) Y[(size_t)j * M + i] = finish(a, b);
                }
            } else if (vec) {
                float* yr = Y + (size_t)i * KN + col0;
#pragma unroll
                for (int b4 = 0; b4 < TN / 4; b4++)
                    *reinterpret_cast<float4*>(yr + 4 * b4) =
                        make_float4(finish(a, 4 * b4), finish(a, 4 * b4 + 1), finish(a, 4 * b4 + 2),
                                    finish(a, 4 * b4 + 3));
            } else {
                const uint32_t img = fastdiv((uint32_t)i, dOHW);
                const uint32_t pix = (uint32_t)i - img * (uint32_t)OHW;
#pragma unroll
                for (int b = 0; b < TN; b++) {
                    const int j = col0 + b;
                    if (j < KN) Y[((size_t)img * KN + j) * OHW + pix] = finish(a, b);
                }
            }
        }
    }
}

template <int MODE, int TM, int TN, int GC, bool IMPL, bool TR, int KS = 0>
hipError_t launch_cfg(const uint32_t* A, const uint32_t* B, float* Y, int64_t M, int KN, int OHW,
                      int G, int K_unpack, float alpha, const ConvGeom& cg, hipStream_t st, const QuantOut& qo) {
    const int64_t gx = (M + 64 * TM - 1) / (64 * TM);
    // with a quantised hand-over every 64-channel word that holds a kernel is written in full
    const int cols = qo.mode != 0 ? (KN + 63) / 64 * 64 : KN;
    constexpr int WC = KS ? TN : 4 * TN;   // columns of a workgroup
    const int64_t gy = (cols + WC - 1) / WC;
    if (gx > 0x7fffffffLL || gy > 65535) return hipErrorInvalidValue;
    static const int tune_panel = getenv("FTNN_MM_PANEL") ? atoi(getenv("FTNN_MM_PANEL")) : 32;   // tuning aid
    const int panel = (gx >= 32 && gy >= 32 && gx * gy < 0x7fffffffLL) ? tune_panel : 0;
    hipLaunchKernelGGL((k_mm<MODE, TM, TN, GC, IMPL, TR, KS>), dim3((unsigned)gx, (unsigned)gy), dim3(KS ? 64 * KS : 256), 0, st,
                       A, B, Y, (int)M, KN, OHW, G, K_unpack, alpha, make_fastdiv((uint32_t)OHW), cg, qo, panel);
    return hipGetLastError();
}

template <int MODE, bool IMPL, bool TR = false>
hipError_t launch_mode(const uint32_t* A, const uint32_t* B, float* Y, int64_t M, int KN, int OHW,
                       int G, int K_unpack, float alpha, const ConvGeom& cg, hipStream_t st,
                       const QuantOut& qo = QuantOut()) {
    // Tile choice (measured on MI355X): 128 x 32 tiles once they give each of the 256 CUs
    // a dozen workgroups; layer-sized problems are one or two waves of workgroups, where
    // smaller tiles finish sooner.
    auto wgs = [&](int tm, int tn) {
        return ((M + 64 * tm - 1) / (64 * tm)) * ((KN + 4 * tn - 1) / (4 * tn));
    };
    static const char* force = getenv("FTNN_MM_TILE");   // tuning aid: "TM,TN" forces a tile
    if (force) {
        int tm = 0, tn = 0;
        sscanf(force, "%d,%d", &tm, &tn);
#define FTNN_TRY(TM_, TN_) \
    if (tm == TM_ && tn == TN_) return launch_cfg<MODE, TM_, TN_, 1, IMPL, TR>(A, B, Y, M, KN, OHW, G, K_unpack, alpha, cg, st, qo);
        FTNN_TRY(2, 8) FTNN_TRY(1, 8) FTNN_TRY(1, 4) FTNN_TRY(1, 2)
#undef FTNN_TRY
    }
    // Few tiles and a K loop worth splitting: the wavefronts of a workgroup share K (KS in the kernel).  Measured on
    // MI355X as device time per call with ten calls queued behind each other: 256 x 256 x 4096 8.7 -> 5.4 us (3.2 us is
    // what the smallest problem takes, 1.7 us the vector ALU's own time for this one), 128 x 1024 x 2048 5.6 -> 5.1,
    // 1024 x 128 x 8192 14 -> 9.5; from 512 x 512 x 4096 on the plain tiles are as fast.  FTNN_MM_KSPLIT = 0 switches
    // it off, "W,TN" forces W = 4 or 8 wavefronts on TN = 2 or 4 columns (tuning aid).
    if constexpr (!IMPL) {
        static const char* tune_ks = getenv("FTNN_MM_KSPLIT");
        int w = 0, tn = 0;
        if (tune_ks) sscanf(tune_ks, "%d,%d", &w, &tn);
        else if (!force && wgs(1, 2) <= 256 && G >= 4) w = G >= 8 ? 8 : 4, tn = ((M + 63) / 64) * ((KN + 3) / 4) < 256 ? 2 : 4;
        if (w && qo.mode == 0) {
#define FTNN_TRY(W_, TN_) \
    if (w == W_ && tn == TN_) return launch_cfg<MODE, 1, TN_, W_, false, TR, W_>(A, B, Y, M, KN, OHW, G, K_unpack, alpha, cg, st, qo);
            FTNN_TRY(4, 2) FTNN_TRY(4, 4) FTNN_TRY(8, 2) FTNN_TRY(8, 4)
#undef FTNN_TRY
        }
    }
    if (wgs(2, 8) >= 3072) return launch_cfg<MODE, 2, 8, 1, IMPL, TR>(A, B, Y, M, KN, OHW, G, K_unpack, alpha, cg, st, qo);
    if (wgs(1, 8) >= 1536) return launch_cfg<MODE, 1, 8, 1, IMPL, TR>(A, B, Y, M, KN, OHW, G, K_unpack, alpha, cg, st, qo);
    if (wgs(1, 4) >= 2048) return launch_cfg<MODE, 1, 4, 1, IMPL, TR>(A, B, Y, M, KN, OHW, G, K_unpack, alpha, cg, st, qo);
    return launch_cfg<MODE, 1, 2, 1, IMPL, TR>(A, B, Y, M, KN, OHW, G, K_unpack, alpha, cg, st, qo);
}

}  // namespace

hipError_t launch_mm(int type, const int64_t* d_a, const int64_t* d_b, int64_t M, int OHW, int KN,
                     int Kw, int K_unpack, float alpha, float* d_y, hipStream_t st, const QuantOut& qo) {
    const uint32_t* A = reinterpret_cast<const uint32_t*>(d_a);
    const uint32_t* B = reinterpret_cast<const uint32_t*>(d_b);
    const int G = Kw / 4;
    const ConvGeom cg = {};
    // A BTN product needs both planes of B next to a plane of A: (a ^ sb) & ~zb.  With B in scalar
    // registers that is two scalar operands in one vector instruction, which the ISA does not
    // encode, so the kernel pays a register copy per dword.  For a row-major result the same sums
    // come from the TBN form with the operands exchanged (ternary B along the lanes, binary A in
    // scalar registers) and the result stored transposed; both types share one PReLU form
    // (src/tnns/mm_p2_final_tbn_avx2.c:72-73, src/tnns/mm_p2_final_btn_avx2.c:72-73).
    if (type == kBTN && OHW == 1 && KN >= 64 && M <= 0x7fffffff && qo.mode == 0)
        return launch_mode<kTBN, false, true>(B, A, d_y, KN, (int)M, 1, G, K_unpack, alpha, cg, st, qo);
    switch (type) {
        case kTNN: return launch_mode<kTNN, false>(A, B, d_y, M, KN, OHW, G, K_unpack, alpha, cg, st, qo);
        case kTBN: return launch_mode<kTBN, false>(A, B, d_y, M, KN, OHW, G, K_unpack, alpha, cg, st, qo);
        case kBTN: return launch_mode<kBTN, false>(A, B, d_y, M, KN, OHW, G, K_unpack, alpha, cg, st, qo);
        case kBNN: return launch_mode<kBNN, false>(A, B, d_y, M, KN, OHW, G, K_unpack, alpha, cg, st, qo);
    }
    return hipErrorInvalidValue;
}

hipError_t launch_mm_implicit(int type, const void* d_p, const int64_t* d_b, const ConvGeom& cg, int N,
                              int KN, int K_unpack, float alpha, float* d_y, hipStream_t st, const QuantOut& qo) {
    const uint32_t* A = static_cast<const uint32_t*>(d_p);
    const uint32_t* B = reinterpret_cast<const uint32_t*>(d_b);
    const int OHW = cg.OH * cg.OW;
    const int64_t M = (int64_t)N * OHW;
    const int G = round4(cg.K) / 4;
    switch (type) {
        case kTNN: return launch_mode<kTNN, true>(A, B, d_y, M, KN, OHW, G, K_unpack, alpha, cg, st, qo);
        case kTBN: return launch_mode<kTBN, true>(A, B, d_y, M, KN, OHW, G, K_unpack, alpha, cg, st, qo);
        case kBTN: return launch_mode<kBTN, true>(A, B, d_y, M, KN, OHW, G, K_unpack, alpha, cg, st, qo);
        case kBNN: return launch_mode<kBNN, true>(A, B, d_y, M, KN, OHW, G, K_unpack, alpha, cg, st, qo);
    }
    return hipErrorInvalidValue;
}

}  // namespace ftnn
