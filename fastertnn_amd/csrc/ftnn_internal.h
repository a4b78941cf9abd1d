// Internal declarations shared by the kernel files and the C-ABI layer.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ftnn {

constexpr int kTNN = 0, kTBN = 1, kBTN = 2, kBNN = 3;

inline int cpack_of(int C) { return (int)(((int64_t)C + 63) / 64); }
inline int round4(int k) { return 4 * ((k + 3) / 4); }
inline int out_dim(int in, int pad, int k, int stride) { return (in + 2 * pad - k) / stride + 1; }

// Division of a 32-bit unsigned n by a fixed d without the ~25-instruction expansion of "/":
// m = floor(2^32 / d) (saturated for d = 1) under-estimates the quotient by at most one, which one
// compare fixes.  Exact for every n < 2^32, d >= 1.
struct FastDiv {
    uint32_t d, m;
};
inline FastDiv make_fastdiv(uint32_t d) {
    FastDiv f;
    f.d = d;
    f.m = d <= 1 ? 0xffffffffu : (uint32_t)((1ull << 32) / d);
    return f;
}
__device__ __forceinline__ uint32_t fastdiv(uint32_t n, const FastDiv& f) {
    uint32_t q = __umulhi(n, f.m);
    if (n - q * f.d >= f.d) q++;
    return q;
}

// geometry of one conv layer as the implicit-im2row GEMM needs it
struct ConvGeom {
    int H, W, CP, OH, OW, KW, K;   // K = C_pack*KH*KW words per plane before rounding
    int H_pad, W_pad, H_stride, W_stride;
    FastDiv dOW, dCP, dKW;
};

// Fused hand-over to a following fp4 layer: instead of the fp32 result, a GEMM kernel writes the
// next layer's quantised input, P4[n][ceil(KN/64)][pixel][32 bytes] (see launch_quantize_f4), from
// the same fp32 values: mode 1 = ternary with thr[n] (strict compares), 2 = binary, 0 = off.
// Kernels past KN in the last 64-channel word get the padding nibble.
struct QuantOut {
    void* p4 = nullptr;
    const float* thr = nullptr;   // one threshold per batch item of the next layer
    int mode = 0;
};

// the E2M1 nibble of one value under QuantOut mode 1 / 2 (src/tnns/ternarize2row_avx2.c:443-449,
// src/tnns/binarize2row_avx2.c:19-21); `live` = false gives the padding lane of that mode
__device__ __forceinline__ uint32_t quant_nibble(float v, float t, bool ternary, bool live) {
    // selects only: a branch per element costs more than the whole computation
    uint32_t r;
    if (ternary) {
        r = v > t ? 0x2u : 0x0u;
        r = v < -t ? 0xAu : r;
        r = live ? r : 0x0u;
    } else {
        r = v < t ? 0xAu : 0x2u;
        r = live ? r : 0x2u;
    }
    return r;
}

// The ternary hand-over without compares, for the slopes and thresholds layers use (anything else takes
// quant_nibble on the PReLU result).  Both PReLU forms leave r > 0 as it is and turn r <= 0 into r * alpha <= 0, so
// for alpha >= 0 and t >= 0: PReLU(r) > t <=> r > t, and PReLU(r) < -t <=> r * alpha < -t (r * alpha is the very
// product PReLU forms; for r > 0 it is >= 0 >= -t).  r is an integer: with 2^-20 <= alpha <= 2^20 (or alpha = 0) and
// t <= 2^40, a difference r - t or -(r * alpha) - t that is positive is at least 2^-44, so 2^60 times it clamps to
// exactly 1, and one that is not positive clamps to +0.  The result is +1, -1 or +0 as a float, which
// v_cvt_scalef32_pk_fp4_f32 turns into the E2M1 nibbles 0x2, 0xA, 0x0, two values per instruction.
__device__ __forceinline__ bool tern_direct_applies(float alpha, float t) {
    return (alpha == 0.0f || (alpha >= 0x1p-20f && alpha <= 0x1p20f)) && t >= 0.0f && t <= 0x1p40f;
}
__device__ __forceinline__ float tern_value_direct(float r, float alpha, float t_big /* t * 2^60 */) {
    const float pos = __builtin_amdgcn_fmed3f(__builtin_fmaf(r, 0x1p60f, -t_big), 0.0f, 1.0f);
    const float neg = __builtin_amdgcn_fmed3f(__builtin_fmaf(r * alpha, -0x1p60f, -t_big), 0.0f, 1.0f);
    return pos - neg;
}
// The binary hand-over the same way: the bit is PReLU(r) < t.  For t > 0 that is r < t (r <= 0 gives PReLU <= 0 < t),
// for t <= 0 it is r * alpha < t (r >= 0 gives PReLU >= 0 >= t).  With alpha = 0 or 2^-20 <= alpha <= 2^20 and t = 0
// or 2^-20 <= |t| <= 2^40 a positive difference t - v is at least 2^-44; the result is -1 (bit set) or +1 as a float.
// `t_pos` must be the same for all lanes of the wavefront.
__device__ __forceinline__ bool bin_direct_applies(float alpha, float t) {
    const float at = __builtin_fabsf(t);
    return (alpha == 0.0f || (alpha >= 0x1p-20f && alpha <= 0x1p20f)) && (t == 0.0f || (at >= 0x1p-20f && at <= 0x1p40f));
}
__device__ __forceinline__ float bin_value_direct(float r, float alpha, float t_big /* t * 2^60 */, bool t_pos) {
    const float v = t_pos ? r : r * alpha;
    const float below = __builtin_amdgcn_fmed3f(__builtin_fmaf(v, -0x1p60f, t_big), 0.0f, 1.0f);
    return __builtin_fmaf(below, -2.0f, 1.0f);
}
// Both hand-overs behind one face: whether the wavefront may take the compare-free form for its thresholds
// (mode 1 ternary, 2 binary; for binary all thresholds must lie on the same side of zero), and the value.
struct DirectQuant {
    bool ok, t_pos;
};
template <int QMODE>
__device__ __forceinline__ DirectQuant direct_quant(float alpha, float t) {
    DirectQuant d = {false, false};
    if constexpr (QMODE == 1) {
        d.ok = __all(tern_direct_applies(alpha, t)) != 0;
    } else if constexpr (QMODE == 2) {
        const bool fits = bin_direct_applies(alpha, t);
        d.t_pos = __all(fits && t > 0.0f) != 0;
        d.ok = d.t_pos || __all(fits && !(t > 0.0f)) != 0;
    }
    return d;
}
template <int QMODE>
__device__ __forceinline__ float direct_value(float r, float alpha, float t_big, bool t_pos, bool live) {
    if constexpr (QMODE == 1) return live ? tern_value_direct(r, alpha, t_big) : 0.0f;
    else return live ? bin_value_direct(r, alpha, t_big, t_pos) : 1.0f;   // padding lanes: 0 / +1
}
// eight values out of {+1, -1, +0} -> one dword of E2M1 nibbles, value k in nibble k
__device__ __forceinline__ uint32_t pack_fp4x8(float z0, float z1, float z2, float z3, float z4, float z5, float z6,
                                               float z7) {
    uint32_t d = 0u;
    d = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(d, z0, z1, 1.0f, 0);
    d = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(d, z2, z3, 1.0f, 1);
    d = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(d, z4, z5, 1.0f, 2);
    d = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(d, z6, z7, 1.0f, 3);
    return d;
}

// Hand-over store of one 32-kernel block: lanes l and l ^ 32 hold the nibbles of one pixel, lane half h those of
// kernels 8 q + 4 h + {0..3}, as d0 (q = 0, 1) and d1 (q = 2, 3), 16 bits per q.  Returns the 8 bytes lane h
// stores at byte 8 h of the block's 16: kernels in order.  v_permlane32_swap exchanges the upper half of d0 with the
// lower half of d1, after which both lane halves combine their pair the same way.
__device__ __forceinline__ uint2 exchange_halves(uint32_t d0, uint32_t d1) {
    const auto r = __builtin_amdgcn_permlane32_swap(d0, d1, false, false);
    // lanes 0..31: r[0] = own d0, r[1] = d0 of lane + 32; lanes 32..63: r[0] = d1 of lane - 32, r[1] = own d1
    uint2 out;
    out.x = (r[0] & 0xffffu) | (r[1] << 16);
    out.y = (r[0] >> 16) | (r[1] & 0xffff0000u);
    return out;
}

// PReLU in the reference's two forms: "f <= 0 -> f *= alpha" (TNN, src/tnns/mm_p2_final_tnn_avx2.c:204-208; a zero
// becomes 0 * alpha) and "r >= 0 ? r : alpha * r" (the others, src/tnns/mm_p2_final_tbn_avx2.c:73)
template <bool FORM0>
__device__ __forceinline__ float prelu_ref(float r, float alpha) {
    const bool scale = FORM0 ? (r <= 0.0f) : (r < 0.0f);
    return scale ? r * alpha : r;
}

// One 32-kernel block of a pixel under the hand-over.  r[e] = this lane's 16 results before PReLU, kernel
// kbase + 8 (e / 4) + 4 h + e % 4 (h = lane half); t = the next layer's threshold for the pixel's image; dq from
// direct_quant.  Returns the 8 bytes this lane stores at byte 8 h of the block's 16.  Every lane of the wavefront
// must call it (exchange_halves crosses lanes).
template <bool FORM0, int QMODE>
__device__ __forceinline__ uint2 hand_over_block(const float (&r)[16], float alpha, float t, const DirectQuant& dq,
                                                 int kbase, int h, int KN) {
    const bool whole = kbase + 32 <= KN;   // wave-uniform: the block holds real kernels only
    uint32_t d0, d1;
    if (dq.ok) {
        // no compares, two nibbles per conversion (see tern_value_direct)
        const float t_big = t * 0x1p60f;
        float z[16];
        if (whole) {
#pragma unroll
            for (int e = 0; e < 16; e++) z[e] = direct_value<QMODE>(r[e], alpha, t_big, dq.t_pos, true);
        } else {   // kernels past KN hold the padding lane
#pragma unroll
            for (int e = 0; e < 16; e++)
                z[e] = direct_value<QMODE>(r[e], alpha, t_big, dq.t_pos, kbase + 8 * (e >> 2) + 4 * h + (e & 3) < KN);
        }
        d0 = pack_fp4x8(z[0], z[1], z[2], z[3], z[4], z[5], z[6], z[7]);
        d1 = pack_fp4x8(z[8], z[9], z[10], z[11], z[12], z[13], z[14], z[15]);
    } else {
        constexpr bool tern = QMODE == 1;
        uint32_t half[4];
        if (whole) {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                half[g] = 0u;
#pragma unroll
                for (int i = 0; i < 4; i++)
                    half[g] |= quant_nibble(prelu_ref<FORM0>(r[4 * g + i], alpha), t, tern, true) << (4 * i);
            }
        } else {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                half[g] = 0u;
#pragma unroll
                for (int i = 0; i < 4; i++)
                    half[g] |= quant_nibble(prelu_ref<FORM0>(r[4 * g + i], alpha), t, tern, kbase + 8 * g + 4 * h + i < KN)
                               << (4 * i);
            }
        }
        d0 = half[0] | (half[1] << 16);
        d1 = half[2] | (half[3] << 16);
    }
    return exchange_halves(d0, d1);
}

// record a failure text for ftnn_last_error(); returns `code`
int fail(int code, const char* fmt, ...);

// shape and size-limit validation shared by every layer entry point; fills OH / OW; FTNN_OK or a recorded failure
int check_conv_shape(int N, int C, int H, int W, int H_pad, int W_pad, int kH, int kW, int H_stride, int W_stride,
                     int* OH, int* OW);

// ---- pack_kernels.hip: launchers (arguments already validated) ----
hipError_t launch_quantize_im2row(bool ternary, const float* d_x, const float* d_thr, int N, int C,
                                  int H, int W, int H_pad, int W_pad, int kH, int kW, int H_stride,
                                  int W_stride, int64_t* d_out, void* d_scratch, hipStream_t st);
hipError_t launch_pack_weights(bool ternary, const float* d_w, const float* d_thr, int KN, int C,
                               int KH, int KW, int64_t* d_out, hipStream_t st);
hipError_t launch_pack_gemm_operand(const float* d_x, int I, int J, int64_t* d_out, hipStream_t st);

// ---- mm_kernels.hip ----
hipError_t launch_mm(int type, const int64_t* d_a, const int64_t* d_b, int64_t M, int OHW, int KN,
                     int Kw /* words per plane, multiple of 4 */, int K_unpack, float alpha,
                     float* d_y, hipStream_t st, const QuantOut& qo = QuantOut());

// GEMM straight from the channel-packed input P (no im2row matrix in memory)
hipError_t launch_mm_implicit(int type, const void* d_p, const int64_t* d_b, const ConvGeom& cg, int N,
                              int KN, int K_unpack, float alpha, float* d_y, hipStream_t st,
                              const QuantOut& qo = QuantOut());
// quantise only: fp32 NCHW -> P
hipError_t launch_quantize(bool ternary, const float* d_x, const float* d_thr, int N, int C, int H, int W,
                           void* d_p, hipStream_t st);

// quantise only, into fp4 nibbles: fp32 NCHW -> P4[n][C_pack][pixel][32 bytes] (operand of launch_conv_f4)
hipError_t launch_quantize_f4(bool ternary, const float* d_x, const float* d_thr, int N, int C, int H, int W,
                              void* d_p4, hipStream_t st);

// dense re-packing of both operands for layers with C <= 32 (several taps per 64-lane word)
bool dense_applies(int C, int KH, int KW, int* T_out, int* Kd_out);
hipError_t launch_dense_rows(bool ternary, const void* d_p, int N, int C, int H, int W, int H_pad, int W_pad,
                             int kH, int kW, int H_stride, int W_stride, int64_t* d_out, hipStream_t st);
hipError_t launch_dense_weights(bool ternary, const int64_t* d_qw, int KN, int C, int kH, int kW,
                                int64_t* d_out, hipStream_t st);

// the same for the fp4 layer kernel (C <= 8): quantise to one nibble dword per pixel (d_pq,
// dense_f4_pq_bytes), then string T taps per 64-lane word into A4[n][Kd][output pixel][32 bytes] (d_a4), the
// operand of launch_conv_f4 for a 1x1 layer with C_pack = Kd over the OH x OW output pixels
bool dense_f4_applies(int C, int KH, int KW);
// stem_kernels.hip: the same layer in one kernel (fp32 input -> result, the rows never stored) where its input
// patch fits the LDS: bytes of LDS it needs, 0 = does not apply
int64_t stem_f4_lds_bytes(int C, int KH, int KW, int H_stride, int W_stride);
hipError_t launch_stem_f4(int type, const float* d_x, const float* d_thr, const void* d_wf, int N, int C, int H,
                          int W, int KN, int KH, int KW, int H_pad, int W_pad, int H_stride, int W_stride,
                          float alpha, float* d_y, hipStream_t st, const QuantOut& qo);
int64_t dense_f4_pq_bytes(int N, int H, int W);
hipError_t launch_dense_rows_f4(bool ternary, const float* d_x, const float* d_thr, int N, int C, int H, int W,
                                int H_pad, int W_pad, int kH, int kW, int H_stride, int W_stride, void* d_pq,
                                void* d_a4, hipStream_t st);

// ---- mfma_kernels.hip: matrix-core formulation (int8 or fp4 operands expanded into d_scratch) ----
int64_t mfma_fragment_bytes(bool f4, int64_t rows, int Kw);
hipError_t launch_mfma_expand(bool f4, bool ternary, const int64_t* d_rows, int rows, int Kw, void* d_out,
                              hipStream_t st);
hipError_t launch_mfma_gemm(bool f4, int type, const void* d_af, const void* d_bf, int64_t M, int OHW, int KN,
                            int Kw, int K_unpack, float alpha, float* d_y, hipStream_t st);
// the fp4 GEMM's own operand form, two bits per lane ("packed4"): what ftnn_expand_rows / ftnn_mm_expanded /
// ftnn_mm_engine use for FTNN_ENGINE_MFMA_F4 (the layer kernels keep the plain fragments above)
int64_t mfma_packed4_bytes(int64_t rows, int Kw);
hipError_t launch_mfma_pack4(bool ternary, const int64_t* d_rows, int rows, int Kw, void* d_out, hipStream_t st);
hipError_t launch_mfma_gemm_packed4(int type, const void* d_ac, const void* d_bc, int64_t M, int OHW, int KN, int Kw, int K_unpack,
                                    float alpha, float* d_y, hipStream_t st);
// scratch of launch_mm_mfma on the fp4 engine (it picks the operand form by shape)
int64_t mfma_f4_mm_scratch_bytes(int64_t M, int KN, int Kw);
hipError_t launch_mm_mfma(bool f4, int type, const int64_t* d_a, const int64_t* d_b, int64_t M, int OHW,
                          int KN, int Kw, int K_unpack, float alpha, float* d_y, void* d_scratch,
                          hipStream_t st);

// conv layer on the fp4 matrix cores: activations from launch_quantize_f4, weights as the fp4 fragments
// launch_mfma_expand(true, ...) makes of the packed weight rows (Kw = round4(cg.K) words per row)
hipError_t launch_conv_f4(int type, const void* d_p4, const void* d_wf, const ConvGeom& cg, int N, int KN,
                          int K_unpack, float alpha, float* d_y, hipStream_t st, const QuantOut& qo = QuantOut());


// the same layer as workgroup tiles of 128 x 128 or 256 x 256 staged through LDS (the GEMM kernel with its activation
// fragments gathered from T4, the quantised input in the layout of launch_quantize_f4_tiled): for layers with
// conv_f4_tile_route() and an fp32 result
int64_t quantize_f4_tiled_bytes(int N, int C, int H, int W, int W_stride);
hipError_t launch_quantize_f4_tiled(bool ternary, const float* d_x, const float* d_thr, int N, int C, int H, int W,
                                    int W_stride, void* d_t4, hipStream_t st);
bool conv_f4_tile_route(int64_t M, int KN, int CP, int taps, int64_t t4_bytes, int W_pad, int W_stride);
hipError_t launch_conv_f4_tiles(int type, const void* d_p4, const void* d_wf, const ConvGeom& cg, int N, int KN,
                                int K_unpack, float alpha, float* d_y, hipStream_t st);

// ---- ftnn_api.hip ----  (arguments already validated)
// The fp4 layer with weights expanded beforehand (d_wf: launch_mfma_expand(true, ...) of the packed rows).
// d_x != null: the input is quantised into d_p4 (N*H*W*C_pack*32 bytes) first; d_x == null: d_p4 already
// holds it (written by the previous layer through its QuantOut).  qo.mode != 0: d_y is not written.
int conv_f4_expanded(int type, const float* d_x, const float* d_thr, const void* d_wf, int N, int C, int H,
                     int W, int KN, int KH, int KW, int H_pad, int W_pad, int H_stride, int W_stride,
                     float prelu_alpha, void* d_p4, float* d_y, hipStream_t st, const QuantOut& qo);
// the vector-ALU layer; d_scratch as for ftnn_conv
// (weights_prepared: for a few-channel layer d_qw already holds the re-packed rows of launch_dense_weights)
int conv_valu(int type, const float* d_x, const float* d_thr, const int64_t* d_qw, int N, int C, int H, int W,
              int KN, int KH, int KW, int H_pad, int W_pad, int H_stride, int W_stride, float prelu_alpha,
              void* d_scratch, float* d_y, hipStream_t st, const QuantOut& qo, bool weights_prepared);
// bytes of the fp4 layer's operand region (d_p4 above) for this shape, rounded up to 256: P4, or for a
// few-channel layer the nibble pixels and dense rows
int64_t conv_f4_operand_bytes(int N, int C, int H, int W, int KH, int KW, int OH, int OW, int KN, int W_stride);
// words per row of the weights as the fp4 layer reads them (the dense re-packing shortens them)
int conv_f4_weight_words(int C, int KH, int KW);

}  // namespace ftnn
