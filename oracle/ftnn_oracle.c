/*
 * ftnn_oracle.c -- TEST INFRASTRUCTURE ONLY.
 *
 * A scalar, plain-C restatement of the FasterTNN "final" (Packing 2) CPU path:
 * weight/operand packers, fused quantise + im2row + bit-pack for activations,
 * the four popcount GEMMs with fused PReLU, and the conv / gemm entry points.
 * It exists to check the HIP library; nothing in the shipped library links or
 * calls it.  Only the test-suite, the smoke check and the CPU-baseline leg of
 * the benchmark may load it.
 *
 * Every routine is written in "gather" form (one loop nest over the OUTPUT
 * words) from the index algebra of the reference, not from its control flow;
 * the reference's scatter loops and AVX2 lanes are not reproduced.  Each
 * routine names the reference lines whose behaviour it restates.
 *
 * Parity pins (all routines are pinned, none is "parity unpinned"):
 *   - byte-for-byte comparison with the compiled reference (oracle/_ref) over
 *     the reference's 12 self-test shapes x 4 network types, run in the build
 *     container, and committed as golden vectors under tests/golden/;
 *   - decode(packed) == quantise(x) brute force on small inputs;
 *   - GEMM == integer matrix product of the decoded {-1,0,+1} operands;
 *   - conv == fp32 direct convolution of the padded, quantised tensors
 *     (pad value 0 for ternary activations, +1 for binary ones), which is the
 *     reference's own self-test (src/timing_layers.c:142-165).
 *
 * All outputs go to caller-provided buffers so that the checker can be driven
 * from numpy through ctypes.
 */
#include <stdint.h>
#include <stddef.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

/* ---------------------------------------------------------------- shapes */

/* C_pack = ceil(C/64) (include/tnns/common.h:12, ternarize2row_avx2.c:722-723) */
static inline int cpack_of(int C) { return (C + 63) / 64; }
/* words per plane rounded up to a multiple of 4
 * (ternarize2row_avx2.c:730-732, mm_p2_final_tnn_avx2.c:385, utils.c:477) */
static inline int round4(int k) { return 4 * ((k + 3) / 4); }

/* OH = (H + 2p - KH)/s + 1, integer division (tnns_cpu_mm_p2.c:7-10) */
ORC_API int orc_out_dim(int in, int pad, int k, int stride)
{
    return (in + 2 * pad - k) / stride + 1;
}

/* number of int64 words per packed row: ternary rows carry two planes */
ORC_API int64_t orc_row_words(int C, int KH, int KW, int ternary)
{
    int64_t kw = round4(cpack_of(C) * KH * KW);
    return ternary ? 2 * kw : kw;
}

/* position of (plane, word idx) inside a Packing-2 ternary row: groups of four
 * sign words followed by their four zero words
 * (ternarize2row_avx2.c:464-469, utils.c:511-514) */
static inline int64_t p2_pos(int64_t idx, int plane)
{
    return (idx / 4) * 8 + (idx % 4) + (plane ? 4 : 0);
}

/* ------------------------------------------------------------ quantisers */

/* activation ternariser, strict compares, negative side tested first
 * (ternarize2row_avx2.c:443-449): returns sign bit in bit0, zero bit in bit1 */
static inline unsigned tern_act(float x, float t)
{
    if (x < -t) return 1u;      /* -1: sign=1 zero=0 */
    if (x > t)  return 0u;      /* +1: sign=0 zero=0 */
    return 2u;                  /*  0: sign=0 zero=1 */
}

/* weight ternariser, positive side tested first (utils.c:503-509) */
static inline unsigned tern_wgt(float x, float t)
{
    if (x > t)  return 0u;
    if (x < -t) return 1u;
    return 2u;
}

/* binariser: bit set (= -1) iff x < t (binarize2row_avx2.c:19-21, utils.c:657-659) */
static inline unsigned bin_bit(float x, float t) { return x < t ? 1u : 0u; }

/* ------------------------------------------------------- weight packers */

/*
 * Ternary weights, fp32 (KN,C,KH,KW) -> Packing 2 rows of 2*round4(KH*KW*C_pack)
 * words.  Restates ternarize_opt_avx2 (utils.c:468-521): channels past C read
 * as 0.0 and go through the same compares (utils.c:498-509); words past the
 * last real one keep the fill (sign 0, zero all-ones) (utils.c:483-490).
 */
ORC_API void orc_pack_weights_ternary(const float *w, const float *thr, int KN, int C,
                                      int KH, int KW, int64_t *out)
{
    const int cp = cpack_of(C);
    const int64_t kw = round4(KH * KW * cp);
    for (int n = 0; n < KN; n++) {
        int64_t *row = out + (int64_t)n * 2 * kw;
        for (int64_t i = 0; i < kw; i++) {
            row[p2_pos(i, 0)] = 0;
            row[p2_pos(i, 1)] = -1;
        }
        for (int h = 0; h < KH; h++)
            for (int x = 0; x < KW; x++)
                for (int ic = 0; ic < cp; ic++) {
                    uint64_t s = 0, z = 0;
                    for (int bit = 0; bit < 64; bit++) {
                        int c = ic * 64 + bit;
                        float v = c < C ? w[(((int64_t)n * C + c) * KH + h) * KW + x] : 0.0f;
                        unsigned q = tern_wgt(v, thr[n]);
                        s |= (uint64_t)(q & 1u) << bit;
                        z |= (uint64_t)(q >> 1) << bit;
                    }
                    int64_t idx = (int64_t)(h * KW + x) * cp + ic;
                    row[p2_pos(idx, 0)] = (int64_t)s;
                    row[p2_pos(idx, 1)] = (int64_t)z;
                }
    }
}

/*
 * Binary weights -> one plane, rows of round4(KH*KW*C_pack) words, tail bits
 * and pad words zero (= +1).  Restates binarize_opt_helper with packing 4
 * (utils.c:634-675).
 */
ORC_API void orc_pack_weights_binary(const float *w, const float *thr, int KN, int C,
                                     int KH, int KW, int64_t *out)
{
    const int cp = cpack_of(C);
    const int64_t kw = round4(KH * KW * cp);
    memset(out, 0, (size_t)KN * kw * sizeof(int64_t));
    for (int n = 0; n < KN; n++)
        for (int h = 0; h < KH; h++)
            for (int x = 0; x < KW; x++)
                for (int ic = 0; ic < cp; ic++) {
                    uint64_t s = 0;
                    for (int bit = 0; bit < 64 && ic * 64 + bit < C; bit++) {
                        int c = ic * 64 + bit;
                        float v = w[(((int64_t)n * C + c) * KH + h) * KW + x];
                        s |= (uint64_t)bin_bit(v, thr[n]) << bit;
                    }
                    out[(int64_t)n * kw + (int64_t)(h * KW + x) * cp + ic] = (int64_t)s;
                }
}

/*
 * GEMM operand packer: fp32 row-major [I][J] with values in {-1,0,+1} ->
 * Packing 2; -1 sets the sign bit, 0 sets the zero bit, anything else is +1.
 * J must be a multiple of 256.  Restates bitpacking2 (utils.c:257-291).
 * Returns -1 if J is not a multiple of 256 (the reference asserts).
 */
ORC_API int orc_pack_gemm_operand(const float *x, int I, int J, int64_t *out)
{
    if (J % 256 != 0) return -1;
    const int64_t kw = J / 64;
    for (int i = 0; i < I; i++)
        for (int64_t wd = 0; wd < kw; wd++) {
            uint64_t s = 0, z = 0;
            for (int bit = 0; bit < 64; bit++) {
                float v = x[(int64_t)i * J + wd * 64 + bit];
                if (v == -1.0f) s |= 1ull << bit;
                else if (v == 0.0f) z |= 1ull << bit;
            }
            out[(int64_t)i * 2 * kw + p2_pos(wd, 0)] = (int64_t)s;
            out[(int64_t)i * 2 * kw + p2_pos(wd, 1)] = (int64_t)z;
        }
    return 0;
}

/* ------------------------------------------ activations: quantise + im2row */

/*
 * Ternarise + im2row + Packing 2.  x is fp32 NCHW, thr[n] per batch item.
 * Row r = (n*OH + oh)*OW + ow; word idx = (kh*KW + kw)*C_pack + ic takes its
 * 64 channels from pixel (oh*s + kh - p, ow*s + kw - p).  Anything not backed
 * by a real (pixel, channel) is (sign 0, zero 1): border pixels, channels past
 * C, and words in [K, round4(K)).  Restates t2r_p2_opt
 * (ternarize2row_avx2.c:715-803) with its helpers :195-314, :316-371, :438-472.
 */
ORC_API void orc_t2r_p2(const float *x, const float *thr, int N, int C, int H, int W,
                        int H_pad, int W_pad, int KH, int KW, int H_stride, int W_stride,
                        int64_t *out)
{
    const int cp = cpack_of(C);
    const int OH = orc_out_dim(H, H_pad, KH, H_stride);
    const int OW = orc_out_dim(W, W_pad, KW, W_stride);
    const int64_t kw = round4(KH * KW * cp);
    for (int n = 0; n < N; n++)
        for (int oh = 0; oh < OH; oh++)
            for (int ow = 0; ow < OW; ow++) {
                int64_t *row = out + (((int64_t)n * OH + oh) * OW + ow) * 2 * kw;
                for (int64_t idx = 0; idx < kw; idx++) {
                    uint64_t s = 0, z = ~0ull;
                    if (idx < (int64_t)KH * KW * cp) {
                        int ic = (int)(idx % cp);
                        int tap = (int)(idx / cp);
                        int ih = oh * H_stride + tap / KW - H_pad;
                        int iw = ow * W_stride + tap % KW - W_pad;
                        if (ih >= 0 && ih < H && iw >= 0 && iw < W)
                            for (int bit = 0; bit < 64 && ic * 64 + bit < C; bit++) {
                                int c = ic * 64 + bit;
                                float v = x[(((int64_t)n * C + c) * H + ih) * W + iw];
                                unsigned q = tern_act(v, thr[n]);
                                s |= (uint64_t)(q & 1u) << bit;
                                if (!(q >> 1)) z &= ~(1ull << bit);
                            }
                    }
                    row[p2_pos(idx, 0)] = (int64_t)s;
                    row[p2_pos(idx, 1)] = (int64_t)z;
                }
            }
}

/*
 * Binarise + im2row, single plane, rows of round4(K) words, no interleave.
 * Border pixels, channels past C and pad words are 0 bits (= +1).  Restates
 * b2r (binarize2row_avx2.c:131-199) with helpers :15-36, :38-81, :83-129.
 */
ORC_API void orc_b2r(const float *x, const float *thr, int N, int C, int H, int W,
                     int H_pad, int W_pad, int KH, int KW, int H_stride, int W_stride,
                     int64_t *out)
{
    const int cp = cpack_of(C);
    const int OH = orc_out_dim(H, H_pad, KH, H_stride);
    const int OW = orc_out_dim(W, W_pad, KW, W_stride);
    const int64_t kw = round4(KH * KW * cp);
    for (int n = 0; n < N; n++)
        for (int oh = 0; oh < OH; oh++)
            for (int ow = 0; ow < OW; ow++) {
                int64_t *row = out + (((int64_t)n * OH + oh) * OW + ow) * kw;
                for (int64_t idx = 0; idx < kw; idx++) {
                    uint64_t s = 0;
                    if (idx < (int64_t)KH * KW * cp) {
                        int ic = (int)(idx % cp);
                        int tap = (int)(idx / cp);
                        int ih = oh * H_stride + tap / KW - H_pad;
                        int iw = ow * W_stride + tap % KW - W_pad;
                        if (ih >= 0 && ih < H && iw >= 0 && iw < W)
                            for (int bit = 0; bit < 64 && ic * 64 + bit < C; bit++) {
                                int c = ic * 64 + bit;
                                float v = x[(((int64_t)n * C + c) * H + ih) * W + iw];
                                s |= (uint64_t)bin_bit(v, thr[n]) << bit;
                            }
                    }
                    row[idx] = (int64_t)s;
                }
            }
}

/* -------------------------------------------------------------- GEMMs */

static inline int pc64(uint64_t v) { return __builtin_popcountll(v); }

/* output position of (row i, column j): NCHW with the image index taken from
 * the row (include/tnns/mm.h:30) */
static inline int64_t y_pos(int64_t i, int j, int64_t OHW, int KN)
{
    return ((i / OHW) * KN + j) * OHW + i % OHW;
}

/*
 * TNN: acc = 64*Kw - sum[ popc(za|zb) + 2*popc((sa^sb) & ~(za|zb)) ]
 * (mm_p2_final_tnn_avx2.c:72-87, :129-178); PReLU as "f=(float)acc; if (f<=0)
 * f*=alpha" (:204-208).  K is the un-rounded word count per plane (:385).
 * acc_out (optional) receives the raw int32 accumulators in the same layout.
 */
ORC_API void orc_mm_tnn(const int64_t *a, const int64_t *b, int N, int OH, int OW, int KN,
                        int K, float alpha, float *y, int32_t *acc_out)
{
    const int64_t kw = round4(K), M = (int64_t)N * OH * OW, OHW = (int64_t)OH * OW;
    for (int64_t i = 0; i < M; i++)
        for (int j = 0; j < KN; j++) {
            const int64_t *ar = a + i * 2 * kw, *br = b + (int64_t)j * 2 * kw;
            int64_t cnt = 0;
            for (int64_t k = 0; k < kw; k++) {
                uint64_t sa = ar[p2_pos(k, 0)], za = ar[p2_pos(k, 1)];
                uint64_t sb = br[p2_pos(k, 0)], zb = br[p2_pos(k, 1)];
                uint64_t z = za | zb;
                cnt += pc64(z) + 2 * pc64((sa ^ sb) & ~z);
            }
            int32_t acc = (int32_t)(64 * kw - cnt);
            float f = (float)acc;
            if (f <= 0) f *= alpha;
            y[y_pos(i, j, OHW, KN)] = f;
            if (acc_out) acc_out[y_pos(i, j, OHW, KN)] = acc;
        }
}

static inline float prelu_ge(int32_t r, float alpha)
{
    return r >= 0 ? (float)r : alpha * r;   /* mm_p2_final_tbn_avx2.c:73 */
}

/*
 * TBN: ternary A (two planes), binary B (one plane, row stride Kw).
 * nonzero_i = 64*Kw - sum popc(za); neg = sum popc((sa ^ b) & ~za);
 * r = nonzero - 2*neg (mm_p2_final_tbn_avx2.c:41-73).
 */
ORC_API void orc_mm_tbn(const int64_t *a, const int64_t *b, int N, int OH, int OW, int KN,
                        int K, float alpha, float *y, int32_t *acc_out)
{
    const int64_t kw = round4(K), M = (int64_t)N * OH * OW, OHW = (int64_t)OH * OW;
    for (int64_t i = 0; i < M; i++) {
        const int64_t *ar = a + i * 2 * kw;
        int64_t zero = 0;
        for (int64_t k = 0; k < kw; k++) zero += pc64((uint64_t)ar[p2_pos(k, 1)]);
        for (int j = 0; j < KN; j++) {
            const int64_t *br = b + (int64_t)j * kw;
            int64_t neg = 0;
            for (int64_t k = 0; k < kw; k++)
                neg += pc64(((uint64_t)ar[p2_pos(k, 0)] ^ (uint64_t)br[k]) &
                            ~(uint64_t)ar[p2_pos(k, 1)]);
            int32_t r = (int32_t)(64 * kw - zero - 2 * neg);
            y[y_pos(i, j, OHW, KN)] = prelu_ge(r, alpha);
            if (acc_out) acc_out[y_pos(i, j, OHW, KN)] = r;
        }
    }
}

/*
 * BTN: binary A (one plane), ternary B (two planes).
 * nonzero_j = 64*Kw - sum popc(zb); neg = sum popc((a ^ sb) & ~zb)
 * (mm_p2_final_btn_avx2.c:41-73).
 */
ORC_API void orc_mm_btn(const int64_t *a, const int64_t *b, int N, int OH, int OW, int KN,
                        int K, float alpha, float *y, int32_t *acc_out)
{
    const int64_t kw = round4(K), M = (int64_t)N * OH * OW, OHW = (int64_t)OH * OW;
    for (int j = 0; j < KN; j++) {
        const int64_t *br = b + (int64_t)j * 2 * kw;
        int64_t zero = 0;
        for (int64_t k = 0; k < kw; k++) zero += pc64((uint64_t)br[p2_pos(k, 1)]);
        for (int64_t i = 0; i < M; i++) {
            const int64_t *ar = a + i * kw;
            int64_t neg = 0;
            for (int64_t k = 0; k < kw; k++)
                neg += pc64(((uint64_t)ar[k] ^ (uint64_t)br[p2_pos(k, 0)]) &
                            ~(uint64_t)br[p2_pos(k, 1)]);
            int32_t r = (int32_t)(64 * kw - zero - 2 * neg);
            y[y_pos(i, j, OHW, KN)] = prelu_ge(r, alpha);
            if (acc_out) acc_out[y_pos(i, j, OHW, KN)] = r;
        }
    }
}

/*
 * BNN: both one plane; r = K_unpack - 2*sum popc(a ^ b) with K_unpack = C*KH*KW
 * (mm_p2_final_bnn_avx2.c:41-60).
 */
ORC_API void orc_mm_bnn(const int64_t *a, const int64_t *b, int N, int OH, int OW, int KN,
                        int K, int K_unpack, float alpha, float *y, int32_t *acc_out)
{
    const int64_t kw = round4(K), M = (int64_t)N * OH * OW, OHW = (int64_t)OH * OW;
    for (int64_t i = 0; i < M; i++)
        for (int j = 0; j < KN; j++) {
            int64_t neg = 0;
            for (int64_t k = 0; k < kw; k++)
                neg += pc64((uint64_t)a[i * kw + k] ^ (uint64_t)b[(int64_t)j * kw + k]);
            int32_t r = (int32_t)(K_unpack - 2 * neg);
            y[y_pos(i, j, OHW, KN)] = prelu_ge(r, alpha);
            if (acc_out) acc_out[y_pos(i, j, OHW, KN)] = r;
        }
}

/* ---------------------------------------------------- layer entry points */

/*
 * One conv layer, type 0=TNN 1=TBN 2=BTN 3=BNN (include/tnns/common.h:16):
 * quantise+im2row then GEMM+PReLU (tnns_cpu_mm_p2.c:6-80, dispatch :83-120).
 * scratch must hold N*OH*OW rows of orc_row_words(C,KH,KW, type<2) words.
 */
ORC_API void orc_tnns_conv(int type, const float *x, const float *thr, const int64_t *qw,
                           int N, int C, int H, int W, int KN, int KH, int KW,
                           int H_pad, int W_pad, int H_stride, int W_stride, float alpha,
                           int64_t *scratch, float *y)
{
    const int OH = orc_out_dim(H, H_pad, KH, H_stride);
    const int OW = orc_out_dim(W, W_pad, KW, W_stride);
    const int K = cpack_of(C) * KH * KW;
    if (type == 0 || type == 1)
        orc_t2r_p2(x, thr, N, C, H, W, H_pad, W_pad, KH, KW, H_stride, W_stride, scratch);
    else
        orc_b2r(x, thr, N, C, H, W, H_pad, W_pad, KH, KW, H_stride, W_stride, scratch);
    switch (type) {
    case 0: orc_mm_tnn(scratch, qw, N, OH, OW, KN, K, alpha, y, NULL); break;
    case 1: orc_mm_tbn(scratch, qw, N, OH, OW, KN, K, alpha, y, NULL); break;
    case 2: orc_mm_btn(scratch, qw, N, OH, OW, KN, K, alpha, y, NULL); break;
    default: orc_mm_bnn(scratch, qw, N, OH, OW, KN, K, C * KH * KW, alpha, y, NULL); break;
    }
}

/* tnns_gemm: TNN GEMM on pre-packed operands with alpha fixed to 1
 * (tnns_cpu_mm_p2.c:122-133) */
ORC_API void orc_tnns_gemm(const int64_t *xp, const int64_t *wp, int m, int n, int p_packed,
                           float *y)
{
    orc_mm_tnn(xp, wp, m, 1, 1, n, p_packed, 1.0f, y, NULL);
}
