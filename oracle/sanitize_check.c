/*
 * sanitize_check.c -- TEST INFRASTRUCTURE ONLY.
 *
 * Drives every routine of the checker (ftnn_oracle.c, ftnn_oracle_avx2.c) on small seeded layers with buffers of
 * exactly the documented sizes, so that a build with AddressSanitizer and UndefinedBehaviorSanitizer
 * (`make -C oracle sanitize`) reports any access outside them, signed overflow or misaligned access.  It also
 * cross-checks what the routines must agree on: the fused layer against quantise + im2row followed by the GEMM,
 * and the AVX2 GEMM against the scalar one.  Prints "sanitize ok" and returns 0 when nothing was found.
 */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

int orc_out_dim(int in, int pad, int k, int stride);
int64_t orc_row_words(int C, int KH, int KW, int ternary);
void orc_pack_weights_ternary(const float *w, const float *thr, int KN, int C, int KH, int KW, int64_t *out);
void orc_pack_weights_binary(const float *w, const float *thr, int KN, int C, int KH, int KW, int64_t *out);
int orc_pack_gemm_operand(const float *x, int I, int J, int64_t *out);
void orc_t2r_p2(const float *x, const float *thr, int N, int C, int H, int W, int H_pad, int W_pad, int KH, int KW,
                int H_stride, int W_stride, int64_t *out);
void orc_b2r(const float *x, const float *thr, int N, int C, int H, int W, int H_pad, int W_pad, int KH, int KW,
             int H_stride, int W_stride, int64_t *out);
void orc_mm_tnn(const int64_t *a, const int64_t *b, int N, int OH, int OW, int KN, int K, float alpha, float *y, int32_t *acc);
void orc_mm_tbn(const int64_t *a, const int64_t *b, int N, int OH, int OW, int KN, int K, float alpha, float *y, int32_t *acc);
void orc_mm_btn(const int64_t *a, const int64_t *b, int N, int OH, int OW, int KN, int K, float alpha, float *y, int32_t *acc);
void orc_mm_bnn(const int64_t *a, const int64_t *b, int N, int OH, int OW, int KN, int K, int K_unpack, float alpha, float *y,
                int32_t *acc);
void orc_tnns_conv(int type, const float *x, const float *thr, const int64_t *qw, int N, int C, int H, int W, int KN, int KH,
                   int KW, int H_pad, int W_pad, int H_stride, int W_stride, float alpha, int64_t *scratch, float *y);
void orc_tnns_gemm(const int64_t *xp, const int64_t *wp, int m, int n, int p_packed, float *y);
void orc_avx2_mm_tnn(const int64_t *a, const int64_t *b, int N, int OH, int OW, int KN, int K, float alpha, float *y);

static uint64_t state = 88172645463325252ull;
static uint32_t rnd(void)
{
    state ^= state << 13;
    state ^= state >> 7;
    state ^= state << 17;
    return (uint32_t)(state >> 11);
}

static void *exact(size_t bytes, size_t align)
{
    /* exactly `bytes` usable: one byte more is a reported overflow */
    void *p = NULL;
    if (posix_memalign(&p, align < sizeof(void *) ? sizeof(void *) : align, bytes ? bytes : 1) != 0) abort();
    return p;
}

static int check_layer(int type, const int shape[8], int batch)
{
    const int C = shape[0], H = shape[1], W = shape[2], KN = shape[3], KW = shape[4], KH = shape[5], pad = shape[6], s = shape[7];
    const int act_t = (type == 0 || type == 1), w_t = (type == 0 || type == 2);
    const int OH = orc_out_dim(H, pad, KH, s), OW = orc_out_dim(W, pad, KW, s);
    const size_t xe = (size_t)batch * C * H * W, we = (size_t)KN * C * KH * KW, ye = (size_t)batch * KN * OH * OW;
    float *x = exact(xe * 4, 32), *w = exact(we * 4, 32), *thr = exact((size_t)batch * 4, 4), *wthr = exact((size_t)KN * 4, 4);
    for (size_t i = 0; i < xe; i++) x[i] = (float)((int)(rnd() % 2001) - 1000) / 500.0f;
    for (size_t i = 0; i < we; i++) w[i] = w_t ? (float)((int)(rnd() % 3) - 1) : (float)(2 * (int)(rnd() % 2) - 1);
    for (int i = 0; i < batch; i++) thr[i] = act_t ? 0.5f + 0.125f * (float)(i % 3) : 0.25f * (float)(i % 3 - 1);
    for (int i = 0; i < KN; i++) wthr[i] = w_t ? 0.5f : 0.0f;
    const size_t qw_words = (size_t)KN * (size_t)orc_row_words(C, KH, KW, w_t);
    const size_t row_words = (size_t)batch * OH * OW * (size_t)orc_row_words(C, KH, KW, act_t);
    int64_t *qw = exact(qw_words * 8, 32), *rows = exact(row_words * 8, 32), *scratch = exact(row_words * 8, 32);
    float *y1 = exact(ye * 4, 4), *y2 = exact(ye * 4, 4);
    if (w_t) orc_pack_weights_ternary(w, wthr, KN, C, KH, KW, qw);
    else orc_pack_weights_binary(w, wthr, KN, C, KH, KW, qw);
    if (act_t) orc_t2r_p2(x, thr, batch, C, H, W, pad, pad, KH, KW, s, s, rows);
    else orc_b2r(x, thr, batch, C, H, W, pad, pad, KH, KW, s, s, rows);
    const int K = ((C + 63) / 64) * KH * KW;
    switch (type) {
        case 0: orc_mm_tnn(rows, qw, batch, OH, OW, KN, K, 0.5f, y1, NULL); break;
        case 1: orc_mm_tbn(rows, qw, batch, OH, OW, KN, K, 0.5f, y1, NULL); break;
        case 2: orc_mm_btn(rows, qw, batch, OH, OW, KN, K, 0.5f, y1, NULL); break;
        default: orc_mm_bnn(rows, qw, batch, OH, OW, KN, K, C * KH * KW, 0.5f, y1, NULL); break;
    }
    orc_tnns_conv(type, x, thr, qw, batch, C, H, W, KN, KH, KW, pad, pad, s, s, 0.5f, scratch, y2);
    int bad = memcmp(y1, y2, ye * 4) != 0;
    if (!bad && type == 0) {   /* the AVX2 GEMM on the same rows */
        orc_avx2_mm_tnn(rows, qw, batch, OH, OW, KN, K, 0.5f, y2);
        bad = memcmp(y1, y2, ye * 4) != 0;
    }
    if (bad) fprintf(stderr, "type %d shape C=%d %dx%d KN=%d %dx%d pad %d stride %d: results disagree\n", type, C, H, W, KN, KH, KW, pad, s);
    free(x); free(w); free(thr); free(wthr); free(qw); free(rows); free(scratch); free(y1); free(y2);
    return bad;
}

static int check_gemm(int m, int n, int p)
{
    const size_t xe = (size_t)m * p, we = (size_t)n * p;
    float *x = exact(xe * 4, 32), *w = exact(we * 4, 32);
    for (size_t i = 0; i < xe; i++) x[i] = (float)((int)(rnd() % 3) - 1);
    for (size_t i = 0; i < we; i++) w[i] = (float)((int)(rnd() % 3) - 1);
    int64_t *xp = exact(xe / 4, 32), *wp = exact(we / 4, 32);   /* 2 bits per value */
    float *y1 = exact((size_t)m * n * 4, 4), *y2 = exact((size_t)m * n * 4, 4);
    int bad = orc_pack_gemm_operand(x, m, p, xp) != 0 || orc_pack_gemm_operand(w, n, p, wp) != 0;
    if (!bad) {
        orc_tnns_gemm(xp, wp, m, n, p / 64, y1);
        orc_avx2_mm_tnn(xp, wp, m, 1, 1, n, p / 64, 1.0f, y2);
        bad = memcmp(y1, y2, (size_t)m * n * 4) != 0;
        /* against the plain product of the unpacked operands on one row */
        for (int j = 0; j < n && !bad; j++) {
            float acc = 0.0f;
            for (int k = 0; k < p; k++) acc += x[k] * w[(size_t)j * p + k];
            bad = acc != y1[j];
        }
    }
    if (bad) fprintf(stderr, "gemm %d x %d x %d: results disagree\n", m, n, p);
    bad = bad || orc_pack_gemm_operand(x, m, 100, xp) == 0;   /* J must be a multiple of 256 */
    free(x); free(w); free(xp); free(wp); free(y1); free(y2);
    return bad;
}

int main(void)
{
    /* C IH IW KN KW KH pad stride: tails below and above a 64-channel word, word counts that round up to 4,
     * non-square windows and inputs, strides, 1x1, a window as large as the padded input */
    static const int shapes[][8] = {
        {32, 7, 7, 32, 3, 3, 0, 1},   {127, 7, 7, 9, 3, 3, 1, 1}, {193, 6, 5, 7, 3, 3, 1, 2}, {64, 9, 4, 5, 3, 5, 1, 2},
        {257, 3, 3, 3, 3, 3, 1, 1},   {3, 12, 12, 6, 7, 7, 3, 2}, {70, 9, 5, 33, 2, 4, 2, 3}, {200, 1, 1, 10, 1, 1, 0, 1},
        {64, 4, 4, 7, 6, 6, 1, 1},    {1, 6, 6, 3, 3, 3, 1, 1},
    };
    int bad = 0;
    for (int type = 0; type < 4; type++)
        for (size_t s = 0; s < sizeof shapes / sizeof shapes[0]; s++)
            for (int batch = 1; batch <= 3; batch += 2) bad += check_layer(type, shapes[s], batch);
    bad += check_gemm(1, 1, 256) + check_gemm(5, 3, 512) + check_gemm(9, 16, 1024);
    if (bad) {
        fprintf(stderr, "sanitize check: %d case(s) failed\n", bad);
        return 1;
    }
    puts("sanitize ok");
    return 0;
}
