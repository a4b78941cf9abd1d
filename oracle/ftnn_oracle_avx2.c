/*
 * ftnn_oracle_avx2.c -- TEST INFRASTRUCTURE ONLY.
 *
 * The TNN popcount GEMM of the FasterTNN "final" build restated with AVX2 intrinsics,
 * so that the benchmark has a CPU baseline of the reference's algorithmic cost on
 * machines where the compiled reference (oracle/_ref) is absent.  It follows the
 * structure of src/tnns/mm_p2_final_tnn_avx2.c: a block of 4 rows of A against one row
 * of B (:100-230, driven per 4 rows and 1 column by :364-382), one 256-bit step = 4 words
 * of both planes, the per-bit count "zero + 2 * negative" kept in carry-save form so that
 * each step costs ONE vector popcount (:44-53), and that popcount done with a nibble
 * look-up and a byte sum (:9-32).  Rows left over after the blocks of 4 run one at a time
 * (:55-97).  Results are the reference's bits: acc = 64*Kw - count, PReLU in the TNN form
 * "f = (float)acc; if (f <= 0) f *= alpha" (:204-208), stored at the NCHW position of
 * include/tnns/mm.h:30.
 *
 * Pinned by tests/test_oracle_avx2.py: bit-identical to the scalar restatement
 * (ftnn_oracle.c, itself pinned against the compiled reference and the golden vectors) on
 * seeded operands including row counts that are no multiple of 4, and to the compiled
 * reference where that is present.  The shipped library never links or calls it.
 */
#include <immintrin.h>
#include <stddef.h>
#include <stdint.h>

#define ORC_API __attribute__((visibility("default")))

/* population count of each 64-bit quarter of v: nibble table, then a byte sum */
static inline __m256i popcount_quarters(__m256i v)
{
    const __m256i table = _mm256_setr_epi8(0, 1, 1, 2, 1, 2, 2, 3, 1, 2, 2, 3, 2, 3, 3, 4,
                                           0, 1, 1, 2, 1, 2, 2, 3, 1, 2, 2, 3, 2, 3, 3, 4);
    const __m256i nib = _mm256_set1_epi8(0x0f);
    const __m256i lo = _mm256_shuffle_epi8(table, _mm256_and_si256(v, nib));
    const __m256i hi = _mm256_shuffle_epi8(table, _mm256_and_si256(_mm256_srli_epi16(v, 4), nib));
    return _mm256_sad_epu8(_mm256_add_epi8(lo, hi), _mm256_setzero_si256());
}

static inline int64_t sum_quarters(__m256i v)
{
    const __m128i s = _mm_add_epi64(_mm256_castsi256_si128(v), _mm256_extracti128_si256(v, 1));
    return _mm_cvtsi128_si64(s) + _mm_extract_epi64(s, 1);
}

/* One 256-bit step of one (row, column) pair.  Per bit position the step adds
 * zero + 2 * negative to the running count, where negative excludes zero.  `ones` carries the
 * weight-1 bits from step to step; what overflows out of it (ones & zero) and the negatives
 * both have weight 2 and can never coincide, so their OR is popcounted once. */
static inline void step(__m256i sa, __m256i za, __m256i sb, __m256i zb, __m256i *ones, __m256i *twos)
{
    const __m256i zero = _mm256_or_si256(za, zb);
    const __m256i neg = _mm256_andnot_si256(zero, _mm256_xor_si256(sa, sb));
    const __m256i weight2 = _mm256_or_si256(_mm256_and_si256(*ones, zero), neg);
    *ones = _mm256_xor_si256(*ones, zero);
    *twos = _mm256_add_epi64(*twos, popcount_quarters(weight2));
}

static inline int64_t y_pos(int64_t i, int j, int64_t OHW, int KN)
{
    return ((i / OHW) * KN + j) * OHW + i % OHW;
}

static inline float finish(int64_t kw, __m256i ones, __m256i twos, float alpha)
{
    const int64_t count = 2 * sum_quarters(twos) + sum_quarters(popcount_quarters(ones));
    float f = (float)(int32_t)(64 * kw - count);
    if (f <= 0) f *= alpha;
    return f;
}

/* a, b: Packing-2 rows of 2 * round4(K) words (groups of 4 sign words then their 4 zero
 * words), 32-byte aligned as the reference requires (:130-133).  y: fp32 (N, KN, OH, OW). */
ORC_API void orc_avx2_mm_tnn(const int64_t *a, const int64_t *b, int N, int OH, int OW, int KN, int K,
                             float alpha, float *y)
{
    const int64_t kw = 4 * (((int64_t)K + 3) / 4), row = 2 * kw;
    const int64_t M = (int64_t)N * OH * OW, OHW = (int64_t)OH * OW;
    int64_t i = 0;
    for (; i + 4 <= M; i += 4) {
        for (int j = 0; j < KN; j++) {
            const int64_t *br = b + (int64_t)j * row;
            __m256i ones[4], twos[4];
            for (int r = 0; r < 4; r++) ones[r] = twos[r] = _mm256_setzero_si256();
            for (int64_t k = 0; k < row; k += 8) {
                const __m256i sb = _mm256_load_si256((const __m256i *)(br + k));
                const __m256i zb = _mm256_load_si256((const __m256i *)(br + k + 4));
                for (int r = 0; r < 4; r++) {
                    const int64_t *ar = a + (i + r) * row + k;
                    step(_mm256_load_si256((const __m256i *)ar), _mm256_load_si256((const __m256i *)(ar + 4)), sb, zb,
                         &ones[r], &twos[r]);
                }
            }
            for (int r = 0; r < 4; r++) y[y_pos(i + r, j, OHW, KN)] = finish(kw, ones[r], twos[r], alpha);
        }
    }
    for (; i < M; i++) {
        for (int j = 0; j < KN; j++) {
            const int64_t *ar = a + i * row, *br = b + (int64_t)j * row;
            __m256i ones = _mm256_setzero_si256(), twos = _mm256_setzero_si256();
            for (int64_t k = 0; k < row; k += 8)
                step(_mm256_load_si256((const __m256i *)(ar + k)), _mm256_load_si256((const __m256i *)(ar + k + 4)),
                     _mm256_load_si256((const __m256i *)(br + k)), _mm256_load_si256((const __m256i *)(br + k + 4)),
                     &ones, &twos);
            y[y_pos(i, j, OHW, KN)] = finish(kw, ones, twos, alpha);
        }
    }
}
