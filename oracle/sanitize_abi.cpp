// sanitize_abi.cpp -- TEST INFRASTRUCTURE ONLY.
//
// The host side of the shipped library (argument checks, shape and size arithmetic, layer-chain validation) under
// AddressSanitizer and UndefinedBehaviorSanitizer: `make -C oracle sanitize` compiles ftnn_api.hip and ftnn_net.hip
// with host-only sanitizers into _san/libftnn_hip_san.so and links this driver against it.  Every call here is
// answered before any device work, so no GPU is needed; what the sanitizers watch is the 32/64-bit arithmetic on
// shapes at and beyond the documented limits.  Prints "sanitize abi ok".
#include <climits>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <initializer_list>

#include "../include/ftnn.h"

static int failures = 0;
#define EXPECT(cond)                                                   \
    do {                                                               \
        if (!(cond)) {                                                 \
            fprintf(stderr, "line %d: %s\n", __LINE__, #cond);         \
            failures++;                                                \
        }                                                              \
    } while (0)

int main() {
    alignas(16) static char buf[4096];
    void* p = buf;
    const int big[] = {1, 3, 63, 64, 65, 1 << 10, 1 << 16, 1 << 20, 1 << 24, (1 << 30) - 1, 1 << 30, INT_MAX};
    // size queries over the whole range of magnitudes: no overflow, refused shapes answer 0
    for (int c : big)
        for (int k : {1, 3, 7, 1 << 12, INT_MAX}) {
            (void)ftnn_row_words(c, k, k, 0);
            (void)ftnn_row_words(c, k, 1, 1);
            (void)ftnn_conv_weights_bytes(TNN, c, 64, k, k);
            for (int hw : {1, 7, 1 << 13, 1 << 20, INT_MAX})
                for (int n : {1, 8, 65535, 65536, INT_MAX}) {
                    for (int type = TNN; type <= BNN; type++) {
                        (void)ftnn_conv_scratch_bytes(type, n, c, hw, hw, 64, k, k, 1, 1, 1, 1);
                        (void)ftnn_conv_scratch_bytes(type, n, c, hw, 3, INT_MAX, k, k, INT_MAX / 2, 0, 2, INT_MAX);
                        (void)ftnn_select_conv_engine(type, n, c, hw, hw, 64, k, k, 1, 1, 1, 1);
                    }
                    (void)ftnn_pack_scratch_bytes(n, c, hw, hw, 1);
                    (void)ftnn_select_engine(TNN, n, hw, 1, c, k);
                    for (int e = FTNN_ENGINE_AUTO; e <= FTNN_ENGINE_MFMA_F4; e++) (void)ftnn_mm_scratch_bytes(e, TNN, n, hw, 1, c, k);
                    (void)ftnn_expand_bytes(FTNN_ENGINE_MFMA_F4, n, k);
                }
        }
    EXPECT(ftnn_out_dim(224, 3, 7, 2) == 112);
    EXPECT(ftnn_row_words(INT_MAX, 3, 3, 1) == 0);
    EXPECT(ftnn_conv_scratch_bytes(TNN, 1, 1, 8192, 8192, 1, 1, 1, 0, 0, 1, 1) == 0);
    // every entry point refuses bad arguments before it touches the device
    EXPECT(ftnn_mm(7, (const int64_t*)p, (const int64_t*)p, 1, 1, 1, 1, 4, 0, 0.5f, (float*)p, nullptr) == FTNN_EINVAL);
    EXPECT(ftnn_mm(TNN, (const int64_t*)p, (const int64_t*)p, INT_MAX, INT_MAX, 1, 1, 4, 0, 0.5f, (float*)p, nullptr) == FTNN_EINVAL);
    EXPECT(ftnn_mm(TNN, nullptr, (const int64_t*)p, 1, 1, 1, 1, 4, 0, 0.5f, (float*)p, nullptr) == FTNN_EINVAL);
    EXPECT(ftnn_mm_engine(9, TNN, (const int64_t*)p, (const int64_t*)p, 1, 1, 1, 1, 4, 0, 0.5f, (float*)p, p, 16, nullptr) == FTNN_EINVAL);
    EXPECT(ftnn_mm_engine(FTNN_ENGINE_MFMA_F4, TNN, (const int64_t*)p, (const int64_t*)p, 64, 1, 1, 64, 4, 0, 0.5f, (float*)p, p, 16,
                          nullptr) == FTNN_EINVAL);   // too little scratch
    EXPECT(ftnn_mm_expanded(FTNN_ENGINE_VALU, TNN, p, p, 1, 1, 1, 1, 4, 0, 0.5f, (float*)p, nullptr) == FTNN_EINVAL);
    EXPECT(ftnn_expand_rows(FTNN_ENGINE_MFMA_F4, 1, (const int64_t*)p, 0, 4, p, nullptr) == FTNN_EINVAL);
    EXPECT(ftnn_quantize_im2row(1, (const float*)p, (const float*)p, 1, 8, 2, 2, 0, 0, 3, 3, 1, 1, (int64_t*)p, p, nullptr) == FTNN_EINVAL);
    EXPECT(ftnn_conv(9, (const float*)p, (const float*)p, (const int64_t*)p, 1, 8, 4, 4, 4, 3, 3, 1, 1, 1, 1, 0.5f, p, (float*)p, nullptr) ==
           FTNN_EINVAL);
    EXPECT(ftnn_conv(TNN, (const float*)p, (const float*)p, (const int64_t*)p, 1, 8, 4, 4, 4, 3, 3, INT_MAX, 1, 1, 1, 0.5f, p, (float*)p,
                     nullptr) == FTNN_EINVAL);
    EXPECT(ftnn_conv_static(TNN, (const float*)p, (const float*)p, (const int64_t*)p, 64, 512, 56, 56, 512, 3, 3, 1, 1, 1, 1, 0.5f,
                            (float*)p, nullptr) == FTNN_EINVAL);   // beyond the fixed work space
    EXPECT(strstr(ftnn_last_error(), "ftnn_conv_static holds") != nullptr);
    EXPECT(ftnn_conv_prepared(TNN, (const float*)p, (const float*)p, p, 0, 8, 4, 4, 4, 3, 3, 1, 1, 1, 1, 0.5f, p, (float*)p, nullptr) ==
           FTNN_EINVAL);
    EXPECT(ftnn_conv_prepare_weights(TNN, (const int64_t*)p, INT_MAX, 4, 3, 3, p, nullptr) == FTNN_EINVAL);
    EXPECT(ftnn_pack_weights(1, (const float*)p, (const float*)p, 0, 8, 3, 3, (int64_t*)p, nullptr) == FTNN_EINVAL);
    EXPECT(ftnn_pack_gemm_operand((const float*)p, 4, 100, (int64_t*)p, nullptr) == FTNN_EINVAL);
    // layer chains: tables refused by validation alone
    ftnn_layer_t l[2] = {{TNN, 64, 8, 8, 64, 3, 3, 1, 1, 0.5f, 0.5f, (const int64_t*)p}, {TNN, 32, 8, 8, 64, 3, 3, 1, 1, 0.5f, 0.5f, (const int64_t*)p}};
    EXPECT(ftnn_net_create(1, 2, l) == nullptr);
    EXPECT(ftnn_net_create(70000, 1, l) == nullptr);
    EXPECT(ftnn_net_create_ex(1, 1, l, 6) == nullptr);
    l[0].pad = 1 << 30;
    EXPECT(ftnn_net_create(1, 1, l) == nullptr);
    l[0].pad = 1;
    l[0].C = INT_MAX;
    EXPECT(ftnn_net_create(1, 1, l) == nullptr);
    EXPECT(ftnn_net_create(0, 1, l) == nullptr);
    EXPECT(ftnn_net_create(1, 0, l) == nullptr);
    if (failures) {
        fprintf(stderr, "sanitize abi: %d check(s) failed\n", failures);
        return 1;
    }
    puts("sanitize abi ok");
    return 0;
}
