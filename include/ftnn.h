/*
 * ftnn.h -- C ABI of libftnn_hip.so, the MI355X (gfx950) implementation of the
 * FasterTNN ternary/binary inference hot path.
 *
 * Two layers:
 *
 *  1. The reference's own entry points, same names, argument meaning, struct
 *     layout and ownership rules, so that the reference's layer drivers link
 *     against this library instead of its tnns_cpu_mm_p2.o / mm_p2_final_*.o /
 *     ternarize2row_*.o / binarize2row_*.o objects.  They take and return host
 *     memory; every returned buffer is ordinary heap memory that the caller
 *     free()s.  Failure handling follows the reference: a message on stderr and
 *     abort().
 *
 *  2. ftnn_* entry points that work on device memory and a caller-supplied HIP
 *     stream (passed as void*, 0 = the null stream).  They return 0 on success
 *     and a negative FTNN_E* code otherwise; ftnn_last_error() gives the text.
 *     They never synchronise the stream.
 *
 * Paths in the comments are relative to the reference tree.
 */
#ifndef FTNN_H
#define FTNN_H

#include <stdint.h>

/* symbols exported by the shared library */
#define FTNN_API __attribute__((visibility("default")))

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ types */

/* include/tnns/common.h:16 */
enum tnns_type { TNN, TBN, BTN, BNN };

/* include/tnns/data.h:4-25 (112 bytes on LP64; field order is part of the ABI) */
typedef struct testcase {
    enum tnns_type type;
    int batchcount;
    int channelcount;
    int inputW;
    int inputH;
    int kernelcount;
    int kernelW;
    int kernelH;
    int paddingW;
    int paddingH;
    int strideW;
    int strideH;
    float preluAlpha;
    float *input_thresholds;            /* one threshold per batch item      */
    float *input;                       /* fp32 NCHW                         */
    float *kernel;                      /* fp32 (KN,C,KH,KW); unused here    */
    int64_t *quantized_kernel_packing0; /* unused here                       */
    int64_t *quantized_kernel_packing1; /* unused here                       */
    int64_t *quantized_kernel_packing2; /* Packing-2 weights (host)          */
    float *output;                      /* overwritten with a fresh buffer   */
} testcase_t;

/* include/tnns/data.h:27-41 (88 bytes on LP64) */
typedef struct testcase_tnns_gemm {
    int m;
    int p;
    int p_packed;
    int n;
    float *x;
    float *w;
    int64_t *x_packing0;
    int64_t *x_packing1;
    int64_t *x_packing2;
    int64_t *w_packing0;
    int64_t *w_packing1;
    int64_t *w_packing2;
    float *output;
} testcase_tnns_gemm_t;

/* ------------------------------------- 1. reference entry points (host memory) */

/* include/tnns/tnns_cpu.h:4, src/tnns/tnns_cpu_mm_p2.c:83-120.  Runs one conv layer
 * of data->type; data->output is replaced by a malloc'd fp32 NCHW tensor. */
FTNN_API void tnns_conv(testcase_t *data);

/* include/tnns/tnns_cpu.h:6, src/tnns/tnns_cpu_mm_p2.c:122-133.  TNN GEMM of the
 * Packing-2 operands with alpha = 1; copies into data->output when it is set,
 * otherwise hands over a malloc'd m x n matrix. */
FTNN_API void tnns_gemm(testcase_tnns_gemm_t *data);

/* include/tnns/ternarize2row.h:7, src/tnns/ternarize2row_avx2.c:715-803.
 * Ternarise + im2row + Packing 2; returns aligned_alloc(32, ...) memory. */
FTNN_API int64_t *t2r_p2_opt(float *x, float *q_thresholds, int N, int C, int H, int W, int H_pad,
                    int W_pad, int kH, int kW, int H_stride, int W_stride);

/* include/tnns/binarize2row.h:4, src/tnns/binarize2row_avx2.c:131-199. */
FTNN_API int64_t *b2r(float *x, float *q_thresholds, int N, int C, int H, int W, int H_pad, int W_pad,
             int kH, int kW, int H_stride, int W_stride);

/* include/tnns/mm.h:5-8; src/tnns/mm_p2_final_{tnn,tbn,btn,bnn}_avx2.c.  K is the
 * number of 64-bit words per plane before rounding up to a multiple of 4.  The
 * result is malloc'd fp32 in (N, KN, OH, OW) order with PReLU(alpha) applied. */
FTNN_API float *mm_tnn(int64_t *a, int64_t *b, int N, int OH, int OW, int KN, int K, float prelu_alpha);
FTNN_API float *mm_tbn(int64_t *a, int64_t *b, int N, int OH, int OW, int KN, int K, float prelu_alpha);
FTNN_API float *mm_btn(int64_t *a, int64_t *b, int N, int OH, int OW, int KN, int K, float prelu_alpha);
FTNN_API float *mm_bnn(int64_t *a, int64_t *b, int N, int OH, int OW, int KN, int K, int K_unpack,
              float prelu_alpha);

/* include/utils.h:17,22,26; src/utils.c:257-291, 468-521, 634-675: the packers the reference's drivers prepare their
 * operands with (src/timing_gemm.c:102-103, src/timing_layers.c:131-134), on host pointers.  bitpacking2 packs an fp32
 * [I][J] matrix of {-1, 0, +1} into Packing 2 (J a multiple of 256); ternarize_opt_avx2 / binarize_opt_avx2 pack fp32
 * weights (N, C, H, W) = (kernels, channels, kernel height, kernel width) with one threshold per kernel.  Each
 * returns aligned_alloc(32, ...) memory that the caller free()s.  A driver that links the reference's own utils.o
 * keeps the reference's definitions (the executable's symbols come first); to take these instead, compile that one
 * file with the three names renamed on the compiler's command line (-Dbitpacking2=ref_bitpacking2 and so on). */
FTNN_API int64_t *bitpacking2(float *x, int I, int J);
FTNN_API int64_t *ternarize_opt_avx2(float *x, float *q_thresholds, int N, int C, int H, int W);
FTNN_API int64_t *binarize_opt_avx2(float *x, float *q_thresholds, int N, int C, int H, int W);

/* State behind the host entry points above (no counterpart in the reference, whose functions keep none).
 * tnns_conv keeps the weights of the layers it has seen on the device in engine form, found again by a 128-bit hash
 * of their contents, their size and the layer shape (never by address): ftnn_host_forget_weights() frees them all;
 * FTNN_HOST_NO_WEIGHT_CACHE=1 in the environment keeps none, FTNN_HOST_WEIGHT_CACHE_MB=n caps them (default 1024;
 * a layer whose prepared weights alone exceed the cap is uploaded and prepared on every call).  Large results are prepared ahead of time by a helper thread once a size
 * repeats (at most 512 MiB waiting, each dropped after 256 large results have passed it by):
 * ftnn_host_release_spares() frees those that are ready and forgets the sizes seen. */
FTNN_API void ftnn_host_forget_weights(void);
FTNN_API void ftnn_host_release_spares(void);
/* device bytes the weight cache holds now */
FTNN_API int64_t ftnn_host_cached_weight_bytes(void);
/* the cache's content hash of `bytes` bytes (out[0] low, out[1] high half); portable != 0 forces the implementation
 * without AES instructions on one thread; ftnn_host_hash_uses_aes() says which one the cache uses on this CPU */
FTNN_API void ftnn_host_hash128(const void *data, int64_t bytes, int portable, uint64_t out[2]);
FTNN_API int ftnn_host_hash_uses_aes(void);

/* ------------------------------------------- 2. device-memory entry points */

#define FTNN_OK 0
#define FTNN_EINVAL (-1)  /* bad argument (shape, alignment, null pointer) */
#define FTNN_EHIP (-2)    /* a HIP call failed                              */
#define FTNN_ENOMEM (-3)  /* device or host allocation failed               */

/* Size limits, all answered with FTNN_EINVAL: batch <= 65535; a padded image plane below
 * 2^26 pixels; at most 2^31-1 output rows (N*OH*OW); at most 2^24-4 words per plane of a row
 * (GEMM K, ceil(C/64)*KH*KW of a layer: 32-bit sums), and below 2^18 on the fp4 engine (exact
 * fp32 accumulation).  Tensors themselves may exceed 2^32 elements: offsets into them are
 * 64-bit. */

/* text of the last failure on the calling thread ("" if none) */
FTNN_API const char *ftnn_last_error(void);

/* library version string, e.g. "ftnn-hip 0.1 gfx950" */
FTNN_API const char *ftnn_version(void);

/* OH = (in + 2*pad - k)/stride + 1 (src/tnns/tnns_cpu_mm_p2.c:7-10) */
FTNN_API int ftnn_out_dim(int in, int pad, int k, int stride);

/* int64 words in one packed row: round4(ceil(C/64)*KH*KW), twice that for a
 * ternary (two-plane) row (src/tnns/ternarize2row_avx2.c:730-732) */
FTNN_API int64_t ftnn_row_words(int C, int KH, int KW, int ternary);

/* Device scratch, in bytes, that ftnn_quantize_im2row / ftnn_conv need for the
 * channel-packed copy of the input (N*H*W*ceil(C/64) words per plane). */
FTNN_API int64_t ftnn_pack_scratch_bytes(int N, int C, int H, int W, int ternary);

/*
 * Quantise + im2row + bit-pack on the device: the work of t2r_p2_opt (ternary != 0,
 * src/tnns/ternarize2row_avx2.c:715-803) or b2r (ternary == 0,
 * src/tnns/binarize2row_avx2.c:131-199).  d_x fp32 NCHW, d_thr[N], d_out holds
 * N*OH*OW rows of ftnn_row_words() words, d_scratch holds
 * ftnn_pack_scratch_bytes() bytes.
 */
FTNN_API int ftnn_quantize_im2row(int ternary, const float *d_x, const float *d_thr, int N, int C, int H,
                         int W, int H_pad, int W_pad, int kH, int kW, int H_stride, int W_stride,
                         int64_t *d_out, void *d_scratch, void *stream);

/*
 * Popcount GEMM + PReLU on the device for type TNN/TBN/BTN/BNN
 * (src/tnns/mm_p2_final_{tnn,tbn,btn,bnn}_avx2.c).  d_a: N*OH*OW packed rows,
 * d_b: KN packed rows, d_y: fp32 (N,KN,OH,OW).  K_unpack is read for BNN only.
 * Both operands must be 16-byte aligned.
 */
FTNN_API int ftnn_mm(int type, const int64_t *d_a, const int64_t *d_b, int N, int OH, int OW, int KN,
            int K, int K_unpack, float prelu_alpha, float *d_y, void *stream);

/*
 * GEMM engines.  The reference has one arithmetic (XOR/AND/popcount on bit-planes); on
 * MI355X the same integer dot products can also run on the matrix cores after the lanes
 * are expanded to int8 or fp4 (E2M1 holds -1, 0, +1 exactly).  All engines give the same
 * bits.  AUTO picks per shape what measured fastest.
 */
#define FTNN_ENGINE_AUTO 0
#define FTNN_ENGINE_VALU 1    /* bit-plane popcount on the vector ALU, no scratch   */
#define FTNN_ENGINE_MFMA_I8 2 /* v_mfma_i32_32x32x32_i8 on expanded operands         */
#define FTNN_ENGINE_MFMA_F4 3 /* v_mfma_f32_32x32x64_f8f6f4 (fp4); GEMM rows of at most 65536 words */

/* the engine FTNN_ENGINE_AUTO resolves to for this shape (never AUTO) */
FTNN_API int ftnn_select_engine(int type, int N, int OH, int OW, int KN, int K);

/* device scratch, in bytes, that ftnn_mm_engine needs for `engine` (0 for the VALU engine;
 * for AUTO the amount of the engine it resolves to) */
FTNN_API int64_t ftnn_mm_scratch_bytes(int engine, int type, int N, int OH, int OW, int KN, int K);

/*
 * ftnn_mm with an explicit engine.  d_scratch (16-byte aligned, scratch_bytes long) holds
 * the expanded operands of the matrix-core engines; it may be NULL for the VALU engine.
 * No counterpart in the reference: its mm_* have a single implementation.
 */
FTNN_API int ftnn_mm_engine(int engine, int type, const int64_t *d_a, const int64_t *d_b, int N, int OH,
                   int OW, int KN, int K, int K_unpack, float prelu_alpha, float *d_y,
                   void *d_scratch, int64_t scratch_bytes, void *stream);

/*
 * The two halves of a matrix-core GEMM, for callers that keep an operand expanded (weights
 * are constant across calls).  ftnn_expand_rows turns `rows` packed rows of K words per
 * plane (ternary != 0: Packing-2, else single-plane binary) into the operand format of
 * `engine` (FTNN_ENGINE_MFMA_I8 or _F4), ftnn_expand_bytes() bytes at d_out;
 * ftnn_mm_expanded multiplies two expanded operands and applies PReLU like ftnn_mm.
 * The fp4 format is opaque: two bits per lane, lane a stored as (a + 1) / 2, followed by
 * one int32 per row with the sum of the row's lanes (the GEMM undoes the offset with it);
 * its sums are exact in fp32 for K <= 65536 words, longer rows are refused (use int8).
 * No counterpart in the reference.
 */
FTNN_API int64_t ftnn_expand_bytes(int engine, int rows, int K);
FTNN_API int ftnn_expand_rows(int engine, int ternary, const int64_t *d_rows, int rows, int K, void *d_out,
                     void *stream);
FTNN_API int ftnn_mm_expanded(int engine, int type, const void *d_a_exp, const void *d_b_exp, int N, int OH,
                     int OW, int KN, int K, int K_unpack, float prelu_alpha, float *d_y, void *stream);

/*
 * One conv layer on the device (src/tnns/tnns_cpu_mm_p2.c:6-80): the input is quantised
 * once into d_scratch (ftnn_conv_scratch_bytes() bytes, 16-byte aligned) and the GEMM gathers
 * its im2row operand from there, so the im2row matrix of t2r_p2_opt / b2r is never written to
 * memory.  Layers with C <= 32 re-pack both operands with several kernel taps per 64-lane word
 * first (an RGB stem uses 3 of 64 lanes otherwise).  Same result as ftnn_quantize_im2row
 * followed by ftnn_mm.
 */
FTNN_API int64_t ftnn_conv_scratch_bytes(int type, int N, int C, int H, int W, int KN, int KH, int KW,
                                int H_pad, int W_pad, int H_stride, int W_stride);
FTNN_API int ftnn_conv(int type, const float *d_x, const float *d_thr, const int64_t *d_qw, int N, int C,
              int H, int W, int KN, int KH, int KW, int H_pad, int W_pad, int H_stride,
              int W_stride, float prelu_alpha, void *d_scratch, float *d_y, void *stream);

/*
 * ftnn_conv without a scratch argument and without any allocation.  No counterpart in the reference; it is for
 * callers that cannot allocate device memory: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  The layer's work space (the quantised input and the weights in engine form) is a fixed array
 * of FTNN_STATIC_SCRATCH_BYTES inside the library's code object: every GPU on which the process loads the library's
 * code holds its copy from that load until the process ends, whether or not the entry point is ever called
 * (ftnn_static_scratch_bytes() returns the size the library was built with).  A layer whose ftnn_conv_scratch_bytes() exceeds that is refused with
 * FTNN_EINVAL.  The call itself performs no hipMalloc / hipFree and synchronises nothing; the first call on a
 * device looks the array's address up (hipGetSymbolAddress), so make that first call outside a graph capture.
 * All calls on one GPU share the one array: calls that overlap on a GPU (two streams, two threads) race, and the
 * array keeps the last call's contents (every call overwrites the part it reads).  Same result as ftnn_conv.
 */
#define FTNN_STATIC_SCRATCH_BYTES (32 << 20)
FTNN_API int64_t ftnn_static_scratch_bytes(void);
FTNN_API int ftnn_conv_static(int type, const float *d_x, const float *d_thr, const int64_t *d_qw, int N, int C,
                              int H, int W, int KN, int KH, int KW, int H_pad, int W_pad, int H_stride,
                              int W_stride, float prelu_alpha, float *d_y, void *stream);

/*
 * The same layer on an explicit engine (no counterpart in the reference; same bits on either):
 * FTNN_ENGINE_VALU      quantise to bit planes, vector-ALU popcount GEMM with implicit im2row;
 * FTNN_ENGINE_MFMA_F4   quantise to fp4 nibbles, expand the weights into matrix-core fragments
 *                       (in d_scratch) and run the fp4 matrix-core layer kernel;
 * FTNN_ENGINE_AUTO      what ftnn_conv does: ftnn_select_conv_engine()'s choice.
 * ftnn_conv_scratch_bytes() covers every engine.
 */
FTNN_API int ftnn_select_conv_engine(int type, int N, int C, int H, int W, int KN, int KH, int KW, int H_pad,
                                     int W_pad, int H_stride, int W_stride);
FTNN_API int ftnn_conv_engine(int engine, int type, const float *d_x, const float *d_thr, const int64_t *d_qw,
                              int N, int C, int H, int W, int KN, int KH, int KW, int H_pad, int W_pad,
                              int H_stride, int W_stride, float prelu_alpha, void *d_scratch, float *d_y,
                              void *stream);

/*
 * Weights prepared once per layer (no counterpart in the reference, whose packed rows are final):
 * ftnn_conv_prepare_weights turns the packed rows of ftnn_pack_weights / the reference's
 * quantized_kernel_packing2 into the form the layer's engine reads -- matrix-core fragments, or
 * the dense re-packing of a few-channel layer -- so that ftnn_conv_prepared does not repeat that
 * work on every call.  d_prepared: ftnn_conv_weights_bytes() bytes, 16-byte aligned.  Result and
 * scratch of ftnn_conv_prepared are those of ftnn_conv.
 */
FTNN_API int64_t ftnn_conv_weights_bytes(int type, int C, int KN, int KH, int KW);
FTNN_API int ftnn_conv_prepare_weights(int type, const int64_t *d_qw, int C, int KN, int KH, int KW,
                                       void *d_prepared, void *stream);
FTNN_API int ftnn_conv_prepared(int type, const float *d_x, const float *d_thr, const void *d_prepared, int N,
                                int C, int H, int W, int KN, int KH, int KW, int H_pad, int W_pad, int H_stride,
                                int W_stride, float prelu_alpha, void *d_scratch, float *d_y, void *stream);

/*
 * A chain of conv layers with device-resident activations: the e2e mode of the reference's
 * layer driver (src/timing_layers.c:182-207 feeds each layer's output to the next one), here
 * without the host round trip per layer.  A layer that feeds a layer on the fp4 matrix-core
 * engine thresholds its own results with that layer's threshold and writes its quantised
 * input directly, so no fp32 tensor exists between them; the chain's output is what the
 * reference's chain of tnns_conv calls returns, bit for bit.  All device memory (activation
 * and operand buffers, work space, per-layer threshold arrays, the weights in engine form) is
 * allocated by ftnn_net_create; a run allocates nothing.  Packed weights stay the caller's and
 * must outlive the net.  From batch 48 on a net runs the two halves of its batch as two chains
 * side by side (the second on a stream of its own, forked from and joined back into the
 * caller's stream inside ftnn_net_run, also under graph capture): the images of a batch never
 * meet, and the launch latencies of one chain overlap with the other's work.
 */
typedef struct ftnn_layer {
    int type;             /* TNN / TBN / BTN / BNN                               */
    int C, H, W;          /* input channels, height, width                       */
    int KN, KH, KW;       /* kernels, kernel height, kernel width                */
    int pad, stride;      /* same in both directions, as the reference's tables  */
    float threshold;      /* activation threshold, applied to every batch item   */
    float prelu_alpha;
    const int64_t *d_qw;  /* packed weights on the device (ftnn_pack_weights)    */
} ftnn_layer_t;

typedef struct ftnn_net ftnn_net_t;

/* NULL on failure (ftnn_last_error() says why): every layer's input must be the previous
 * layer's output shape */
FTNN_API ftnn_net_t *ftnn_net_create(int batch, int n_layers, const ftnn_layer_t *layers);
/* The same with flags.  FTNN_NET_REREAD_PREFIX accepts a layer whose input shape is not the
 * previous layer's output shape, provided it is no larger: the layer then takes the leading
 * N*C*H*W floats of the previous fp32 output as its NCHW input.  That is what the reference's e2e
 * driver does on its tables that leave out the pooling layers (ResNet-34, VGG-16, VGG-19 of
 * include/timing/shapes_e2e.h: src/timing_layers.c:187-200 hands the output buffer on whatever
 * the next row says); without the flag such a table is refused. */
#define FTNN_NET_REREAD_PREFIX 1
FTNN_API ftnn_net_t *ftnn_net_create_ex(int batch, int n_layers, const ftnn_layer_t *layers, int flags);
FTNN_API void ftnn_net_destroy(ftnn_net_t *net);
/* elements of the final output (batch * KN * OH * OW of the last layer) */
FTNN_API int64_t ftnn_net_output_elems(const ftnn_net_t *net);
/* d_x: fp32 NCHW input of layer 0; d_y: fp32 NCHW output of the last layer.  use_graph != 0
 * records the layer launches into a HIP graph on first use (and again whenever d_x, d_y or
 * the stream change) and replays it afterwards. */
FTNN_API int ftnn_net_run(ftnn_net_t *net, const float *d_x, float *d_y, int use_graph, void *stream);

/*
 * Weight packers on the device: fp32 (KN,C,KH,KW) -> Packing-2 rows.  ternary != 0 is
 * ternarize_opt_avx2 (src/utils.c:468-521), ternary == 0 is binarize_opt_avx2
 * (src/utils.c:634-675).  d_thr[KN].
 */
FTNN_API int ftnn_pack_weights(int ternary, const float *d_w, const float *d_thr, int KN, int C, int KH,
                      int KW, int64_t *d_out, void *stream);

/*
 * GEMM operand packer on the device: fp32 row-major [I][J] with values in
 * {-1,0,+1} -> Packing 2 (bitpacking2, src/utils.c:257-291).  J % 256 must be 0.
 */
FTNN_API int ftnn_pack_gemm_operand(const float *d_x, int I, int J, int64_t *d_out, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FTNN_H */
