/*
 * C ABI of the MI355X (gfx950) backend for dabnn's binary-convolution path.
 *
 * Every entry point is the device-side replacement of one function of the
 * reference (cited per declaration).  All tensor pointers are DEVICE pointers
 * into contiguous buffers in the reference's layouts:
 *
 *   fp32 activations   [N][H][W][C]            (dabnn/mat.h:36, NHWC)
 *   packed activations [N][H][W][C/64] uint64  bit j of word i = (x[64*i+j] > 0)
 *                                              (common/common_bitpack.h:26,110-174)
 *   packed weights     [Cout][words per filter] uint64, tap order (kh, kw, c)
 *                                              (tools/onnx2bnn/OnnxConverter.cpp:121-156)
 *
 * The batch dimension N is an extension: the reference processes one image
 * per call (dabnn/net.cpp:64-65); N images here give exactly the results of N
 * reference calls.
 *
 * Calls are asynchronous on `stream` (a hipStream_t passed as void*; NULL is
 * the default stream).  Return value: DAB_OK or a negative DAB_E* code; the
 * functions never throw and never abort.  dab_last_error() returns a
 * thread-local message for the last failing call.  The reference signals the
 * same conditions with BNN_ASSERT -> std::runtime_error (common/helper.h:69-77);
 * the C++ layer on top of this header rethrows them as that type.
 */
#ifndef DABNN_HIP_H
#define DABNN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define DAB_API __attribute__((visibility("default")))
#else
#define DAB_API
#endif

#define DAB_OK 0
#define DAB_EINVAL (-1)      /* argument violates a reference assertion (shape, alignment, null) */
#define DAB_EUNSUPPORTED (-2) /* valid request outside what this entry point implements */
#define DAB_EHIP (-3)        /* a HIP runtime call failed; message holds hipGetErrorString */

typedef void *dab_stream_t;

/* Library / device information. */
DAB_API const char *dab_last_error(void);
DAB_API int dab_version(void);
/* CU count and shader clock (kHz) of the current device; feeds the roofline figures. */
DAB_API int dab_device_info(int *cu_count, int *clock_khz);

/*
 * pack_mat -> pack_mat_64 (dabnn/bitpack.h:254-293): sign-pack n_pix pixels of
 * c channels (c % 64 == 0) along the channel axis.  out holds n_pix * c/64 words.
 */
DAB_API int dab_bitpack_nhwc(const float *x, uint64_t *out, int64_t n_pix, int c, dab_stream_t stream);

/*
 * Same output words from an NCHW tensor [n][c][h][w].  No counterpart in the
 * reference (its tensors are NHWC only, dabnn/mat.h:36); specified as
 * dab_bitpack_nhwc applied to the NHWC permutation of x.
 */
DAB_API int dab_bitpack_nchw(const float *x, uint64_t *out, int n, int c, int h, int w, dab_stream_t stream);

/*
 * pad, Bit branch (dabnn/pad.h:7-19): copy [n][h][w][cw] words into the
 * centre of a zero-filled [n][h+2*pad_h][w+2*pad_w][cw] buffer.
 */
DAB_API int dab_pad_bit(const uint64_t *x, int n, int h, int w, int cw, int pad_h, int pad_w, uint64_t *out,
                dab_stream_t stream);

/*
 * Split::forward_impl (dabnn/layers/Split.cpp:6-21) on packed activations: the cw words of each of the n_pix pixels
 * are cut in two, out1 takes words [0, cw/2), out2 words [cw/2, cw); both hold n_pix * cw/2 words.  cw * 64 channels
 * must be a multiple of 128 and at most 512 (dabnn/layers/Split.h:22-23), i.e. cw in {2, 4, 6, 8}.
 */
DAB_API int dab_split_bit(const uint64_t *x, int64_t n_pix, int cw, uint64_t *out1, uint64_t *out2, dab_stream_t stream);

/*
 * Shuffle::forward_impl (dabnn/layers/Shuffle.cpp:6-43), in place on packed activations of elem_c channels
 * (a multiple of 128, at most 512, dabnn/layers/Shuffle.h:19-20): the channel shuffle of a two-group network at the
 * granularity the reference has -- 128 channels: the 32-bit quarters 1 and 2 of every pixel change places; 256: words
 * 1 and 2; 512: words 2,3 and 4,5; 384 channels pass unchanged, as in the reference.
 */
DAB_API int dab_shuffle_bit_inplace(uint64_t *x, int64_t n_pix, int elem_c, dab_stream_t stream);

/*
 * fused_binarize_im2col (dabnn/fused_binarize_im2col.h:6-68): for every
 * output pixel gather kh*kw runs of c floats (zeros outside the image),
 * zero-extend to a multiple of 128 floats and sign-pack.
 * col holds n*oh*ow rows of dab_col_row_words(kh, kw, c) words.
 * Fails with DAB_EINVAL when kh*kw*c >= 60000 (reference assertion, :14).
 */
DAB_API int dab_fused_binarize_im2col(const float *x, int n, int h, int w, int c, int kh, int kw, int pad_h, int pad_w,
                              int stride_h, int stride_w, int dil_h, int dil_w, uint64_t *col, dab_stream_t stream);
DAB_API int dab_col_row_words(int kh, int kw, int c);

/*
 * bgemm / bgemm_naive (dabnn/bgemm.h:46-66,587-597): column-major
 * C(i,j) += float(popcount(A(i,h) ^ B(h,j))), A(i,h) = a[h*lda+i],
 * B(h,j) = b[j*ldb+h], C(i,j) = c[j*ldc+i].  C is accumulated into, as in the
 * reference (callers zero-fill it first, dabnn/layers/BinConv.cpp:153,168).
 * Bit-exact with the reference whenever C holds integer-valued floats and
 * every sum stays below 2^24 (always true for zero-filled C and k <= 2^18).
 */
DAB_API int dab_bgemm(int m, int n, int k, const uint64_t *a, int lda, const uint64_t *b, int ldb, float *c, int ldc,
              dab_stream_t stream);

/*
 * What the reference's pair output_mat->fill<float>(0.f) + bgemm leaves in C (dabnn/layers/BinConv.cpp:153-165,
 * 168-189): C(i,j) = float(popcount(A(i,h) ^ B(h,j))) summed over h, written without reading C.  Bit for bit the
 * result of dab_fill_f32(c, 0) followed by dab_bgemm (0.f + count == count), in one launch and without the read of C.
 */
DAB_API int dab_bgemm_overwrite(int m, int n, int k, const uint64_t *a, int lda, const uint64_t *b, int ldb, float *c,
                                int ldc, dab_stream_t stream);

/*
 * Weight transpose done by the BinConv constructor for its bgemm method
 * (dabnn/layers/BinConv.cpp:59-76): wt[i*m + j] = w[j*k + i].
 */
DAB_API int dab_weight_transpose(const uint64_t *w, int m, int k, uint64_t *wt, dab_stream_t stream);

/*
 * bconv_3x3 on top of pad (dabnn/bconv.h:855-931 with dabnn/pad.h, i.e. the
 * DIRECT_CONV arm of dabnn/layers/BinConv.cpp:145-150) == baseline_bconv
 * (common/baseline.h:77-116) with a 3x3 kernel: x is the UNPADDED packed
 * activation [n][h][w][cin/64]; taps outside the image read a zero word.
 * wgt is [cout][9*cin/64] words.  out is fp32 [n][oh][ow][cout] holding the
 * mismatch counts, oh = (h + 2*pad - 3)/stride + 1.
 * Implemented for cin in {64, 128, 256, 512, 1024} (the reference's list,
 * dabnn/layers/BinConv.cpp:118; 1024 as two passes over 512 channels each, the
 * second adding to the first) and cout % 8 == 0; other shapes return
 * DAB_EUNSUPPORTED (use dab_fused_binarize_im2col + dab_bgemm, as the
 * reference's BGEMM arm does).
 */
DAB_API int dab_bconv3x3(const uint64_t *x, int n, int h, int w, int cin, const uint64_t *wgt, int cout, int stride,
                 int pad, float *out, dab_stream_t stream);

/*
 * dab_bconv3x3 followed in the same pass by the two layers that always follow a
 * BinConv in a residual block: affine_inplace (dabnn/layers/Affine.cpp:10-23)
 * and add_inplace (dabnn/layers/Add.cpp:7-17):
 *   out[p][c] = (a[c] * cnt[p][c] + b[c]) + shortcut[p][c]
 * with the three operations rounded one by one, so the result equals running
 * the three reference layers in sequence bit for bit.  shortcut may be NULL
 * (affine only); it has the layout of out and must not overlap it.
 */
DAB_API int dab_bconv3x3_affine_add(const uint64_t *x, int n, int h, int w, int cin, const uint64_t *wgt, int cout,
                                    int stride, int pad, const float *a, const float *b, const float *shortcut,
                                    float *out, dab_stream_t stream);

/*
 * dab_bconv3x3_affine_add that also writes pack_mat (dabnn/bitpack.h:277-293) of its own result:
 *   out_packed[p][c/64] bit c%64 = (out[p][c] > 0)
 * i.e. the words BinConv::forward_impl of the next layer would make from out (dabnn/layers/BinConv.cpp:146), so
 * that layer can skip reading the fp32 blob again.  cout must be a multiple of 64.
 */
DAB_API int dab_bconv3x3_affine_add_sign(const uint64_t *x, int n, int h, int w, int cin, const uint64_t *wgt, int cout,
                                         int stride, int pad, const float *a, const float *b, const float *shortcut,
                                         float *out, uint64_t *out_packed, dab_stream_t stream);

/*
 * BinConv::forward_impl (dabnn/layers/BinConv.cpp:144-191) for a batch of
 * fp32 NHWC images: binarise + binary convolution, fp32 mismatch counts out.
 * Method selection mirrors BinConv::method() (:80-98): 3x3 with cin in
 * {64,128,256,512,1024} takes the direct kernel (pack + bconv), anything else
 * takes fused_binarize_im2col + bgemm on `wgt_t` (the transposed weights;
 * may be NULL when the direct kernel applies).
 * hwc_words = words per filter (weight.total()/weight.n).
 * workspace must hold dab_binconv_workspace_bytes(...) bytes.
 * method_out (optional) receives 0 = DIRECT_CONV, 1 = BGEMM.
 */
DAB_API size_t dab_binconv_workspace_bytes(int n, int h, int w, int c, int kh, int kw, int pad_h, int pad_w, int stride_h,
                                   int stride_w);
DAB_API int dab_binconv_forward(const float *x, int n, int h, int w, int c, const uint64_t *wgt, const uint64_t *wgt_t,
                        int hwc_words, int kh, int kw, int pad_h, int pad_w, int stride_h, int stride_w, int cout,
                        float *out, void *workspace, size_t workspace_bytes, int *method_out, dab_stream_t stream);

/*
 * No counterpart in the reference.  dab_binconv_forward for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the workspace is a buffer of
 * DAB_BINCONV_STATIC_SCRATCH_BYTES that lives inside the library's code object, one copy per GPU, held until the
 * process ends.  Same arguments, results and error codes as dab_binconv_forward without the workspace pair; problems
 * whose dab_binconv_workspace_bytes(...) exceeds the buffer return DAB_EUNSUPPORTED.  The call allocates and frees
 * nothing on the device.  All calls on one GPU share that GPU's buffer: two calls that overlap in time on the same
 * GPU (different streams or threads) race; calls on one stream are ordered and safe.  The first call on a device
 * resolves the buffer's address (hipGetSymbolAddress); make it outside a graph capture.
 */
#define DAB_BINCONV_STATIC_SCRATCH_BYTES (16u << 20)
DAB_API int dab_binconv_forward_static(const float *x, int n, int h, int w, int c, const uint64_t *wgt,
                                       const uint64_t *wgt_t, int hwc_words, int kh, int kw, int pad_h, int pad_w,
                                       int stride_h, int stride_w, int cout, float *out, int *method_out,
                                       dab_stream_t stream);

/* ------------------------------------------------------------------ float glue */

/*
 * fconv (dabnn/fconv.h:14-76): fp32 convolution, weights [cout][kh][kw][c],
 * optional bias (NULL for none).  Agreement with the reference is to fp32
 * rounding (1e-4 relative), the summation order differs from Eigen's.
 */
DAB_API int dab_fconv(const float *x, int n, int h, int w, int c, const float *wgt, const float *bias, int kh, int kw,
              int pad_h, int pad_w, int stride_h, int stride_w, int dil_h, int dil_w, int cout, float *out,
              dab_stream_t stream);

/*
 * dab_fconv followed in the same pass by the Affine (a, b; both NULL for none) and Relu (relu != 0) layers that
 * follow a float convolution in the stem of a network: out = relu(a[c]*(conv + bias[c]) + b[c]), each operation
 * rounded as the separate layers round it (dabnn/layers/Affine.cpp:10-23, dabnn/layers/Relu.cpp).
 */
DAB_API int dab_fconv_affine_relu(const float *x, int n, int h, int w, int c, const float *wgt, const float *bias,
                                  const float *a, const float *b, int relu, int kh, int kw, int pad_h, int pad_w,
                                  int stride_h, int stride_w, int dil_h, int dil_w, int cout, float *out,
                                  dab_stream_t stream);

/*
 * AvePool 2x2, stride 2, no padding (ave_pool_fallback, dabnn/layers/AvePool.cpp:84-123) followed by a 1x1 FpConv2D
 * (dabnn/fconv.h:14-76) and the optional Affine and Relu of dab_fconv_affine_relu, in one launch: the shortcut branch
 * of a down-sampling block.  pooled [n][(h-2)/2+1][(w-2)/2+1][c] receives the pooled tensor exactly as dab_ave_pool
 * writes it, out the convolution of it exactly as dab_fconv_affine_relu computes it from that tensor.
 * pooled may be NULL when nobody reads the pooled tensor (it is then not written; out is the same), except for
 * eight pooled pixels or fewer with cout >= 64, which run as the two launches and need the buffer (DAB_EINVAL).
 * wgt is [cout][1][1][c].  c must be a multiple of 4 and x, wgt, pooled 16-byte aligned (DAB_EUNSUPPORTED otherwise).
 */
DAB_API int dab_ave_pool2_fconv1x1(const float *x, int n, int h, int w, int c, const float *wgt, const float *bias,
                                   const float *a, const float *b, int relu, int cout, float *pooled, float *out,
                                   dab_stream_t stream);

/*
 * A global AvePool -- one h x w window, stride 1, no padding, a 1 x 1 result per image (ave_pool_fallback,
 * dabnn/layers/AvePool.cpp:84-123; Net::prepare builds the layer at dabnn/net.cpp:221-229) -- followed by a 1x1
 * FpConv2D (dabnn/fconv.h:14-76) and the optional Affine and Relu of dab_fconv_affine_relu, in one launch: the end of
 * a classifier at small batch.  pooled [n][1][1][c] receives the pooled tensor exactly as dab_ave_pool writes it, out
 * [n][1][1][cout] the convolution of it exactly as dab_fconv_affine_relu computes it from that tensor.  wgt is
 * [cout][1][1][c].  dab_global_ave_pool_fconv1x1_takes (dabnn_hip_tuning.h) returns 1 for the shapes the launch covers (n <= 8,
 * h * w <= 64, c a multiple of 4 up to 1024, cout >= 64); others, and x, wgt or pooled not 16-byte aligned, are
 * DAB_EUNSUPPORTED: the two separate calls serve them.
 */
DAB_API int dab_global_ave_pool_fconv1x1(const float *x, int n, int h, int w, int c, const float *wgt, const float *bias,
                                         const float *a, const float *b, int relu, int cout, float *pooled, float *out,
                                         dab_stream_t stream);

/*
 * FpConv2D (dabnn/fconv.h:14-76) with the optional Affine and Relu of dab_fconv_affine_relu, followed by MaxPool 3x3,
 * stride 2, pad 1 (max_pool_fallback, dabnn/layers/MaxPool.cpp:209-246), in one pass that never writes the
 * convolution's output: the stem of a Bi-Real-style net.  pooled [n][oh/2][ow/2][cout] receives what dab_max_pool
 * computes from the convolution's result; pooled_packed, when not null (cout % 64 == 0), pack_mat of it
 * (dabnn/bitpack.h:277-293) as dab_max_pool_sign writes it (where a window's maximum is a zero of either sign, pooled
 * may hold the zero of the other sign than dab_max_pool's: equal as numbers, and the same bit in pooled_packed).  carry is
 * a workspace of dab_fconv_maxpool_carry_floats(...) floats, whose contents after the call are unspecified.  Shapes: the convolution's output width ow must divide 448 into an even
 * number of rows (28, 56, 112 or 224), oh must be a multiple of 448/ow, c must be 3 or a multiple of 4, cout a
 * multiple of 4, all buffers 16-byte aligned (DAB_EUNSUPPORTED otherwise).
 * dab_fconv_maxpool_carry_floats returns 0 for shapes the pass does not take; dab_fconv_maxpool_pays (dabnn_hip_tuning.h) returns 1 when
 * the problem is also large enough on the current device for the pass to beat dab_fconv_affine_relu + dab_max_pool_sign.
 */
DAB_API int dab_fconv_maxpool(const float *x, int n, int h, int w, int c, const float *wgt, const float *bias,
                              const float *a, const float *b, int relu, int kh, int kw, int pad_h, int pad_w,
                              int stride_h, int stride_w, int dil_h, int dil_w, int cout, float *pooled,
                              uint64_t *pooled_packed, float *carry, dab_stream_t stream);
DAB_API int64_t dab_fconv_maxpool_carry_floats(int n, int h, int w, int c, int kh, int kw, int pad_h, int pad_w,
                                               int stride_h, int stride_w, int dil_h, int dil_w, int cout);

/* affine_inplace (dabnn/layers/Affine.cpp:10-23): x[..., ch] = a[ch]*x[..., ch] + b[ch]. */
DAB_API int dab_affine_inplace(float *x, int64_t n_pix, int c, const float *a, const float *b, dab_stream_t stream);

/* add_inplace (dabnn/layers/Add.cpp:7-17): a += b over n_elem floats. */
DAB_API int dab_add_inplace(float *a, const float *b, int64_t n_elem, dab_stream_t stream);

/* Relu::forward_impl (dabnn/layers/Relu.cpp): x = max(x, 0) in place over n_elem floats. */
DAB_API int dab_relu_inplace(float *x, int64_t n_elem, dab_stream_t stream);

/*
 * PRelu::forward_impl (dabnn/layers/PRelu.cpp:6-30): x = x < 0 ? x*slope : x in place, with one slope for the whole
 * tensor (slope_n == 1) or one per channel (slope_n == c); any other slope_n is DAB_EINVAL as the reference asserts.
 */
DAB_API int dab_prelu_inplace(float *x, int64_t n_pix, int c, const float *slope, int slope_n, dab_stream_t stream);

/*
 * Concat::forward_impl (dabnn/layers/Concat.cpp:7-21; axis 3 only, dabnn/net.cpp:230-236): out[p] = a[p][0..ca) followed
 * by b[p][0..cb) for each of the n_pix pixels.  out must not alias a or b.
 */
DAB_API int dab_concat_channels(const float *a, int ca, const float *b, int cb, int64_t n_pix, float *out,
                                dab_stream_t stream);

/* Mat::fill<float> (dabnn/mat.h:351-443): x[i] = value; the zero-fill before bgemm (dabnn/layers/BinConv.cpp:153). */
DAB_API int dab_fill_f32(float *x, int64_t n_elem, float value, dab_stream_t stream);

/* ave_pool_fallback (dabnn/layers/AvePool.cpp:84-123): mean over in-bounds taps. */
DAB_API int dab_ave_pool(const float *x, int n, int h, int w, int c, int kh, int kw, int pad_h, int pad_w, int stride_h,
                 int stride_w, float *out, dab_stream_t stream);

/* max_pool_fallback (dabnn/layers/MaxPool.cpp:209-246): max over in-bounds taps from -FLT_MAX. */
DAB_API int dab_max_pool(const float *x, int n, int h, int w, int c, int kh, int kw, int pad_h, int pad_w, int stride_h,
                 int stride_w, float *out, dab_stream_t stream);

/*
 * dab_max_pool that also writes pack_mat (dabnn/bitpack.h:277-293) of its result, the packed input of a BinConv that
 * reads the pooled blob (the first block of a Bi-Real net): out_packed[p][c/64] bit c%64 = (out[p][c] > 0).
 * c must be a multiple of 64, x and out 16-byte aligned.
 */
DAB_API int dab_max_pool_sign(const float *x, int n, int h, int w, int c, int kh, int kw, int pad_h, int pad_w,
                              int stride_h, int stride_w, float *out, uint64_t *out_packed, dab_stream_t stream);

#ifdef __cplusplus
}
#endif

#endif /* DABNN_HIP_H */
