/*
 * Dispatch probes of the MI355X (gfx950) backend: which kernel an entry point of dabnn_hip.h would run for a problem
 * on the current device.  None of them has a counterpart in the reference and none computes anything: they exist so
 * that a caller that plans a layer sequence (Net::prepare) can link layers the way the kernels prefer, and so that a
 * parity test can name the build it means to cover.  The reference's surface, and the documented extensions of it,
 * are in dabnn_hip.h; a drop-in caller needs nothing from this file.
 */
#ifndef DABNN_HIP_TUNING_H
#define DABNN_HIP_TUNING_H

#include "dabnn_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * 1 when dab_bconv3x3* would run this problem (n_out_pixels = N*OH*OW) with its small-problem kernel, whose work
 * items are whole bytes of sign bits -- dab_bconv3x3_affine_add_sign then costs no more than dab_bconv3x3_affine_add,
 * also for 512 input channels, where the large kernel makes the packed copy dearer than a separate dab_bitpack_nhwc.
 * 0 otherwise (cin 64, 128, 256 or 512; other values answer 0).  Net::prepare uses it to decide which layers to link.
 */
DAB_API int dab_bconv3x3_splits_depth(int64_t n_out_pixels, int cin, int cout);

/*
 * Which of the three builds of the direct kernel dab_bconv3x3_affine_add(_sign) runs for a problem of
 * n_out_pixels = N*OH*OW on the current device: 0 = the small-problem kernel (a block splits the depth over its
 * waves), 1 = the unit kernel's build for mid-sized problems, 2 = its build for large ones (four waves per SIMD and
 * whole-line stores for 64 and 128 input channels, units of twice the channels for 256 and 512; taken when a wave
 * gets many units); -1 for shapes the direct kernel does not take.  For tests and tuning: a parity test names the
 * build it means to cover.
 */
DAB_API int dab_bconv3x3_build(int64_t n_out_pixels, int cin, int cout);

/*
 * The same for dab_bconv3x3 itself (raw counts), which has a fourth build for 256 and 512 input channels from a
 * single tile up to mid-sized problems: 3 = the row-split kernel, whose blocks are three waves that count one kernel
 * row each and add their partial counts in LDS.  dab_bconv3x3_build answers for dab_bconv3x3_affine_add at stride 1
 * and never says 3; dab_bconv3x3_epilogue_build knows stride and sign bits.
 */
DAB_API int dab_bconv3x3_counts_build(int64_t n_out_pixels, int cin, int cout, int stride);

/*
 * The same for dab_bconv3x3_affine_add (with_sign = 0) and dab_bconv3x3_affine_add_sign (with_sign = 1) at a given
 * stride: 0, 1, 2 as dab_bconv3x3_build names them, 3 = the row-split kernel, which these entry points take for 256
 * and 512 input channels between the small and the mid-sized problems.  Net::prepare asks it for producers with 512
 * input channels: where the answer is 3, the packed copy for the next binary convolution costs no separate pass.
 */
DAB_API int dab_bconv3x3_epilogue_build(int64_t n_out_pixels, int cin, int cout, int stride, int with_sign);

/*
 * Whether dab_bconv3x3_affine_add(_sign) runs a problem of n_out_pixels = N*OH*OW on
 * the kernel whose blocks share a tile of 64 pixels x 64 output channels and write it as one piece (64 input channels,
 * cout a multiple of 64, at least 32 tiles per CU: the first stage of a residual net at large batch, bound by the fp32
 * shortcut it reads and the result it writes) instead of the build dab_bconv3x3_build names.  1 or 0.  For tests.
 */
DAB_API int dab_bconv3x3_fused_shares_tiles(int64_t n_out_pixels, int cin, int cout);

/*
 * 1 for the shapes dab_global_ave_pool_fconv1x1 covers (n <= 8, h * w <= 64, c a multiple of 4 up to 1024,
 * cout >= 64), 0 for those the two separate calls serve.
 */
DAB_API int dab_global_ave_pool_fconv1x1_takes(int n, int h, int w, int c, int cout);

/*
 * 1 when dab_fconv_maxpool takes the shape and the problem is large enough on the current device for the one pass to
 * beat dab_fconv_affine_relu + dab_max_pool_sign, 0 otherwise.
 */
DAB_API int dab_fconv_maxpool_pays(int n, int h, int w, int c, int kh, int kw, int pad_h, int pad_w, int stride_h,
                                   int stride_w, int dil_h, int dil_w, int cout);

#ifdef __cplusplus
}
#endif

#endif /* DABNN_HIP_TUNING_H */
