/*
 * CPU oracle for the binary-convolution hot path of dabnn.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is a from-scratch plain-C restatement
 * of the algorithms in the reference's portable (non-ARM) code path.  It is
 * the checker that the HIP kernels are compared against and the "port" CPU
 * baseline that bench.py times; the shipped library never links, loads or
 * calls it.  Every function names the reference lines it restates.
 *
 * All tensors are contiguous: fp32 activations are [H][W][C], packed
 * activations are [H][W][C/64] 64-bit words, one image per call (the
 * reference has no batch dimension, dabnn/net.cpp:64-65); callers loop over
 * images.  The reference's Mat requires w*c*elemsize % 16 == 0 and then has
 * hstep == w*c (dabnn/mat.h:246-247,605-617), i.e. exactly this layout.
 *
 * How each function is pinned (see tests/test_oracle_*.py):
 *   orc_pack_64 / orc_pack_mat     closed form bit j = (x > 0); known answer
 *                                  0x8000000000000001; numpy packbits
 *   orc_pack_nchw                  defined as transpose + orc_pack_mat
 *   orc_pad_bit                    numpy pad with zero words
 *   orc_baseline_bconv             +-1 float convolution with -1 padding
 *                                  (K - 2*cnt identity), brute force, corner
 *                                  and complement invariants
 *   orc_im2col                     the 288-value vector held by the
 *                                  reference's tests/im2col_test.cpp:22-38
 *   orc_fused_binarize_im2col      pack(im2col) identity on top of the above
 *   orc_bgemm_naive                numpy unpackbits integer matmul
 *   orc_weight_transpose           construction in tests/bgemm_test.cpp:60-77
 *   orc_binconv_forward            both dispatch arms agree with each other
 *                                  and with the +-1 float convolution
 *   orc_fconv / pools / affine     torch.nn.functional on NCHW-permuted data;
 *                                  ramp cases of tests/fconv_test.cpp
 *   orc_prelu_inplace              torch.nn.functional.prelu (scalar and per-
 *                                  channel slope)
 *   orc_concat                     numpy.concatenate along the channel axis
 *   orc_split_bit                  numpy slicing of the word axis
 *   orc_shuffle_bit                a channel permutation of the unpacked bits:
 *                                  two groups, 32 / 64 / 128 channels a piece
 *   orc_pack_weight / orc_bn_fold  K - 2*cnt end-to-end identity
 */
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <float.h>
#include <math.h>

#define ORC_API __attribute__((visibility("default")))

/* common/baseline.h:12-19: population count of a 64-bit word. */
static inline unsigned orc_bitcount(uint64_t x) {
    unsigned n = 0;
    while (x) {
        x &= x - 1;
        ++n;
    }
    return n;
}

/* Same count, fast form for the timed baseline loops (identical result). */
static inline unsigned orc_bitcount_fast(uint64_t x) {
    return (unsigned)__builtin_popcountll(x);
}

/*
 * common/common_bitpack.h:12-34 (pack_64_bitset) and :36-175
 * (pack_64_bitfield): bit j (LSB = 0) is 1 iff f[j] > 0; bits >= eff_bits
 * are 0.  +0, -0, NaN and negatives give 0.
 */
ORC_API uint64_t orc_pack_64(const float *f, size_t eff_bits) {
    uint64_t w = 0;
    for (size_t j = 0; j < 64 && j < eff_bits; ++j) {
        if (f[j] > 0) w |= (uint64_t)1 << j;
    }
    return w;
}

/*
 * dabnn/bitpack.h:254-293 (pack_mat -> pack_mat_64): pack every run of 64
 * consecutive floats of a [H][W][C] tensor, C % 64 == 0.  n_float is the
 * total element count; returns -1 when it is not a multiple of 64
 * (the reference asserts w*c % 64 == 0 and c % 64 == 0).
 */
ORC_API int orc_pack_mat(const float *x, size_t n_float, uint64_t *out) {
    if (n_float % 64 != 0) return -1;
    for (size_t i = 0; i < n_float / 64; ++i) out[i] = orc_pack_64(x + 64 * i, 64);
    return 0;
}

/*
 * NCHW-input variant: same output words as orc_pack_mat applied to the
 * NHWC permutation of x.  The reference has no NCHW tensors
 * (dabnn/mat.h:36); this is the specification of the added entry point.
 */
ORC_API int orc_pack_nchw(const float *x, int c, int h, int w, uint64_t *out) {
    if (c % 64 != 0) return -1;
    const int cw = c / 64;
    for (int y = 0; y < h; ++y)
        for (int xx = 0; xx < w; ++xx)
            for (int k = 0; k < cw; ++k) {
                uint64_t word = 0;
                for (int j = 0; j < 64; ++j) {
                    const float v = x[((size_t)(k * 64 + j) * h + y) * w + xx];
                    if (v > 0) word |= (uint64_t)1 << j;
                }
                out[((size_t)y * w + xx) * cw + k] = word;
            }
    return 0;
}

/*
 * dabnn/pad.h:7-19, Bit branch: zero words around the image; a zero word
 * stands for 64 values of -1.
 */
ORC_API void orc_pad_bit(const uint64_t *x, int h, int w, int cw, int pad_h, int pad_w, uint64_t *out) {
    const int ow = w + 2 * pad_w, oh = h + 2 * pad_h;
    memset(out, 0, (size_t)oh * ow * cw * sizeof(uint64_t));
    for (int y = 0; y < h; ++y)
        memcpy(out + ((size_t)(y + pad_h) * ow + pad_w) * cw, x + (size_t)y * w * cw,
               (size_t)w * cw * sizeof(uint64_t));
}

/* dabnn/pad.h:20-26, Float branch. */
ORC_API void orc_pad_float(const float *x, int h, int w, int c, int pad_h, int pad_w, float val, float *out) {
    const int ow = w + 2 * pad_w, oh = h + 2 * pad_h;
    for (size_t i = 0; i < (size_t)oh * ow * c; ++i) out[i] = val;
    for (int y = 0; y < h; ++y)
        memcpy(out + ((size_t)(y + pad_h) * ow + pad_w) * c, x + (size_t)y * w * c, (size_t)w * c * sizeof(float));
}

static int orc_out_dim(int in, int pad, int k, int dil, int stride) {
    return (in + 2 * pad - (dil * (k - 1) + 1)) / stride + 1;
}

/*
 * common/baseline.h:77-116 (baseline_bconv): direct binary convolution.
 * x is [h][w][cw] words, wgt is cout filters of hwc_words words each
 * (hwc_words = weight.total()/weight.n, >= kh*kw*cw when filters are padded
 * to 128 bits), tap order (kh, kw, cw).  Out-of-range taps read a zero word.
 * out is [oh][ow][cout] fp32 holding the mismatch count.
 */
ORC_API void orc_baseline_bconv(const uint64_t *x, int h, int w, int cw, const uint64_t *wgt, int hwc_words, int kh,
                                int kw, int pad_h, int pad_w, int stride_h, int stride_w, int dil_h, int dil_w,
                                int cout, float *out, int oh, int ow) {
    int input_y = 0;
    for (int th = 0; th < oh; ++th) {
        int input_x = 0;
        for (int tw = 0; tw < ow; ++tw) {
            for (int tc = 0; tc < cout; ++tc) {
                uint32_t acc = 0;
                for (int wh = 0; wh < kh; ++wh) {
                    const int y = input_y - pad_h + wh * dil_h;
                    for (int ww = 0; ww < kw; ++ww) {
                        const int xx = input_x - pad_w + ww * dil_w;
                        const int oob = y < 0 || y >= h || xx < 0 || xx >= w;
                        for (int wc = 0; wc < cw; ++wc) {
                            const uint64_t wv = wgt[(size_t)tc * hwc_words + (size_t)wh * kw * cw + ww * cw + wc];
                            const uint64_t bv = oob ? 0 : x[((size_t)y * w + xx) * cw + wc];
                            acc += orc_bitcount_fast(wv ^ bv);
                        }
                    }
                }
                out[((size_t)th * ow + tw) * cout + tc] = (float)acc;
            }
            input_x += stride_w;
        }
        input_y += stride_h;
    }
}

/* Same loop with the bit-by-bit count, for cross-checking the fast form. */
ORC_API uint32_t orc_xor_popcount_slow(const uint64_t *a, const uint64_t *b, size_t n) {
    uint32_t acc = 0;
    for (size_t i = 0; i < n; ++i) acc += orc_bitcount(a[i] ^ b[i]);
    return acc;
}

/*
 * dabnn/bconv.h:927-930: on non-ARM targets bconv_3x3 of an already padded
 * bit tensor is baseline_bconv with pad 0 and equal strides.
 */
ORC_API void orc_bconv_3x3_padded(const uint64_t *xp, int hp, int wp, int cw, const uint64_t *wgt, int hwc_words,
                                  int stride, int cout, float *out) {
    const int oh = orc_out_dim(hp, 0, 3, 1, stride), ow = orc_out_dim(wp, 0, 3, 1, stride);
    orc_baseline_bconv(xp, hp, wp, cw, wgt, hwc_words, 3, 3, 0, 0, stride, stride, 1, 1, cout, out, oh, ow);
}

/*
 * dabnn/im2col.h:14-47: for every output pixel, the kh*kw runs of c
 * elements (elemsize bytes each) at the tap positions, zero bytes where the
 * tap is outside the image.  Works on bytes, so it serves fp32 and packed
 * words alike.
 */
ORC_API void orc_im2col(const void *im, int h, int w, int c, int elemsize, int kh, int kw, int pad_h, int pad_w,
                        int stride_h, int stride_w, int dil_h, int dil_w, void *col) {
    const int oh = orc_out_dim(h, pad_h, kh, dil_h, stride_h), ow = orc_out_dim(w, pad_w, kw, dil_w, stride_w);
    const size_t run = (size_t)c * elemsize;
    char *dst = (char *)col;
    int input_y = 0;
    for (int oy = 0; oy < oh; ++oy) {
        int input_x = 0;
        for (int ox = 0; ox < ow; ++ox) {
            for (int a = 0; a < kh; ++a) {
                const int y = input_y - pad_h + a * dil_h;
                for (int b = 0; b < kw; ++b) {
                    const int xx = input_x - pad_w + b * dil_w;
                    if (y < 0 || y >= h || xx < 0 || xx >= w)
                        memset(dst, 0, run);
                    else
                        memcpy(dst, (const char *)im + ((size_t)y * w + xx) * run, run);
                    dst += run;
                }
            }
            input_x += stride_w;
        }
        input_y += stride_h;
    }
}

/* Words per fused-im2col row: kh*kw*c bits rounded up to 128, in words. */
ORC_API int orc_col_row_words(int kh, int kw, int c) { return (kh * kw * c + 127) / 128 * 2; }

/*
 * dabnn/fused_binarize_im2col.h:6-68: gather the kh*kw*c floats of every
 * output pixel (zeros outside), zero-extend the run to a multiple of 128
 * floats, pack by sign.  Returns -1 when kh*kw*c >= 60000 (reference
 * assertion, :14).
 */
ORC_API int orc_fused_binarize_im2col(const float *im, int h, int w, int c, int kh, int kw, int pad_h, int pad_w,
                                      int stride_h, int stride_w, int dil_h, int dil_w, uint64_t *col) {
    const int len = kh * kw * c;
    if (len >= 60000) return -1;
    const int oh = orc_out_dim(h, pad_h, kh, dil_h, stride_h), ow = orc_out_dim(w, pad_w, kw, dil_w, stride_w);
    const int len128 = (len + 127) / 128 * 128;
    float *buf = (float *)malloc((size_t)len128 * sizeof(float));
    if (!buf) return -2;
    int input_y = 0;
    for (int oy = 0; oy < oh; ++oy) {
        int input_x = 0;
        for (int ox = 0; ox < ow; ++ox) {
            float *p = buf;
            for (int a = 0; a < kh; ++a) {
                const int y = input_y - pad_h + a * dil_h;
                for (int b = 0; b < kw; ++b) {
                    const int xx = input_x - pad_w + b * dil_w;
                    if (y < 0 || y >= h || xx < 0 || xx >= w)
                        memset(p, 0, (size_t)c * sizeof(float));
                    else
                        memcpy(p, im + ((size_t)y * w + xx) * c, (size_t)c * sizeof(float));
                    p += c;
                }
            }
            memset(p, 0, (size_t)(len128 - len) * sizeof(float));
            for (int i = 0; i < len128 / 64; ++i) *col++ = orc_pack_64(buf + 64 * i, 64);
            input_x += stride_w;
        }
        input_y += stride_h;
    }
    free(buf);
    return 0;
}

/*
 * dabnn/layers/BinConv.cpp:59-76: weights [m][k] -> [k][m], which is the
 * column-major m x k operand A of bgemm (lda = m).
 */
ORC_API void orc_weight_transpose(const uint64_t *w, int m, int k, uint64_t *wt) {
    for (int i = 0; i < k; ++i)
        for (int j = 0; j < m; ++j) wt[(size_t)i * m + j] = w[(size_t)j * k + i];
}

/*
 * dabnn/bgemm.h:22-24,587-597 (bgemm_naive; bgemm on non-NEON targets,
 * :63-65): column-major C(i,j) += float(popcount(A(i,h) ^ B(h,j))), the sum
 * running over h in increasing order in fp32.
 */
ORC_API void orc_bgemm_naive(int m, int n, int k, const uint64_t *a, int lda, const uint64_t *b, int ldb, float *c,
                             int ldc) {
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j)
            for (int h = 0; h < k; ++h)
                c[(size_t)j * ldc + i] += (float)orc_bitcount_fast(a[(size_t)h * lda + i] ^ b[(size_t)j * ldb + h]);
}

/*
 * dabnn/layers/BinConv.cpp:80-98,167-189 on a non-ARM target: the layer's
 * forward for one fp32 [h][w][c] image.  c == 64 takes pack_mat +
 * baseline_bconv; anything else zero-fills the output and runs
 * fused_binarize_im2col + bgemm_naive on the transposed weights.
 * wgt holds cout filters of hwc_words words (tools/onnx2bnn/
 * OnnxConverter.cpp:121-156 layout).  Returns the method taken (2 =
 * BCONV_NAIVE, 3 = BGEMM_NAIVE) or a negative error.
 */
ORC_API int orc_binconv_forward(const float *x, int h, int w, int c, const uint64_t *wgt, int hwc_words, int kh,
                                int kw, int pad_h, int pad_w, int stride_h, int stride_w, int cout, float *out) {
    const int oh = orc_out_dim(h, pad_h, kh, 1, stride_h), ow = orc_out_dim(w, pad_w, kw, 1, stride_w);
    if (c % 64 != 0) return -1;
    if (c == 64) {
        uint64_t *bin = (uint64_t *)malloc((size_t)h * w * sizeof(uint64_t));
        if (!bin) return -2;
        orc_pack_mat(x, (size_t)h * w * c, bin);
        orc_baseline_bconv(bin, h, w, 1, wgt, hwc_words, kh, kw, pad_h, pad_w, stride_h, stride_w, 1, 1, cout, out,
                           oh, ow);
        free(bin);
        return 2;
    }
    const int k = hwc_words;
    if (k != orc_col_row_words(kh, kw, c)) return -3;
    uint64_t *col = (uint64_t *)malloc((size_t)oh * ow * k * sizeof(uint64_t));
    uint64_t *wt = (uint64_t *)malloc((size_t)cout * k * sizeof(uint64_t));
    if (!col || !wt) {
        free(col);
        free(wt);
        return -2;
    }
    memset(out, 0, (size_t)oh * ow * cout * sizeof(float));
    orc_fused_binarize_im2col(x, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, 1, 1, col);
    orc_weight_transpose(wgt, cout, k, wt);
    orc_bgemm_naive(cout, oh * ow, k, wt, cout, col, k, out, cout);
    free(col);
    free(wt);
    return 3;
}

/*
 * tools/onnx2bnn/OnnxConverter.cpp:121-156 (bitpack of a weight tensor
 * already in [n][kh][kw][c] order, hwc = kh*kw*c floats per filter).  When
 * c != 64 every filter is zero-bit padded to a multiple of 128 bits.
 * Returns the number of words written per filter.
 */
ORC_API int orc_pack_weight(const float *wf, int n, int hwc, int c, uint64_t *out) {
    if (c == 64) {
        const size_t total = (size_t)n * hwc;
        for (size_t i = 0; i < total / 64; ++i) out[i] = orc_pack_64(wf + 64 * i, 64);
        return hwc / 64;
    }
    const int per = (hwc + 127) / 128 * 2;
    for (int f = 0; f < n; ++f)
        for (int i = 0, wi = 0; i < hwc; i += 128, wi += 2) {
            const int eff = hwc - i < 128 ? hwc - i : 128;
            out[(size_t)f * per + wi] = orc_pack_64(wf + (size_t)f * hwc + i, eff < 64 ? eff : 64);
            out[(size_t)f * per + wi + 1] = eff > 64 ? orc_pack_64(wf + (size_t)f * hwc + i + 64, eff - 64) : 0;
        }
    return per;
}

/*
 * tools/onnx2bnn/OnnxConverter.cpp:583-639 (CalculateCoeff): batch-norm to
 * per-channel a, b; when the BN follows a binary conv with k_bits inputs per
 * output, fold count -> +-1 dot product: b += k_bits*a (+ a*bias), a *= -2.
 */
ORC_API void orc_bn_fold(const float *scale, const float *bias_bn, const float *mean, const float *var, float eps,
                         int n, int k_bits, const float *conv_bias, float *a, float *b) {
    for (int i = 0; i < n; ++i) {
        const float t = sqrtf(var[i] + eps);
        a[i] = scale[i] / t;
        b[i] = bias_bn[i] - scale[i] * mean[i] / t;
    }
    if (k_bits > 0) {
        for (int i = 0; i < n; ++i) {
            b[i] = b[i] + (float)k_bits * a[i];
            if (conv_bias) b[i] += a[i] * conv_bias[i];
        }
        for (int i = 0; i < n; ++i) a[i] *= -2;
    }
}

/*
 * common/baseline.h:37-75 (baseline_fconv): direct fp32 convolution,
 * weights [cout][kh][kw][c], accumulating into out in (kh, kw, c) order.
 * out must be zero-filled by the caller, as in tests/fconv_test.cpp:33-35.
 */
ORC_API void orc_baseline_fconv(const float *x, int h, int w, int c, const float *wgt, int kh, int kw, int pad_h,
                                int pad_w, int stride_h, int stride_w, int dil_h, int dil_w, int cout, float *out,
                                int oh, int ow) {
    int input_y = 0;
    for (int th = 0; th < oh; ++th) {
        int input_x = 0;
        for (int tw = 0; tw < ow; ++tw) {
            for (int tc = 0; tc < cout; ++tc)
                for (int a = 0; a < kh; ++a) {
                    const int y = input_y - pad_h + a * dil_h;
                    for (int b = 0; b < kw; ++b) {
                        const int xx = input_x - pad_w + b * dil_w;
                        const int oob = y < 0 || y >= h || xx < 0 || xx >= w;
                        for (int wc = 0; wc < c; ++wc) {
                            const float wv = wgt[((size_t)tc * kh * kw + (size_t)a * kw + b) * c + wc];
                            const float bv = oob ? 0 : x[((size_t)y * w + xx) * c + wc];
                            out[((size_t)th * ow + tw) * cout + tc] += wv * bv;
                        }
                    }
                }
            input_x += stride_w;
        }
        input_y += stride_h;
    }
}

/*
 * dabnn/fconv.h:14-76: im2col followed by out[n][m] = sum_k W[m][k] *
 * col[n][k] (+ bias[m]); k order (kh, kw, c).  The reference multiplies
 * with Eigen, whose summation order is unspecified; this restatement sums
 * in increasing k with an fp32 accumulator, so agreement with the reference
 * is to rounding (1e-4 relative), not bit-exact.  bias may be NULL.
 */
ORC_API int orc_fconv(const float *x, int h, int w, int c, const float *wgt, const float *bias, int kh, int kw,
                      int pad_h, int pad_w, int stride_h, int stride_w, int dil_h, int dil_w, int cout, float *out) {
    const int oh = orc_out_dim(h, pad_h, kh, dil_h, stride_h), ow = orc_out_dim(w, pad_w, kw, dil_w, stride_w);
    const int K = kh * kw * c, N = oh * ow;
    float *col = (float *)malloc((size_t)N * K * sizeof(float));
    if (!col) return -2;
    orc_im2col(x, h, w, c, 4, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, col);
    for (int n = 0; n < N; ++n)
        for (int m = 0; m < cout; ++m) {
            float acc = 0.f;
            const float *wr = wgt + (size_t)m * K, *cr = col + (size_t)n * K;
            for (int k = 0; k < K; ++k) acc += wr[k] * cr[k];
            out[(size_t)n * cout + m] = bias ? acc + bias[m] : acc;
        }
    free(col);
    return 0;
}

/* dabnn/layers/Affine.cpp:10-23: x[..., c] = a[c] * x[..., c] + b[c]. */
ORC_API void orc_affine_inplace(float *x, size_t n_pix, int c, const float *a, const float *b) {
    for (size_t p = 0; p < n_pix; ++p)
        for (int i = 0; i < c; ++i) x[p * c + i] = a[i] * x[p * c + i] + b[i];
}

/* dabnn/layers/Add.cpp:7-17: a += b. */
ORC_API void orc_add_inplace(float *a, const float *b, size_t n) {
    for (size_t i = 0; i < n; ++i) a[i] += b[i];
}

/*
 * dabnn/layers/PRelu.cpp:6-30: a negative value is multiplied by the slope
 * (slope_n == 1) or by its channel's slope (slope_n == c).  Returns nonzero
 * for any other slope_n, where the reference asserts.
 */
ORC_API int orc_prelu_inplace(float *x, size_t n_pix, int c, const float *slope, int slope_n) {
    if (slope_n != 1 && slope_n != c) return 1;
    for (size_t p = 0; p < n_pix; ++p)
        for (int i = 0; i < c; ++i) {
            float *v = x + p * c + i;
            if (*v < 0) *v = *v * slope[slope_n == 1 ? 0 : i];
        }
    return 0;
}

/* dabnn/layers/Concat.cpp:7-21: per pixel, the ca values of a and then the cb values of b. */
ORC_API void orc_concat(const float *a, int ca, const float *b, int cb, size_t n_pix, float *out) {
    for (size_t p = 0; p < n_pix; ++p) {
        memcpy(out, a + p * ca, (size_t)ca * sizeof(float));
        out += ca;
        memcpy(out, b + p * cb, (size_t)cb * sizeof(float));
        out += cb;
    }
}

/*
 * dabnn/layers/Split.cpp:6-21: per pixel, the first c/2 words go to out1, the
 * other c/2 to out2 (c = words per pixel).
 */
ORC_API void orc_split_bit(const uint64_t *x, size_t n_pix, int c, uint64_t *out1, uint64_t *out2) {
    const int c_per_output = c / 2;
    for (size_t p = 0; p < n_pix; ++p) {
        memcpy(out1, x, (size_t)c_per_output * sizeof(uint64_t));
        out1 += c_per_output;
        x += c_per_output;
        memcpy(out2, x, (size_t)c_per_output * sizeof(uint64_t));
        out2 += c_per_output;
        x += c_per_output;
    }
}

/*
 * dabnn/layers/Shuffle.cpp:6-43, in place: 128 channels -- 32-bit quarters 1
 * and 2 of a pixel change places; 256 -- words 1 and 2; 512 -- words 2,3 and
 * 4,5; other channel counts are left alone (the reference has no branch for
 * them).  n_pix pixels of elem_c / 64 words.
 */
ORC_API void orc_shuffle_bit(uint64_t *x, size_t n_pix, int elem_c) {
    if (elem_c == 128) {
        uint32_t *ptr = (uint32_t *)x;
        for (size_t p = 0; p < n_pix; ++p) {
            const uint32_t tmp = ptr[1];
            ptr[1] = ptr[2];
            ptr[2] = tmp;
            ptr += 4;
        }
    } else if (elem_c == 256) {
        for (size_t p = 0; p < n_pix; ++p) {
            const uint64_t tmp = x[1];
            x[1] = x[2];
            x[2] = tmp;
            x += 4;
        }
    } else if (elem_c == 512) {
        for (size_t p = 0; p < n_pix; ++p) {
            const uint64_t tmp1 = x[2], tmp2 = x[3];
            x[2] = x[4];
            x[3] = x[5];
            x[4] = tmp1;
            x[5] = tmp2;
            x += 8;
        }
    }
}

/*
 * dabnn/layers/AvePool.cpp:84-123 (ave_pool_fallback): mean over the taps
 * that fall inside the image (divisor = in-bounds tap count).
 */
ORC_API void orc_ave_pool(const float *x, int h, int w, int c, int pad_h, int pad_w, int stride_h, int stride_w,
                          int kh, int kw, float *out) {
    const int oh = orc_out_dim(h, pad_h, kh, 1, stride_h), ow = orc_out_dim(w, pad_w, kw, 1, stride_w);
    int input_y = 0;
    for (int oy = 0; oy < oh; ++oy) {
        int input_x = 0;
        for (int ox = 0; ox < ow; ++ox) {
            for (int oc = 0; oc < c; ++oc) {
                size_t n = 0;
                float sum = 0;
                for (int a = 0; a < kh; ++a) {
                    const int y = input_y - pad_h + a;
                    for (int b = 0; b < kw; ++b) {
                        const int xx = input_x - pad_w + b;
                        if (!(y < 0 || y >= h || xx < 0 || xx >= w)) {
                            sum += x[((size_t)y * w + xx) * c + oc];
                            n++;
                        }
                    }
                }
                out[((size_t)oy * ow + ox) * c + oc] = sum / n;
            }
            input_x += stride_w;
        }
        input_y += stride_h;
    }
}

/*
 * dabnn/layers/MaxPool.cpp:209-246 (max_pool_fallback): max over in-bounds
 * taps starting from -FLT_MAX.
 */
ORC_API void orc_max_pool(const float *x, int h, int w, int c, int pad_h, int pad_w, int stride_h, int stride_w,
                          int kh, int kw, float *out) {
    const int oh = orc_out_dim(h, pad_h, kh, 1, stride_h), ow = orc_out_dim(w, pad_w, kw, 1, stride_w);
    int input_y = 0;
    for (int oy = 0; oy < oh; ++oy) {
        int input_x = 0;
        for (int ox = 0; ox < ow; ++ox) {
            for (int oc = 0; oc < c; ++oc) {
                float m = -FLT_MAX;
                for (int a = 0; a < kh; ++a) {
                    const int y = input_y - pad_h + a;
                    for (int b = 0; b < kw; ++b) {
                        const int xx = input_x - pad_w + b;
                        if (!(y < 0 || y >= h || xx < 0 || xx >= w)) {
                            const float v = x[((size_t)y * w + xx) * c + oc];
                            m = v > m ? v : m;
                        }
                    }
                }
                out[((size_t)oy * ow + ox) * c + oc] = m;
            }
            input_x += stride_w;
        }
        input_y += stride_h;
    }
}
