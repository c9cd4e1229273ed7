// BinConv::forward_impl (dabnn/layers/BinConv.cpp:144-191) as one call:
// binarise the fp32 input and run the binary convolution, choosing between
// the direct 3x3 kernel and im2col + bgemm the way BinConv::method() (:80-98)
// does on the reference's optimised targets.
#include <mutex>

#include "common.h"

namespace dab {

// Scratch of dab_binconv_forward_static: the packed activations (direct arm) or the column matrix (bgemm arm) of one
// call.  One copy per GPU, held until the process ends; the array's name is only a handle for hipGetSymbolAddress in
// host code, the kernels get the device address that call returns.
static __device__ __align__(256) unsigned char scratch[DAB_BINCONV_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
static void *scratch_ptr[kMaxDevices];  // device address of `scratch` on each GPU, resolved on the first call there
static std::mutex scratch_mutex;

// Device address of this GPU's copy of `scratch` (the current device's).
static int static_scratch(void **out) {
    int dev = 0;
    DAB_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(DAB_EUNSUPPORTED, "dab_binconv_forward_static: device index %d", dev);
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (scratch_ptr[dev] == nullptr) {
        void *p = nullptr;
        DAB_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (p == nullptr) return fail(DAB_EHIP, "dab_binconv_forward_static: no device address for the scratch array");
        scratch_ptr[dev] = p;
    }
    *out = scratch_ptr[dev];
    return DAB_OK;
}


static bool direct_ok(int c, int kh, int kw, int pad_h, int pad_w, int stride_h, int stride_w, int cout) {
    // dabnn/layers/BinConv.cpp:100-126: 3x3, equal strides, 64/128/256/512/1024 input channels
    return kh == 3 && kw == 3 && stride_h == stride_w && pad_h == pad_w &&
           (c == 64 || c == 128 || c == 256 || c == 512 || c == 1024) && cout % 8 == 0;
}
}  // namespace dab

extern "C" size_t dab_binconv_workspace_bytes(int n, int h, int w, int c, int kh, int kw, int pad_h, int pad_w,
                                              int stride_h, int stride_w) {
    using namespace dab;
    if (n <= 0 || h <= 0 || w <= 0 || c <= 0 || kh <= 0 || kw <= 0 || stride_h <= 0 || stride_w <= 0) return 0;
    const size_t packed = (size_t)n * h * w * ((c + 63) / 64) * 8;
    const int oh = out_dim(h, pad_h, kh, 1, stride_h), ow = out_dim(w, pad_w, kw, 1, stride_w);
    const size_t col = (size_t)n * (oh > 0 ? oh : 0) * (ow > 0 ? ow : 0) * dab_col_row_words(kh, kw, c) * 8;
    return packed > col ? packed : col;
}

extern "C" int dab_binconv_forward(const float *x, int n, int h, int w, int c, const uint64_t *wgt, const uint64_t *wgt_t,
                                   int hwc_words, int kh, int kw, int pad_h, int pad_w, int stride_h, int stride_w,
                                   int cout, float *out, void *workspace, size_t workspace_bytes, int *method_out,
                                   dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(x && out && workspace, "dab_binconv_forward: null pointer");
    DAB_REQUIRE(n > 0 && h > 0 && w > 0 && c > 0 && cout > 0 && kh > 0 && kw > 0, "dab_binconv_forward: non-positive dimension");
    DAB_REQUIRE(c % 64 == 0, "dab_binconv_forward: c %d is not a multiple of 64", c);
    DAB_REQUIRE(workspace_bytes >= dab_binconv_workspace_bytes(n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w),
                "dab_binconv_forward: workspace too small");
    const int oh = out_dim(h, pad_h, kh, 1, stride_h), ow = out_dim(w, pad_w, kw, 1, stride_w);
    DAB_REQUIRE(oh > 0 && ow > 0, "dab_binconv_forward: empty output");

    if (direct_ok(c, kh, kw, pad_h, pad_w, stride_h, stride_w, cout)) {
        DAB_REQUIRE(wgt, "dab_binconv_forward: direct method needs wgt");
        DAB_REQUIRE(hwc_words == 9 * (c / 64), "dab_binconv_forward: %d words per filter, expected %d", hwc_words,
                    9 * (c / 64));
        uint64_t *packed = static_cast<uint64_t *>(workspace);
        int rc = dab_bitpack_nhwc(x, packed, (int64_t)n * h * w, c, stream);
        if (rc != DAB_OK) return rc;
        rc = dab_bconv3x3(packed, n, h, w, c, wgt, cout, stride_h, pad_h, out, stream);
        if (rc == DAB_OK && method_out) *method_out = 0;
        return rc;
    }

    DAB_REQUIRE(wgt_t, "dab_binconv_forward: bgemm method needs the transposed weights");
    const int row_words = dab_col_row_words(kh, kw, c);
    DAB_REQUIRE(hwc_words <= row_words && hwc_words * 64 >= kh * kw * c,
                "dab_binconv_forward: %d words per filter does not match a %dx%dx%d filter", hwc_words, kh, kw, c);
    uint64_t *col = static_cast<uint64_t *>(workspace);
    const long long npix = (long long)n * oh * ow;
    if (npix >= (1ll << 31)) return fail(DAB_EUNSUPPORTED, "dab_binconv_forward: too many output pixels");
    // output_mat->fill<float>(0.f) and the accumulation into it (BinConv.cpp:153-165) are one store: 0.f + count == count
    int rc = dab_fused_binarize_im2col(x, n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, 1, 1, col, stream);
    if (rc != DAB_OK) return rc;
    rc = dab_bgemm_overwrite(cout, (int)npix, hwc_words, wgt_t, cout, col, row_words, out, cout, stream);
    if (rc == DAB_OK && method_out) *method_out = 1;
    return rc;
}

extern "C" int dab_binconv_forward_static(const float *x, int n, int h, int w, int c, const uint64_t *wgt,
                                          const uint64_t *wgt_t, int hwc_words, int kh, int kw, int pad_h, int pad_w,
                                          int stride_h, int stride_w, int cout, float *out, int *method_out,
                                          dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(n > 0 && h > 0 && w > 0 && c > 0 && kh > 0 && kw > 0 && stride_h > 0 && stride_w > 0,
                "dab_binconv_forward_static: non-positive dimension");
    const size_t need = dab_binconv_workspace_bytes(n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w);
    if (need > (size_t)DAB_BINCONV_STATIC_SCRATCH_BYTES)
        return fail(DAB_EUNSUPPORTED,
                    "dab_binconv_forward_static: this problem needs %zu bytes of scratch, the static buffer holds %zu; "
                    "use dab_binconv_forward with a workspace of your own",
                    need, (size_t)DAB_BINCONV_STATIC_SCRATCH_BYTES);
    void *ws = nullptr;
    const int rc = static_scratch(&ws);
    if (rc != DAB_OK) return rc;
    // both arms overwrite every word of the scratch they read, so nothing of the previous call has to be cleared
    return dab_binconv_forward(x, n, h, w, c, wgt, wgt_t, hwc_words, kh, kw, pad_h, pad_w, stride_h, stride_w, cout, out,
                               ws, (size_t)DAB_BINCONV_STATIC_SCRATCH_BYTES, method_out, stream);
}
