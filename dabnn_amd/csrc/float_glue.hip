// fp32 layers that sit between the binary convolutions of a Bi-Real-style net:
// fconv, per-channel affine, add, average and max pooling.  All NHWC.
#include <float.h>

#include "common.h"

namespace dab {

// ---------------------------------------------------------------- fconv
// Implicit GEMM: rows = output pixels (N*OH*OW), columns = output channels,
// depth = kh*kw*c in the reference's (kh, kw, c) order (dabnn/fconv.h:33-41,
// dabnn/im2col.h:14-47).  64x64 output tile per 256-thread block, 16-deep
// slices staged in LDS, 4x4 accumulators per thread.
struct FconvArgs {
    const float *x;
    const float *w;
    const float *bias;
    float *out;
    int n, h, wd, c;
    int kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w;
    int oh, ow, cout;
    int K;        // kh*kw*c
    int M;        // n*oh*ow
    FastDiv div_c, div_kw, div_ow, div_oh;
};

constexpr int kFTile = 64, kFDepth = 16;

__global__ __launch_bounds__(256) void fconv_kernel(const FconvArgs p) {
    __shared__ float As[kFDepth][kFTile + 4];  // [k][pixel]
    __shared__ float Bs[kFDepth][kFTile + 4];  // [k][cout]
    const int tid = threadIdx.x;
    const int m0 = blockIdx.x * kFTile, n0 = blockIdx.y * kFTile;
    const int tx = tid & 15, ty = tid >> 4;  // 16 x 16 threads, 4 x 4 outputs each

    // loader roles: each thread fetches 4 elements of A and 4 of B per slice
    const int l_row = tid >> 2;        // 0..63: pixel (A) or cout (B) within the tile
    const int l_k = (tid & 3) * 4;     // 0,4,8,12: first k of this thread's 4
    const int pix = m0 + l_row;
    const bool pix_ok = pix < p.M;
    int oy = 0, ox = 0, img = 0;
    if (pix_ok) {
        const uint32_t t = p.div_ow.div((uint32_t)pix);
        ox = pix - t * p.ow;
        img = p.div_oh.div(t);
        oy = t - img * p.oh;
    }
    const int y0 = oy * p.stride_h - p.pad_h, x0 = ox * p.stride_w - p.pad_w;
    const int co_l = n0 + l_row;

    float acc[4][4] = {};
    for (int k0 = 0; k0 < p.K; k0 += kFDepth) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + l_k + i;
            float av = 0.f, bv = 0.f;
            if (k < p.K) {
                if (pix_ok) {
                    const uint32_t tap = p.div_c.div((uint32_t)k);
                    const int ch = k - tap * p.c;
                    const uint32_t a = p.div_kw.div(tap);
                    const int b = tap - a * p.kw;
                    const int y = y0 + (int)a * p.dil_h, xx = x0 + b * p.dil_w;
                    if (y >= 0 && y < p.h && xx >= 0 && xx < p.wd) av = p.x[(((size_t)img * p.h + y) * p.wd + xx) * p.c + ch];
                }
                if (co_l < p.cout) bv = p.w[(size_t)co_l * p.K + k];
            }
            As[l_k + i][l_row] = av;
            Bs[l_k + i][l_row] = bv;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < kFDepth; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i], b[i] = Bs[kk][tx * 4 + i];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= p.M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int co = n0 + tx * 4 + j;
            if (co < p.cout) p.out[(size_t)m * p.cout + co] = p.bias ? acc[i][j] + p.bias[co] : acc[i][j];
        }
    }
}

// ---------------------------------------------------------------- elementwise
// Affine.cpp:10-23.  Multiply and add are kept as two roundings, as the
// reference's x86 build does, so results match it bit for bit.
__global__ __launch_bounds__(256) void affine_kernel(float *__restrict__ x, long long total, int c,
                                                     const float *__restrict__ a, const float *__restrict__ b) {
#pragma clang fp contract(off)
    const long long stride = (long long)gridDim.x * 256;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
        const int ch = (int)(i % c);
        const float prod = a[ch] * x[i];  // no contraction under the pragma above: two roundings
        x[i] = prod + b[ch];
    }
}

__global__ __launch_bounds__(256) void add_kernel(float *__restrict__ a, const float *__restrict__ b, long long total) {
    const long long stride = (long long)gridDim.x * 256;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) a[i] = __fadd_rn(a[i], b[i]);
}

__global__ __launch_bounds__(256) void relu_kernel(float *__restrict__ x, long long total) {
    const long long stride = (long long)gridDim.x * 256;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) x[i] = x[i] > 0.f ? x[i] : 0.f;
}

__global__ __launch_bounds__(256) void fill_kernel(float *__restrict__ x, long long total, float v) {
    const long long stride = (long long)gridDim.x * 256;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) x[i] = v;
}

// ---------------------------------------------------------------- pooling
struct PoolArgs {
    const float *x;
    float *out;
    int n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, oh, ow;
};

// AvePool.cpp:84-123 (MAX = false) and MaxPool.cpp:209-246 (MAX = true);
// taps are visited in the reference's order so the fp32 sum rounds alike.
template <bool MAX>
__global__ __launch_bounds__(256) void pool_kernel(const PoolArgs p) {
    const long long total = (long long)p.n * p.oh * p.ow * p.c;
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int ch = (int)(idx % p.c);
    long long t = idx / p.c;
    const int ox = (int)(t % p.ow);
    t /= p.ow;
    const int oy = (int)(t % p.oh);
    const long long img = t / p.oh;
    float m = -FLT_MAX, sum = 0.f;
    int cnt = 0;
    for (int a = 0; a < p.kh; ++a) {
        const int y = oy * p.stride_h - p.pad_h + a;
        for (int b = 0; b < p.kw; ++b) {
            const int xx = ox * p.stride_w - p.pad_w + b;
            if (y >= 0 && y < p.h && xx >= 0 && xx < p.w) {
                const float v = p.x[((img * p.h + y) * p.w + xx) * p.c + ch];
                if (MAX)
                    m = v > m ? v : m;
                else
                    sum = __fadd_rn(sum, v), ++cnt;
            }
        }
    }
    p.out[idx] = MAX ? m : __fdiv_rn(sum, (float)cnt);
}

static unsigned grid_for(long long total) {
    long long b = (total + 255) / 256;
    const long long cap = (long long)simd_count() * 16;
    if (b > cap) b = cap;
    return (unsigned)(b < 1 ? 1 : b);
}

int fill_f32(float *x, long long total, float v, hipStream_t s) {
    hipLaunchKernelGGL(fill_kernel, dim3(grid_for(total)), dim3(256), 0, s, x, total, v);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

}  // namespace dab

extern "C" int dab_fconv(const float *x, int n, int h, int w, int c, const float *wgt, const float *bias, int kh, int kw,
                         int pad_h, int pad_w, int stride_h, int stride_w, int dil_h, int dil_w, int cout, float *out,
                         dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(x && wgt && out, "dab_fconv: null pointer");
    DAB_REQUIRE(n > 0 && h > 0 && w > 0 && c > 0 && kh > 0 && kw > 0 && cout > 0, "dab_fconv: non-positive dimension");
    DAB_REQUIRE(pad_h >= 0 && pad_w >= 0 && stride_h > 0 && stride_w > 0 && dil_h > 0 && dil_w > 0,
                "dab_fconv: bad pad/stride/dilation");
    FconvArgs a;
    a.x = x, a.w = wgt, a.bias = bias, a.out = out;
    a.n = n, a.h = h, a.wd = w, a.c = c;
    a.kh = kh, a.kw = kw, a.pad_h = pad_h, a.pad_w = pad_w, a.stride_h = stride_h, a.stride_w = stride_w;
    a.dil_h = dil_h, a.dil_w = dil_w;
    a.oh = out_dim(h, pad_h, kh, dil_h, stride_h), a.ow = out_dim(w, pad_w, kw, dil_w, stride_w);
    DAB_REQUIRE(a.oh > 0 && a.ow > 0, "dab_fconv: empty output");
    a.cout = cout;
    a.K = kh * kw * c;
    const long long M = (long long)n * a.oh * a.ow;
    if (M >= (1ll << 31) - 64) return fail(DAB_EUNSUPPORTED, "dab_fconv: too many output pixels");
    a.M = (int)M;
    a.div_c = FastDiv((uint32_t)c), a.div_kw = FastDiv((uint32_t)kw);
    a.div_ow = FastDiv((uint32_t)a.ow), a.div_oh = FastDiv((uint32_t)a.oh);
    dim3 grid((unsigned)((M + kFTile - 1) / kFTile), (unsigned)((cout + kFTile - 1) / kFTile));
    hipLaunchKernelGGL(fconv_kernel, grid, dim3(256), 0, as_stream(stream), a);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

extern "C" int dab_affine_inplace(float *x, int64_t n_pix, int c, const float *a, const float *b, dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(x && a && b, "dab_affine_inplace: null pointer");
    DAB_REQUIRE(n_pix > 0 && c > 0, "dab_affine_inplace: n_pix %lld c %d", (long long)n_pix, c);
    const long long total = (long long)n_pix * c;
    hipLaunchKernelGGL(affine_kernel, dim3(grid_for(total)), dim3(256), 0, as_stream(stream), x, total, c, a, b);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

extern "C" int dab_add_inplace(float *a, const float *b, int64_t n_elem, dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(a && b, "dab_add_inplace: null pointer");
    DAB_REQUIRE(n_elem > 0, "dab_add_inplace: n_elem %lld", (long long)n_elem);
    hipLaunchKernelGGL(add_kernel, dim3(grid_for(n_elem)), dim3(256), 0, as_stream(stream), a, b, (long long)n_elem);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

extern "C" int dab_relu_inplace(float *x, int64_t n_elem, dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(x, "dab_relu_inplace: null pointer");
    DAB_REQUIRE(n_elem > 0, "dab_relu_inplace: n_elem %lld", (long long)n_elem);
    hipLaunchKernelGGL(relu_kernel, dim3(grid_for(n_elem)), dim3(256), 0, as_stream(stream), x, (long long)n_elem);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

extern "C" int dab_fill_f32(float *x, int64_t n_elem, float value, dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(x, "dab_fill_f32: null pointer");
    DAB_REQUIRE(n_elem > 0, "dab_fill_f32: n_elem %lld", (long long)n_elem);
    return fill_f32(x, (long long)n_elem, value, as_stream(stream));
}

static int pool_common(bool is_max, const float *x, int n, int h, int w, int c, int kh, int kw, int pad_h, int pad_w,
                       int stride_h, int stride_w, float *out, dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(x && out, "dab_pool: null pointer");
    DAB_REQUIRE(n > 0 && h > 0 && w > 0 && c > 0 && kh > 0 && kw > 0, "dab_pool: non-positive dimension");
    DAB_REQUIRE(pad_h >= 0 && pad_w >= 0 && stride_h > 0 && stride_w > 0, "dab_pool: bad pad/stride");
    PoolArgs a;
    a.x = x, a.out = out;
    a.n = n, a.h = h, a.w = w, a.c = c, a.kh = kh, a.kw = kw;
    a.pad_h = pad_h, a.pad_w = pad_w, a.stride_h = stride_h, a.stride_w = stride_w;
    a.oh = out_dim(h, pad_h, kh, 1, stride_h), a.ow = out_dim(w, pad_w, kw, 1, stride_w);
    DAB_REQUIRE(a.oh > 0 && a.ow > 0, "dab_pool: empty output");
    const long long total = (long long)n * a.oh * a.ow * c;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (is_max)
        hipLaunchKernelGGL(pool_kernel<true>, dim3(blocks), dim3(256), 0, as_stream(stream), a);
    else
        hipLaunchKernelGGL(pool_kernel<false>, dim3(blocks), dim3(256), 0, as_stream(stream), a);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

extern "C" int dab_ave_pool(const float *x, int n, int h, int w, int c, int kh, int kw, int pad_h, int pad_w,
                            int stride_h, int stride_w, float *out, dab_stream_t stream) {
    return pool_common(false, x, n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, out, stream);
}

extern "C" int dab_max_pool(const float *x, int n, int h, int w, int c, int kh, int kw, int pad_h, int pad_w,
                            int stride_h, int stride_w, float *out, dab_stream_t stream) {
    return pool_common(true, x, n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, out, stream);
}
