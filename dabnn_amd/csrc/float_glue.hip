// fp32 layers that sit between the binary convolutions of a Bi-Real-style net:
// fconv, per-channel affine, add, average and max pooling.  All NHWC.
#include <float.h>

#include "common.h"

namespace dab {

// ---------------------------------------------------------------- fconv
// Implicit GEMM: rows = output pixels (N*OH*OW), columns = output channels,
// depth = kh*kw*c in the reference's (kh, kw, c) order (dabnn/fconv.h:33-41,
// dabnn/im2col.h:14-47).  This is the one GEMM-shaped fp32 layer of the path, so
// it runs on the matrix cores: v_mfma_f32_32x32x2_f32, fp32 in and fp32 accumulate.
// A 256-thread block owns a 128 x BN output tile (BN = 32, 64 or 128) as four
// wave tiles; 16-deep slices of the gathered image patch and of the weights are
// staged in two LDS buffers, the next slice fetched into registers while the
// current one is multiplied.  A depth index is the same for all lanes of a wave
// while it loads, so its decoding into (tap row, tap column, channel) runs once
// per wave on the scalar unit.
// Epilogue: + bias, then optionally the Affine (a*v + b, two roundings) and Relu
// layers that follow the convolution, in the reference's order of operations.
struct FconvArgs {
    const float *x;
    const float *w;
    const float *bias;
    const float *aff_a;
    const float *aff_b;
    float *out;
    int n, h, wd, c;
    int kw, dil_h, dil_w;
    int pad_h, pad_w, stride_h, stride_w;
    int oh, ow, cout;
    int K;  // kh*kw*c
    int M;  // n*oh*ow
    int relu;
    FastDiv div_ow, div_oh, div_c, div_kw;
};

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kFM = 128, kFK = 16;

template <int BN>
__global__ __launch_bounds__(256) void fconv_kernel(const FconvArgs p) {
    constexpr int WAVES_N = BN >= 64 ? 2 : 1, WAVES_M = 4 / WAVES_N;
    constexpr int WTM = kFM / WAVES_M, WTN = BN / WAVES_N;  // wave tile
    constexpr int TM = WTM / 32, TN = WTN / 32;             // 32 x 32 matrix-core tiles per wave
    constexpr int BPT = BN / 16;                            // weights fetched per thread and slice
    // row strides of 32 (mod 64) floats: the two half-waves of a fragment read land in different banks
    constexpr int AS = kFM + 32, BS = (BN % 64 == 32) ? BN : BN + 32;
    __shared__ float As[2][kFK][AS];  // [k][pixel]
    __shared__ float Bs[2][kFK][BS];  // [k][cout]
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int m0 = blockIdx.x * kFM, n0 = blockIdx.y * BN;

    // A loader: this thread always fetches pixel (tid % 128), depth rows (tid / 128) + 2*i
    const int l_m = tid & 127, l_kk = __builtin_amdgcn_readfirstlane(tid >> 7);
    const int pix = m0 + l_m;
    const bool pix_ok = pix < p.M;
    int y0 = 0, x0 = 0;
    const float *xpix = p.x;
    if (pix_ok) {
        const uint32_t t = p.div_ow.div((uint32_t)pix);
        const int ox = pix - t * p.ow;
        const uint32_t img = p.div_oh.div(t);
        const int oy = t - img * p.oh;
        y0 = oy * p.stride_h - p.pad_h, x0 = ox * p.stride_w - p.pad_w;
        // signed 64-bit arithmetic: y0 and x0 are negative inside the padding; the pointer is only used in bounds
        xpix = p.x + (((long long)img * p.h + y0) * p.wd + x0) * p.c;
    }
    // B loader: depth (tid % 16), output channels (tid / 16) + 16*j
    const int b_k = tid & 15, b_n = tid >> 4;

    float a_reg[8], b_reg[BPT];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int k = k0 + l_kk + 2 * i;
            float v = 0.f;
            if (k < p.K) {
                const int tap = (int)p.div_c.div((uint32_t)k), ch = k - tap * p.c;
                const int ty = (int)p.div_kw.div((uint32_t)tap), tx = tap - ty * p.kw;
                const int dy = ty * p.dil_h, dx = tx * p.dil_w;
                const int y = y0 + dy, xx = x0 + dx;
                if (pix_ok && (unsigned)y < (unsigned)p.h && (unsigned)xx < (unsigned)p.wd)
                    v = xpix[(dy * p.wd + dx) * p.c + ch];
            }
            a_reg[i] = v;
        }
#pragma unroll
        for (int j = 0; j < BPT; ++j) {
            const int co = n0 + b_n + 16 * j, k = k0 + b_k;
            b_reg[j] = (co < p.cout && k < p.K) ? p.w[(size_t)co * p.K + k] : 0.f;
        }
    };
    auto commit = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 8; ++i) As[buf][l_kk + 2 * i][l_m] = a_reg[i];
#pragma unroll
        for (int j = 0; j < BPT; ++j) Bs[buf][b_k][b_n + 16 * j] = b_reg[j];
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    // fragment addressing of v_mfma_f32_32x32x2_f32: lane l supplies row/column l % 32 at depth l / 32
    const int f_k = lane >> 5, f_i = lane & 31;
    fetch(0);
    commit(0);
    __syncthreads();
    int buf = 0;
    for (int k0 = 0; k0 < p.K; k0 += kFK, buf ^= 1) {
        const bool more = k0 + kFK < p.K;
        if (more) fetch(k0 + kFK);
#pragma unroll
        for (int kp = 0; kp < kFK / 2; ++kp) {
            float a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) a[i] = As[buf][kp * 2 + f_k][wm * WTM + i * 32 + f_i];
#pragma unroll
            for (int j = 0; j < TN; ++j) b[j] = Bs[buf][kp * 2 + f_k][wn * WTN + j * 32 + f_i];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        // the other buffer was last read before the barrier that ended the previous slice
        if (more) commit(buf ^ 1);
        __syncthreads();
    }

    // accumulator element e of lane l: row 8*(e/4) + 4*(l/32) + e%4, column l % 32
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int co = n0 + wn * WTN + j * 32 + f_i;
        if (co >= p.cout) continue;
        const float bias = p.bias ? p.bias[co] : 0.f;
        const float fa = p.aff_a ? p.aff_a[co] : 0.f, fb = p.aff_a ? p.aff_b[co] : 0.f;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm * WTM + i * 32 + 8 * (e / 4) + 4 * f_k + (e % 4);
                if (m >= p.M) continue;
                {
#pragma clang fp contract(off)
                    float v = acc[i][j][e];
                    if (p.bias) v = v + bias;
                    if (p.aff_a) {
                        const float prod = fa * v;
                        v = prod + fb;
                    }
                    if (p.relu) v = v > 0.f ? v : 0.f;
                    p.out[(size_t)m * p.cout + co] = v;
                }
            }
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

// Same pooling for c % 4 == 0 and fewer than 2^31 outputs: four channels per thread through 16-byte accesses and
// multiply-high divisions in place of 64-bit ones.
struct PoolVecArgs {
    PoolArgs g;
    int c4;         // c / 4
    uint32_t total; // n*oh*ow*c4
    FastDiv div_c4, div_ow, div_oh;
};

template <bool MAX>
__global__ __launch_bounds__(256) void pool_vec4_kernel(const float4 *__restrict__ x, float4 *__restrict__ out,
                                                        const PoolVecArgs p) {
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    if (idx >= p.total) return;
    uint32_t t = p.div_c4.div(idx);
    const int ch = (int)(idx - t * p.c4);
    uint32_t t2 = p.div_ow.div(t);
    const int ox = (int)(t - t2 * p.g.ow);
    const uint32_t img = p.div_oh.div(t2);
    const int oy = (int)(t2 - img * p.g.oh);
    float4 m = make_float4(-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX), sum = make_float4(0.f, 0.f, 0.f, 0.f);
    int cnt = 0;
    const int ys = oy * p.g.stride_h - p.g.pad_h, xs = ox * p.g.stride_w - p.g.pad_w;
    for (int a = 0; a < p.g.kh; ++a) {
        const int y = ys + a;
        if ((unsigned)y >= (unsigned)p.g.h) continue;
        const float4 *row = x + ((size_t)img * p.g.h + y) * p.g.w * p.c4 + ch;
        for (int b = 0; b < p.g.kw; ++b) {
            const int xx = xs + b;
            if ((unsigned)xx >= (unsigned)p.g.w) continue;
            const float4 v = row[(size_t)xx * p.c4];
            if (MAX) {
                m.x = v.x > m.x ? v.x : m.x, m.y = v.y > m.y ? v.y : m.y;
                m.z = v.z > m.z ? v.z : m.z, m.w = v.w > m.w ? v.w : m.w;
            } else {
#pragma clang fp contract(off)
                sum.x = sum.x + v.x, sum.y = sum.y + v.y, sum.z = sum.z + v.z, sum.w = sum.w + v.w;
                ++cnt;
            }
        }
    }
    if (MAX) {
        out[idx] = m;
    } else {
        const float d = (float)cnt;
        out[idx] = make_float4(__fdiv_rn(sum.x, d), __fdiv_rn(sum.y, d), __fdiv_rn(sum.z, d), __fdiv_rn(sum.w, d));
    }
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

static int fconv_impl(const char *fn, const float *x, int n, int h, int w, int c, const float *wgt, const float *bias,
                      const float *aff_a, const float *aff_b, int relu, int kh, int kw, int pad_h, int pad_w, int stride_h,
                      int stride_w, int dil_h, int dil_w, int cout, float *out, dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(x && wgt && out, "%s: null pointer", fn);
    DAB_REQUIRE(n > 0 && h > 0 && w > 0 && c > 0 && kh > 0 && kw > 0 && cout > 0, "%s: non-positive dimension", fn);
    DAB_REQUIRE(pad_h >= 0 && pad_w >= 0 && stride_h > 0 && stride_w > 0 && dil_h > 0 && dil_w > 0,
                "%s: bad pad/stride/dilation", fn);
    DAB_REQUIRE((aff_a == nullptr) == (aff_b == nullptr), "%s: affine needs both coefficient vectors", fn);
    FconvArgs a;
    a.x = x, a.w = wgt, a.bias = bias, a.aff_a = aff_a, a.aff_b = aff_b, a.relu = relu, a.out = out;
    a.n = n, a.h = h, a.wd = w, a.c = c;
    a.pad_h = pad_h, a.pad_w = pad_w, a.stride_h = stride_h, a.stride_w = stride_w;
    a.oh = out_dim(h, pad_h, kh, dil_h, stride_h), a.ow = out_dim(w, pad_w, kw, dil_w, stride_w);
    DAB_REQUIRE(a.oh > 0 && a.ow > 0, "%s: empty output", fn);
    a.cout = cout;
    a.K = kh * kw * c;
    const long long M = (long long)n * a.oh * a.ow;
    if (M >= (1ll << 31) - kFM || (long long)n * h * w * c >= (1ll << 31))
        return fail(DAB_EUNSUPPORTED, "%s: tensor too large for 32-bit indexing", fn);
    a.M = (int)M;
    a.div_ow = FastDiv((uint32_t)a.ow), a.div_oh = FastDiv((uint32_t)a.oh);
    a.kw = kw, a.dil_h = dil_h, a.dil_w = dil_w;
    a.div_c = FastDiv((uint32_t)c), a.div_kw = FastDiv((uint32_t)kw);
    hipStream_t s = as_stream(stream);
    const unsigned gx = (unsigned)((M + kFM - 1) / kFM);
    if (cout <= 32) {
        hipLaunchKernelGGL(fconv_kernel<32>, dim3(gx, 1), dim3(256), 0, s, a);
    } else if (cout <= 64) {
        hipLaunchKernelGGL(fconv_kernel<64>, dim3(gx, 1), dim3(256), 0, s, a);
    } else {
        hipLaunchKernelGGL(fconv_kernel<128>, dim3(gx, (unsigned)((cout + 127) / 128)), dim3(256), 0, s, a);
    }
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

extern "C" int dab_fconv(const float *x, int n, int h, int w, int c, const float *wgt, const float *bias, int kh, int kw,
                         int pad_h, int pad_w, int stride_h, int stride_w, int dil_h, int dil_w, int cout, float *out,
                         dab_stream_t stream) {
    return fconv_impl("dab_fconv", x, n, h, w, c, wgt, bias, nullptr, nullptr, 0, kh, kw, pad_h, pad_w, stride_h, stride_w,
                      dil_h, dil_w, cout, out, stream);
}

extern "C" int dab_fconv_affine_relu(const float *x, int n, int h, int w, int c, const float *wgt, const float *bias,
                                     const float *a, const float *b, int relu, int kh, int kw, int pad_h, int pad_w,
                                     int stride_h, int stride_w, int dil_h, int dil_w, int cout, float *out,
                                     dab_stream_t stream) {
    return fconv_impl("dab_fconv_affine_relu", x, n, h, w, c, wgt, bias, a, b, relu, kh, kw, pad_h, pad_w, stride_h,
                      stride_w, dil_h, dil_w, cout, out, stream);
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
    if (c % 4 == 0 && total / 4 < (1ll << 31) - 256 && (reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) % 16 == 0) {
        PoolVecArgs v;
        v.g = a, v.c4 = c / 4, v.total = (uint32_t)(total / 4);
        v.div_c4 = FastDiv((uint32_t)v.c4), v.div_ow = FastDiv((uint32_t)a.ow), v.div_oh = FastDiv((uint32_t)a.oh);
        const unsigned vb = (v.total + 255u) / 256u;
        const float4 *x4 = reinterpret_cast<const float4 *>(x);
        float4 *o4 = reinterpret_cast<float4 *>(out);
        if (is_max)
            hipLaunchKernelGGL(pool_vec4_kernel<true>, dim3(vb), dim3(256), 0, as_stream(stream), x4, o4, v);
        else
            hipLaunchKernelGGL(pool_vec4_kernel<false>, dim3(vb), dim3(256), 0, as_stream(stream), x4, o4, v);
        DAB_LAUNCH_CHECK();
        return DAB_OK;
    }
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
