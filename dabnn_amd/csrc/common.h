// Shared host/device helpers of the gfx950 backend.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include <string>
#include <utility>

#include "../../include/dabnn_hip_tuning.h"

namespace dab {

// ---------------------------------------------------------------- errors
// Thread-local message behind dab_last_error().
std::string &last_error();
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define DAB_REQUIRE(cond, ...)                               \
    do {                                                     \
        if (!(cond)) return ::dab::fail(DAB_EINVAL, __VA_ARGS__); \
    } while (0)

#define DAB_HIP(call)                                                                                \
    do {                                                                                             \
        hipError_t e__ = (call);                                                                     \
        if (e__ != hipSuccess) return ::dab::fail(DAB_EHIP, "%s: %s", #call, hipGetErrorString(e__)); \
    } while (0)

// Checks the launch that was just enqueued.
#define DAB_LAUNCH_CHECK() DAB_HIP(hipGetLastError())

inline hipStream_t as_stream(dab_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// Number of SIMDs on the current device (4 per CU); cached.
int simd_count();
// fconv_c32.hip: the 3x3, stride 1, 32-input-channel float convolution on the bf16 matrix cores; 1 = done, 0 = not its
// shapes (the caller takes the general kernel), negative = error.
bool fconv_c32_takes(int n, int h, int w, int c, int kh, int kw, int pad_h, int pad_w, int stride_h, int stride_w, int dil_h,
                     int dil_w, int cout, int oh, int ow);
int fconv_c32_try(const float *x, int n, int h, int w, int c, const float *wgt, const float *bias, const float *aff_a,
                  const float *aff_b, int relu, int kh, int kw, int pad_h, int pad_w, int stride_h, int stride_w, int dil_h,
                  int dil_w, int cout, int oh, int ow, float *out, hipStream_t s);
bool fconv_c32_pool_takes(int n, int h, int w, int c, int kh, int kw, int pad_h, int pad_w, int stride_h, int stride_w, int dil_h,
                          int dil_w, int cout, int oh, int ow);
long long fconv_c32_pool_workspace_floats(int n, int oh, int ow, int cout);
int fconv_c32_pool_run(const float *x, int n, int h, int w, const float *wgt, const float *bias, const float *aff_a,
                       const float *aff_b, int relu, int pad_h, int pad_w, int cout, int oh, int ow, float *pooled,
                       uint64_t *pooled_packed, float *work, hipStream_t s);

// Output extent of a convolution / pooling window (common/Shaper.cpp:34-54).
inline int out_dim(int in, int pad, int k, int dil, int stride) { return (in + 2 * pad - (dil * (k - 1) + 1)) / stride + 1; }

// ---------------------------------------------------------------- compile-time loops
template <int... Is, class F>
__host__ __device__ __forceinline__ void static_for_impl(std::integer_sequence<int, Is...>, F &&f) {
    (f(std::integral_constant<int, Is>{}), ...);
}
// Calls f(integral_constant<int, i>) for i in [0, N); i is usable as a constant expression.
template <int N, class F>
__host__ __device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

// ---------------------------------------------------------------- division by a runtime constant
// q = n / d for 0 <= n < 2^31 and 1 <= d < 2^31 through one mul-hi and a shift.
struct FastDiv {
    uint32_t mul;
    uint32_t shift;
    uint32_t d;
    FastDiv() : mul(0), shift(0), d(1) {}
    explicit FastDiv(uint32_t div) : d(div) {
        if (div == 1) {
            mul = 0;
            shift = 0;
            return;
        }
        uint32_t l = 0;
        while ((1ull << l) < div) ++l;  // ceil(log2(d))
        shift = l - 1;
        mul = (uint32_t)(((1ull << (32 + shift)) + div - 1) / div);
    }
    __device__ __forceinline__ uint32_t div(uint32_t n) const { return d == 1 ? n : (__umulhi(n, mul) >> shift); }
};

// ---------------------------------------------------------------- blocks and XCDs
// The blocks of a launch are dealt to the eight XCDs in turn (block b runs on XCD b % 8) and every XCD has an L2 of
// its own.  This renumbering gives every XCD a contiguous range of numbers, so that blocks whose work is adjacent
// (neighbouring runs of rows of an image) read the same lines through the same L2.  Not for the xor/popcount kernels:
// their waves' ranges, renumbered this way, took 4-25 % longer per launch (every XCD then walks all filters for an
// eighth of the pixels, and the remainder units land on one XCD unless they are spread, which breaks whole staging
// windows apart).
__device__ __forceinline__ uint32_t xcd_contiguous_block(uint32_t b, uint32_t grid) {
    const uint32_t q = grid >> 3, r = grid & 7u, x = b & 7u;
    return x * q + (x < r ? x : r) + (b >> 3);
}

// ---------------------------------------------------------------- write-through stores
// *p = v, written through the L2 at device scope (sc1).  An ordinary store leaves a dirty line in the L2 until it
// is evicted or the kernel ends, and a kernel's end waits for all of them to be written back; these lines leave as
// they are written and stay readable in the L2.  For output that a wave writes in contiguous pieces of 128 bytes or
// more and that the same kernel does not write again: measured on the pack, im2col and GEMM kernels, 3-20 % less
// time per launch at 3-100 MB of output.  4, 8 or 16 bytes per lane.
template <class T, class U>
__device__ __forceinline__ void store_through(T *p, const U &value) {
    const T v = value;
    static_assert(sizeof(T) == 4 || sizeof(T) == 8 || sizeof(T) == 16, "one, two or four dwords per lane");
    if constexpr (sizeof(T) == 4)
        asm volatile("global_store_dword %0, %1, off sc1" : : "v"(p), "v"(v) : "memory");
    else if constexpr (sizeof(T) == 8)
        asm volatile("global_store_dwordx2 %0, %1, off sc1" : : "v"(p), "v"(v) : "memory");
    else
        // A store of more than 8 bytes still reads its data registers for two cycles after it has issued, and a
        // vector instruction that overwrites them in that time changes what is stored.  The compiler keeps that
        // distance for the stores it emits itself; it cannot see into this statement, so the statement keeps it.
        asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
}

// ---------------------------------------------------------------- sign bits of results
// Bit i = (component i > 0): the packing rule of pack_64 (common/common_bitpack.h:12-34) for four channels.
__device__ __forceinline__ uint32_t sign_nibble(float4 r) {
    return (uint32_t)(r.x > 0.0f) | ((uint32_t)(r.y > 0.0f) << 1) | ((uint32_t)(r.z > 0.0f) << 2) | ((uint32_t)(r.w > 0.0f) << 3);
}
// v | (v of lane + N within the row of 16 lanes; zero past the row's end): DPP row_shl:N
template <int N>
__device__ __forceinline__ uint32_t or_from_lane_above(uint32_t v) {
    return v | (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x100 + N, 0xF, 0xF, true);
}

// ---------------------------------------------------------------- fp32 products on the bf16 matrix cores
// An fp32 value is the exact sum of three bf16 values (8 + 8 + 8 significand bits, fp32's exponent range):
// hi = the upper 16 bits of x, mid = the upper 16 bits of x - hi, lo = x - hi - mid.  A product x*w is then
// hi*hi + (hi*mid + mid*hi) + (hi*lo + mid*mid + lo*hi) + terms below 2^-24 of it: six bf16 matrix instructions,
// accumulated in fp32 from the smallest term up, give a dot product whose error is that of an fp32 loop (measured on
// a 160-deep product against fp64: 1.6e-7 of the sum of magnitudes, an fp32 loop 2.0e-7; the three leading terms
// alone: 1.1e-5) at up to 2.6 times the rate of the fp32 matrix instruction (v_mfma_f32_32x32x16_bf16 issues in 33
// cycles, six of them for 16 depths: 404 TFLOP/s fp32-equivalent against 156; v_mfma_f32_16x16x32_bf16 in 16-19 for
// 32 depths; the splitting runs on the vector pipe while another wave's matrix instructions are in flight).
// An infinity or a NaN stays whole in hi and takes part in the hi*hi term only, where it meets the other operand's
// leading part -- the same sign, and zero where the operand is zero -- so x*w is infinite or NaN where the fp32
// product is, as long as the other operand's leading part is a normal bf16 or an exact zero; the cross terms use
// `hif`, hi with non-finite values replaced by zero (an infinity times a zero mid or lo part would be a NaN).  A NaN
// keeps a quiet bit in its upper half.
// Limits: the leading part of a nonzero |w| below 2^-126 (an fp32 denormal) is zero or a bf16 denormal, which the
// matrix core may flush, so inf * w can come out as NaN or 0 where fp32 arithmetic gives an infinity; and for finite
// operands within 2^16 of the smallest normal the mid and lo parts are bf16 denormals, so the fp32-equivalent error
// bound above holds only for magnitudes of 2^-110 and more.  Float weights and activations of that size do not occur
// in the networks this path serves, and no fixture of the reference covers them.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4w __attribute__((ext_vector_type(4)));

struct SplitParts {
    uint32_t hi, hif, mid, lo;  // bf16 in the upper halves
};
__device__ __forceinline__ SplitParts split_bf16x3(float x) {
    const uint32_t xb = __builtin_bit_cast(uint32_t, x);
    const bool special = !(__builtin_fabsf(x) < __builtin_inff());  // infinity or NaN
    const uint32_t hb = (x != x) ? 0x7fc00000u : (xb & 0xffff0000u);
    float r = x - __builtin_bit_cast(float, hb);
    r = special ? 0.f : r;
    const uint32_t rb = __builtin_bit_cast(uint32_t, r);
    const float l = r - __builtin_bit_cast(float, rb & 0xffff0000u);
    return SplitParts{hb, special ? 0u : hb, rb, __builtin_bit_cast(uint32_t, l)};
}
// the upper halves of two dwords as one: a in the lower 16 bits, b in the upper
__device__ __forceinline__ uint32_t pack_upper_halves(uint32_t a, uint32_t b) { return __builtin_amdgcn_perm(b, a, 0x07060302u); }

// The same split for a pair of finite values with the hardware's round-to-nearest conversions (v_cvt_pk_bf16_f32
// packs two): hi = bf16(x), mid = bf16(x - hi), lo = bf16(x - hi - mid), both subtractions and the last conversion
// exact.  5.5 vector instructions per value against about 10 for the truncating form with its tests.  An infinity or a
// NaN would come out as NaN in mid and lo: callers check with bf16_pair_max / bf16_pairs_finite and take the
// truncating form for the rare group that holds one.
typedef __bf16 bf16x2v __attribute__((ext_vector_type(2)));
typedef float f32x2v __attribute__((ext_vector_type(2)));
typedef unsigned short u16x2v __attribute__((ext_vector_type(2)));
struct SplitPair {
    uint32_t hi, mid, lo;  // two bf16 each, the first value in the lower half
};
__device__ __forceinline__ SplitPair split_pair_finite(float x0, float x1) {
    auto widen = [](uint32_t w) { return f32x2v{__builtin_bit_cast(float, w << 16), __builtin_bit_cast(float, w & 0xffff0000u)}; };
    const f32x2v x = {x0, x1};
    SplitPair s;
    s.hi = __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2v));
    const f32x2v r = x - widen(s.hi);
    s.mid = __builtin_bit_cast(uint32_t, __builtin_convertvector(r, bf16x2v));
    const f32x2v r2 = r - widen(s.mid);
    s.lo = __builtin_bit_cast(uint32_t, __builtin_convertvector(r2, bf16x2v));
    return s;
}
// Running maximum of the magnitudes of bf16 pairs (as 16-bit integers, half by half), and the test of the result.
__device__ __forceinline__ uint32_t bf16_pair_max(uint32_t running, uint32_t pair) {
    const u16x2v a = __builtin_bit_cast(u16x2v, running), b = __builtin_bit_cast(u16x2v, pair & 0x7fff7fffu);
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a, b));
}
__device__ __forceinline__ bool bf16_pairs_finite(uint32_t running) {
    return (running & 0xffffu) < 0x7f80u && (running >> 16) < 0x7f80u;
}

// Two bf16 in a dword, each replaced by zero when it is an infinity or a NaN.
__device__ __forceinline__ uint32_t finite_bf16_pair(uint32_t w) {
    const uint32_t lo_ok = (w & 0x00007f80u) != 0x00007f80u ? 0x0000ffffu : 0u;
    const uint32_t hi_ok = (w & 0x7f800000u) != 0x7f800000u ? 0xffff0000u : 0u;
    return w & (lo_ok | hi_ok);
}

// Eight consecutive depths of one row or column as four planes of eight bf16.
struct SplitFrag8 {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    u4 hi, hif, mid, lo;
    // finite values only (see split_pair_finite); hif = hi; returns the running magnitude maximum with these values in
    __device__ __forceinline__ uint32_t set_finite(const float (&x)[8], uint32_t running) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const SplitPair s = split_pair_finite(x[2 * i], x[2 * i + 1]);
            hi[i] = s.hi, mid[i] = s.mid, lo[i] = s.lo;
            running = bf16_pair_max(running, s.hi);
        }
        hif = hi;
        return running;
    }
    __device__ __forceinline__ void set(const float (&x)[8]) {
        SplitParts s[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) s[i] = split_bf16x3(x[i]);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            hi[i] = pack_upper_halves(s[2 * i].hi, s[2 * i + 1].hi);
            hif[i] = pack_upper_halves(s[2 * i].hif, s[2 * i + 1].hif);
            mid[i] = pack_upper_halves(s[2 * i].mid, s[2 * i + 1].mid);
            lo[i] = pack_upper_halves(s[2 * i].lo, s[2 * i + 1].lo);
        }
    }
};

// acc += A * B over 32 depths for two 16 x 16 tiles that share A: lane l holds row / column l % 16, depths
// 8 * (l / 16) .. + 7 (any assignment of depths to lanes and elements works as long as A and B use the same one).
// The two accumulators alternate so that no instruction waits for the one before it.
__device__ __forceinline__ void mfma6_16x16x32(f32x4w &acc0, f32x4w &acc1, const SplitFrag8 &a, const SplitFrag8 &b0,
                                               const SplitFrag8 &b1) {
    auto v = [](SplitFrag8::u4 w) { return __builtin_bit_cast(bf16x8, w); };
#define DAB_MFMA2(A, B)                                                               \
    acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v(a.A), v(b0.B), acc0, 0, 0, 0);  \
    acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v(a.A), v(b1.B), acc1, 0, 0, 0);
    DAB_MFMA2(lo, hif)
    DAB_MFMA2(hif, lo)
    DAB_MFMA2(mid, mid)
    DAB_MFMA2(mid, hif)
    DAB_MFMA2(hif, mid)
    DAB_MFMA2(hi, hi)
#undef DAB_MFMA2
}

// ---------------------------------------------------------------- buffer resources
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x16 __attribute__((ext_vector_type(16)));

// Raw buffer descriptor over [p, p + bytes): loads with an offset at or beyond
// `bytes` return zero, which is how out-of-image taps read a zero word.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, 0x00020000);
}

}  // namespace dab
