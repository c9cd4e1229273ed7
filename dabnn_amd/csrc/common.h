// Shared host/device helpers of the gfx950 backend.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include <string>
#include <utility>

#include "../../include/dabnn_hip.h"

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
