// Device building blocks of the xor/popcount kernels (bconv3x3 and bgemm).
//
// Work decomposition shared by both kernels
// -----------------------------------------
// A "unit" is 64 output pixels (one per lane of a wave) times 8 output
// channels.  A lane keeps the packed activations of its pixel in VGPRs for as
// long as the wave stays on the same 64-pixel tile; the weights of the 8
// channels are wave-uniform, so they are fetched with scalar loads
// (s_load_dwordx16 through the scalar data cache) and enter v_xor_b32 as SGPR
// operands: no VGPR, no LDS traffic and no per-lane address arithmetic for the
// weight operand.  Per 32 bits of K and per output the wave issues exactly one
// v_xor_b32 and one v_bcnt_u32_b32 (whose third operand is the running sum).
//
// Every wave owns a contiguous range of units (ordered tile-major, channel
// group minor), so all SIMDs get the same amount of work to within one unit
// and activations are reloaded only when the range crosses a tile boundary.
//
// The inner loop is written with small asm statements: the compiler otherwise
// hoists all scalar loads of an unrolled unit to its top and spills SGPRs.
// Statement order is the schedule: load vector j+1, consume vector j, wait.
#pragma once

#include "common.h"

namespace dab {

// 16 dwords of weights through the scalar cache, immediate byte offset.
template <int OFF>
__device__ __forceinline__ void sload16(u32x16 &v, const void *p) {
    asm volatile("s_load_dwordx16 %0, %1, %2" : "=s"(v) : "s"(p), "n"(OFF));
}
// Same with a wave-uniform register byte offset.
__device__ __forceinline__ void sload16_off(u32x16 &v, const void *p, uint32_t off) {
    asm volatile("s_load_dwordx16 %0, %1, %2" : "=s"(v) : "s"(p), "s"(off));
}
// Scalar loads return out of order: the only usable wait is "all of them".
// Tying the vector to the statement keeps its consumers behind the wait.
__device__ __forceinline__ void swait(u32x16 &v) { asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(v)); }

// acc += popcount(w0 ^ a0) + popcount(w1 ^ a1), weights in SGPRs.
__device__ __forceinline__ void xp2(uint32_t &acc, uint32_t w0, uint32_t w1, uint32_t a0, uint32_t a1) {
    uint32_t t0, t1;
    asm volatile(
        "v_xor_b32 %1, %3, %5\n\t"
        "v_xor_b32 %2, %4, %6\n\t"
        "v_bcnt_u32_b32 %0, %1, %0\n\t"
        "v_bcnt_u32_b32 %0, %2, %0"
        : "+v"(acc), "=&v"(t0), "=&v"(t1)
        : "s"(w0), "s"(w1), "v"(a0), "v"(a1));
}

// Accumulators start at the bit pattern of 2^23: adding an integer count
// c < 2^23 to that pattern yields the float 2^23 + c exactly, so one
// subtraction replaces the integer-to-float conversion.
constexpr uint32_t kAccInit = 0x4B000000u;
constexpr float kAccBias = 8388608.0f;
constexpr int kMaxCount = (1 << 23) - 1;

// ---------------------------------------------------------------- unit bodies

// 8 channels whose K32 weight dwords each lie contiguously ([channel][K32],
// the reference's weight layout): the 8*K32 dwords are K32/2 vectors of 16.
template <int K32>
__device__ __forceinline__ void unit_rowmajor(const void *wbase, const uint32_t (&a)[K32], uint32_t (&acc)[8]) {
    constexpr int NV = K32 / 2;
    static_assert(K32 % 2 == 0, "a dword pair never straddles two channels");
    u32x16 buf[2];
    sload16<0>(buf[0], wbase);
    swait(buf[0]);
    static_for<NV>([&](auto j_) {
        constexpr int j = j_;
        if constexpr (j + 1 < NV) sload16<(j + 1) * 64>(buf[(j + 1) & 1], wbase);
        static_for<8>([&](auto e_) {
            constexpr int d = j * 16 + e_ * 2;  // dword index within the 8-channel block
            constexpr int q = d / K32, k = d % K32;
            xp2(acc[q], buf[j & 1][e_ * 2], buf[j & 1][e_ * 2 + 1], a[k], a[k + 1]);
        });
        if constexpr (j + 1 < NV) swait(buf[(j + 1) & 1]);
    });
}

// 8 channels stored channel-minor ([k word][channel], bgemm's column-major A):
// vector h holds word h of channels 0..7; consecutive words are `stride`
// bytes apart.
template <int K64>
__device__ __forceinline__ void unit_colmajor(const void *wbase, uint32_t stride, const uint32_t *a, uint32_t (&acc)[8]) {
    u32x16 buf[2];
    sload16<0>(buf[0], wbase);
    swait(buf[0]);
    uint32_t off = 0;
    static_for<K64>([&](auto h_) {
        constexpr int h = h_;
        if constexpr (h + 1 < K64) {
            off += stride;
            sload16_off(buf[(h + 1) & 1], wbase, off);
        }
        static_for<8>([&](auto q_) {
            xp2(acc[q_], buf[h & 1][q_ * 2], buf[h & 1][q_ * 2 + 1], a[2 * h], a[2 * h + 1]);
        });
        if constexpr (h + 1 < K64) swait(buf[(h + 1) & 1]);
    });
}

// ---------------------------------------------------------------- output staging
// A wave parks up to 32 channels (4 units) of its 64 pixels in LDS, one row
// per pixel, and writes them out transposed: 8 consecutive lanes cover the
// 128 contiguous bytes of one pixel, so every store instruction writes whole
// cache lines instead of 64 scattered 16-byte pieces.
constexpr int kStageRow = 144;                // 32 channels * 4 B + 16 B pad: conflict-free b128 access
constexpr int kStageBytes = 64 * kStageRow;   // per wave

__device__ __forceinline__ void stage_put(unsigned char *stage, int lane, int slot, const uint32_t (&acc)[8]) {
    float4 *dst = reinterpret_cast<float4 *>(stage + lane * kStageRow + slot * 32);
    dst[0] = make_float4(__uint_as_float(acc[0]) - kAccBias, __uint_as_float(acc[1]) - kAccBias,
                         __uint_as_float(acc[2]) - kAccBias, __uint_as_float(acc[3]) - kAccBias);
    dst[1] = make_float4(__uint_as_float(acc[4]) - kAccBias, __uint_as_float(acc[5]) - kAccBias,
                         __uint_as_float(acc[6]) - kAccBias, __uint_as_float(acc[7]) - kAccBias);
}

// Writes staged channel groups [g_lo, g_hi] of the 32-channel window that
// starts at channel cbase.  out is [pixel][ld] floats; pixels >= total are
// skipped.  ACCUM adds to what out already holds (bgemm's C +=).
template <bool ACCUM>
__device__ __forceinline__ void stage_flush(const unsigned char *stage, int lane, float *__restrict__ out, int ld,
                                            int tile, int total, int cbase, int g_lo, int g_hi) {
    __builtin_amdgcn_wave_barrier();
    const int np = 2 * (g_hi - g_lo + 1);  // 16-byte parts per pixel row
    if (np == 8 && (tile + 1) * 64 <= total) {
        const int pr0 = lane >> 3, part = lane & 7;
        const unsigned char *src = stage + pr0 * kStageRow + part * 16;
        float *dst = out + ((size_t)tile * 64 + pr0) * ld + cbase + part * 4;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float4 v = *reinterpret_cast<const float4 *>(src + i * 8 * kStageRow);
            float4 *d = reinterpret_cast<float4 *>(dst + (size_t)i * 8 * ld);
            if (ACCUM) {
                const float4 o = *d;
                v.x += o.x, v.y += o.y, v.z += o.z, v.w += o.w;
            }
            *d = v;
        }
    } else {
        const int magic = (65536 + np - 1) / np;  // c / np for c < 512
        for (int i = 0; i < np; ++i) {
            const int c = lane + 64 * i;
            const int pr = (c * magic) >> 16;
            const int part = 2 * g_lo + (c - pr * np);
            const int pix = tile * 64 + pr;
            if (pix < total) {
                float4 v = *reinterpret_cast<const float4 *>(stage + pr * kStageRow + part * 16);
                float4 *d = reinterpret_cast<float4 *>(out + (size_t)pix * ld + cbase + part * 4);
                if (ACCUM) {
                    const float4 o = *d;
                    v.x += o.x, v.y += o.y, v.z += o.z, v.w += o.w;
                }
                *d = v;
            }
        }
    }
    __builtin_amdgcn_wave_barrier();
}

// Contiguous unit range [u0, u1) of wave `wv` out of `n_waves`.
__device__ __forceinline__ void unit_range(int wv, int n_waves, int n_units, int &u0, int &u1) {
    u0 = (int)(((long long)wv * n_units) / n_waves);
    u1 = (int)(((long long)(wv + 1) * n_units) / n_waves);
}

// Host side: how many waves to launch for n_units units.
inline int pick_wave_count(int n_units, int waves_per_simd, int waves_per_block) {
    long long w = (long long)simd_count() * waves_per_simd;
    if (w > n_units) w = n_units;
    if (w < 1) w = 1;
    return (int)((w + waves_per_block - 1) / waves_per_block * waves_per_block);
}

}  // namespace dab
