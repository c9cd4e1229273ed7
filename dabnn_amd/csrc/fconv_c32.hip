// FpConv2D (dabnn/fconv.h:14-76) for 3x3, stride 1 convolutions over 32 input channels -- the second and third
// convolution of a three-convolution stem -- on the bf16 matrix cores with split operands (common.h: six products
// per depth group, fp32 accuracy), with the optional Affine and Relu of dab_fconv_affine_relu in the same pass.
//
// A depth group of the matrix instruction (32 depths) is one tap's 32 channels, so there is no im2col stage and no
// pixel tile in LDS: a wave owns 64 output pixels (four tiles of 16 along an image row) and all output channels, and
// for every tap a lane fetches the eight channels 8 * (lane / 16) .. + 7 of its pixel of each tile straight from the
// image -- 16 lanes x 4 groups read 16 pixels x 128 contiguous bytes -- and splits them in registers.  Out-of-image taps
// read zero through the buffer descriptor.  The filters are split once per block into three planes of bf16 in LDS
// ([plane][output channel][tap][32] with eight elements of padding per channel: a quarter wave's 16-byte reads hit
// all banks); a filter fragment (16 channels x 32 depths of one tap) is read once per tap and used for the wave's four
// pixel tiles.  The output channels are the rows of the matrix instruction and the pixels its columns, so a lane ends
// up with four consecutive channels of one pixel: one 16-byte store.  Waves are independent (no barrier after the
// filters are in place) and persistent over their share of the 64-pixel items.
#include <cfloat>
#include <type_traits>

#include "common.h"

namespace dab {

struct FconvC32Args {
    const float *x, *w, *bias, *aff_a, *aff_b;
    float *out;
    int relu;
    int h, wd, oh, ow, cout, pad_h, pad_w;
    uint32_t x_bytes;
    int tiles;          // 16-pixel tiles of the output: n * oh * ow / 16
    int items;          // groups of four tiles
    FastDiv div_tiles_per_row, div_oh;
    int tiles_per_row;
};

constexpr int kC32Threads = 512, kC32PixelTiles = 4;
constexpr uint32_t kC32Oob = 0x80000000u;  // beyond the descriptor (images here are shorter than 2^31 bytes)

template <int NT, int KH, int KW>  // NT: 16-channel tiles of the output (cout = 16 * NT)
__global__ __launch_bounds__(kC32Threads) void fconv_c32_kernel(const FconvC32Args p) {
    constexpr int TAPS = KH * KW, PT = kC32PixelTiles, COUT = 16 * NT;
    constexpr int ROW = TAPS * 32 + 8;     // bf16 elements per output channel in a plane
    constexpr int PLANE = COUT * ROW;      // elements per plane (hi, mid, lo)
    __shared__ __attribute__((aligned(16))) uint16_t planes[3 * PLANE];
    __shared__ int filter_special;  // a filter value is an infinity or a NaN

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 4, f_i = lane & 15;

    if (tid == 0) filter_special = 0;
    __syncthreads();
    {
        bool special = false;
        // pairs of consecutive depths: one dword per plane
        for (int idx = tid; idx < COUT * TAPS * 16; idx += kC32Threads) {
            const int co = idx / (TAPS * 16), r = idx - co * (TAPS * 16);  // r: pair index in the channel's 288 depths
            const float2 v = *reinterpret_cast<const float2 *>(p.w + (size_t)co * (TAPS * 32) + 2 * r);
            const SplitParts s0 = split_bf16x3(v.x), s1 = split_bf16x3(v.y);
            special |= s0.hif != s0.hi || s1.hif != s1.hi;
            uint32_t *d = reinterpret_cast<uint32_t *>(planes + co * ROW + 2 * r);
            d[0] = pack_upper_halves(s0.hi, s1.hi);
            d[PLANE / 2] = pack_upper_halves(s0.mid, s1.mid);
            d[2 * (PLANE / 2)] = pack_upper_halves(s0.lo, s1.lo);
        }
        if (special) filter_special = 1;
    }
    __syncthreads();
    const bool w_special = __builtin_amdgcn_readfirstlane(filter_special) != 0;

    const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(p.x, p.x_bytes);
    typedef float f32x4r __attribute__((ext_vector_type(4)));
    // A block works through a contiguous range of items, its waves side by side: the image rows above and below the
    // ones it is on were fetched by the block itself a moment ago and are still in its L2 (with the items dealt to all
    // waves in turn every row was fetched from memory twice, by blocks on different XCDs).
    const int per = p.items / (int)gridDim.x, extra = p.items - per * (int)gridDim.x, b = (int)blockIdx.x;
    const int first = b * per + (b < extra ? b : extra), last = first + per + (b < extra ? 1 : 0);

    for (int item = first + wave; item < last; item += kC32Threads / 64) {
        // the lane's pixel of each tile: byte offset of its window's first tap (may lie outside the image: then the
        // row or column test below sends the load out of range), and its coordinates for those tests
        int off0[PT], iy0[PT], ix0[PT];
#pragma unroll
        for (int t = 0; t < PT; ++t) {
            const int T = item * PT + t;
            const uint32_t row = p.div_tiles_per_row.div((uint32_t)T);
            const int xt = T - (int)row * p.tiles_per_row;
            const uint32_t img = p.div_oh.div(row);
            const int oy = (int)(row - img * (uint32_t)p.oh);
            const bool tile_ok = T < p.tiles;
            iy0[t] = tile_ok ? oy - p.pad_h : -0x40000000;  // a tile past the end reads nothing
            ix0[t] = xt * 16 + f_i - p.pad_w;
            off0[t] = tile_ok ? (((int)img * p.h + iy0[t]) * p.wd + ix0[t]) * 128 + g * 32 : 0;
        }
        auto fetch = [&](int tap, f32x4r (&lo)[PT], f32x4r (&hi)[PT]) {
            const int ty = tap / KW, tx = tap - ty * KW;
#pragma unroll
            for (int t = 0; t < PT; ++t) {
                const bool ok = (unsigned)(iy0[t] + ty) < (unsigned)p.h && (unsigned)(ix0[t] + tx) < (unsigned)p.wd;
                const uint32_t off = ok ? (uint32_t)(off0[t] + (ty * p.wd + tx) * 128) : kC32Oob;
                lo[t] = __builtin_bit_cast(f32x4r, __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, (int)off, 0, 0));
                hi[t] = __builtin_bit_cast(f32x4r, __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, (int)(off + 16u), 0, 0));
            }
        };
        // a filter fragment: output channels 16 * nt + f_i, depths 8 * g .. + 7 of the tap
        auto filter_frag = [&](auto filters_special, int nt, int tap) {
            const uint16_t *src = planes + (nt * 16 + f_i) * ROW + tap * 32 + 8 * g;
            SplitFrag8 f;
            f.hi = *reinterpret_cast<const SplitFrag8::u4 *>(src);
            f.mid = *reinterpret_cast<const SplitFrag8::u4 *>(src + PLANE);
            f.lo = *reinterpret_cast<const SplitFrag8::u4 *>(src + 2 * PLANE);
            f.hif = f.hi;
            if constexpr (decltype(filters_special)::value) {
#pragma unroll
                for (int e = 0; e < 4; ++e) f.hif[e] = finite_bf16_pair(f.hi[e]);
            }
            return f;
        };

        f32x4w acc[PT][NT];
#pragma unroll
        for (int t = 0; t < PT; ++t)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) acc[t][nt] = f32x4w{0.f, 0.f, 0.f, 0.f};

        f32x4r raw_lo[PT], raw_hi[PT];
        fetch(0, raw_lo, raw_hi);
        auto all_taps = [&](auto filters_special) {
        // the taps one after the other (not unrolled: the compiler would otherwise start all nine taps' loads at once
        // and spill); the next tap's pixels are on their way while this tap is multiplied
#pragma unroll 1
        for (int tap = 0; tap < TAPS; ++tap) {
            SplitFrag8 px[PT];
            uint32_t magnitude = 0;
#pragma unroll
            for (int t = 0; t < PT; ++t) {
                const float v[8] = {raw_lo[t][0], raw_lo[t][1], raw_lo[t][2], raw_lo[t][3],
                                    raw_hi[t][0], raw_hi[t][1], raw_hi[t][2], raw_hi[t][3]};
                magnitude = px[t].set_finite(v, magnitude);
            }
            if (__builtin_amdgcn_ballot_w64(!bf16_pairs_finite(magnitude)) != 0) {
                // an infinity or a NaN among the wave's pixels of this tap: the split that keeps it out of the cross terms
#pragma unroll
                for (int t = 0; t < PT; ++t) {
                    const float v[8] = {raw_lo[t][0], raw_lo[t][1], raw_lo[t][2], raw_lo[t][3],
                                        raw_hi[t][0], raw_hi[t][1], raw_hi[t][2], raw_hi[t][3]};
                    px[t].set(v);
                }
            }
            if (tap + 1 < TAPS) fetch(tap + 1, raw_lo, raw_hi);
            // rows of the product = output channels (the filter fragment), columns = pixels
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const SplitFrag8 f = filter_frag(filters_special, nt, tap);
                mfma6_16x16x32(acc[0][nt], acc[1][nt], f, px[0], px[1]);
                mfma6_16x16x32(acc[2][nt], acc[3][nt], f, px[2], px[3]);
            }
        }
        };
        if (w_special)
            all_taps(std::true_type{});
        else
            all_taps(std::false_type{});

        // accumulator element e of lane l: output channel 16 * nt + 4 * (l / 16) + e of pixel l % 16
        auto store_all = [&]() {
#pragma clang fp contract(off)
            float bs[NT][4], as[NT][4], bb[NT][4];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const int co = nt * 16 + 4 * g;
                const float4 bias = p.bias ? *reinterpret_cast<const float4 *>(p.bias + co) : make_float4(0.f, 0.f, 0.f, 0.f);
                const float4 fa = p.aff_a ? *reinterpret_cast<const float4 *>(p.aff_a + co) : make_float4(0.f, 0.f, 0.f, 0.f);
                const float4 fb = p.aff_a ? *reinterpret_cast<const float4 *>(p.aff_b + co) : make_float4(0.f, 0.f, 0.f, 0.f);
                bs[nt][0] = bias.x, bs[nt][1] = bias.y, bs[nt][2] = bias.z, bs[nt][3] = bias.w;
                as[nt][0] = fa.x, as[nt][1] = fa.y, as[nt][2] = fa.z, as[nt][3] = fa.w;
                bb[nt][0] = fb.x, bb[nt][1] = fb.y, bb[nt][2] = fb.z, bb[nt][3] = fb.w;
            }
            // a pixel's channel tiles one after the other: its 64-byte pieces complete 128-byte lines while they are
            // still in the write path
#pragma unroll
            for (int t = 0; t < PT; ++t) {
                const int T = item * PT + t;
                if (T >= p.tiles) continue;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    float v[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        v[e] = acc[t][nt][e];
                        if (p.bias) v[e] = v[e] + bs[nt][e];
                        if (p.aff_a) {
                            const float prod = as[nt][e] * v[e];
                            v[e] = prod + bb[nt][e];
                        }
                        if (p.relu) v[e] = v[e] < 0.f ? 0.f : v[e];  // std::max(v, 0.f): a NaN stays
                    }
                    *reinterpret_cast<float4 *>(p.out + ((size_t)T * 16 + f_i) * COUT + nt * 16 + 4 * g) =
                        make_float4(v[0], v[1], v[2], v[3]);
                }
            }
        };
        store_all();
    }
}

// Whether the shapes are this kernel's and the problem is large enough to fill its persistent waves (buffer alignment
// aside, which only the call itself can check).
bool fconv_c32_takes(int n, int h, int w, int c, int kh, int kw, int pad_h, int pad_w, int stride_h, int stride_w, int dil_h,
                     int dil_w, int cout, int oh, int ow) {
    if (c != 32 || kh != 3 || kw != 3 || stride_h != 1 || stride_w != 1 || dil_h != 1 || dil_w != 1) return false;
    if ((cout != 32 && cout != 64) || oh <= 0 || ow <= 0 || ow % 16 != 0 || pad_h > 2 || pad_w > 2) return false;
    const long long in_bytes = (long long)n * h * w * 128, tiles = (long long)n * oh * ow / 16;
    if (in_bytes >= (1ll << 31) || tiles >= (1ll << 30)) return false;
    const long long waves = (long long)(simd_count() / 4) * (kC32Threads / 64);
    // smaller problems: the general kernel's tiles fill the chip better
    return (tiles + kC32PixelTiles - 1) / kC32PixelTiles >= 2 * waves;
}

// Runs the convolution if fconv_c32_takes says so and the buffers are 16-byte aligned; returns 1 when it did, 0 when
// the caller must take the general kernel, a negative error code on failure.
int fconv_c32_try(const float *x, int n, int h, int w, int c, const float *wgt, const float *bias, const float *aff_a,
                  const float *aff_b, int relu, int kh, int kw, int pad_h, int pad_w, int stride_h, int stride_w, int dil_h,
                  int dil_w, int cout, int oh, int ow, float *out, hipStream_t s) {
    if (!fconv_c32_takes(n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, cout, oh, ow)) return 0;
    uintptr_t align = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(wgt) | reinterpret_cast<uintptr_t>(out);
    if (bias) align |= reinterpret_cast<uintptr_t>(bias);
    if (aff_a) align |= reinterpret_cast<uintptr_t>(aff_a) | reinterpret_cast<uintptr_t>(aff_b);
    if (align % 16 != 0) return 0;
    const long long tiles = (long long)n * oh * ow / 16;
    const int blocks = simd_count() / 4;  // one block of eight waves per CU (the filter planes take most of its LDS)
    FconvC32Args a;
    a.x = x, a.w = wgt, a.bias = bias, a.aff_a = aff_a, a.aff_b = aff_b, a.out = out, a.relu = relu;
    a.h = h, a.wd = w, a.oh = oh, a.ow = ow, a.cout = cout, a.pad_h = pad_h, a.pad_w = pad_w;
    a.x_bytes = (uint32_t)((long long)n * h * w * 128);
    a.tiles = (int)tiles, a.items = (int)((tiles + kC32PixelTiles - 1) / kC32PixelTiles);
    a.tiles_per_row = ow / 16;
    a.div_tiles_per_row = FastDiv((uint32_t)a.tiles_per_row), a.div_oh = FastDiv((uint32_t)oh);
    if (cout == 32)
        hipLaunchKernelGGL((fconv_c32_kernel<2, 3, 3>), dim3(blocks), dim3(kC32Threads), 0, s, a);
    else
        hipLaunchKernelGGL((fconv_c32_kernel<4, 3, 3>), dim3(blocks), dim3(kC32Threads), 0, s, a);
    return hipGetLastError() == hipSuccess ? 1 : fail(DAB_EHIP, "fconv_c32: launch failed");
}

}  // namespace dab
