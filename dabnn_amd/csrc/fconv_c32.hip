// FpConv2D (dabnn/fconv.h:14-76) for 3x3, stride 1 convolutions over 32 input channels -- the second and third
// convolution of a three-convolution stem -- on the bf16 matrix cores with split operands (common.h: six products
// per depth group, fp32 accuracy), with the optional Affine and Relu of dab_fconv_affine_relu in the same pass.
//
// A depth group of the matrix instruction (32 depths) is one tap's 32 channels, so there is no im2col stage and no
// pixel tile in LDS: a wave owns a column of four 16-pixel tiles (four consecutive output rows at one x tile) and all
// output channels.  A lane fetches the eight channels 8 * (lane / 16) .. + 7 of its pixel in each of the six input
// rows under the column straight from the image -- 16 lanes x 4 groups read 16 pixels x 128 contiguous bytes -- and
// splits them in registers, once: a split row serves the three output rows it is a vertical tap of, and the three
// horizontal taps are the same values one lane over (lane-shifting moves, with the two pixels beside the tile fetched
// and split as a seventh row).  Out-of-image taps read zero through the buffer descriptor.  The next item's rows are
// in flight while this one's last products are made.  The filters are split once per block into three planes of bf16
// in LDS ([plane][output channel][tap][32] with eight elements of padding per channel: a quarter wave's 16-byte reads
// hit all banks); a filter fragment (16 channels x 32 depths of one tap) is read once per tap and used for the wave's
// four tiles.  The output channels are the rows of the matrix instruction and the pixels its columns, so a lane ends
// up with four consecutive channels of one pixel: one 16-byte store.  Waves are independent (no barrier after the
// filters are in place) and take their items from a counter of the block.
#include <cfloat>
#include <type_traits>

#include "common.h"

namespace dab {

struct FconvC32Args {
    const float *x, *w, *bias, *aff_a, *aff_b;
    float *out;
    float *brow, *bcol;  // POOL: every fourth output row and every sixteenth output column, for the pass that completes the pooling
    uint64_t *bits;      // the completing pass: pack_mat of the pooled tensor, or null
    int relu;
    int h, wd, oh, ow, cout, pad_h, pad_w;
    uint32_t x_bytes;
    int items;          // columns of four tiles: n * ceil(oh / 4) * (ow / 16)
    int row_groups;     // ceil(oh / 4)
    FastDiv div_tiles_per_row, div_row_groups;
    int tiles_per_row;
};

constexpr int kC32Threads = 512, kC32PixelTiles = 4;
constexpr uint32_t kC32Oob = 0x80000000u;  // beyond the descriptor (images here are shorter than 2^31 bytes)

// POOL: a MaxPool 3x3, stride 2, pad 1 (max_pool_fallback, dabnn/layers/MaxPool.cpp:209-246) follows and the convolution's
// own result is not wanted.  A wave's column of four output rows x 16 pixels holds two pooled rows x eight pooled pixels:
// it pools what it has -- rows as elementwise maxima of its accumulators, columns as maxima with the two neighbouring
// lanes -- and writes that to p.out, now [n][oh / 2][ow / 2][cout].  What it lacks is the output row above the column
// (for its first pooled row) and the output pixel left of it (for its first pooled pixel): every column also writes its
// last output row to p.brow [n][oh / 4][ow][cout] and its last pixel of each row to p.bcol [n][oh / 4][ow / 16][4][cout],
// and c32_pool_complete_kernel takes the maxima with those afterwards.  oh must be a multiple of 4.
template <int NT, int KH, int KW, bool POOL = false>  // NT: 16-channel tiles of the output (cout = 16 * NT)
__global__ __launch_bounds__(kC32Threads) void fconv_c32_kernel(const FconvC32Args p) {
    constexpr int TAPS = KH * KW, PT = kC32PixelTiles, COUT = 16 * NT;
    constexpr int ROW = TAPS * 32 + 8;     // bf16 elements per output channel in a plane
    constexpr int PLANE = COUT * ROW;      // elements per plane (hi, mid, lo)
    __shared__ __attribute__((aligned(16))) uint16_t planes[3 * PLANE];
    __shared__ int filter_special;  // a filter value is an infinity or a NaN
    __shared__ int next_item;       // the first item of the block's range that no wave has taken
    // bias, Affine a and b per output channel (zeros where the layer has none): read from here when an item is written,
    // so that no load is outstanding among the stores -- loads and stores share one counter and complete in no fixed
    // order, and a wait for such a load would also wait for every store before it to be acknowledged
    __shared__ __attribute__((aligned(16))) float per_channel[3][COUT];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 4, f_i = lane & 15;

    // A block works through a contiguous range of items, its waves side by side: the image rows above and below the
    // ones it is on were fetched by the block itself a moment ago and are still in its L2 (with the items dealt to all
    // waves in turn every row was fetched from memory twice, by blocks on different XCDs).  A wave takes its next item
    // from a counter: of the two waves of a SIMD the older one is served first and gets through its items faster, and
    // with equal shares the other would finish its last quarter alone, its vector and matrix instructions no longer
    // overlapping with anyone's.
    const int per = p.items / (int)gridDim.x, extra = p.items - per * (int)gridDim.x, b = (int)blockIdx.x;
    const int first = b * per + (b < extra ? b : extra), last = first + per + (b < extra ? 1 : 0);
    if (tid == 0) filter_special = 0, next_item = first + kC32Threads / 64;
    if (tid < COUT) {
        per_channel[0][tid] = p.bias ? p.bias[tid] : 0.f;
        per_channel[1][tid] = p.aff_a ? p.aff_a[tid] : 0.f;
        per_channel[2][tid] = p.aff_a ? p.aff_b[tid] : 0.f;
    }
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
    typedef SplitFrag8::u4 u4;
    // An item is a column of four tiles: output rows oy0 .. oy0 + 3 of one image at the 16 pixels of one x tile.  An
    // input row's pixels at horizontal tap tx then serve three of the item's output rows (vertical taps 0, 1, 2), so a
    // fetched and split fragment is used for three tiles' products: KH + 3 fragments per horizontal tap instead of
    // 4 * KH -- the splitting, which bounds the kernel with few output channels, is halved.
    constexpr int ROWS = PT + KH - 1;
    struct Place {
        int img, oy0, xt;
        int off0;  // byte offset of this lane's eight channels at input row oy0 - pad, column of tap 0 (may lie outside the image)
    };
    auto locate = [&](int item) {
        Place q;
        const uint32_t rowg = p.div_tiles_per_row.div((uint32_t)item);
        q.xt = item - (int)rowg * p.tiles_per_row;
        q.img = (int)p.div_row_groups.div(rowg);
        q.oy0 = ((int)rowg - q.img * p.row_groups) * PT;
        q.off0 = ((q.img * p.h + q.oy0 - p.pad_h) * p.wd + q.xt * 16 + f_i - p.pad_w) * 128 + g * 32;
        return q;
    };
    // the eight channels of this lane's pixel at input row (oy0 - pad + j), horizontal tap tx; zero outside the image
    // and for an item beyond the block's range
    auto fetch = [&](const Place &q, bool item_ok, int j, int tx, f32x4r (&r)[2]) __attribute__((always_inline)) {
        const bool ok = item_ok && (unsigned)(q.xt * 16 + f_i - p.pad_w + tx) < (unsigned)p.wd && (unsigned)(q.oy0 - p.pad_h + j) < (unsigned)p.h;
        const uint32_t off = ok ? (uint32_t)(q.off0 + (j * p.wd + tx) * 128) : kC32Oob;
        r[0] = __builtin_bit_cast(f32x4r, __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, (int)off, 0, 0));
        r[1] = __builtin_bit_cast(f32x4r, __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, (int)(off + 16u), 0, 0));
    };
    auto filter_at = [&](int nt, int ty, int tx) { return planes + (nt * 16 + f_i) * ROW + (ty * KW + tx) * 32 + 8 * g; };
    // accumulator element e of lane l: output channel 16 * nt + 4 * (l / 16) + e of pixel l % 16
    auto finish = [&](float v, float bias, float fa, float fb) {
#pragma clang fp contract(off)
        if (p.bias) v = v + bias;
        if (p.aff_a) {
            const float prod = fa * v;
            v = prod + fb;
        }
        if (p.relu) v = v < 0.f ? 0.f : v;  // std::max(v, 0.f): a NaN stays
        return v;
    };

    static_assert(KW == 3, "the horizontal taps are the fetched pixels and their two neighbours");
    // The halo of an item: lane l % 16 = j < 6 fetches the pixel left of the item's 16 (horizontal tap 0 of the first
    // pixel) in input row j, lane l % 16 = 8 + j the pixel right of them (tap 2 of the last).
    auto fetch_halo = [&](const Place &q, bool item_ok, f32x4r (&r)[2]) __attribute__((always_inline)) {
        const int j = f_i & 7, col = q.xt * 16 - p.pad_w + (f_i >> 3) * 17;
        const bool ok = item_ok && j < ROWS && (unsigned)col < (unsigned)p.wd && (unsigned)(q.oy0 - p.pad_h + j) < (unsigned)p.h;
        const uint32_t off = ok ? (uint32_t)(q.off0 + (j * p.wd + (f_i >> 3) * 17 - f_i) * 128) : kC32Oob;
        r[0] = __builtin_bit_cast(f32x4r, __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, (int)off, 0, 0));
        r[1] = __builtin_bit_cast(f32x4r, __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, (int)(off + 16u), 0, 0));
    };
    Place here = locate(first + wave);
    // the next item's six input rows (the pixels of horizontal tap 1) and halo, in flight while this one's last
    // products are made
    f32x4r raw[ROWS][2], raw_halo[2];
#pragma unroll
    for (int j = 0; j < ROWS; ++j) fetch(here, first + wave < last, j, 1, raw[j]);
    fetch_halo(here, first + wave < last, raw_halo);

    f32x4w acc[PT][NT];
    // max_pool's step, `v > m ? v : m` from -FLT_MAX on, as the hardware's maximum: a NaN is passed over either way (the
    // running maximum never is one); where +0 and -0 tie the hardware gives +0 and max_pool the earlier tap, which no
    // comparison and no sign bit of the result can tell apart
    // (the instructions by name: fmaxf would come with an instruction per operand that quiets signalling NaNs, which
    // these values -- results of arithmetic -- never are)
    auto later_max = [](float m, float v) {
        float r;
        asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(m), "v"(v));
        return r;
    };
    auto max_of_three = [](float a, float b, float c) {
        float r;
        asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
        return r;
    };
    // POOL: a tile column's two pooled rows for channel tile nt from the maxima over its output rows {0, 1} (v0) and
    // {1, 2, 3} (v1): lane f (even) takes the maximum over pixels f - 1, f, f + 1 of the tile and stores pooled pixel f / 2
    auto pool_store = [&](const Place &at, int nt, int g_now, const f32x4w &v0, const f32x4w &v1) __attribute__((always_inline)) {
        const int lowest = __float_as_int(-FLT_MAX);
        float h[2][4];
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const f32x4w &v = half ? v1 : v0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float left = __int_as_float(__builtin_amdgcn_update_dpp(lowest, __float_as_int(v[e]), 0x111, 0xf, 0xf, false));
                const float right = __int_as_float(__builtin_amdgcn_update_dpp(lowest, __float_as_int(v[e]), 0x101, 0xf, 0xf, false));
                h[half][e] = max_of_three(left, v[e], right);
            }
        }
        // one store for both rows: the odd lanes take the second row's cell from the even lane below them
        float out[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float second = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(h[1][e]), 0x111, 0xf, 0xf, true));
            out[e] = (f_i & 1) ? second : h[0][e];
        }
        const size_t cell = ((size_t)at.img * (p.oh >> 1) + (at.oy0 >> 1) + (f_i & 1)) * (p.ow >> 1) + at.xt * 8 + (f_i >> 1);
        *reinterpret_cast<float4 *>(p.out + cell * COUT + nt * 16 + 4 * g_now) = make_float4(out[0], out[1], out[2], out[3]);
    };
    // Writes the item at `at`, whose sums are in acc (special: an infinity or a NaN among its pixels or in the filters).
    auto write_item = [&](const Place &at, bool special) __attribute__((always_inline)) {
        int g_now = g;
        asm volatile("" : "+v"(g_now));  // what follows is read per item: hoisted out of the item loop it would be spilled
        if (!special) {
            float bs[NT][4], as[NT][4], bb[NT][4];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const int co = nt * 16 + 4 * g_now;
                const float4 bias = *reinterpret_cast<const float4 *>(per_channel[0] + co);
                const float4 fa = *reinterpret_cast<const float4 *>(per_channel[1] + co);
                const float4 fb = *reinterpret_cast<const float4 *>(per_channel[2] + co);
                bs[nt][0] = bias.x, bs[nt][1] = bias.y, bs[nt][2] = bias.z, bs[nt][3] = bias.w;
                as[nt][0] = fa.x, as[nt][1] = fa.y, as[nt][2] = fa.z, as[nt][3] = fa.w;
                bb[nt][0] = fb.x, bb[nt][1] = fb.y, bb[nt][2] = fb.z, bb[nt][3] = fb.w;
            }
            // bias, Affine and Relu each over all of the item's values under one test of its wave-uniform flag (tested
            // per value they become a select per value and stage: 9 instead of 5 instructions per value)
            {
#pragma clang fp contract(off)
                if (p.bias) {
#pragma unroll
                    for (int t = 0; t < PT; ++t)
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                            for (int e = 0; e < 4; ++e) acc[t][nt][e] = acc[t][nt][e] + bs[nt][e];
                }
                if (p.aff_a) {
#pragma unroll
                    for (int t = 0; t < PT; ++t)
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const float prod = as[nt][e] * acc[t][nt][e];
                                acc[t][nt][e] = prod + bb[nt][e];
                            }
                }
                if (p.relu) {
#pragma unroll
                    for (int t = 0; t < PT; ++t)
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                            for (int e = 0; e < 4; ++e) acc[t][nt][e] = acc[t][nt][e] < 0.f ? 0.f : acc[t][nt][e];  // std::max(v, 0.f): a NaN stays
                }
            }
            if constexpr (POOL) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    f32x4w v0, v1;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        v0[e] = later_max(acc[0][nt][e], acc[1][nt][e]);
                        v1[e] = max_of_three(acc[1][nt][e], acc[2][nt][e], acc[3][nt][e]);
                    }
                    pool_store(at, nt, g_now, v0, v1);
                    // the last row as it is; the last pixel of the four rows gathered into lanes 12..15 of each group
                    float *row = p.brow + ((((size_t)at.img * p.row_groups + (at.oy0 >> 2)) * p.ow + at.xt * 16 + f_i) * COUT + nt * 16 + 4 * g_now);
                    *reinterpret_cast<float4 *>(row) = make_float4(acc[3][nt][0], acc[3][nt][1], acc[3][nt][2], acc[3][nt][3]);
                    float w[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int r2 = __builtin_amdgcn_update_dpp(0, __float_as_int(acc[2][nt][e]), 0x101, 0xf, 0xf, true);  // lane 14 <- 15
                        const int r1 = __builtin_amdgcn_update_dpp(0, __float_as_int(acc[1][nt][e]), 0x102, 0xf, 0xf, true);  // lane 13 <- 15
                        const int r0 = __builtin_amdgcn_update_dpp(0, __float_as_int(acc[0][nt][e]), 0x103, 0xf, 0xf, true);  // lane 12 <- 15
                        w[e] = f_i == 15 ? acc[3][nt][e] : __int_as_float(f_i == 14 ? r2 : f_i == 13 ? r1 : r0);
                    }
                    if (f_i >= 12) {
                        float *col = p.bcol + (((((size_t)at.img * p.row_groups + (at.oy0 >> 2)) * p.tiles_per_row + at.xt) * 4 + (f_i - 12)) * COUT + nt * 16 + 4 * g_now);
                        *reinterpret_cast<float4 *>(col) = make_float4(w[0], w[1], w[2], w[3]);
                    }
                }
            } else {
            // a pixel's channel tiles one after the other: its 64-byte pieces complete 128-byte lines while they are
            // still in the write path
#pragma unroll
            for (int t = 0; t < PT; ++t) {
                if (at.oy0 + t >= p.oh) continue;
                const size_t m = ((size_t)at.img * p.oh + at.oy0 + t) * p.ow + at.xt * 16 + f_i;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
                    *reinterpret_cast<float4 *>(p.out + m * COUT + 4 * g_now + nt * 16) =
                        make_float4(acc[t][nt][0], acc[t][nt][1], acc[t][nt][2], acc[t][nt][3]);
            }
            }
        } else {
            // The item is made again, one tile and one tap at a time, with the split that keeps an infinity or a NaN
            // whole in hi and takes copies with the non-finite values zeroed for the cross terms (Inf * 0 would make a
            // NaN of a sum that is an infinity).
#pragma unroll 1
            for (int nt = 0; nt < NT; ++nt) {
                const int co = nt * 16 + 4 * g_now;
                const float4 bias = *reinterpret_cast<const float4 *>(per_channel[0] + co);
                const float4 fa = *reinterpret_cast<const float4 *>(per_channel[1] + co);
                const float4 fb = *reinterpret_cast<const float4 *>(per_channel[2] + co);
                f32x4w v0 = f32x4w{-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX}, v1 = v0;
#pragma unroll 1
                for (int t = 0; t < PT; ++t) {
                    if (at.oy0 + t >= p.oh) break;
                    f32x4w one = f32x4w{0.f, 0.f, 0.f, 0.f}, none = one;
#pragma unroll 1
                    for (int tap = 0; tap < TAPS; ++tap) {
                        const int ty = tap / KW, tx = tap - ty * KW;
                        f32x4r r[2];
                        fetch(at, true, t + ty, tx, r);
                        const float v[8] = {r[0][0], r[0][1], r[0][2], r[0][3], r[1][0], r[1][1], r[1][2], r[1][3]};
                        SplitFrag8 px, f;
                        px.set(v);
                        const uint16_t *src = filter_at(nt, ty, tx);
                        f.hi = *reinterpret_cast<const u4 *>(src), f.mid = *reinterpret_cast<const u4 *>(src + PLANE);
                        f.lo = *reinterpret_cast<const u4 *>(src + 2 * PLANE);
#pragma unroll
                        for (int e = 0; e < 4; ++e) f.hif[e] = finite_bf16_pair(f.hi[e]);
                        mfma6_16x16x32(one, none, f, px, px);
                    }
                    const float4 fin = make_float4(finish(one[0], bias.x, fa.x, fb.x), finish(one[1], bias.y, fa.y, fb.y),
                                                   finish(one[2], bias.z, fa.z, fb.z), finish(one[3], bias.w, fa.w, fb.w));
                    if constexpr (POOL) {
                        const float fv[4] = {fin.x, fin.y, fin.z, fin.w};
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            if (t <= 1) v0[e] = later_max(v0[e], fv[e]);
                            if (t >= 1) v1[e] = later_max(v1[e], fv[e]);
                        }
                        const size_t group = (size_t)at.img * p.row_groups + (at.oy0 >> 2);
                        if (t == PT - 1) *reinterpret_cast<float4 *>(p.brow + ((group * p.ow + at.xt * 16 + f_i) * COUT + co)) = fin;
                        if (f_i == 15) *reinterpret_cast<float4 *>(p.bcol + (((group * p.tiles_per_row + at.xt) * 4 + t) * COUT + co)) = fin;
                    } else {
                        const size_t m = ((size_t)at.img * p.oh + at.oy0 + t) * p.ow + at.xt * 16 + f_i;
                        *reinterpret_cast<float4 *>(p.out + m * COUT + co) = fin;
                    }
                }
                if constexpr (POOL) pool_store(at, nt, g_now, v0, v1);
            }
        }
    };

    // An item's results are written after the split of the next item, just before a long run of products: the wait
    // for the next fetched rows also waits for every store before it to be acknowledged (one counter covers both, and
    // loads and stores complete in no fixed order), which by then has long happened.
    Place done = here;
    bool have_done = false, done_special = false;
    struct Row {
        u4 hi, mid, lo;
    };
    auto split_row = [&](const f32x4r (&r)[2], uint32_t &magnitude) __attribute__((always_inline)) {
        const float v[8] = {r[0][0], r[0][1], r[0][2], r[0][3], r[1][0], r[1][1], r[1][2], r[1][3]};
        Row out;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const SplitPair sp = split_pair_finite(v[2 * e], v[2 * e + 1]);
            out.hi[e] = sp.hi, out.mid[e] = sp.mid, out.lo[e] = sp.lo;
            magnitude = bf16_pair_max(magnitude, sp.hi);
        }
        return out;
    };
    for (int item = first + wave; item < last;) {
        int taken = 0;
        if (lane == 0) taken = atomicAdd(&next_item, 1);
        const int next_index = __builtin_amdgcn_readfirstlane(taken);
        const Place next = locate(next_index);
        const bool next_ok = next_index < last;
        uint32_t magnitude = 0;
        // Every pixel is fetched and split once: the pixels of horizontal tap 1, and the halo.  Taps 0 and 2 are the
        // same values one lane over (a lane's neighbours in its group of 16 hold the neighbouring pixels' same eight
        // channels), moved with the lane-shifting form of v_mov; the end lane takes its value from the halo row.
        Row centre[ROWS];
#pragma unroll
        for (int j = 0; j < ROWS; ++j) centre[j] = split_row(raw[j], magnitude);
        const Row halo = split_row(raw_halo, magnitude);

        if (have_done) write_item(done, done_special);
#pragma unroll
        for (int t = 0; t < PT; ++t)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) acc[t][nt] = f32x4w{0.f, 0.f, 0.f, 0.f};

        // input row j as horizontal tap TX sees it
        auto shifted = [&](auto tx_c, auto j_c) __attribute__((always_inline)) {
            constexpr int TX = decltype(tx_c)::value, J = decltype(j_c)::value;
            if constexpr (TX == 1) {
                return centre[J];
            } else {
                Row out;
                auto move = [&](uint32_t c, uint32_t h) {
                    // row_shl:n (0x100 + n): lane i takes lane i + n's; row_shr:n (0x110 + n): lane i - n's; a lane
                    // without a source keeps the first argument
                    if constexpr (TX == 0) {
                        const int end = J == 0 ? (int)h : __builtin_amdgcn_update_dpp(0, (int)h, 0x100 + (J == 0 ? 1 : J), 0xf, 0xf, true);
                        return (uint32_t)__builtin_amdgcn_update_dpp(end, (int)c, 0x111, 0xf, 0xf, false);
                    } else {
                        const int end = __builtin_amdgcn_update_dpp(0, (int)h, 0x110 + (7 - J), 0xf, 0xf, true);
                        return (uint32_t)__builtin_amdgcn_update_dpp(end, (int)c, 0x101, 0xf, 0xf, false);
                    }
                };
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    out.hi[e] = move(centre[J].hi[e], halo.hi[e]);
                    out.mid[e] = move(centre[J].mid[e], halo.mid[e]);
                    out.lo[e] = move(centre[J].lo[e], halo.lo[e]);
                }
                return out;
            }
        };
        auto frag = [](const u4 &h, const u4 &m, const u4 &l) {
            SplitFrag8 f;
            f.hi = h, f.hif = h, f.mid = m, f.lo = l;
            return f;
        };
        auto of_row = [&](const Row &r) { return frag(r.hi, r.mid, r.lo); };
        // rows of the product = output channels (the filter fragment), columns = pixels; output row t takes input row
        // t + ty.  The rows of a tap are made as the vertical taps first need them: four, then one, then one.
        auto phase = [&](auto tx_c, auto &&after_first) __attribute__((always_inline)) {
            constexpr int TX = decltype(tx_c)::value;
            Row r0 = shifted(tx_c, std::integral_constant<int, 0>{}), r1 = shifted(tx_c, std::integral_constant<int, 1>{});
            Row r2 = shifted(tx_c, std::integral_constant<int, 2>{}), r3 = shifted(tx_c, std::integral_constant<int, 3>{});
            auto products = [&](int ty, const Row &a, const Row &b, const Row &c, const Row &d) __attribute__((always_inline)) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const uint16_t *src = filter_at(nt, ty, TX);
                    const SplitFrag8 f = frag(*reinterpret_cast<const u4 *>(src), *reinterpret_cast<const u4 *>(src + PLANE),
                                              *reinterpret_cast<const u4 *>(src + 2 * PLANE));
                    mfma6_16x16x32(acc[0][nt], acc[1][nt], f, of_row(a), of_row(b));
                    mfma6_16x16x32(acc[2][nt], acc[3][nt], f, of_row(c), of_row(d));
                }
                __builtin_amdgcn_sched_barrier(0);  // rows and filter fragments are made as they are needed, not up front
            };
            products(0, r0, r1, r2, r3);
            after_first();
            const Row r4 = shifted(tx_c, std::integral_constant<int, 4>{});
            products(1, r1, r2, r3, r4);
            const Row r5 = shifted(tx_c, std::integral_constant<int, 5>{});
            products(2, r2, r3, r4, r5);
        };
        phase(std::integral_constant<int, 1>{}, [] {});
        phase(std::integral_constant<int, 0>{}, [] {});
        phase(std::integral_constant<int, 2>{}, [&]() __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < ROWS; ++j) fetch(next, next_ok, j, 1, raw[j]);
            fetch_halo(next, next_ok, raw_halo);
        });

        done = here, have_done = true;
        done_special = w_special || __builtin_amdgcn_ballot_w64(!bf16_pairs_finite(magnitude)) != 0;
        here = next, item = next_index;
    }
    if (have_done) write_item(done, done_special);
}

// The pass behind fconv_c32_kernel<..., POOL>: a pooled cell of an even pooled row (the first of its tile column) takes
// the maxima with the three output pixels above it, which are in the last row of the tile column above (brow); a cell
// that is the first of its tile takes them with the output pixels left of it, the last pixels of the tile to the left
// (bcol).  The other cells are final as they are.  SIGN: pack_mat of the pooled tensor (cout a multiple of 64) -- the 16
// threads that hold the 64 channels of a word are one row of lanes, as in pool_vec4_kernel.
struct C32PoolCompleteArgs {
    float4 *pooled;
    const float4 *brow, *bcol;
    uint64_t *bits;
    int ph, pw, c4, ow, groups, tiles;
    uint32_t total;
    FastDiv div_c4, div_pw, div_ph;
};

template <bool SIGN>
__global__ __launch_bounds__(256) void c32_pool_complete_kernel(const C32PoolCompleteArgs p) {
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    if (idx >= p.total) return;
    const uint32_t t = p.div_c4.div(idx);
    const int ch = (int)(idx - t * (uint32_t)p.c4);
    const uint32_t t2 = p.div_pw.div(t);
    const int c = (int)(t - t2 * (uint32_t)p.pw);
    const uint32_t img = p.div_ph.div(t2);
    const int r = (int)(t2 - img * (uint32_t)p.ph), m = r >> 1;
    auto later_max = [](float4 a, float4 v) {
        return make_float4(v.x > a.x ? v.x : a.x, v.y > a.y ? v.y : a.y, v.z > a.z ? v.z : a.z, v.w > a.w ? v.w : a.w);
    };
    float4 v = p.pooled[idx];
    bool changed = false;
    if (!(r & 1) && m > 0) {
        const float4 *row = p.brow + ((size_t)img * p.groups + (m - 1)) * p.ow * p.c4 + ch;
#pragma unroll
        for (int dx = -1; dx <= 1; ++dx) {
            const int x = 2 * c + dx;
            if ((unsigned)x < (unsigned)p.ow) v = later_max(v, row[(size_t)x * p.c4]);
        }
        changed = true;
    }
    if (!(c & 7) && c > 0) {
        const float4 *col = p.bcol + ((((size_t)img * p.groups + m) * p.tiles + ((c >> 3) - 1)) * 4) * p.c4 + ch;
        if (r & 1) {
            v = later_max(later_max(later_max(v, col[p.c4]), col[2 * p.c4]), col[3 * p.c4]);
        } else {
            v = later_max(later_max(v, col[0]), col[p.c4]);
        }
        changed = true;
    }
    if (changed) p.pooled[idx] = v;
    if constexpr (SIGN) {
        const int part = (int)(idx & 15u);
        const uint32_t nib = sign_nibble(v);
        uint32_t lo = part < 8 ? nib << (4 * part) : 0u, hi = part >= 8 ? nib << (4 * (part - 8)) : 0u;
        lo = or_from_lane_above<1>(lo), hi = or_from_lane_above<1>(hi);
        lo = or_from_lane_above<2>(lo), hi = or_from_lane_above<2>(hi);
        lo = or_from_lane_above<4>(lo), hi = or_from_lane_above<4>(hi);
        lo = or_from_lane_above<8>(lo), hi = or_from_lane_above<8>(hi);
        if (part == 0) p.bits[idx >> 4] = ((uint64_t)hi << 32) | lo;
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
    return (long long)n * ((oh + kC32PixelTiles - 1) / kC32PixelTiles) * (ow / 16) >= 2 * waves;
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
    const int blocks = simd_count() / 4;  // one block of eight waves per CU (the filter planes take most of its LDS)
    FconvC32Args a;
    a.x = x, a.w = wgt, a.bias = bias, a.aff_a = aff_a, a.aff_b = aff_b, a.out = out, a.relu = relu;
    a.brow = nullptr, a.bcol = nullptr, a.bits = nullptr;
    a.h = h, a.wd = w, a.oh = oh, a.ow = ow, a.cout = cout, a.pad_h = pad_h, a.pad_w = pad_w;
    a.x_bytes = (uint32_t)((long long)n * h * w * 128);
    a.row_groups = (oh + kC32PixelTiles - 1) / kC32PixelTiles, a.tiles_per_row = ow / 16;
    a.items = n * a.row_groups * a.tiles_per_row;
    a.div_tiles_per_row = FastDiv((uint32_t)a.tiles_per_row), a.div_row_groups = FastDiv((uint32_t)a.row_groups);
    if (cout == 32)
        hipLaunchKernelGGL((fconv_c32_kernel<2, 3, 3>), dim3(blocks), dim3(kC32Threads), 0, s, a);
    else
        hipLaunchKernelGGL((fconv_c32_kernel<4, 3, 3>), dim3(blocks), dim3(kC32Threads), 0, s, a);
    return hipGetLastError() == hipSuccess ? 1 : fail(DAB_EHIP, "fconv_c32: launch failed");
}

// The convolution with the MaxPool 3x3, stride 2, pad 1 behind it (fconv_c32_kernel<..., POOL> and the completing pass):
// the shapes of fconv_c32_takes with an output height that is a multiple of 4.  workspace_floats: what `work` must hold.
bool fconv_c32_pool_takes(int n, int h, int w, int c, int kh, int kw, int pad_h, int pad_w, int stride_h, int stride_w, int dil_h,
                          int dil_w, int cout, int oh, int ow) {
    return oh % 4 == 0 && fconv_c32_takes(n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, cout, oh, ow) &&
           (long long)n * (oh / 2) * (ow / 2) * (cout / 4) < (1ll << 32) - 256;  // the completing pass counts cells in 32 bits
}

long long fconv_c32_pool_workspace_floats(int n, int oh, int ow, int cout) {
    return (long long)n * (oh / 4) * ow * cout + (long long)n * (oh / 4) * (ow / 16) * 4 * cout;
}

// Returns 1 when it ran, 0 when the buffers are not 16-byte aligned (the caller takes another path), negative on failure.
int fconv_c32_pool_run(const float *x, int n, int h, int w, const float *wgt, const float *bias, const float *aff_a,
                       const float *aff_b, int relu, int pad_h, int pad_w, int cout, int oh, int ow, float *pooled,
                       uint64_t *pooled_packed, float *work, hipStream_t s) {
    uintptr_t align = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(wgt) | reinterpret_cast<uintptr_t>(pooled) |
                      reinterpret_cast<uintptr_t>(work);
    if (bias) align |= reinterpret_cast<uintptr_t>(bias);
    if (aff_a) align |= reinterpret_cast<uintptr_t>(aff_a) | reinterpret_cast<uintptr_t>(aff_b);
    if (align % 16 != 0) return 0;
    const int blocks = simd_count() / 4;
    FconvC32Args a;
    a.x = x, a.w = wgt, a.bias = bias, a.aff_a = aff_a, a.aff_b = aff_b, a.out = pooled, a.relu = relu;
    a.brow = work, a.bcol = work + (size_t)n * (oh / 4) * ow * cout, a.bits = nullptr;
    a.h = h, a.wd = w, a.oh = oh, a.ow = ow, a.cout = cout, a.pad_h = pad_h, a.pad_w = pad_w;
    a.x_bytes = (uint32_t)((long long)n * h * w * 128);
    a.row_groups = oh / kC32PixelTiles, a.tiles_per_row = ow / 16;
    a.items = n * a.row_groups * a.tiles_per_row;
    a.div_tiles_per_row = FastDiv((uint32_t)a.tiles_per_row), a.div_row_groups = FastDiv((uint32_t)a.row_groups);
    if (cout == 32)
        hipLaunchKernelGGL((fconv_c32_kernel<2, 3, 3, true>), dim3(blocks), dim3(kC32Threads), 0, s, a);
    else
        hipLaunchKernelGGL((fconv_c32_kernel<4, 3, 3, true>), dim3(blocks), dim3(kC32Threads), 0, s, a);
    if (hipGetLastError() != hipSuccess) return fail(DAB_EHIP, "fconv_c32 (pooled): launch failed");
    C32PoolCompleteArgs f;
    f.pooled = reinterpret_cast<float4 *>(pooled), f.brow = reinterpret_cast<const float4 *>(a.brow);
    f.bcol = reinterpret_cast<const float4 *>(a.bcol), f.bits = pooled_packed;
    f.ph = oh / 2, f.pw = ow / 2, f.c4 = cout / 4, f.ow = ow, f.groups = a.row_groups, f.tiles = a.tiles_per_row;
    f.total = (uint32_t)((long long)n * f.ph * f.pw * f.c4);
    f.div_c4 = FastDiv((uint32_t)f.c4), f.div_pw = FastDiv((uint32_t)f.pw), f.div_ph = FastDiv((uint32_t)f.ph);
    const unsigned grid = (f.total + 255u) / 256u;
    if (pooled_packed)
        hipLaunchKernelGGL(c32_pool_complete_kernel<true>, dim3(grid), dim3(256), 0, s, f);
    else
        hipLaunchKernelGGL(c32_pool_complete_kernel<false>, dim3(grid), dim3(256), 0, s, f);
    return hipGetLastError() == hipSuccess ? 1 : fail(DAB_EHIP, "fconv_c32 (pooled): launch failed");
}

}  // namespace dab
