// fp32 convolution (+ Affine, Relu) and the 3x3 stride-2 pad-1 MaxPool behind it in one pass: the stem of a
// Bi-Real-style net (dabnn/fconv.h:14-76, dabnn/layers/Affine.cpp:10-23, dabnn/layers/MaxPool.cpp:209-246).  The
// convolution's output -- four times the size of the pooled tensor -- never goes to memory.
//
// A 512-thread block owns a band of R whole rows of the convolution's output of one image, R * OW = 448 pixels, and
// 64 output channels.  It multiplies like the plain float convolution (implicit GEMM, rows = pixels, depth = (kh, kw,
// c), two LDS buffers of SK-deep slices, v_mfma_f32_16x16x4_f32; eight waves as 4 x 2, a wave holds 112 pixels x 32
// channels), leaves the band in LDS and pools it there.  A pooled row 2*py-1 .. 2*py+1 lies inside the band for all
// but the band's first pooled row, which also needs the last row of the band above.  A block is persistent and makes
// consecutive bands of an image, so the horizontal maxima of a band's last row wait in the registers of the threads
// that pool the same columns of the next band.  Where another block made the band above (the first band of a
// block's range; every band when there are several 64-channel tiles), that block writes the row to a carry buffer,
// and a second, small kernel folds it into the first pooled row of the band below (a maximum does not depend on the
// order of its operands).  With the pooled tensor the kernels can write its sign bits, the packed input of the
// binary convolution that follows (dabnn/bitpack.h:277-293).
#include <float.h>

#include <type_traits>

#include "common.h"

namespace dab {

struct FconvPoolArgs {
    const float *x;
    const float *w;
    const float *bias;
    const float *aff_a;
    const float *aff_b;
    float *pooled;    // [n][ph][pw][cout]
    float *carry;     // [n][bands][pw][cout]
    uint64_t *bits;   // [n][ph][pw][cout/64] or null
    int n, h, wd, c;
    int kw, dil_h, dil_w;
    int pad_h, pad_w, stride_h, stride_w;
    int oh, ow, cout;
    int K;  // kh*kw*c
    int relu;
    int band_rows, bands;  // R, bands per image
    int ph, pw;
    int ytiles;  // 64-channel tiles of cout
    // chained: block b takes the items [b*per + min(b, extra), ...) one after the other (ytiles == 1: consecutive
    // bands of an image) and keeps a band's last row for the next one in registers; otherwise the items gridDim.x apart
    int chained, per, extra;
    FastDiv div_ow, div_c, div_kw, div_bands, div_ytiles;
};

// The work items of a block: first, one past the last, and the distance between two of them.
struct BandRange {
    int first, end, step;
};
__device__ __forceinline__ BandRange band_range(const FconvPoolArgs &p) {
    const int b = (int)blockIdx.x;
    if (!p.chained) return BandRange{b, p.n * p.bands * p.ytiles, (int)gridDim.x};
    const int first = b * p.per + (b < p.extra ? b : p.extra);
    return BandRange{first, first + p.per + (b < p.extra ? 1 : 0), 1};
}
constexpr int kKeepSlots = 4;  // pooled columns x 16 channel groups per thread: at most 112 * 16 / 512

typedef float f32x4v __attribute__((ext_vector_type(4)));

constexpr uint32_t kPoolOob = 0x80000000u;  // beyond every descriptor used here (all shorter than 2^30 bytes)
constexpr int kBandPixels = 448, kBandChannels = 64, kBandThreads = 512;
constexpr int kStageStride = 68;  // floats per pixel row of the staged band: the 64 lanes of a store hit 64 banks

template <int CV>
struct BandSlice {
    static constexpr int depth = CV == 3 ? 24 : 32;  // eight taps of three channels / eight groups of four channels
    static constexpr int stride = depth + 4;         // LDS row stride in floats
    static constexpr int loop_floats = 2 * (kBandPixels + kBandChannels) * stride;
    static constexpr int stage_floats = kBandPixels * kStageStride;
    static constexpr int lds_floats = loop_floats > stage_floats ? loop_floats : stage_floats;
};

// max of three values as the reference's loop computes it for results of arithmetic (v > m ? v : m skips a NaN; a
// convolution's result is never a signalling NaN, the only kind the instruction treats differently)
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
__device__ __forceinline__ float4 max3(float4 a, float4 b, float4 c) {
    return make_float4(max3(a.x, b.x, c.x), max3(a.y, b.y, c.y), max3(a.z, b.z, c.z), max3(a.w, b.w, c.w));
}

// What the epilogue needs to know of a finished band.
struct BandOut {
    int img, band, row0, n0, ytile;
};

// Pooling down the rows of a staged band: a thread takes four channels of one pooled column; column(px, c4) gives a
// function h(r), the maximum of row r's three columns 2*px-1 .. 2*px+1.  Pooled row q is max(h[2q-1], h[2q], h[2q+1]);
// for q = 0 the row above the band is left out: row -1 of the image does not exist, and the last row of the band
// above arrives through the carry, which is this band's h[R-1] -- or, when this block made the band above just before
// (fold), it is in `keep`: a thread has the same columns and channels in every band.
// ROWS: the band's rows when the kernel knows them (all loads of a column are then asked for at once).
template <bool SIGN, int SLOTS, int ROWS, class Column>
__device__ __forceinline__ void pool_band_rows(const FconvPoolArgs &p, const BandOut o, int tid, float4 (&keep)[SLOTS], bool fold,
                                               bool write_carry, Column column) {
#pragma unroll
    for (int slot = 0; slot < SLOTS; ++slot) {
        const int it = tid + slot * kBandThreads;
        if (it >= p.pw * 16) break;
        const int c4 = it & 15, px = it >> 4;
        const int co = o.n0 + c4 * 4;
        const auto h_of = column(px, c4);
        const float4 lowest = make_float4(-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX);
        float4 prev = fold ? keep[slot] : lowest, even = lowest;
        const int rows = ROWS ? ROWS : p.band_rows;
        constexpr int kUnrollRows = ROWS > 0 ? ROWS : 1;
#pragma unroll kUnrollRows
        for (int r = 0; r < rows; ++r) {
            const float4 h = h_of(r);
            if (r & 1) {
                const float4 m = max3(even, h, lowest);
                if (co < p.cout) {
                    const size_t pix = (size_t)(o.img * p.ph + ((o.row0 + r) >> 1)) * p.pw + px;
                    *reinterpret_cast<float4 *>(p.pooled + pix * p.cout + co) = m;
                    if constexpr (SIGN) {
                        // cout % 64 == 0: the 16 lanes of a pixel are one row of lanes, all of them here
                        const uint32_t nib = sign_nibble(m);
                        uint32_t lo = c4 < 8 ? nib << (4 * c4) : 0u, hi = c4 >= 8 ? nib << (4 * (c4 - 8)) : 0u;
                        lo = or_from_lane_above<1>(lo), hi = or_from_lane_above<1>(hi);
                        lo = or_from_lane_above<2>(lo), hi = or_from_lane_above<2>(hi);
                        lo = or_from_lane_above<4>(lo), hi = or_from_lane_above<4>(hi);
                        lo = or_from_lane_above<8>(lo), hi = or_from_lane_above<8>(hi);
                        if (c4 == 0) p.bits[pix * (p.cout >> 6) + o.ytile] = ((uint64_t)hi << 32) | lo;
                    }
                }
            } else {
                even = max3(prev, h, lowest);  // r == 0 without fold: prev is the lowest value, the row above is left out
            }
            prev = h;
        }
        keep[slot] = prev;
        if (write_carry && co < p.cout) {
            const float4 m = max3(prev, lowest, lowest);
            *reinterpret_cast<float4 *>(p.carry + ((size_t)(o.img * p.bands + o.band) * p.pw + px) * p.cout + co) = m;
        }
    }
}

// A finished band (a wave's accumulators: 7 x 2 tiles of 16 pixels x 16 channels, wave (wm, wn) = pixels 112*wm ..,
// channels 32*wn ..) goes through LDS to the pooled tensor, the carry and the sign bits.  All threads of the block
// call it after a barrier that ended every other use of `stage`.
template <bool SIGN, int SLOTS, int ROWS = 0>
__device__ __forceinline__ void band_epilogue(const FconvPoolArgs &p, float *stage, const f32x4v (&acc)[7][2], const BandOut o,
                                              int tid, int wm, int wn, int f_s, int f_i, float4 (&keep)[SLOTS],
                                              bool fold, bool write_carry) {
    constexpr int TM = 7, TN = 2;
    // The band goes to LDS (the slices are dead: the loop ended with a barrier): + bias, Affine (a*v + b, two
    // roundings), Relu, in the reference's order.  Accumulator element e of lane l: pixel 4*(l/16) + e, channel l % 16.
    auto stage_all = [&](auto has_bias, auto has_affine, auto has_relu) {
#pragma clang fp contract(off)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int col = wn * (TN * 16) + j * 16 + f_i, co = o.n0 + col;
            const bool co_ok = co < p.cout;
            const float bias = (decltype(has_bias)::value && co_ok) ? p.bias[co] : 0.f;
            const float fa = (decltype(has_affine)::value && co_ok) ? p.aff_a[co] : 0.f;
            const float fb = (decltype(has_affine)::value && co_ok) ? p.aff_b[co] : 0.f;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float v = acc[i][j][e];
                    if constexpr (decltype(has_bias)::value) v = v + bias;
                    if constexpr (decltype(has_affine)::value) {
                        const float prod = fa * v;
                        v = prod + fb;
                    }
                    if constexpr (decltype(has_relu)::value) v = v < 0.f ? 0.f : v;  // std::max(v, 0.f): a NaN stays
                    stage[(wm * (TM * 16) + i * 16 + 4 * f_s + e) * kStageStride + col] = v;
                }
        }
    };
    using T = std::true_type;
    using F = std::false_type;
    switch ((p.bias ? 4 : 0) | (p.aff_a ? 2 : 0) | (p.relu ? 1 : 0)) {
        case 0: stage_all(F{}, F{}, F{}); break;
        case 1: stage_all(F{}, F{}, T{}); break;
        case 2: stage_all(F{}, T{}, F{}); break;
        case 3: stage_all(F{}, T{}, T{}); break;
        case 4: stage_all(T{}, F{}, F{}); break;
        case 5: stage_all(T{}, F{}, T{}); break;
        case 6: stage_all(T{}, T{}, F{}); break;
        default: stage_all(T{}, T{}, T{}); break;
    }
    __syncthreads();
    const int ow = ROWS ? kBandPixels / ROWS : p.ow;
    // h of row r = the maximum of the row's three columns 2*px-1 .. 2*px+1 (the first pooled column has two; one is
    // read twice)
    pool_band_rows<SIGN, SLOTS, ROWS>(p, o, tid, keep, fold, write_carry, [&](int px, int c4) {
        const float *col0 = &stage[(px == 0 ? 0 : 2 * px - 1) * kStageStride + c4 * 4];
        const float *col1 = &stage[(2 * px) * kStageStride + c4 * 4];
        return [=](int r) {
            const int ro = r * ow * kStageStride;
            return max3(*reinterpret_cast<const float4 *>(col0 + ro), *reinterpret_cast<const float4 *>(col1 + ro),
                        *reinterpret_cast<const float4 *>(col1 + ro + kStageStride));
        };
    });
}

template <int CV, bool SIGN>
__global__ __launch_bounds__(kBandThreads) void fconv_maxpool_kernel(const FconvPoolArgs p) {
    constexpr int BM = kBandPixels, BN = kBandChannels;
    constexpr int SK = BandSlice<CV>::depth, RS = BandSlice<CV>::stride;
    constexpr int LK = SK / CV;              // loader lanes along the depth
    constexpr int RP = kBandThreads / LK;    // tile rows fetched per pass of the block
    constexpr int APT = BM / RP;             // pixel rows per thread and slice
    constexpr int TM = 7, TN = 2;            // 16 x 16 matrix-core tiles per wave
    static_assert(LK == 8 && RP == 64 && APT == 7 && RP == BN, "loader shape");
    __shared__ __attribute__((aligned(16))) float smem[BandSlice<CV>::lds_floats];
    auto As = [&](int buf, int row, int k) -> float & { return smem[(buf * (BM + BN) + row) * RS + k]; };
    auto Bs = [&](int buf, int row, int k) -> float & { return smem[(buf * (BM + BN) + BM + row) * RS + k]; };

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int l_k = tid % LK, l_r = tid / LK;  // loader: depth group l_k of the slice, tile rows l_r + RP*i
    const uint32_t img_bytes = (uint32_t)(p.h * p.wd * p.c) * 4u;
    const uint32_t b_row = (uint32_t)l_r * p.K * 4u;

    // the band of the loader (the one whose slices are being fetched) and its addresses
    int img, band, row0, n0, rows_n;
    __amdgpu_buffer_rsrc_t x_rsrc, w_rsrc;
    uint32_t a_base[APT];  // byte offset of (y0, x0, channel 0) in the image, modulo 2^32
    int a_x0[APT];
    int a_lr[APT], a_ox[APT];  // the thread's pixels inside a band, the same for every band
#pragma unroll
    for (int i = 0; i < APT; ++i) {
        const int r = l_r + RP * i;
        a_lr[i] = (int)p.div_ow.div((uint32_t)r), a_ox[i] = r - a_lr[i] * p.ow;
    }
    auto enter = [&](int item) {
        const int bi = (int)p.div_ytiles.div((uint32_t)item);
        n0 = (item - bi * p.ytiles) * BN;
        img = (int)p.div_bands.div((uint32_t)bi);
        band = bi - img * p.bands;
        row0 = band * p.band_rows;
        // The descriptor covers one image: a tap above or below the image has an offset that is negative modulo
        // 2^32 or at least the image's size, and reads as zero without a test; only the column needs one.
        x_rsrc = make_rsrc(p.x + (size_t)img * p.h * p.wd * p.c, img_bytes);
        rows_n = p.cout - n0 < BN ? p.cout - n0 : BN;
        w_rsrc = make_rsrc(p.w + (size_t)n0 * p.K, (uint32_t)rows_n * p.K * 4u);
#pragma unroll
        for (int i = 0; i < APT; ++i) {
            const int y0 = (row0 + a_lr[i]) * p.stride_h - p.pad_h, x0 = a_ox[i] * p.stride_w - p.pad_w;
            a_base[i] = (uint32_t)((y0 * p.wd + x0) * p.c) * 4u;
            a_x0[i] = x0;
        }
    };

    typedef float f32xcv __attribute__((ext_vector_type(CV)));
    f32xcv a_reg[APT], b_reg;
    auto load_cv = [](__amdgpu_buffer_rsrc_t rsrc, uint32_t off) -> f32xcv {
        // bit-cast as a whole: casting single elements of a vector buffer load makes the compiler shrink the load
        if constexpr (CV == 3)
            return __builtin_bit_cast(f32xcv, __builtin_amdgcn_raw_buffer_load_b96(rsrc, (int)off, 0, 0));
        else
            return __builtin_bit_cast(f32xcv, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)off, 0, 0));
    };
    auto fetch = [&](int k0) {
        // CV == 3: lane group = tap, channels 0..2 (c == 3).  CV == 4: four consecutive channels of a tap (c % 4 == 0).
        const int k = k0 + CV * l_k;
        const bool k_ok = k < p.K;
        int tap, ch;
        if constexpr (CV == 3) {
            tap = (int)((uint32_t)k0 / 3u) + l_k, ch = 0;
        } else {
            tap = (int)p.div_c.div((uint32_t)k), ch = k - tap * p.c;
        }
        const int ty = (int)p.div_kw.div((uint32_t)tap), tx = tap - ty * p.kw;
        const int dy = ty * p.dil_h, dx = tx * p.dil_w;
        // a depth past the end: 2^31 added to an offset of magnitude below 2^30 stays out of range
        const uint32_t delta = k_ok ? (uint32_t)((dy * p.wd + dx) * p.c + ch) * 4u : kPoolOob;
#pragma unroll
        for (int i = 0; i < APT; ++i)
            a_reg[i] = load_cv(x_rsrc, (unsigned)(a_x0[i] + dx) < (unsigned)p.wd ? a_base[i] + delta : kPoolOob);
        b_reg = load_cv(w_rsrc, (k_ok && l_r < rows_n) ? b_row + (uint32_t)k * 4u : kPoolOob);
    };
    auto commit = [&](int buf) {
#pragma unroll
        for (int i = 0; i < APT; ++i)
#pragma unroll
            for (int c = 0; c < CV; ++c) As(buf, l_r + RP * i, l_k * CV + c) = a_reg[i][c];
#pragma unroll
        for (int c = 0; c < CV; ++c) Bs(buf, l_r, l_k * CV + c) = b_reg[c];
    };

    // operand lane l of the instruction: row / column l % 16, depth slot l / 16.  Which depth sits in which of the
    // four slots does not matter as long as both operands agree: a lane reads two consecutive depths at once and
    // uses them in two instructions.
    const int f_s = lane >> 4, f_i = lane & 15;
    const BandRange range = band_range(p);
    int item = range.first;
    if (item >= range.end) return;
    float4 keep[kKeepSlots];
#pragma unroll
    for (int slot = 0; slot < kKeepSlots; ++slot) keep[slot] = make_float4(-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX);
    bool fold = false;
    enter(item);
    fetch(0);
    for (;;) {
        // here: the first slice of `item` is in registers, every thread is past its last read of the LDS
        commit(0);
        __syncthreads();
        f32x4v acc[TM][TN];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = f32x4v{0.f, 0.f, 0.f, 0.f};
        int buf = 0;
        for (int k0 = 0; k0 < p.K; k0 += SK, buf ^= 1) {
            const bool more = k0 + SK < p.K;
            if (more) fetch(k0 + SK);
#pragma unroll
            for (int g = 0; g < SK / 8; ++g) {
                // the last slice may end early: groups that lie wholly past the depth hold zeros on both sides
                if (g > 0 && k0 + g * 8 >= p.K) break;
                const int kb = g * 8 + 2 * f_s;
                float2 a2[TM], b2[TN];
#pragma unroll
                for (int i = 0; i < TM; ++i) a2[i] = *reinterpret_cast<const float2 *>(&As(buf, wm * (TM * 16) + i * 16 + f_i, kb));
#pragma unroll
                for (int j = 0; j < TN; ++j) b2[j] = *reinterpret_cast<const float2 *>(&Bs(buf, wn * (TN * 16) + j * 16 + f_i, kb));
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j) {
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a2[i].x, b2[j].x, acc[i][j], 0, 0, 0);
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a2[i].y, b2[j].y, acc[i][j], 0, 0, 0);
                    }
            }
            // the other buffer was last read before the barrier that ended the previous slice
            if (more) commit(buf ^ 1);
            __syncthreads();
        }

        // what the epilogue needs of this band, then the next band's first slice is asked for: its latency hides
        // behind the epilogue
        const int e_img = img, e_band = band, e_row0 = row0, e_n0 = n0;
        const int next = item + range.step;
        const bool has_next = next < range.end;
        if (has_next) {
            enter(next);
            fetch(0);
        }

        // chained: the band above was this block's previous item unless this is its first one or an image's first
        // band; the carry goes to memory only where another block continues
        band_epilogue<SIGN, kKeepSlots>(p, smem, acc, BandOut{e_img, e_band, e_row0, e_n0, e_n0 / BN}, tid, wm, wn, f_s, f_i, keep,
                            fold && e_band > 0, !p.chained || !has_next);
        if (!has_next) break;
        fold = p.chained != 0;
        item = next;
        __syncthreads();  // the staged band is dead
    }
}

// The ImageNet stem itself -- 7x7, stride 2, pad 3 on three-channel images whose output is 112 pixels wide -- without
// an im2col stage: a band's 13 input rows go to LDS as they are (230 pixels from x = -3, zeros outside the image), and
// the matrix-core operands are read straight from them.  Wave (wm, wn) owns output row wm of the band and 32
// channels; an output pixel's 21 values of one kernel row are contiguous (tile elements 6*ox + k', k' = 3*tx + ch),
// so a lane's operand addresses are a base plus constants.
//
// The products run on the bf16 matrix cores with fp32 accuracy (split operands, six v_mfma_f32_16x16x32_bf16 per 32
// depths; common.h): the instruction takes 19 cycles where the eight fp32 ones for the same depth take 256.  The tile
// is split once, on its way into LDS, into three planes of bf16 (hi, mid, lo), and so are the block's 64 filters, once
// for all of its bands, in the order the instruction wants them (a lane's eight depths are 16 contiguous bytes).  The
// cross terms need hi with non-finite values taken out (common.h); a band with an infinity or a NaN in its rows or in
// the filters -- flags in LDS say so -- takes a second copy of the loop that derives it from hi in registers, all
// other bands use hi as it is.  A depth group is
// four slots of eight depths, slot g = lane / 16; the 147 depths make 19 slots: q = 0..13: kernel row q / 2, k' = 0..7
// or 8..15; q = 14..17: k' = 16..19 of kernel rows (0, 1), (2, 3), (4, 5), (6, none); q = 18: k' = 20 of the seven
// kernel rows, which a second small array per plane holds transposed (T20[ox][tile row]) so that they are contiguous
// too; q = 19 is empty.  Empty halves read a zero area of the plane; the eighth element of slot 18 is masked (it is a
// real tile value, and zero times an infinity would be a NaN).  160 depths for 147, five groups.
// The next band's rows are fetched into registers while the current one is pooled.  Pooling starts in registers: a
// lane holds four neighbouring pixels of a row, so the maxima over the columns 2*px-1 .. 2*px+1 of two pooled columns
// need one value from the lane 16 below; only those maxima -- half of the band -- are staged in LDS for the pass
// down the rows.
constexpr int kTileStride = 692;                    // elements per tile row: 115 pixel pairs x 6, + 2
constexpr int kTileRows = 13, kTilePairs = 115;
constexpr int kPlaneZero = 9000;                    // eight zeros behind the 13 x 692 tile elements
constexpr int kPlaneT20 = kPlaneZero + 8;           // [112 output columns][16]: tile rows of element 6 * ox + 20
constexpr int kPlane = kPlaneT20 + 112 * 16;        // bf16 elements per plane
constexpr int kStemDepth = 160;                     // 5 groups x 4 slots x 8
constexpr int kFilterRow = kStemDepth + 8;          // bf16 elements per filter in a plane
constexpr int kFilterPlane = kBandChannels * kFilterRow;
constexpr int kStemStageStride = 72;                // floats per pooled column of the staged maxima: two columns on are 16 banks on
constexpr int kStemStageFloats = 4 * 56 * kStemStageStride;
constexpr int kStemWorkBytes = 3 * kPlane * 2 > kStemStageFloats * 4 ? 3 * kPlane * 2 : kStemStageFloats * 4;  // the planes share the staged maxima's space
constexpr int kPairLoads = (kTileRows * kTilePairs + kBandThreads - 1) / kBandThreads;
constexpr int kStemKeepSlots = 2;  // 56 pooled columns x 16 channel groups on 512 threads
static_assert(56 * 16 <= kStemKeepSlots * kBandThreads, "pooled columns of the stem");
static_assert(kTileStride * kTileRows <= kPlaneZero && (kPlaneT20 * 2) % 16 == 0 && (kPlane * 2) % 16 == 0, "plane layout");
static_assert((kFilterRow * 2) % 16 == 0 && kStemWorkBytes % 16 == 0, "filter rows and the work area are 16-byte aligned");

// The stem's finished band (accumulator element e of lane l: pixel 16*i + 4*(l/16) + e of row wm, channel l % 16 of
// tile j): + bias, Affine (a*v + b, two roundings), Relu, in the reference's order; then the maxima over the columns
// of the two pooled columns 8*i + 2*(l/16) and the next one go to LDS, and pool_band_rows walks down the four rows.
// All threads of the block call it after a barrier that ended every other use of `stage`.
template <bool SIGN>
__device__ __forceinline__ void stem_epilogue(const FconvPoolArgs &p, float *stage, const f32x4v (&acc)[7][2], const BandOut o,
                                              int tid, int wm, int wn, int f_s, int f_i, float4 (&keep)[kStemKeepSlots],
                                              bool fold, bool write_carry) {
    constexpr int TM = 7, TN = 2;
    const int below = (((tid & 63) - 16) & 63) * 4;  // ds_bpermute address of the lane 16 below (lanes 0..15: 48 above)
    auto stage_all = [&](auto has_bias, auto has_affine, auto has_relu) {
#pragma clang fp contract(off)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int col = wn * (TN * 16) + j * 16 + f_i, co = o.n0 + col;
            const bool co_ok = co < p.cout;
            const float bias = (decltype(has_bias)::value && co_ok) ? p.bias[co] : 0.f;
            const float fa = (decltype(has_affine)::value && co_ok) ? p.aff_a[co] : 0.f;
            const float fb = (decltype(has_affine)::value && co_ok) ? p.aff_b[co] : 0.f;
            float left = -FLT_MAX;  // lanes 0..15: the last pixel of the tile before (none before the first)
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = acc[i][j][e];
                    if constexpr (decltype(has_bias)::value) v[e] = v[e] + bias;
                    if constexpr (decltype(has_affine)::value) {
                        const float prod = fa * v[e];
                        v[e] = prod + fb;
                    }
                    if constexpr (decltype(has_relu)::value) v[e] = v[e] < 0.f ? 0.f : v[e];  // std::max(v, 0.f): a NaN stays
                }
                const float from_below = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(below, __builtin_bit_cast(int, v[3])));
                const float before = f_s > 0 ? from_below : left;
                left = from_below;
                float *d = &stage[(wm * 56 + i * 8 + 2 * f_s) * kStemStageStride + col];
                d[0] = max3(before, v[0], v[1]);
                d[kStemStageStride] = max3(v[1], v[2], v[3]);
            }
        }
    };
    using T = std::true_type;
    using F = std::false_type;
    switch ((p.bias ? 4 : 0) | (p.aff_a ? 2 : 0) | (p.relu ? 1 : 0)) {
        case 0: stage_all(F{}, F{}, F{}); break;
        case 1: stage_all(F{}, F{}, T{}); break;
        case 2: stage_all(F{}, T{}, F{}); break;
        case 3: stage_all(F{}, T{}, T{}); break;
        case 4: stage_all(T{}, F{}, F{}); break;
        case 5: stage_all(T{}, F{}, T{}); break;
        case 6: stage_all(T{}, T{}, F{}); break;
        default: stage_all(T{}, T{}, T{}); break;
    }
    __syncthreads();
    pool_band_rows<SIGN, kStemKeepSlots, 4>(p, o, tid, keep, fold, write_carry, [&](int px, int c4) {
        const float *col = &stage[px * kStemStageStride + c4 * 4];
        return [=](int r) { return *reinterpret_cast<const float4 *>(col + r * (56 * kStemStageStride)); };
    });
}

template <bool SIGN>
__global__ __launch_bounds__(kBandThreads) void fconv7x7s2_maxpool_kernel(const FconvPoolArgs p) {
    constexpr int BN = kBandChannels, TM = 7, TN = 2;
    typedef uint32_t u32x2a __attribute__((ext_vector_type(2), aligned(4)));
    __shared__ __attribute__((aligned(16))) uint16_t fplanes[3 * kFilterPlane];  // the filters: hi, mid, lo
    __shared__ __attribute__((aligned(16))) float stage[kStemWorkBytes / 4];
    uint16_t *const planes = reinterpret_cast<uint16_t *>(stage);  // the band's rows: hi, mid, lo, kPlane elements each
    __shared__ int special_flag;    // the band's rows hold an infinity or a NaN
    __shared__ int special_filters;  // 1 + the first channel of a channel tile whose filters hold one, or 0

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int f_s = lane >> 4, f_i = lane & 15;
    const uint32_t img_bytes = (uint32_t)(p.h * p.wd * 3) * 4u;
    const BandRange range = band_range(p);
    int item = range.first;
    if (item >= range.end) return;
    float4 keep[kStemKeepSlots];
#pragma unroll
    for (int slot = 0; slot < kStemKeepSlots; ++slot) keep[slot] = make_float4(-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX);
    bool fold = false;

    // the thread's pixel pairs of a tile (pair u = tid + 512 * j: tile row u / 115, pixels 2 * (u % 115) - 3 and the
    // next): byte offsets from the tile's first row in the image and places in a plane, worked out again wherever
    // they are needed rather than held in registers across the multiplication
    struct PairPlace {
        uint32_t off0, off1;
        int lds, t20;
    };
    auto pair_place = [&](int j) {
        int u = tid + kBandThreads * j;
        asm volatile("" : "+v"(u));  // worked out here every time: hoisted out of the band loop these values are spilled
        const int ry = u / kTilePairs, pr = u - ry * kTilePairs, x0 = 2 * pr - 3;
        const bool in = u < kTileRows * kTilePairs;
        PairPlace q;
        q.off0 = in && (unsigned)x0 < (unsigned)p.wd ? (uint32_t)((ry * p.wd + x0) * 12) : kPoolOob;
        q.off1 = in && (unsigned)(x0 + 1) < (unsigned)p.wd ? (uint32_t)((ry * p.wd + x0 + 1) * 12) : kPoolOob;
        q.lds = in ? ry * kTileStride + 6 * pr : -1;
        q.t20 = in && pr >= 3 ? kPlaneT20 + (pr - 3) * 16 + ry : -1;  // the pair's third element is tile element 6 * (pr - 3) + 20
        return q;
    };
    typedef float f32x3v __attribute__((ext_vector_type(3)));
    f32x3v pf0[kPairLoads], pf1[kPairLoads];
    int img, band, row0, n0;
    auto enter = [&](int it) {
        const int bi = (int)p.div_ytiles.div((uint32_t)it);
        n0 = (it - bi * p.ytiles) * BN;
        img = (int)p.div_bands.div((uint32_t)bi);
        band = bi - img * p.bands;
        row0 = band * 4;
    };
    auto fetch_tile = [&]() {
        // One descriptor per image: rows above and below it have offsets that are negative modulo 2^32 or at least
        // the image's size, and read as zero; columns outside carry kPoolOob, which stays out of range after the
        // addition of a row offset of magnitude below 2^30.
        const auto x_rsrc = make_rsrc(p.x + (size_t)img * p.h * p.wd * 3, img_bytes);
        const uint32_t base = (uint32_t)((2 * row0 - 3) * p.wd * 12);
#pragma unroll
        for (int j = 0; j < kPairLoads; ++j) {
            const PairPlace q = pair_place(j);
            pf0[j] = __builtin_bit_cast(f32x3v, __builtin_amdgcn_raw_buffer_load_b96(x_rsrc, (int)(base + q.off0), 0, 0));
            pf1[j] = __builtin_bit_cast(f32x3v, __builtin_amdgcn_raw_buffer_load_b96(x_rsrc, (int)(base + q.off1), 0, 0));
        }
    };

    // lane constants of the tile reads: the plane elements of a slot's two halves of four (tile i of the wave's
    // row: + 96 * i; slot 18: + 256 * i; the zero area: + 0).  Groups 0..2 and the first two slots of group 3 are
    // eight consecutive k' of kernel row 2 * G + g / 2: group 0's offsets plus a constant.  The other slots of group
    // 3 and group 4 have offsets of their own.  (The filter planes are laid out slot by slot when they are filled.)
    const int base_a = 2 * wm * kTileStride + 6 * f_i;
    const int a_main = base_a + (f_s >> 1) * kTileStride + 8 * (f_s & 1);
    // group 3: slots 12, 13 (kernel row 6), 14, 15 (k' = 16..19 of kernel rows (0, 1) and (2, 3))
    const int a0_g3 = f_s < 2 ? a_main + 6 * kTileStride : base_a + 2 * (f_s - 2) * kTileStride + 16;
    const int a1_g3 = a0_g3 + (f_s < 2 ? 4 : kTileStride);
    // group 4: slots 16 (kernel rows 4, 5), 17 (row 6, nothing), 18 (k' = 20 of all rows), 19 (nothing)
    const int a0_g4 = f_s < 2 ? base_a + (4 + 2 * f_s) * kTileStride + 16 : f_s == 2 ? kPlaneT20 + f_i * 16 + 2 * wm : kPlaneZero;
    const int a1_g4 = f_s == 0 ? a0_g4 + kTileStride : f_s == 2 ? a0_g4 + 4 : kPlaneZero;
    const int s0_g4 = f_s < 2 ? 96 : f_s == 2 ? 256 : 0, s1_g4 = f_s == 0 ? 96 : f_s == 2 ? 256 : 0;
    const uint32_t keep_g4 = f_s == 2 ? 0x0000ffffu : 0xffffffffu;  // slot 18: seven kernel rows, the eighth element out

    enter(item);
    fetch_tile();
    if (tid == 0) special_flag = 0, special_filters = 0;
    __syncthreads();
    int filters_of = -1;  // the channel tile whose filters are in LDS
    for (;;) {
        // here: the band's rows are in registers (or on their way), every thread is past its last read of the LDS
        if (n0 != filters_of) {
            filters_of = n0;
            const int rows_n = p.cout - n0 < BN ? p.cout - n0 : BN;
            bool special = false;
            // two consecutive places of a filter's 160: slot q = place / 8, element t = place % 8
            for (int idx = tid; idx < BN * (kStemDepth / 2); idx += kBandThreads) {
                const int co = idx / (kStemDepth / 2), pr = idx - co * (kStemDepth / 2);
                SplitParts sp[2];
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const int q = (2 * pr + e) >> 3, t = (2 * pr + e) & 7;
                    int k = -1;  // the place's depth in the filter's (kernel row, k') order
                    if (q < 14) {
                        k = (q >> 1) * 21 + 8 * (q & 1) + t;
                    } else if (q < 18) {
                        const int ky = 2 * (q - 14) + (t >> 2);
                        if (ky < 7) k = ky * 21 + 16 + (t & 3);
                    } else if (q == 18 && t < 7) {
                        k = t * 21 + 20;
                    }
                    sp[e] = split_bf16x3((co < rows_n && k >= 0) ? p.w[(size_t)(n0 + co) * 147 + k] : 0.f);
                    special |= sp[e].hif != sp[e].hi;
                }
                uint32_t *d = reinterpret_cast<uint32_t *>(fplanes + co * kFilterRow + 2 * pr);
                d[0] = pack_upper_halves(sp[0].hi, sp[1].hi);
                d[kFilterPlane / 2] = pack_upper_halves(sp[0].mid, sp[1].mid);
                d[2 * (kFilterPlane / 2)] = pack_upper_halves(sp[0].lo, sp[1].lo);
            }
            if (special) special_filters = n0 + 1;
        }
        if (tid < 12) reinterpret_cast<uint32_t *>(planes + (tid >> 2) * kPlane + kPlaneZero)[tid & 3] = 0u;
        bool any_special = false;
#pragma unroll
        for (int j = 0; j < kPairLoads; ++j) {
            const PairPlace q = pair_place(j);
            if (q.lds >= 0) {
                // the six values as three pairs through the packed conversions; a triple with an infinity, a NaN or a
                // value that rounds up to an infinity is split again the slow way (and sends the band through the
                // loop that derives the finite parts, which is right for finite values too)
                const float v[6] = {pf0[j][0], pf0[j][1], pf0[j][2], pf1[j][0], pf1[j][1], pf1[j][2]};
                SplitPair sp[3];
                uint32_t magnitudes = 0;
#pragma unroll
                for (int e = 0; e < 3; ++e) {
                    sp[e] = split_pair_finite(v[2 * e], v[2 * e + 1]);
                    magnitudes = bf16_pair_max(magnitudes, sp[e].hi);
                }
                if (!bf16_pairs_finite(magnitudes)) {
                    any_special = true;
#pragma unroll
                    for (int e = 0; e < 3; ++e) {
                        const SplitParts s0 = split_bf16x3(v[2 * e]), s1 = split_bf16x3(v[2 * e + 1]);
                        sp[e].hi = pack_upper_halves(s0.hi, s1.hi);
                        sp[e].mid = pack_upper_halves(s0.mid, s1.mid);
                        sp[e].lo = pack_upper_halves(s0.lo, s1.lo);
                    }
                }
                uint32_t *d = reinterpret_cast<uint32_t *>(planes + q.lds);
#pragma unroll
                for (int e = 0; e < 3; ++e) {
                    d[e] = sp[e].hi;
                    d[kPlane / 2 + e] = sp[e].mid;
                    d[2 * (kPlane / 2) + e] = sp[e].lo;
                }
                if (q.t20 >= 0) {  // the pair's third value: the first of the second pair
                    planes[q.t20] = (uint16_t)sp[1].hi;
                    planes[kPlane + q.t20] = (uint16_t)sp[1].mid;
                    planes[2 * kPlane + q.t20] = (uint16_t)sp[1].lo;
                }
            }
        }
        if (any_special) special_flag = 1;
        __syncthreads();

        const BandOut o{img, band, row0, n0, n0 / BN};
        const int next = item + range.step;
        const bool has_next = next < range.end;

        f32x4v acc[TM][TN];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = f32x4v{0.f, 0.f, 0.f, 0.f};
        // a slot's eight bf16 of every plane: two halves of four (each 4-byte aligned)
        auto a_frag = [&](auto derive_finite, int e0, int e1, uint32_t keep_mask) {
            SplitFrag8 f;
            const u32x2a h0 = *reinterpret_cast<const u32x2a *>(planes + e0), h1 = *reinterpret_cast<const u32x2a *>(planes + e1);
            const u32x2a m0 = *reinterpret_cast<const u32x2a *>(planes + kPlane + e0), m1 = *reinterpret_cast<const u32x2a *>(planes + kPlane + e1);
            const u32x2a l0 = *reinterpret_cast<const u32x2a *>(planes + 2 * kPlane + e0), l1 = *reinterpret_cast<const u32x2a *>(planes + 2 * kPlane + e1);
            f.hi = SplitFrag8::u4{h0.x, h0.y, h1.x, h1.y & keep_mask};
            f.mid = SplitFrag8::u4{m0.x, m0.y, m1.x, m1.y & keep_mask};
            f.lo = SplitFrag8::u4{l0.x, l0.y, l1.x, l1.y & keep_mask};
            if constexpr (decltype(derive_finite)::value) {
#pragma unroll
                for (int e = 0; e < 4; ++e) f.hif[e] = finite_bf16_pair(f.hi[e]);
            } else {
                f.hif = f.hi;
            }
            return f;
        };
        auto b_frag = [&](auto derive_finite, int G, int j) {
            const uint16_t *row = fplanes + (wn * 32 + j * 16 + f_i) * kFilterRow + G * 32 + f_s * 8;
            SplitFrag8 f;
            f.hi = *reinterpret_cast<const SplitFrag8::u4 *>(row);
            f.mid = *reinterpret_cast<const SplitFrag8::u4 *>(row + kFilterPlane);
            f.lo = *reinterpret_cast<const SplitFrag8::u4 *>(row + 2 * kFilterPlane);
            if constexpr (decltype(derive_finite)::value) {
#pragma unroll
                for (int e = 0; e < 4; ++e) f.hif[e] = finite_bf16_pair(f.hi[e]);
            } else {
                f.hif = f.hi;
            }
            return f;
        };
        auto tile_frag = [&](auto derive_finite, int G, int i) {
            return G < 3    ? a_frag(derive_finite, a_main + 2 * G * kTileStride + 96 * i, a_main + 2 * G * kTileStride + 96 * i + 4, 0xffffffffu)
                   : G == 3 ? a_frag(derive_finite, a0_g3 + 96 * i, a1_g3 + 96 * i, 0xffffffffu)
                            : a_frag(derive_finite, a0_g4 + s0_g4 * i, a1_g4 + s1_g4 * i, keep_g4);
        };
        // 35 steps of twelve matrix instructions (depth group G = step / 7, pixel tile i = step % 7); a step's reads are
        // the next step's tile fragment (six reads) and, in the middle of a group, the next group's filter fragments
        // (six more), dealt out between its matrix instructions
        auto multiply = [&](auto derive_finite) {
            SplitFrag8 a[2], b[2][TN];
#pragma unroll
            for (int j = 0; j < TN; ++j) b[0][j] = b_frag(derive_finite, 0, j);
            a[0] = tile_frag(derive_finite, 0, 0);
#pragma unroll
            for (int step = 0; step < 5 * TM; ++step) {
                const int G = step / TM, i = step - G * TM;
                const bool more_tiles = step + 1 < 5 * TM, more_filters = i == 3 && G + 1 < 5;
                if (more_tiles) a[(step + 1) & 1] = tile_frag(derive_finite, (step + 1) / TM, (step + 1) % TM);
                if (more_filters) {
#pragma unroll
                    for (int j = 0; j < TN; ++j) b[(G + 1) & 1][j] = b_frag(derive_finite, G + 1, j);
                }
                mfma6_16x16x32(acc[i][0], acc[i][1], a[step & 1], b[G & 1][0], b[G & 1][1]);
                if constexpr (!decltype(derive_finite)::value) {
#pragma unroll
                    for (int k = 0; k < 6; ++k) {
                        if (more_tiles) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);    // one LDS read
                        if (more_filters) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // and one of the filters'
                        __builtin_amdgcn_sched_group_barrier(0x8, 2, 0);                      // two matrix instructions
                    }
                }
            }
        };
        if (__builtin_amdgcn_readfirstlane(special_flag) != 0 || __builtin_amdgcn_readfirstlane(special_filters) == n0 + 1)
            multiply(std::true_type{});
        else
            multiply(std::false_type{});
        int tid_band = tid;
        asm volatile("" : "+v"(tid_band));  // the epilogue's addresses are worked out per band, not held (spilled) across the loop
        // the next band's rows come while this band is pooled (their registers are free of the multiplication)
        if (has_next) {
            enter(next);
            fetch_tile();
        }
        __syncthreads();  // the planes are dead: the staged band takes their place
        if (tid == 0) special_flag = 0;  // the next band's rows set it again, after the barrier that ends this pass
        stem_epilogue<SIGN>(p, stage, acc, o, tid_band, wm, wn, f_s, f_i, keep, fold && o.band > 0, !p.chained || !has_next);
        if (!has_next) break;
        fold = p.chained != 0;
        item = next;
        __syncthreads();  // the staged band is dead
    }
}

struct CarryArgs {
    float4 *pooled;
    const float4 *carry;
    uint64_t *bits;
    uint32_t total;  // n * (bands - 1) * pw * c4, chained: (blocks of the band kernel - 1) * pw * c4
    int bands, ph, pw, c4, half;
    int chained, per, extra;  // as in FconvPoolArgs: only the first band of a block's range is left to do
    FastDiv div_c4, div_pw, div_bm1, div_bands;
};

// pooled[first row of band b] = max(itself, carry of band b - 1), b >= 1; SIGN: and that row's sign bits again.
template <bool SIGN>
__global__ __launch_bounds__(256) void maxpool_carry_kernel(const CarryArgs p) {
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    if (idx >= p.total) return;
    uint32_t t = p.div_c4.div(idx);
    const int ch = (int)(idx - t * p.c4);
    uint32_t t2 = p.div_pw.div(t);
    const int px = (int)(t - t2 * p.pw);
    uint32_t img;
    int b;
    if (p.chained) {
        const int blk = (int)t2 + 1;  // block 0 starts with an image's first band
        const uint32_t item = (uint32_t)(blk * p.per + (blk < p.extra ? blk : p.extra));
        img = p.div_bands.div(item);
        b = (int)(item - img * p.bands);
        if (b == 0) return;  // the 16 lanes of a pixel's word leave together
    } else {
        img = p.div_bm1.div(t2);
        b = (int)(t2 - img * (p.bands - 1)) + 1;
    }
    const size_t pix = ((size_t)img * p.ph + (size_t)b * p.half) * p.pw + px;
    const float4 m = p.pooled[pix * p.c4 + ch];
    const float4 v = p.carry[(((size_t)img * p.bands + (b - 1)) * p.pw + px) * p.c4 + ch];
    float4 r;
    r.x = v.x > m.x ? v.x : m.x, r.y = v.y > m.y ? v.y : m.y, r.z = v.z > m.z ? v.z : m.z, r.w = v.w > m.w ? v.w : m.w;
    p.pooled[pix * p.c4 + ch] = r;
    if constexpr (SIGN) {
        // c4 % 16 == 0 and total % 16 == 0: a row of lanes is one word's channels, complete or returned as a whole
        const int part = ch & 15;
        const uint32_t nib = sign_nibble(r);
        uint32_t lo = part < 8 ? nib << (4 * part) : 0u, hi = part >= 8 ? nib << (4 * (part - 8)) : 0u;
        lo = or_from_lane_above<1>(lo), hi = or_from_lane_above<1>(hi);
        lo = or_from_lane_above<2>(lo), hi = or_from_lane_above<2>(hi);
        lo = or_from_lane_above<4>(lo), hi = or_from_lane_above<4>(hi);
        lo = or_from_lane_above<8>(lo), hi = or_from_lane_above<8>(hi);
        if (part == 0) p.bits[(pix * p.c4 + ch) >> 4] = ((uint64_t)hi << 32) | lo;
    }
}

// Geometry of the fused pass, or false when the shapes do not fit it.
struct BandPlan {
    int oh, ow, band_rows, bands, ph, pw;
};
static bool plan_bands(int h, int w, int c, int kh, int kw, int pad_h, int pad_w, int stride_h, int stride_w, int dil_h,
                       int dil_w, int cout, BandPlan &b) {
    if (h <= 0 || w <= 0 || c <= 0 || kh <= 0 || kw <= 0 || pad_h < 0 || pad_w < 0 || stride_h <= 0 || stride_w <= 0 ||
        dil_h <= 0 || dil_w <= 0 || cout <= 0)
        return false;
    b.oh = out_dim(h, pad_h, kh, dil_h, stride_h), b.ow = out_dim(w, pad_w, kw, dil_w, stride_w);
    if (b.oh <= 0 || b.ow <= 0 || kBandPixels % b.ow != 0) return false;
    b.band_rows = kBandPixels / b.ow;
    if (b.band_rows % 2 != 0 || b.ow % 2 != 0 || b.oh % b.band_rows != 0) return false;
    b.bands = b.oh / b.band_rows;
    b.ph = b.oh / 2, b.pw = b.ow / 2;  // out_dim(oh, 1, 3, 1, 2) for even oh
    if (b.pw * 16 > kKeepSlots * kBandThreads) return false;  // (ow <= 224 here: never)
    if (cout % 4 != 0 || !(c == 3 || c % 4 == 0)) return false;
    // one image, 64 filters and 64 output pixels' worth of offsets stay below 2^30 bytes
    if (((long long)h + (long long)kh * dil_h + pad_h) * w * c * 4 >= (1ll << 30) || 64ll * kh * kw * c * 4 >= (1ll << 30)) return false;
    return true;
}

// The shapes of the kernel that reads its operands from the raw input rows.
static bool takes_raw_tile(int c, int kh, int kw, int pad_h, int pad_w, int stride_h, int stride_w, int dil_h, int dil_w,
                           const BandPlan &b) {
    return c == 3 && kh == 7 && kw == 7 && stride_h == 2 && stride_w == 2 && pad_h == 3 && pad_w == 3 && dil_h == 1 &&
           dil_w == 1 && b.ow == 112;
}

}  // namespace dab

extern "C" int64_t dab_fconv_maxpool_carry_floats(int n, int h, int w, int c, int kh, int kw, int pad_h, int pad_w,
                                                  int stride_h, int stride_w, int dil_h, int dil_w, int cout) {
    dab::BandPlan b;
    if (n <= 0 || !dab::plan_bands(h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, cout, b)) return 0;
    // the split-operand kernel's pooled form keeps a quarter of the output rows and a sixteenth of its columns instead
    if (dab::fconv_c32_pool_takes(n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, cout, b.oh, b.ow))
        return dab::fconv_c32_pool_workspace_floats(n, b.oh, b.ow, cout);
    return (int64_t)n * b.bands * b.pw * cout;
}

extern "C" int dab_fconv_maxpool_pays(int n, int h, int w, int c, int kh, int kw, int pad_h, int pad_w, int stride_h,
                                      int stride_w, int dil_h, int dil_w, int cout) {
    dab::BandPlan b;
    if (n <= 0 || !dab::plan_bands(h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, cout, b)) return 0;
    // A band is a long work item (17-45 us) and a CU holds one block, so a launch takes whole rounds of bands.  The
    // raw-tile stem kernel beats the two launches from 140 bands on (measured at 84 to 812 bands: 31 against 33 us at
    // 140, 33 against 46 at 224, 87 against 103 at 812; 2 us behind only at 280, just past a round; at 112 bands
    // equal alone and 4 % behind inside Bi-Real-18, whose next layer then starts late).  The im2col band
    // kernel gains a few per cent over full rounds and loses as much as the last round is empty (32 -> 64 channels at
    // 112 x 112, one pass against two launches: 127 / 128 us at 672 bands, 166 / 143 at 784, 166 / 166 at 896,
    // 205 / 187 at 1036): it runs when the last round leaves less than an eighth of all slots idle.
    // 3x3 convolutions over 32 channels that are large enough for the split-operand kernel: its pooled form where the
    // output height allows it; otherwise that kernel and a separate MaxPool beat the one pass over im2col slices
    // (32 -> 64 at 112 x 112, batch 256: 0.76 + 0.21 against 1.35 ms)
    if (dab::fconv_c32_pool_takes(n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, cout, b.oh, b.ow)) return 1;
    if (dab::fconv_c32_takes(n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, cout, b.oh, b.ow)) return 0;
    const long long blocks = (long long)n * b.bands * ((cout + dab::kBandChannels - 1) / dab::kBandChannels);
    const long long cus = dab::simd_count() / 4;
    if (dab::takes_raw_tile(c, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, b)) return 2 * blocks > cus ? 1 : 0;
    const long long rounds = (blocks + cus - 1) / cus;
    return 8 * blocks > 7 * rounds * cus ? 1 : 0;
}

extern "C" int dab_fconv_maxpool(const float *x, int n, int h, int w, int c, const float *wgt, const float *bias,
                                 const float *aff_a, const float *aff_b, int relu, int kh, int kw, int pad_h, int pad_w,
                                 int stride_h, int stride_w, int dil_h, int dil_w, int cout, float *pooled,
                                 uint64_t *pooled_packed, float *carry, dab_stream_t stream) {
    using namespace dab;
    const char *fn = "dab_fconv_maxpool";
    DAB_REQUIRE(x && wgt && pooled && carry, "%s: null pointer", fn);
    DAB_REQUIRE(n > 0 && h > 0 && w > 0 && c > 0 && kh > 0 && kw > 0 && cout > 0, "%s: non-positive dimension", fn);
    DAB_REQUIRE(pad_h >= 0 && pad_w >= 0 && stride_h > 0 && stride_w > 0 && dil_h > 0 && dil_w > 0,
                "%s: bad pad/stride/dilation", fn);
    DAB_REQUIRE((aff_a == nullptr) == (aff_b == nullptr), "%s: affine needs both coefficient vectors", fn);
    BandPlan b;
    if (!plan_bands(h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, cout, b))
        return fail(DAB_EUNSUPPORTED,
                    "%s: needs an output width that divides 448 into an even number of rows, an output height that is a "
                    "multiple of it, 3 or a multiple of 4 input channels and cout %% 4 == 0 (got %dx%dx%d -> %dx%dx%d)",
                    fn, h, w, c, out_dim(h, pad_h, kh, dil_h, stride_h), out_dim(w, pad_w, kw, dil_w, stride_w), cout);
    if (pooled_packed && cout % 64 != 0) return fail(DAB_EUNSUPPORTED, "%s: sign bits need cout %% 64 == 0", fn);
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(wgt) | reinterpret_cast<uintptr_t>(pooled) |
         reinterpret_cast<uintptr_t>(carry)) % 16 != 0)
        return fail(DAB_EUNSUPPORTED, "%s: needs 16-byte aligned buffers", fn);
    if (fconv_c32_pool_takes(n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, cout, b.oh, b.ow)) {
        // alignment of the optional vectors decides at the call: unaligned ones take the band kernel below
        const int rc = fconv_c32_pool_run(x, n, h, w, wgt, bias, aff_a, aff_b, relu, pad_h, pad_w, cout, b.oh, b.ow, pooled,
                                          pooled_packed, carry, as_stream(stream));
        if (rc != 0) return rc < 0 ? rc : DAB_OK;
    }
    const long long pooled_elems = (long long)n * b.ph * b.pw * cout;
    if ((long long)n * b.oh >= (1ll << 31) || pooled_elems >= (1ll << 33))
        return fail(DAB_EUNSUPPORTED, "%s: tensor too large for 32-bit indexing", fn);
    FconvPoolArgs a;
    a.x = x, a.w = wgt, a.bias = bias, a.aff_a = aff_a, a.aff_b = aff_b, a.relu = relu;
    a.pooled = pooled, a.carry = carry, a.bits = pooled_packed;
    a.n = n, a.h = h, a.wd = w, a.c = c;
    a.kw = kw, a.dil_h = dil_h, a.dil_w = dil_w;
    a.pad_h = pad_h, a.pad_w = pad_w, a.stride_h = stride_h, a.stride_w = stride_w;
    a.oh = b.oh, a.ow = b.ow, a.cout = cout, a.K = kh * kw * c;
    a.band_rows = b.band_rows, a.bands = b.bands, a.ph = b.ph, a.pw = b.pw;
    a.div_ow = FastDiv((uint32_t)b.ow), a.div_c = FastDiv((uint32_t)c), a.div_kw = FastDiv((uint32_t)kw);
    a.ytiles = (cout + kBandChannels - 1) / kBandChannels;
    a.div_bands = FastDiv((uint32_t)b.bands), a.div_ytiles = FastDiv((uint32_t)a.ytiles);
    hipStream_t s = as_stream(stream);
    // one block per CU (its LDS holds one), each walking through the work items gridDim.x apart
    const long long items = (long long)n * b.bands * a.ytiles;
    if (items >= (1ll << 31)) return fail(DAB_EUNSUPPORTED, "%s: tensor too large for 32-bit indexing", fn);
    const int cus = simd_count() / 4;
    const dim3 grid((unsigned)(items < cus ? items : cus));
    a.chained = a.ytiles == 1 && b.bands > 1;
    a.per = (int)(items / grid.x), a.extra = (int)(items % grid.x);
    if (takes_raw_tile(c, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, b)) {
        if (pooled_packed)
            hipLaunchKernelGGL(fconv7x7s2_maxpool_kernel<true>, grid, dim3(kBandThreads), 0, s, a);
        else
            hipLaunchKernelGGL(fconv7x7s2_maxpool_kernel<false>, grid, dim3(kBandThreads), 0, s, a);
    } else if (c == 3) {
        if (pooled_packed)
            hipLaunchKernelGGL((fconv_maxpool_kernel<3, true>), grid, dim3(kBandThreads), 0, s, a);
        else
            hipLaunchKernelGGL((fconv_maxpool_kernel<3, false>), grid, dim3(kBandThreads), 0, s, a);
    } else {
        if (pooled_packed)
            hipLaunchKernelGGL((fconv_maxpool_kernel<4, true>), grid, dim3(kBandThreads), 0, s, a);
        else
            hipLaunchKernelGGL((fconv_maxpool_kernel<4, false>), grid, dim3(kBandThreads), 0, s, a);
    }
    DAB_LAUNCH_CHECK();
    if (b.bands > 1) {
        CarryArgs ca;
        ca.pooled = reinterpret_cast<float4 *>(pooled), ca.carry = reinterpret_cast<const float4 *>(carry);
        ca.bits = pooled_packed;
        ca.bands = b.bands, ca.ph = b.ph, ca.pw = b.pw, ca.c4 = cout / 4, ca.half = b.band_rows / 2;
        ca.chained = a.chained, ca.per = a.per, ca.extra = a.extra;
        const long long total = (a.chained ? (long long)grid.x - 1 : (long long)n * (b.bands - 1)) * b.pw * ca.c4;
        if (total >= (1ll << 31)) return fail(DAB_EUNSUPPORTED, "%s: tensor too large for 32-bit indexing", fn);
        ca.total = (uint32_t)total;
        ca.div_c4 = FastDiv((uint32_t)ca.c4), ca.div_pw = FastDiv((uint32_t)b.pw), ca.div_bm1 = FastDiv((uint32_t)(b.bands - 1));
        ca.div_bands = FastDiv((uint32_t)b.bands);
        const unsigned blocks = (unsigned)((total + 255) / 256);
        bool any = !a.chained && total > 0;
        for (unsigned blk = 1; a.chained && !any && blk < grid.x; ++blk)
            any = (blk * (long long)a.per + (blk < (unsigned)a.extra ? blk : a.extra)) % b.bands != 0;
        if (!any) {
            // every block's range starts with an image's first band (one block, or whole images per block)
        } else if (pooled_packed)
            hipLaunchKernelGGL(maxpool_carry_kernel<true>, dim3(blocks), dim3(256), 0, s, ca);
        else
            hipLaunchKernelGGL(maxpool_carry_kernel<false>, dim3(blocks), dim3(256), 0, s, ca);
        DAB_LAUNCH_CHECK();
    }
    return DAB_OK;
}
