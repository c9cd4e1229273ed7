// fp32 layers that sit between the binary convolutions of a Bi-Real-style net:
// fconv, per-channel affine, add, average and max pooling.  All NHWC.
#include <float.h>

#include <type_traits>

#include "common.h"

namespace dab {

// ---------------------------------------------------------------- fconv
// Implicit GEMM: rows = output pixels (N*OH*OW), columns = output channels,
// depth = kh*kw*c in the reference's (kh, kw, c) order (dabnn/fconv.h:33-41,
// dabnn/im2col.h:14-47).  This is the one GEMM-shaped fp32 layer of the path, so
// it runs on the matrix cores: v_mfma_f32_32x32x2_f32, fp32 in and fp32 accumulate.
//
// A 256-thread block owns a BM x BN output tile.  SK-deep slices of the gathered
// image patch and of the weights are staged in two LDS buffers, rows = pixel /
// output channel, depth contiguous; the next slice is fetched into registers
// while the current one is multiplied.  Lanes of a load run along the depth,
// which is contiguous in memory for both operands (channels, then the taps of a
// kernel row), so a wave touches a few cache lines per load.
// The four waves split the tile (KSPLIT = 1) or, for problems too small to give
// every CU a big tile, all work on one 32 x 32 tile and split each slice's depth
// (KSPLIT = 4); their partial sums are then added in a fixed order through LDS.
// Which depth index sits in which of the instruction's two depth slots does not
// matter as long as both operands agree: a lane takes four consecutive depths
// with one 16-byte LDS read and uses them in four instructions.
// Epilogue: + bias, then optionally the Affine (a*v + b, two roundings) and Relu
// layers that follow the convolution, in the reference's order of operations.
// CV = 3 is the loader for three-channel images (the 7x7 stem): a lane fetches
// the three channels of one tap with one 12-byte load, so a slice (8 taps = 24
// depths) takes a third of the load instructions and of the address and bounds
// arithmetic per depth.  CV = 4 does the same with 16-byte loads of four
// consecutive channels when the channel count is a multiple of 4.  POOL (1x1
// convolutions with CV = 4) averages 2x2 windows of the input on the way in --
// an AvePool 2x2 stride 2 followed by the convolution, the shortcut branch of a
// down-sampling block, in one launch; the pooled tensor is written too unless
// p.pooled is null.
struct FconvArgs {
    const float *x;
    const float *w;
    const float *bias;
    const float *aff_a;
    const float *aff_b;
    float *out;
    float *pooled;  // POOL kernels: the 2x2-averaged input, written as a side product
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

// Addressing: all three tensors are reached through buffer descriptors that start at the block's own first image /
// weight row / output row, so 32-bit byte offsets suffice for tensors of any size, reads past the end of the
// descriptor (rows beyond the last pixel or channel) return zero and such writes are dropped.  An element that is
// padding, or whose depth index is past K, gets the offset kOob, which is out of range for every descriptor.
constexpr uint32_t kOob = 0x80000000u;     // descriptors here are shorter than 2^30 bytes
constexpr uint32_t kOobRow = 0x40000000u;  // kOobRow + kOob and kOobRow + (anything < 2^30) stay out of range

template <int BM, int BN, int SK, int KSPLIT, bool PADDED, int CV = 1, bool POOL = false>
__global__ __launch_bounds__(256) void fconv_kernel(const FconvArgs p) {
    constexpr int WAVES_MN = 4 / KSPLIT;
    constexpr int WAVES_N = (WAVES_MN >= 2 && BN >= 64) ? 2 : 1, WAVES_M = WAVES_MN / WAVES_N;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;  // wave tile
    constexpr int TM = WTM / 32, TN = WTN / 32;            // 32 x 32 matrix-core tiles per wave
    constexpr int LK = SK / CV;                            // loader lanes along the depth (taps when CV == 3)
    constexpr int RP = 256 / LK;                           // tile rows fetched per pass of the block
    constexpr int APT = BM / RP, BPT = (BN + RP - 1) / RP;  // loads per thread and slice
    constexpr int RS = SK + 4;                             // LDS row stride: 16-byte reads of 16 lanes hit 64 banks once
    constexpr int WK = SK / KSPLIT;                        // depths of a slice one wave multiplies
    static_assert(TM >= 1 && TN >= 1 && WTM % 32 == 0 && WTN % 32 == 0, "wave tile");
    static_assert(WK % 8 == 0 && 256 % LK == 0 && APT >= 1 && BPT >= 1, "slice");
    static_assert(CV == 1 || CV == 4 || (CV == 3 && KSPLIT == 1), "channel-vector loader");
    static_assert(KSPLIT == 1 || (KSPLIT == 4 && BM == 32 && BN == 32), "a split depth: the four waves share one 32 x 32 tile");
    static_assert(!POOL || (CV == 4 && !PADDED), "the pooling loader takes whole 2x2 windows of four channels");
    constexpr int NW = POOL ? 4 : 1;  // loads per tile element: the window of the pooled input
    constexpr bool B_PARTIAL = BN < RP;  // fewer weight rows than loader rows: the upper loader rows fetch nothing
    __shared__ __attribute__((aligned(16))) float As[2][BM][RS];
    __shared__ __attribute__((aligned(16))) float Bs[2][BN][RS];
    __shared__ float red[KSPLIT > 1 ? KSPLIT * 16 * 64 : 1];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ks = wave / WAVES_MN, wm = (wave % WAVES_MN) / WAVES_N, wn = wave % WAVES_N;
    const int m0 = blockIdx.x * BM, n0 = blockIdx.y * BN;

    // descriptors relative to this block's first image, first weight row and first output row
    const int img0 = (int)p.div_oh.div(p.div_ow.div((uint32_t)m0));
    const int img_elems = p.h * p.wd * p.c;
    const long long x_left = (long long)(p.n - img0) * img_elems * 4;
    const auto x_rsrc = make_rsrc(p.x + (size_t)img0 * img_elems, (uint32_t)(x_left < kOobRow ? x_left : kOobRow));
    const int rows_n = p.cout - n0 < BN ? p.cout - n0 : BN, rows_m = p.M - m0 < BM ? p.M - m0 : BM;
    const auto w_rsrc = make_rsrc(p.w + (size_t)n0 * p.K, (uint32_t)rows_n * p.K * 4u);
    const auto o_rsrc = make_rsrc(p.out + (size_t)m0 * p.cout, (uint32_t)rows_m * p.cout * 4u);

    // loader: depth l_k of the slice, tile rows l_r + RP*i
    const int l_k = tid % LK, l_r = tid / LK;
    uint32_t a_base[APT];  // byte offset of (image, y0, x0, channel 0) from the descriptor's start, modulo 2^32
    int a_y0[PADDED ? APT : 1], a_x0[PADDED ? APT : 1];
    {
        // the thread's first pixel by division, the others by stepping RP pixels on (one row wrap at most when the
        // output is at least RP wide; by division again otherwise)
        const int pix0 = m0 + l_r;
        const uint32_t t0 = p.div_ow.div((uint32_t)pix0);
        int ox = pix0 - (int)t0 * p.ow;
        int img = (int)p.div_oh.div(t0);
        int oy = (int)t0 - img * p.oh;
        const bool step_ok = p.ow >= RP;
#pragma unroll
        for (int i = 0; i < APT; ++i) {
            const int pix = pix0 + RP * i;
            if (i > 0) {
                if (step_ok) {
                    ox += RP;
                    const bool wrap = ox >= p.ow;
                    ox = wrap ? ox - p.ow : ox;
                    oy += wrap ? 1 : 0;
                    const bool wrap2 = oy >= p.oh;
                    oy = wrap2 ? 0 : oy;
                    img += wrap2 ? 1 : 0;
                } else {
                    const uint32_t t = p.div_ow.div((uint32_t)pix);
                    ox = pix - (int)t * p.ow;
                    img = (int)p.div_oh.div(t);
                    oy = (int)t - img * p.oh;
                }
            }
            if (pix < p.M) {
                const int y0 = oy * p.stride_h - p.pad_h, x0 = ox * p.stride_w - p.pad_w;
                a_base[i] = (uint32_t)((((img - img0) * p.h + y0) * p.wd + x0) * p.c) * 4u;
                if (PADDED) a_y0[i] = y0, a_x0[i] = x0;
            } else {
                a_base[i] = kOobRow;
                if (PADDED) a_y0[i] = -(1 << 30), a_x0[i] = 0;  // every tap fails the bounds test
            }
        }
    }
    uint32_t b_row[BPT];
#pragma unroll
    for (int j = 0; j < BPT; ++j) b_row[j] = (uint32_t)(l_r + RP * j) * p.K * 4u;

    typedef float f32xcv __attribute__((ext_vector_type(CV)));
    f32xcv a_reg[APT][NW], b_reg[BPT];
    auto load_cv = [](__amdgpu_buffer_rsrc_t rsrc, uint32_t off) -> f32xcv {
        // the result is bit-cast as a whole: casting single elements of a vector buffer load makes the compiler
        // replace it by one 4-byte load
        if constexpr (CV == 1)
            return __builtin_bit_cast(f32xcv, __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)off, 0, 0));
        else if constexpr (CV == 3)
            return __builtin_bit_cast(f32xcv, __builtin_amdgcn_raw_buffer_load_b96(rsrc, (int)off, 0, 0));
        else
            return __builtin_bit_cast(f32xcv, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)off, 0, 0));
    };
    auto fetch = [&](int k0) {
        // CV == 1: lane = depth index k -> (tap, channel).  CV == 4: four consecutive channels of a tap (c % 4 == 0).
        // CV == 3: lane = tap, channels 0..2 (c == 3, k0 % 24 == 0).
        const int k = k0 + CV * l_k;
        const bool k_ok = k < p.K;
        int tap, ch;
        if constexpr (CV != 3) {
            tap = (int)p.div_c.div((uint32_t)k), ch = k - tap * p.c;
        } else {
            tap = (int)((uint32_t)k0 / 3u) + l_k, ch = 0;
        }
        const int ty = (int)p.div_kw.div((uint32_t)tap), tx = tap - ty * p.kw;
        const int dy = ty * p.dil_h, dx = tx * p.dil_w;
        const uint32_t delta = k_ok ? (uint32_t)((dy * p.wd + dx) * p.c + ch) * 4u : kOob;
#pragma unroll
        for (int i = 0; i < APT; ++i) {
            uint32_t off = a_base[i] + delta;
            if (PADDED) {
                const int y = a_y0[i] + dy, xx = a_x0[i] + dx;
                off = ((unsigned)y < (unsigned)p.h && (unsigned)xx < (unsigned)p.wd) ? off : kOob;
            }
            a_reg[i][0] = load_cv(x_rsrc, off);
            if constexpr (POOL) {
                // the window's other three pixels: right, below, below right (out-of-range elements carry kOob and
                // stay out of range with these small additions)
                const uint32_t right = (uint32_t)p.c * 4u, below = (uint32_t)p.wd * right;
                a_reg[i][1] = load_cv(x_rsrc, off + right);
                a_reg[i][2] = load_cv(x_rsrc, off + below);
                a_reg[i][3] = load_cv(x_rsrc, off + below + right);
            }
        }
        const uint32_t k4 = k_ok ? (uint32_t)k * 4u : kOob;
#pragma unroll
        for (int j = 0; j < BPT; ++j) b_reg[j] = load_cv(w_rsrc, (!B_PARTIAL || l_r < BN) ? b_row[j] + k4 : kOob);
    };
    auto commit = [&](int buf, int k0) {
#pragma unroll
        for (int i = 0; i < APT; ++i) {
            f32xcv v = a_reg[i][0];
            if constexpr (POOL) {
                // ave_pool_fallback (dabnn/layers/AvePool.cpp:84-123) for a 2x2 window without padding: the taps are
                // added to zero in row-major order and divided by 4 (a multiplication by 0.25 rounds the same way)
#pragma clang fp contract(off)
                f32xcv sum = {0.f, 0.f, 0.f, 0.f};
                sum = sum + a_reg[i][0];
                sum = sum + a_reg[i][1];
                sum = sum + a_reg[i][2];
                sum = sum + a_reg[i][3];
                v = sum * 0.25f;
                const int pix = m0 + l_r + RP * i, k = k0 + CV * l_k;
                if (p.pooled != nullptr && blockIdx.y == 0 && pix < p.M && k < p.K)
                    *reinterpret_cast<f32xcv *>(p.pooled + (size_t)pix * p.K + k) = v;
            }
#pragma unroll
            for (int c = 0; c < CV; ++c) As[buf][l_r + RP * i][l_k * CV + c] = v[c];
        }
        if (!B_PARTIAL || l_r < BN) {
#pragma unroll
            for (int j = 0; j < BPT; ++j)
#pragma unroll
                for (int c = 0; c < CV; ++c) Bs[buf][l_r + RP * j][l_k * CV + c] = b_reg[j][c];
        }
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    // operand lane l of the instruction: row / column l % 32, depth slot l / 32
    const int f_k = lane >> 5, f_i = lane & 31;
    fetch(0);
    commit(0, 0);
    __syncthreads();
    int buf = 0;
    for (int k0 = 0; k0 < p.K; k0 += SK, buf ^= 1) {
        const bool more = k0 + SK < p.K;
        if (more) fetch(k0 + SK);
#pragma unroll
        for (int g = 0; g < WK / 8; ++g) {  // this wave's depths of the slice, 8 at a time
            // the last slice may end early: groups that lie wholly past the depth hold zeros on both sides
            if (KSPLIT == 1 && g > 0 && k0 + g * 8 >= p.K) break;
            const int kb = ks * WK + g * 8 + f_k * 4;
            float4 a4[TM], b4[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) a4[i] = *reinterpret_cast<const float4 *>(&As[buf][wm * WTM + i * 32 + f_i][kb]);
#pragma unroll
            for (int j = 0; j < TN; ++j) b4[j] = *reinterpret_cast<const float4 *>(&Bs[buf][wn * WTN + j * 32 + f_i][kb]);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a4[i].x, b4[j].x, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a4[i].y, b4[j].y, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a4[i].z, b4[j].z, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a4[i].w, b4[j].w, acc[i][j], 0, 0, 0);
                }
        }
        // the other buffer was last read before the barrier that ended the previous slice
        if (more) commit(buf ^ 1, k0 + SK);
        __syncthreads();
    }

    // Epilogue.  The three optional steps are decided once per launch, so the per-element code is straight-line:
    // (+ bias) (a*v + b, two roundings) (relu) and one store.  An element's byte offset is the lane's own part (its
    // column, its share of the row index) plus a wave-uniform multiple of the row pitch; rows past the last pixel are
    // past the end of the output descriptor and a column past the last channel carries kOob.
    const uint32_t row_bytes = (uint32_t)p.cout * 4u;
    auto emit = [&](auto has_bias, auto has_affine, auto has_relu, uint32_t off, float v, float bias, float fa, float fb) {
#pragma clang fp contract(off)
        if constexpr (decltype(has_bias)::value) v = v + bias;
        if constexpr (decltype(has_affine)::value) {
            const float prod = fa * v;
            v = prod + fb;
        }
        if constexpr (decltype(has_relu)::value) v = v < 0.f ? 0.f : v;  // std::max(v, 0.f): a NaN stays
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), o_rsrc, (int)off, 0, 0);
    };
    // accumulator element e of lane l: row 8*(e/4) + 4*(l/32) + e%4, column l % 32
    auto emit_all = [&](auto has_bias, auto has_affine, auto has_relu) {
        if constexpr (KSPLIT == 1) {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int co = n0 + wn * WTN + j * 32 + f_i;
                const bool co_ok = co < p.cout;
                const float bias = (decltype(has_bias)::value && co_ok) ? p.bias[co] : 0.f;
                const float fa = (decltype(has_affine)::value && co_ok) ? p.aff_a[co] : 0.f;
                const float fb = (decltype(has_affine)::value && co_ok) ? p.aff_b[co] : 0.f;
                const uint32_t lane_off = (co_ok ? (uint32_t)co * 4u : kOob) + (uint32_t)(wm * WTM + 4 * f_k) * row_bytes;
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int e = 0; e < 16; ++e)
                        emit(has_bias, has_affine, has_relu, lane_off + (uint32_t)(i * 32 + 8 * (e / 4) + (e % 4)) * row_bytes,
                             acc[i][j][e], bias, fa, fb);
            }
        } else {
            // one 32 x 32 tile: the waves' partial sums are added in wave order, four accumulator elements per thread
            const int co = n0 + f_i;
            const bool co_ok = co < p.cout;
            const float bias = (decltype(has_bias)::value && co_ok) ? p.bias[co] : 0.f;
            const float fa = (decltype(has_affine)::value && co_ok) ? p.aff_a[co] : 0.f;
            const float fb = (decltype(has_affine)::value && co_ok) ? p.aff_b[co] : 0.f;
            const uint32_t lane_off = (co_ok ? (uint32_t)co * 4u : kOob) + (uint32_t)(4 * f_k) * row_bytes;
#pragma unroll
            for (int q = 0; q < 16 / KSPLIT; ++q) {
                const int e = wave * (16 / KSPLIT) + q;
                float v = red[e * 64 + lane];
#pragma unroll
                for (int s = 1; s < KSPLIT; ++s) v = __fadd_rn(v, red[(s * 16 + e) * 64 + lane]);
                emit(has_bias, has_affine, has_relu, lane_off + (uint32_t)(8 * (e / 4) + (e % 4)) * row_bytes, v, bias, fa, fb);
            }
        }
    };
    if constexpr (KSPLIT > 1) {
#pragma unroll
        for (int e = 0; e < 16; ++e) red[(ks * 16 + e) * 64 + lane] = acc[0][0][e];
        __syncthreads();
    }
    using T = std::true_type;
    using F = std::false_type;
    switch ((p.bias ? 4 : 0) | (p.aff_a ? 2 : 0) | (p.relu ? 1 : 0)) {
        case 0: emit_all(F{}, F{}, F{}); break;
        case 1: emit_all(F{}, F{}, T{}); break;
        case 2: emit_all(F{}, T{}, F{}); break;
        case 3: emit_all(F{}, T{}, T{}); break;
        case 4: emit_all(T{}, F{}, F{}); break;
        case 5: emit_all(T{}, F{}, T{}); break;
        case 6: emit_all(T{}, T{}, F{}); break;
        default: emit_all(T{}, T{}, T{}); break;
    }
}

// AvePool 2x2 stride 2 + 1x1 convolution over K input channels (a multiple of 64; built for 64) when the launch is
// bound by the input it reads.  fconv_kernel<..., POOL> pools a tile's pixels once per column tile and fetches a
// pixel's channels slice by slice.  Here a block pools its BM pixels once, whole pixels at a time (4K contiguous bytes
// per window pixel), into an LDS tile that holds all K depths, and walks the column tiles of 128 output channels over
// it while the filters stream through a double buffer in slices of 32 depths.  Every sum takes its depths in the
// order fconv_kernel takes them (eight at a time, the pairs d and d + 4 in one matrix instruction), so the results
// are the same bit for bit.  p.pooled may be null: then the pooled tensor is not written.
template <int K, int BM>
__global__ __launch_bounds__(256) void pool2_fconv1x1_kernel(const FconvArgs p) {
    constexpr int BN = 128, SK = 32, RS = SK + 4, AS = K + 4;  // row strides of 4 mod 64 floats: no bank conflicts
    constexpr int THREADS = 256, WAVES_M = BM / 32, WAVES_N = 4 / WAVES_M, WTN = BN / WAVES_N, TN = WTN / 32;
    constexpr int KV = K / 4;           // 16-byte pieces of a pixel
    constexpr int A4 = BM * KV / THREADS;   // pieces of the pooled tile per thread
    constexpr int AB = A4 < 4 ? A4 : 4;  // of which this many are in flight at a time (four loads each)
    constexpr int SLICES = K / SK;
    static_assert(BM == 32 || BM == 64, "one or two rows of waves");
    constexpr int BJ = BN * 8 / THREADS;  // 16-byte pieces of a filter slice per thread
    static_assert(K % SK == 0 && (BM * KV) % THREADS == 0 && A4 % AB == 0 && TN >= 1, "tile");
    __shared__ __attribute__((aligned(16))) float As[BM][AS];
    __shared__ __attribute__((aligned(16))) float Bs[2][BN][RS];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int m0 = blockIdx.x * BM;
    const int img0 = (int)p.div_oh.div(p.div_ow.div((uint32_t)m0));
    const int img_elems = p.h * p.wd * K;
    const long long x_left = (long long)(p.n - img0) * img_elems * 4;
    const auto x_rsrc = make_rsrc(p.x + (size_t)img0 * img_elems, (uint32_t)(x_left < kOobRow ? x_left : kOobRow));
    const auto w_rsrc = make_rsrc(p.w, (uint32_t)p.cout * K * 4u);
    const int rows_m = p.M - m0 < BM ? p.M - m0 : BM;
    const auto o_rsrc = make_rsrc(p.out + (size_t)m0 * p.cout, (uint32_t)rows_m * p.cout * 4u);
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    auto load4 = [](__amdgpu_buffer_rsrc_t rsrc, uint32_t off) -> f32x4 {
        return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)off, 0, 0));
    };

    // filters: slice `it` = column tile it / SLICES, depths 32 * (it % SLICES) ...; thread = 16 bytes of four rows
    const int b_k = tid & 7, b_r = tid >> 3;
    constexpr int BR = THREADS / 8;  // filter rows per pass of the block
    const int tiles_n = (p.cout + BN - 1) / BN, total = tiles_n * SLICES;
    // two slices ahead, through registers: a slice is asked for two iterations before it is multiplied (the first
    // touch of a slice by any block comes from memory) and goes to the LDS buffer that the iteration before it freed
    f32x4 b_reg[2][BJ];
    auto fetch_b = [&](int it, int slot) {
        const int nt = it / SLICES, ks = it - nt * SLICES;
#pragma unroll
        for (int j = 0; j < BJ; ++j) {
            const int row = nt * BN + b_r + BR * j;
            b_reg[slot][j] = load4(w_rsrc, row < p.cout ? (uint32_t)((row * K + ks * SK + 4 * b_k) * 4) : kOob);
        }
    };
    auto commit_b = [&](int slot) {
#pragma unroll
        for (int j = 0; j < BJ; ++j) *reinterpret_cast<f32x4 *>(&Bs[slot][b_r + BR * j][4 * b_k]) = b_reg[slot][j];
    };
    fetch_b(0, 0);
    if (total > 1) fetch_b(1, 1);

    // the pooled tile: ave_pool_fallback (dabnn/layers/AvePool.cpp:84-123) for a 2x2 window without padding, the taps
    // added to zero in row-major order and divided by 4 (a multiplication by 0.25 rounds the same way)
    {
        const uint32_t right = (uint32_t)K * 4u, below = (uint32_t)p.wd * right;
#pragma unroll
        for (int i0 = 0; i0 < A4; i0 += AB) {
            f32x4 win[AB][4];
#pragma unroll
            for (int i = 0; i < AB; ++i) {
                const int piece = tid + THREADS * (i0 + i), r = piece / KV, c4 = piece % KV;
                const int pix = m0 + r;
                const uint32_t t0 = p.div_ow.div((uint32_t)pix);
                const int ox = pix - (int)t0 * p.ow, img = (int)p.div_oh.div(t0), oy = (int)t0 - img * p.oh;
                const uint32_t off =
                    pix < p.M ? (uint32_t)((((img - img0) * p.h + 2 * oy) * p.wd + 2 * ox) * K + 4 * c4) * 4u : kOobRow;
                win[i][0] = load4(x_rsrc, off);
                win[i][1] = load4(x_rsrc, off + right);
                win[i][2] = load4(x_rsrc, off + below);
                win[i][3] = load4(x_rsrc, off + below + right);
            }
#pragma unroll
            for (int i = 0; i < AB; ++i) {
#pragma clang fp contract(off)
                const int piece = tid + THREADS * (i0 + i), r = piece / KV, c4 = piece % KV;
                f32x4 sum = {0.f, 0.f, 0.f, 0.f};
                sum = sum + win[i][0];
                sum = sum + win[i][1];
                sum = sum + win[i][2];
                sum = sum + win[i][3];
                const f32x4 v = sum * 0.25f;
                *reinterpret_cast<f32x4 *>(&As[r][4 * c4]) = v;
                if (p.pooled != nullptr && m0 + r < p.M)
                    __builtin_nontemporal_store(v, reinterpret_cast<f32x4 *>(p.pooled + (size_t)(m0 + r) * K + 4 * c4));
            }
        }
    }
    commit_b(0);
    __syncthreads();

    const uint32_t row_bytes = (uint32_t)p.cout * 4u;
    const int f_k = lane >> 5, f_i = lane & 31;
    // accumulator element e of lane l: row 8*(e/4) + 4*(l/32) + e%4, column l % 32
    auto emit_tile = [&](auto has_bias, auto has_affine, auto has_relu, int n0, const f32x16 (&acc)[TN]) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int co = n0 + wn * WTN + j * 32 + f_i;
            const bool co_ok = co < p.cout;
            const float bias = (decltype(has_bias)::value && co_ok) ? p.bias[co] : 0.f;
            const float fa = (decltype(has_affine)::value && co_ok) ? p.aff_a[co] : 0.f;
            const float fb = (decltype(has_affine)::value && co_ok) ? p.aff_b[co] : 0.f;
            const uint32_t lane_off = (co_ok ? (uint32_t)co * 4u : kOob) + (uint32_t)(wm * 32 + 4 * f_k) * row_bytes;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
#pragma clang fp contract(off)
                float v = acc[j][e];
                if constexpr (decltype(has_bias)::value) v = v + bias;
                if constexpr (decltype(has_affine)::value) {
                    const float prod = fa * v;
                    v = prod + fb;
                }
                if constexpr (decltype(has_relu)::value) v = v < 0.f ? 0.f : v;  // std::max(v, 0.f): a NaN stays
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), o_rsrc,
                                                      (int)(lane_off + (uint32_t)(8 * (e / 4) + (e % 4)) * row_bytes), 0, 0);
            }
        }
    };
    using T = std::true_type;
    using F = std::false_type;
    const int epilogue = (p.bias ? 4 : 0) | (p.aff_a ? 2 : 0) | (p.relu ? 1 : 0);

    static_assert(SLICES % 2 == 0, "a slice's buffer is its number modulo 2 in every column tile");
    f32x16 acc[TN];
    for (int nt = 0; nt < tiles_n; ++nt) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;
#pragma unroll
        for (int ks = 0; ks < SLICES; ++ks) {
            const int it = nt * SLICES + ks;
            if (it + 2 < total) fetch_b(it + 2, ks & 1);
#pragma unroll
            for (int g = 0; g < SK / 8; ++g) {
                const int kb = g * 8 + f_k * 4;
                const float4 a4 = *reinterpret_cast<const float4 *>(&As[wm * 32 + f_i][ks * SK + kb]);
                float4 b4[TN];
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    b4[j] = *reinterpret_cast<const float4 *>(&Bs[ks & 1][wn * WTN + j * 32 + f_i][kb]);
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a4.x, b4[j].x, acc[j], 0, 0, 0);
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a4.y, b4[j].y, acc[j], 0, 0, 0);
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a4.z, b4[j].z, acc[j], 0, 0, 0);
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a4.w, b4[j].w, acc[j], 0, 0, 0);
                }
            }
            if (ks == SLICES - 1) {
                switch (epilogue) {
                    case 0: emit_tile(F{}, F{}, F{}, nt * BN, acc); break;
                    case 1: emit_tile(F{}, F{}, T{}, nt * BN, acc); break;
                    case 2: emit_tile(F{}, T{}, F{}, nt * BN, acc); break;
                    case 3: emit_tile(F{}, T{}, T{}, nt * BN, acc); break;
                    case 4: emit_tile(T{}, F{}, F{}, nt * BN, acc); break;
                    case 5: emit_tile(T{}, F{}, T{}, nt * BN, acc); break;
                    case 6: emit_tile(T{}, T{}, F{}, nt * BN, acc); break;
                    default: emit_tile(T{}, T{}, T{}, nt * BN, acc); break;
                }
            }
            // the other buffer was last read before the barrier that ended the previous slice
            if (it + 1 < total) commit_b((ks + 1) & 1);
            __syncthreads();
        }
    }
}

// The classifier at small batch: a 1x1 convolution over a handful of pixels is a matrix-vector product, and the
// 32 x 32 tiles above would leave all but 32 blocks idle.  One wave per output channel: lanes stride over the depth
// with 16-byte loads (c % 4 == 0), the partial sums are added across the wave, lane 0 applies the epilogue.
__global__ __launch_bounds__(256) void fconv_gemv_kernel(const FconvArgs p) {
    constexpr int MR = 4;  // pixels that share one pass over a weight row
    const int lane = threadIdx.x & 63;
    const int co = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (co >= p.cout) return;
    const float4 *w4 = reinterpret_cast<const float4 *>(p.w + (size_t)co * p.K);
    const int k4n = p.K >> 2;
    for (int m0 = 0; m0 < p.M; m0 += MR) {
        float acc[MR] = {0.f, 0.f, 0.f, 0.f};
        for (int k4 = lane; k4 < k4n; k4 += 64) {
            const float4 wv = w4[k4];
#pragma unroll
            for (int r = 0; r < MR; ++r) {
                const int m = m0 + r < p.M ? m0 + r : p.M - 1;  // a valid row; its sum is not stored
                const float4 xv = reinterpret_cast<const float4 *>(p.x + (size_t)m * p.K)[k4];
                acc[r] += wv.x * xv.x + wv.y * xv.y + wv.z * xv.z + wv.w * xv.w;
            }
        }
#pragma unroll
        for (int r = 0; r < MR; ++r) {
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) acc[r] += __shfl_xor(acc[r], d, 64);
        }
        if (lane == 0) {
#pragma clang fp contract(off)
#pragma unroll
            for (int r = 0; r < MR; ++r) {
                if (m0 + r >= p.M) break;
                float v = acc[r];
                if (p.bias) v = v + p.bias[co];
                if (p.aff_a) {
                    const float prod = p.aff_a[co] * v;
                    v = prod + p.aff_b[co];
                }
                if (p.relu) v = v < 0.f ? 0.f : v;
                p.out[(size_t)(m0 + r) * p.cout + co] = v;
            }
        }
    }
}

// The same at the end of a net: a global AvePool (one window over the whole h x w image) and the classifier's 1x1
// convolution in one launch, for the few images of a small batch.  Block (b, img) first averages image img into LDS --
// thread t sums channels 4t .. 4t + 3 over the taps in ave_pool's order with ave_pool's rounding, so the pooled blob it
// writes (block 0 of the image) is the one dab_ave_pool writes -- and then its four waves make kGlobalPoolChannels output
// channels each, with fconv_gemv_kernel's arithmetic (lanes stride over the depth, sums added across the wave).  The
// weights are asked for before the image: the two round trips to memory overlap.
constexpr int kGlobalPoolChannels = 4;  // output channels per wave
constexpr int kGlobalPoolTaps = 64;     // h * w at most
constexpr int kGlobalPoolDepth4 = 256;  // c / 4 at most
// D4: float4 of the depth per lane (c <= 256 * D4); U: taps asked for at once (49: a 7x7 window in one round trip)
template <int D4, int U>
__global__ __launch_bounds__(256) void global_avepool_gemv_kernel(const FconvArgs p) {
    constexpr int CH = kGlobalPoolChannels;
    __shared__ float4 pooled4[kGlobalPoolDepth4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, img = blockIdx.y;
    const int k4n = p.K >> 2, taps = p.h * p.wd;
    const int co0 = (blockIdx.x * 4 + wave) * CH;
    float4 wv[CH][D4];
#pragma unroll
    for (int j = 0; j < CH; ++j) {
        const int co = co0 + j < p.cout ? co0 + j : p.cout - 1;  // a valid row; its sum is not stored
        const float4 *w4 = reinterpret_cast<const float4 *>(p.w + (size_t)co * p.K);
#pragma unroll
        for (int i = 0; i < D4; ++i) wv[j][i] = lane + 64 * i < k4n ? w4[lane + 64 * i] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    if ((int)threadIdx.x < k4n) {
        const float4 *x4 = reinterpret_cast<const float4 *>(p.x) + (size_t)img * taps * k4n + threadIdx.x;
        float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int t0 = 0; t0 < taps; t0 += U) {
            float4 v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) v[u] = x4[(size_t)(t0 + u < taps ? t0 + u : taps - 1) * k4n];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (t0 + u < taps) {
#pragma clang fp contract(off)
                    sum.x = sum.x + v[u].x, sum.y = sum.y + v[u].y, sum.z = sum.z + v[u].z, sum.w = sum.w + v[u].w;
                }
            }
        }
        const float d = (float)taps;
        const float4 r = make_float4(__fdiv_rn(sum.x, d), __fdiv_rn(sum.y, d), __fdiv_rn(sum.z, d), __fdiv_rn(sum.w, d));
        pooled4[threadIdx.x] = r;
        if (blockIdx.x == 0) reinterpret_cast<float4 *>(p.pooled)[(size_t)img * k4n + threadIdx.x] = r;
    }
    __syncthreads();
    float acc[CH];
#pragma unroll
    for (int j = 0; j < CH; ++j) acc[j] = 0.f;
#pragma unroll
    for (int i = 0; i < D4; ++i) {
        if (lane + 64 * i < k4n) {
            const float4 xv = pooled4[lane + 64 * i];
#pragma unroll
            for (int j = 0; j < CH; ++j) acc[j] += wv[j][i].x * xv.x + wv[j][i].y * xv.y + wv[j][i].z * xv.z + wv[j][i].w * xv.w;
        }
    }
#pragma unroll
    for (int j = 0; j < CH; ++j) {
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) acc[j] += __shfl_xor(acc[j], d, 64);
    }
    if (lane == 0) {
#pragma clang fp contract(off)
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            const int co = co0 + j;
            if (co >= p.cout) break;
            float v = acc[j];
            if (p.bias) v = v + p.bias[co];
            if (p.aff_a) {
                const float prod = p.aff_a[co] * v;
                v = prod + p.aff_b[co];
            }
            if (p.relu) v = v < 0.f ? 0.f : v;
            p.out[(size_t)img * p.cout + co] = v;
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
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) x[i] = x[i] < 0.f ? 0.f : x[i];
}

// PRelu.cpp:6-30: negative values are scaled by one slope or by their channel's slope (slope_n = 1 or c).
__global__ __launch_bounds__(256) void prelu_kernel(float *__restrict__ x, long long total, int c,
                                                    const float *__restrict__ slope, int slope_n) {
    const long long stride = (long long)gridDim.x * 256;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
        const float v = x[i];
        if (v < 0.f) x[i] = v * slope[slope_n == 1 ? 0 : (int)(i % c)];
    }
}

// Concat.cpp:7-21: per pixel the ca floats of a, then the cb floats of b.
__global__ __launch_bounds__(256) void concat_kernel(const float *__restrict__ a, int ca, const float *__restrict__ b, int cb,
                                                     float *__restrict__ out, long long total) {
    const long long stride = (long long)gridDim.x * 256;
    const int c = ca + cb;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
        const long long pix = i / c;
        const int ch = (int)(i - pix * c);
        out[i] = ch < ca ? a[pix * ca + ch] : b[pix * cb + (ch - ca)];
    }
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

// SIGN (c % 64 == 0): the 16 threads that hold the 64 channels of a word are one row of lanes; their sign nibbles are
// gathered with DPP and the first of them stores pack_mat's word of the pooled pixel (dabnn/bitpack.h:277-293).
template <bool MAX, bool SIGN, int U>
__global__ __launch_bounds__(256) void pool_vec4_kernel(const float4 *__restrict__ x, float4 *__restrict__ out,
                                                        uint64_t *__restrict__ out_packed, const PoolVecArgs p) {
    const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= p.total) return;
    uint32_t t = p.div_c4.div(idx);
    const int ch = (int)(idx - t * p.c4);
    uint32_t t2 = p.div_ow.div(t);
    const int ox = (int)(t - t2 * p.g.ow);
    const uint32_t img = p.div_oh.div(t2);
    const int oy = (int)(t2 - img * p.g.oh);
    float4 m = make_float4(-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX), sum = make_float4(0.f, 0.f, 0.f, 0.f);
    const int ys = oy * p.g.stride_h - p.g.pad_h, xs = ox * p.g.stride_w - p.g.pad_w;
    // in-bounds part of the window: the taps are walked in the reference's order, U loads at a time, all of them in
    // flight before the first is used (a 7x7 window is five waits for memory, not 49)
    const int a_lo = ys < 0 ? -ys : 0, a_hi = ys + p.g.kh > p.g.h ? p.g.h - ys : p.g.kh;
    const int b_lo = xs < 0 ? -xs : 0, b_hi = xs + p.g.kw > p.g.w ? p.g.w - xs : p.g.kw;
    const int cnt = (a_hi > a_lo && b_hi > b_lo) ? (a_hi - a_lo) * (b_hi - b_lo) : 0;
    const float4 *img0 = x + (size_t)img * p.g.h * p.g.w * p.c4 + ch;
    int a = a_lo, b = b_lo;
    for (int t0 = 0; t0 < cnt; t0 += U) {
        float4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            // past the last tap (a, b) stays on it: a load of a valid address whose value is not used
            v[u] = img0[((size_t)(ys + a) * p.g.w + (xs + b)) * p.c4];
            if (t0 + u + 1 < cnt && ++b == b_hi) b = b_lo, ++a;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (t0 + u < cnt) {
                if (MAX) {
                    m.x = v[u].x > m.x ? v[u].x : m.x, m.y = v[u].y > m.y ? v[u].y : m.y;
                    m.z = v[u].z > m.z ? v[u].z : m.z, m.w = v[u].w > m.w ? v[u].w : m.w;
                } else {
#pragma clang fp contract(off)
                    sum.x = sum.x + v[u].x, sum.y = sum.y + v[u].y, sum.z = sum.z + v[u].z, sum.w = sum.w + v[u].w;
                }
            }
        }
    }
    float4 r;
    if (MAX) {
        r = m;
    } else {
        const float d = (float)cnt;
        r = make_float4(__fdiv_rn(sum.x, d), __fdiv_rn(sum.y, d), __fdiv_rn(sum.z, d), __fdiv_rn(sum.w, d));
    }
    out[idx] = r;
    if constexpr (SIGN) {
        // total is a multiple of 16 here, so a row of lanes is either complete or has returned above as a whole
        const int part = (int)(idx & 15u);
        const uint32_t nib = sign_nibble(r);
        uint32_t lo = part < 8 ? nib << (4 * part) : 0u, hi = part >= 8 ? nib << (4 * (part - 8)) : 0u;
        lo = or_from_lane_above<1>(lo), hi = or_from_lane_above<1>(hi);
        lo = or_from_lane_above<2>(lo), hi = or_from_lane_above<2>(hi);
        lo = or_from_lane_above<4>(lo), hi = or_from_lane_above<4>(hi);
        lo = or_from_lane_above<8>(lo), hi = or_from_lane_above<8>(hi);
        if (part == 0) out_packed[idx >> 4] = ((uint64_t)hi << 32) | lo;
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

// 1x1 convolutions to 128 channels or more with fewer 128 x 128 tiles than CUs (the shortcut branches of a residual
// net below batch 64 or so): the tile that still gives three quarters of the CUs a block -- 1: 64 x 128 with 32-deep
// slices, 2: 64 x 64 with 32-deep slices, 3: 32 x 32 with 64-deep slices split over the four waves -- or 0 for other
// shapes.  Measured inside a graph, AvePool 2x2 in the loader, against the 64 x 64 tiles with 16-deep slices that ran
// before: 28 x 28 x 128 -> 256 at batch 64 / 32 / 16: 18.3 / 11.5 / 8.0 against 20.5 / 15.0 / 9.1 us; 14 x 14 x 256 ->
// 512 at batch 64 / 32: 18.9 / 14.1 against 23.8 / 17.9.
static int small_1x1_tiles(int taps, long long M, int cout) {
    if (taps != 1 || cout < 128) return 0;
    const long long want = 3ll * dab::simd_count() / 16;  // three quarters of the CUs
    if (((M + 63) / 64) * ((cout + 127) / 128) >= want) return 1;
    if (((M + 63) / 64) * ((cout + 63) / 64) >= want) return 2;
    return 3;
}

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
    a.pooled = nullptr;
    a.n = n, a.h = h, a.wd = w, a.c = c;
    a.pad_h = pad_h, a.pad_w = pad_w, a.stride_h = stride_h, a.stride_w = stride_w;
    a.oh = out_dim(h, pad_h, kh, dil_h, stride_h), a.ow = out_dim(w, pad_w, kw, dil_w, stride_w);
    DAB_REQUIRE(a.oh > 0 && a.ow > 0, "%s: empty output", fn);
    a.cout = cout;
    a.K = kh * kw * c;
    const long long M = (long long)n * a.oh * a.ow;
    if (M >= (1ll << 31) - 128 || (long long)n * h * w * c >= (1ll << 31))
        return fail(DAB_EUNSUPPORTED, "%s: tensor too large for 32-bit indexing", fn);
    a.M = (int)M;
    a.div_ow = FastDiv((uint32_t)a.ow), a.div_oh = FastDiv((uint32_t)a.oh);
    a.kw = kw, a.dil_h = dil_h, a.dil_w = dil_w;
    a.div_c = FastDiv((uint32_t)c), a.div_kw = FastDiv((uint32_t)kw);
    hipStream_t s = as_stream(stream);
    // byte offsets inside a block's descriptors stay below 2^30: the images its 128 pixels come from, 128 weight
    // rows, 128 output rows
    const long long span_imgs = 128 / ((long long)a.oh * a.ow) + 2;
    if (span_imgs * h * w * c * 4 >= (1ll << 30) || 128ll * a.K * 4 >= (1ll << 30) || 128ll * cout * 4 >= (1ll << 30))
        return fail(DAB_EUNSUPPORTED, "%s: image, filter or channel count too large for 32-bit tile offsets", fn);
    {
        const int rc = fconv_c32_try(x, n, h, w, c, wgt, bias, aff_a, aff_b, relu, kh, kw, pad_h, pad_w, stride_h, stride_w,
                                     dil_h, dil_w, cout, a.oh, a.ow, out, s);
        if (rc != 0) return rc < 0 ? rc : DAB_OK;
    }
    // without padding every tap of every window is inside the image and the bounds test is dropped
    const bool padded = pad_h != 0 || pad_w != 0 || (a.oh - 1) * stride_h + (kh - 1) * dil_h >= h ||
                        (a.ow - 1) * stride_w + (kw - 1) * dil_w >= w;
    const int bn = cout <= 32 ? 32 : cout <= 64 ? 64 : 128;
    const long long big_tiles = ((M + 127) / 128) * ((cout + bn - 1) / bn);
#define DAB_FCONV_LAUNCH(BM, BN, SK, KSPLIT, CV)                                                         \
    do {                                                                                                 \
        const dim3 grid((unsigned)((M + BM - 1) / BM), (unsigned)((cout + BN - 1) / BN));                \
        if (padded)                                                                                      \
            hipLaunchKernelGGL((fconv_kernel<BM, BN, SK, KSPLIT, true, CV>), grid, dim3(256), 0, s, a);  \
        else                                                                                             \
            hipLaunchKernelGGL((fconv_kernel<BM, BN, SK, KSPLIT, false, CV>), grid, dim3(256), 0, s, a); \
    } while (0)
    // Loader: 16-byte loads of four channels when the channel count allows it; for three-channel images one 12-byte
    // load per tap if the window has enough taps that slices of eight taps waste little (7x7: 56 for 49); else
    // element by element.
    const int taps = kh * kw;
    const bool vec4 = c % 4 == 0 && (reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(wgt)) % 16 == 0;
    const bool vec3 = c == 3 && bn == 64 && (taps + 7) / 8 * 24 * 10 <= (a.K + 15) / 16 * 16 * 11;
    if (M <= 8 && kh == 1 && kw == 1 && pad_h == 0 && pad_w == 0 && stride_h == 1 && stride_w == 1 && vec4 && cout >= 64) {
        // a matrix-vector product (the classifier at small batch): one wave per output channel
        hipLaunchKernelGGL(fconv_gemv_kernel, dim3((unsigned)((cout + 3) / 4)), dim3(256), 0, s, a);
    } else if (big_tiles < simd_count() / 4 && vec3 && (M + 63) / 64 >= simd_count() / 8) {
        // a three-channel image too small for 128-pixel tiles (the stem at batch 1): 64-pixel tiles keep the
        // one-load-per-tap loader and still give most CUs a block
        DAB_FCONV_LAUNCH(64, 64, 24, 1, 3);
    } else if (big_tiles < simd_count() / 4 && vec4 && small_1x1_tiles(kh * kw, M, cout) == 1) {
        DAB_FCONV_LAUNCH(64, 128, 32, 1, 4);
    } else if (big_tiles < simd_count() / 4 && vec4 && small_1x1_tiles(kh * kw, M, cout) == 2) {
        DAB_FCONV_LAUNCH(64, 64, 32, 1, 4);
    } else if (big_tiles < simd_count() / 4 && vec4 && small_1x1_tiles(kh * kw, M, cout) == 3) {
        DAB_FCONV_LAUNCH(32, 32, 64, 4, 4);
    } else if (big_tiles < simd_count() / 4 && vec4 && ((M + 63) / 64) * ((cout + 63) / 64) >= simd_count() / 8) {
        // fewer big tiles than CUs, but enough 64 x 64 ones for half of them: a wave still multiplies a whole 32 x 32 tile
        DAB_FCONV_LAUNCH(64, 64, 16, 1, 4);
    } else if (big_tiles < simd_count() / 4) {
        // fewer big tiles than CUs: 32 x 32 tiles, each slice's depth split over the block's waves
        if (vec4)
            DAB_FCONV_LAUNCH(32, 32, 64, 4, 4);
        else
            DAB_FCONV_LAUNCH(32, 32, 64, 4, 1);
    } else if (vec3) {
        DAB_FCONV_LAUNCH(128, 64, 24, 1, 3);
    } else if (c == 3 && bn == 32) {
        // few output channels: the launch is bound by its loads and stores, and one 12-byte load per tap beats three
        // 4-byte ones even where two slices of eight taps hold only nine (3x3 stride 2, 3 -> 32 at 224 x 224, batch
        // 256: 162 against 178 us)
        DAB_FCONV_LAUNCH(128, 32, 24, 1, 3);
    } else if (bn == 32) {
        if (vec4)
            DAB_FCONV_LAUNCH(128, 32, 16, 1, 4);
        else
            DAB_FCONV_LAUNCH(128, 32, 16, 1, 1);
    } else if (bn == 64) {
        if (vec4)
            DAB_FCONV_LAUNCH(128, 64, 16, 1, 4);
        else
            DAB_FCONV_LAUNCH(128, 64, 16, 1, 1);
    } else {
        if (vec4)
            DAB_FCONV_LAUNCH(128, 128, 16, 1, 4);
        else
            DAB_FCONV_LAUNCH(128, 128, 16, 1, 1);
    }
#undef DAB_FCONV_LAUNCH
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

// Whether dab_global_ave_pool_fconv1x1 takes the shapes: the few images of a small batch (more of them are a matrix
// product, which the pooling kernel and fconv_kernel do better), a window and a depth that fit the kernel's registers
// and LDS, 16-byte rows.
extern "C" int dab_global_ave_pool_fconv1x1_takes(int n, int h, int w, int c, int cout) {
    using namespace dab;
    return n >= 1 && n <= 8 && h >= 1 && w >= 1 && h * w <= kGlobalPoolTaps && c >= 4 && c % 4 == 0 &&
           c / 4 <= kGlobalPoolDepth4 && cout >= 64;
}

extern "C" int dab_global_ave_pool_fconv1x1(const float *x, int n, int h, int w, int c, const float *wgt, const float *bias,
                                            const float *aff_a, const float *aff_b, int relu, int cout, float *pooled,
                                            float *out, dab_stream_t stream) {
    using namespace dab;
    const char *fn = "dab_global_ave_pool_fconv1x1";
    DAB_REQUIRE(x && wgt && pooled && out, "%s: null pointer", fn);
    DAB_REQUIRE(n > 0 && h > 0 && w > 0 && c > 0 && cout > 0, "%s: non-positive dimension", fn);
    DAB_REQUIRE((aff_a == nullptr) == (aff_b == nullptr), "%s: affine needs both coefficient vectors", fn);
    if (!dab_global_ave_pool_fconv1x1_takes(n, h, w, c, cout) ||
        (reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(wgt) | reinterpret_cast<uintptr_t>(pooled)) % 16 != 0)
        return fail(DAB_EUNSUPPORTED, "%s: needs n <= 8, h * w <= %d, c %% 4 == 0, c <= %d, cout >= 64 and 16-byte aligned buffers", fn,
                    kGlobalPoolTaps, 4 * kGlobalPoolDepth4);
    FconvArgs a = {};
    a.x = x, a.w = wgt, a.bias = bias, a.aff_a = aff_a, a.aff_b = aff_b, a.relu = relu, a.out = out, a.pooled = pooled;
    a.n = n, a.h = h, a.wd = w, a.c = c, a.cout = cout, a.K = c, a.M = n;
    const unsigned blocks = (unsigned)((cout + 4 * kGlobalPoolChannels - 1) / (4 * kGlobalPoolChannels));
    const dim3 grid(blocks, (unsigned)n);
    hipStream_t s = as_stream(stream);
    if (c <= 512 && h * w <= 49)
        hipLaunchKernelGGL((global_avepool_gemv_kernel<2, 49>), grid, dim3(256), 0, s, a);
    else if (c <= 512)
        hipLaunchKernelGGL((global_avepool_gemv_kernel<2, 32>), grid, dim3(256), 0, s, a);
    else
        hipLaunchKernelGGL((global_avepool_gemv_kernel<4, 32>), grid, dim3(256), 0, s, a);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

extern "C" int dab_ave_pool2_fconv1x1(const float *x, int n, int h, int w, int c, const float *wgt, const float *bias,
                                      const float *aff_a, const float *aff_b, int relu, int cout, float *pooled, float *out,
                                      dab_stream_t stream) {
    using namespace dab;
    const char *fn = "dab_ave_pool2_fconv1x1";
    DAB_REQUIRE(x && wgt && out, "%s: null pointer", fn);
    DAB_REQUIRE(n > 0 && h >= 2 && w >= 2 && c > 0 && cout > 0, "%s: bad dimension (the input must hold a 2x2 window)", fn);
    DAB_REQUIRE((aff_a == nullptr) == (aff_b == nullptr), "%s: affine needs both coefficient vectors", fn);
    if (c % 4 != 0 ||
        (reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(wgt) | reinterpret_cast<uintptr_t>(pooled)) % 16 != 0)
        return fail(DAB_EUNSUPPORTED, "%s: needs c %% 4 == 0 and 16-byte aligned buffers", fn);
    FconvArgs a;
    a.x = x, a.w = wgt, a.bias = bias, a.aff_a = aff_a, a.aff_b = aff_b, a.relu = relu, a.out = out, a.pooled = pooled;
    a.n = n, a.h = h, a.wd = w, a.c = c;
    a.pad_h = 0, a.pad_w = 0, a.stride_h = 2, a.stride_w = 2;  // a pooled pixel's window starts at twice its coordinates
    a.oh = out_dim(h, 0, 2, 1, 2), a.ow = out_dim(w, 0, 2, 1, 2);
    a.cout = cout;
    a.K = c;
    const long long M = (long long)n * a.oh * a.ow;
    if (M >= (1ll << 31) - 128 || (long long)n * h * w * c >= (1ll << 31))
        return fail(DAB_EUNSUPPORTED, "%s: tensor too large for 32-bit indexing", fn);
    a.M = (int)M;
    if (M <= 8 && cout >= 64) {
        DAB_REQUIRE(pooled, "%s: eight pooled pixels or fewer run as two launches and need the pooled tensor's buffer", fn);
        // a handful of pooled pixels: dab_fconv_affine_relu makes them with its matrix-vector kernel, whose sums are
        // added in another order than a tile's -- two launches, so that the result stays what the two calls give
        int rc = dab_ave_pool(x, n, h, w, c, 2, 2, 0, 0, 2, 2, pooled, stream);
        if (rc != DAB_OK) return rc;
        return dab_fconv_affine_relu(pooled, n, a.oh, a.ow, c, wgt, bias, aff_a, aff_b, relu, 1, 1, 0, 0, 1, 1, 1, 1, cout, out, stream);
    }
    a.div_ow = FastDiv((uint32_t)a.ow), a.div_oh = FastDiv((uint32_t)a.oh);
    a.kw = 1, a.dil_h = 1, a.dil_w = 1;
    a.div_c = FastDiv((uint32_t)c), a.div_kw = FastDiv(1u);
    const long long span_imgs = 128 / ((long long)a.oh * a.ow) + 2;
    if (span_imgs * h * w * c * 4 >= (1ll << 30) || 128ll * a.K * 4 >= (1ll << 30) || 128ll * cout * 4 >= (1ll << 30))
        return fail(DAB_EUNSUPPORTED, "%s: image, filter or channel count too large for 32-bit tile offsets", fn);
    hipStream_t s = as_stream(stream);
    const int bn = cout <= 32 ? 32 : cout <= 64 ? 64 : 128;
    const long long big_tiles = ((M + 127) / 128) * ((cout + bn - 1) / bn);
#define DAB_POOLED_LAUNCH(BM, BN, SK, KSPLIT)                                                                     \
    hipLaunchKernelGGL((fconv_kernel<BM, BN, SK, KSPLIT, false, 4, true>),                                        \
                       dim3((unsigned)((M + BM - 1) / BM), (unsigned)((cout + BN - 1) / BN)), dim3(256), 0, s, a)
    // the same tiles as dab_fconv_affine_relu takes for the 1x1 convolution of the pooled tensor: the sums of a tile
    // whose depth is split over waves are added in another order
    const bool few = big_tiles < simd_count() / 4;
    const int small = few ? small_1x1_tiles(1, M, cout) : 0;
    const bool depth_split = few && (small == 3 || (small == 0 && ((M + 63) / 64) * ((cout + 63) / 64) < simd_count() / 8));
    if (c == 64 && cout > 64 && !depth_split && (long long)cout * c * 4 < (1ll << 30))
        // 64 input channels: the launch is bound by the input it reads, and the kernel that pools whole pixels once
        // into LDS reads it at the rate of a copy (256 x 56 x 56 x 64 -> 128: 66 us against 85, 58 without the pooled
        // tensor; batch 8: 5.2 against 6.1).  With 128 and 256 channels the two forms take the same time at batch
        // 256 (50 / 50 and 50 / 46 us), both at half of what the fp32 matrix instructions could do, and the tile
        // kernel wins below.
        hipLaunchKernelGGL((pool2_fconv1x1_kernel<64, 32>), dim3((unsigned)((M + 31) / 32)), dim3(256), 0, s, a);
    else if (big_tiles < simd_count() / 4 && small_1x1_tiles(1, M, cout) == 1)
        DAB_POOLED_LAUNCH(64, 128, 32, 1);
    else if (big_tiles < simd_count() / 4 && small_1x1_tiles(1, M, cout) == 2)
        DAB_POOLED_LAUNCH(64, 64, 32, 1);
    else if (big_tiles < simd_count() / 4 && small_1x1_tiles(1, M, cout) == 3)
        DAB_POOLED_LAUNCH(32, 32, 64, 4);
    else if (big_tiles < simd_count() / 4 && ((M + 63) / 64) * ((cout + 63) / 64) >= simd_count() / 8)
        DAB_POOLED_LAUNCH(64, 64, 16, 1);
    else if (big_tiles < simd_count() / 4)
        DAB_POOLED_LAUNCH(32, 32, 64, 4);
    else if (bn == 32)
        DAB_POOLED_LAUNCH(128, 32, 16, 1);
    else if (bn == 64)
        DAB_POOLED_LAUNCH(128, 64, 16, 1);
    else if (cout <= 128)
        // one column tile: the launch is bound by the input it reads, and a 32-deep slice takes whole 128-byte
        // lines of a pixel where a 16-deep one fetches every line twice, a slice apart (97 -> 83 us for
        // 256 x 56 x 56 x 64 -> 128)
        DAB_POOLED_LAUNCH(128, 128, 32, 1);
    else
        // several column tiles: every one of them pools the input again, so the tile is as wide as the accumulators
        // allow and 64 rows high (256 x 28 x 28 x 128 -> 256: 60 -> 55 us, 256 x 14 x 14 x 256 -> 512: 59 -> 48 us;
        // 128 x 64 tiles: 90 us)
        DAB_POOLED_LAUNCH(64, 256, 16, 1);
#undef DAB_POOLED_LAUNCH
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

extern "C" int dab_prelu_inplace(float *x, int64_t n_pix, int c, const float *slope, int slope_n, dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(x && slope, "dab_prelu_inplace: null pointer");
    DAB_REQUIRE(n_pix > 0 && c > 0, "dab_prelu_inplace: n_pix %lld c %d", (long long)n_pix, c);
    DAB_REQUIRE(slope_n == 1 || slope_n == c, "dab_prelu_inplace: slope must have size 1 or c (%d), got %d", c, slope_n);
    const long long total = (long long)n_pix * c;
    hipLaunchKernelGGL(prelu_kernel, dim3(grid_for(total)), dim3(256), 0, as_stream(stream), x, total, c, slope, slope_n);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

extern "C" int dab_concat_channels(const float *a, int ca, const float *b, int cb, int64_t n_pix, float *out,
                                   dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(a && b && out, "dab_concat_channels: null pointer");
    DAB_REQUIRE(n_pix > 0 && ca > 0 && cb > 0, "dab_concat_channels: n_pix %lld ca %d cb %d", (long long)n_pix, ca, cb);
    DAB_REQUIRE(out != a && out != b, "dab_concat_channels: out must not alias an input");
    const long long total = (long long)n_pix * (ca + cb);
    hipLaunchKernelGGL(concat_kernel, dim3(grid_for(total)), dim3(256), 0, as_stream(stream), a, ca, b, cb, out, total);
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
                       int stride_h, int stride_w, float *out, uint64_t *out_packed, bool want_sign, dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(x && out && (out_packed || !want_sign), "dab_pool: null pointer");
    DAB_REQUIRE(n > 0 && h > 0 && w > 0 && c > 0 && kh > 0 && kw > 0, "dab_pool: non-positive dimension");
    DAB_REQUIRE(pad_h >= 0 && pad_w >= 0 && stride_h > 0 && stride_w > 0, "dab_pool: bad pad/stride");
    PoolArgs a;
    a.x = x, a.out = out;
    a.n = n, a.h = h, a.w = w, a.c = c, a.kh = kh, a.kw = kw;
    a.pad_h = pad_h, a.pad_w = pad_w, a.stride_h = stride_h, a.stride_w = stride_w;
    a.oh = out_dim(h, pad_h, kh, 1, stride_h), a.ow = out_dim(w, pad_w, kw, 1, stride_w);
    DAB_REQUIRE(a.oh > 0 && a.ow > 0, "dab_pool: empty output");
    const long long total = (long long)n * a.oh * a.ow * c;
    const bool vec_ok = c % 4 == 0 && total / 4 < (1ll << 31) - 256 &&
                        (reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) % 16 == 0;
    if (want_sign) {
        if (c % 64 != 0 || !vec_ok || !is_max)
            return fail(DAB_EUNSUPPORTED, "dab_max_pool_sign: needs c %% 64 == 0, 16-byte aligned buffers and fewer than 2^33 outputs");
        DAB_REQUIRE(reinterpret_cast<uintptr_t>(out_packed) % 8 == 0, "dab_max_pool_sign: misaligned packed output");
    }
    if (vec_ok) {
        PoolVecArgs v;
        v.g = a, v.c4 = c / 4, v.total = (uint32_t)(total / 4);
        v.div_c4 = FastDiv((uint32_t)v.c4), v.div_ow = FastDiv((uint32_t)a.ow), v.div_oh = FastDiv((uint32_t)a.oh);
        // windows of more than 16 taps are long chains of waits: one wave per block there, so that a launch of a few
        // hundred waves spreads over all CUs (the global 7x7 average at batch 256: 128 blocks of 256 threads before)
        const unsigned bs = kh * kw > 16 ? 64u : 256u;
        const unsigned vb = (v.total + bs - 1u) / bs;
        const float4 *x4 = reinterpret_cast<const float4 *>(x);
        float4 *o4 = reinterpret_cast<float4 *>(out);
        // loads kept in flight: the whole window up to 3x3, 16 at a time beyond, 32 when the launch is too small to
        // fill the chip and the chain of waits is all there is to it
        const int taps = kh * kw;
        const int batch_taps = taps <= 4 ? 4 : taps <= 9 ? 9 : (taps <= 16 || v.total > 65536u) ? 16 : 32;
        auto launch = [&](auto kernel) {
            hipLaunchKernelGGL(kernel, dim3(vb), dim3(bs), 0, as_stream(stream), x4, o4, out_packed, v);
        };
#define DAB_POOL_LAUNCH(MAX, SIGN)                                               \
    switch (batch_taps) {                                                        \
        case 4: launch(pool_vec4_kernel<MAX, SIGN, 4>); break;                   \
        case 9: launch(pool_vec4_kernel<MAX, SIGN, 9>); break;                   \
        case 16: launch(pool_vec4_kernel<MAX, SIGN, 16>); break;                 \
        default: launch(pool_vec4_kernel<MAX, SIGN, 32>); break;                 \
    }
        if (!is_max && taps > 32 && taps <= 49 && v.total <= 4096u) {
            // a global 7x7 average at batch 1-8: a few waves whose whole life is waiting for their taps -- ask for
            // all 49 at once
            launch(pool_vec4_kernel<false, false, 49>);
        } else if (want_sign) {
            DAB_POOL_LAUNCH(true, true)
        } else if (is_max) {
            DAB_POOL_LAUNCH(true, false)
        } else {
            DAB_POOL_LAUNCH(false, false)
        }
#undef DAB_POOL_LAUNCH
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
    return pool_common(false, x, n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, out, nullptr, false, stream);
}

extern "C" int dab_max_pool(const float *x, int n, int h, int w, int c, int kh, int kw, int pad_h, int pad_w,
                            int stride_h, int stride_w, float *out, dab_stream_t stream) {
    return pool_common(true, x, n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, out, nullptr, false, stream);
}

extern "C" int dab_max_pool_sign(const float *x, int n, int h, int w, int c, int kh, int kw, int pad_h, int pad_w,
                                 int stride_h, int stride_w, float *out, uint64_t *out_packed, dab_stream_t stream) {
    return pool_common(true, x, n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, out, out_packed, true, stream);
}
