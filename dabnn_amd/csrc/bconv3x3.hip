// Direct 3x3 binary convolution for 64/128/256/512 input channels.
//
// Replaces the reference's pack -> pad -> bconv_3x3 chain
// (dabnn/layers/BinConv.cpp:145-150, dabnn/bconv.h:855-931) on packed input;
// results equal baseline_bconv (common/baseline.h:77-116) bit for bit.
//
// Data layout: x [N][H][W][CW] uint64 (CW = cin/64), weights in the reference's
// own order [cout][3][3][CW] (no repacking), out [N][OH][OW][cout] fp32.
// A lane owns one output pixel and keeps its 9*CW input words (18*CW VGPRs)
// resident; out-of-image taps are fetched through a buffer descriptor with an
// out-of-range offset, which the hardware answers with zero -- the zero word
// that stands for 64 values of -1 (dabnn/pad.h:12).
#include <type_traits>

#include "xnor_core.h"
#include "bconv3x3_rows.h"

namespace dab {

struct BconvArgs {
    const uint64_t *x;
    const uint64_t *w;
    float *out;
    int total;     // N*OH*OW output pixels
    int H, W, OH, OW;
    int cout;
    int stride, pad;
    int n_groups;  // cout / Q channel groups per tile
    int items_per_wave, items_extra;  // split of the work items over the waves
    uint32_t x_bytes;
    int half;      // HALF kernels: which 512 of the 1024 input channels (0 or 1)
    int gran;      // row-split kernel: channels per work item (4, or 8 when sign bits are written)
    int through;   // raw counts: written through the L2 instead of as streaming (windows) and ordinary (pieces) stores
    FastDiv div_ow, div_oh, div_groups;
    // fused epilogue (MODE >= 1 kernels only): out = a*cnt + b (+ shortcut); MODE 2 also writes sign bits of out
    const float *epi_a;
    const float *epi_b;
    const float *epi_shortcut;
    unsigned char *epi_bits;
};

constexpr int kWavesPerBlock = 4;

// Channels per unit for CW words per pixel: units stay near 600 VALU instructions, so that the tail of a launch (one
// unit on a lone wave) stays short and the SIMDs' loads differ by little.  256 and 512 input channels have a second
// build with units twice that size for problems large enough that neither matters (BIG: eight channels for 256,
// four for 512): a unit starts with a wait for its first vector of filters that only other waves can hide and ends
// with a staging write, and half as many of both are worth 2.5 % (256 channels) and 11 % (512) at batch 256, against
// a loss of 3-8 % at batch 64.
template <int CW, bool BIG>
struct UnitChannels {
    static constexpr int value = CW == 8 ? (BIG ? 4 : 2) : (CW == 4 ? (BIG ? 8 : 4) : 8);
};

// Work items handed to waves are runs of S units so that a wave's share of a
// pixel row always starts and ends on a 16-byte boundary (4 channels) -- on
// 8 channels when the epilogue also writes sign bits, one whole byte of them.
template <int Q, bool EMIT>
struct ItemUnits {
    static constexpr int align = EMIT ? 8 : 4;
    static constexpr int value = Q >= align ? 1 : align / Q;
};

// MODE 0: raw counts.  1: + Affine (+ Add).  2: the same and a sign-packed copy of the result.
constexpr int kModeCounts = 0, kModeAffineAdd = 1, kModeAffineAddSign = 2;
// 3: out += counts, the second pass over a depth that is counted in two halves (1024 input channels)
constexpr int kModeAccumulate = 3;

// Resident waves per SIMD the kernel is built for, and the staging window that lets them fit the CU's LDS:
// the activations take 18*CW VGPRs, so 64 and 128 channels leave room for 8 and 6 waves (with the 16-channel
// window, 5 KB per wave), 256 channels for 4 and 512 channels (144 of 512/3 = 168 VGPRs) for 3.
// 64 and 128 channels have a second build (NARROW): 4 waves, the 32-channel window (whole 128-byte lines, no extra
// write traffic) and wave priorities.  Measured: faster when a wave gets enough units (64 channels, 6 per wave:
// 17.2 against 18.4 us; 128 channels, 12 per wave: 51 against 55 us), slower when it gets few (64 channels, 3 per
// wave: 11.2 against 10.2 us; 128 channels, 3 per wave: 17.3 against 16.1 us).
// For 256 and 512 input channels the flag selects the large-unit build instead (same residency).
template <int CW, bool NARROW>
struct Residency {
    static constexpr int waves_per_simd = CW == 8 ? 3 : CW == 4 ? 4 : NARROW ? 4 : (CW == 1 ? 8 : 6);
    static constexpr int window = (CW <= 2 && !NARROW) ? 16 : 32;
    static constexpr bool priorities = waves_per_simd <= 4;
};

// HALF: the tensors have 1024 channels (16 words per pixel and per filter tap) and the kernel counts one half of them,
// words 8 * p.half .. + 7: the reference lists 1024 input channels as direct-convolution compatible
// (dabnn/layers/BinConv.cpp:118); two passes of the 512-channel kernel, the second adding to the first's result.
template <int CW, int MODE, bool NARROW, bool HALF = false>
__global__ __launch_bounds__(64 * kWavesPerBlock, (Residency<CW, NARROW>::waves_per_simd)) void bconv3x3_kernel(const BconvArgs p) {
    static_assert(!HALF || CW == 8, "halves of 1024 channels only");
    constexpr int K32 = 18 * CW;
    constexpr int kPixelBytes = HALF ? 128 : CW * 8;       // one pixel's words
    constexpr int kFilterWords = HALF ? 9 * 16 : 9 * CW;   // one output channel's words
    constexpr int Q = UnitChannels<CW, NARROW>::value;
    constexpr int S = ItemUnits<Q, MODE == kModeAffineAddSign>::value;
    constexpr int WCH = Residency<CW, NARROW>::window;
    constexpr int WU = WCH / Q;  // units per staging window
    constexpr int kStageBytes = Stage<WCH>::bytes;
    constexpr bool kPrefetchFilters = true;
    constexpr int kFlushGroup = CW == 1 ? 8 : CW == 2 ? (NARROW ? 8 : 2) : CW == 4 ? 4 : 1;  // shortcut loads in flight, as the register budget allows
    __shared__ __attribute__((aligned(16))) unsigned char stage_all[kWavesPerBlock * kStageBytes];
    const int lane = threadIdx.x & 63;
    const int wib = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    unsigned char *stage = stage_all + wib * kStageBytes;
    const int wv = blockIdx.x * kWavesPerBlock + wib;

    int i0, i1;
    item_range(wv, p.items_per_wave, p.items_extra, i0, i1);
    if (i0 >= i1) return;
    const int u0 = i0 * S, u1 = i1 * S;

    if constexpr (kPrefetchFilters) {
        // Every wave walks the filters with scalar loads.  When other kernels have run in between they are in no L2
        // any more, and the first wave of an XCD to need a row waits for memory in the middle of its unit.  So the
        // launch first touches every 128-byte line of the filters once per XCD (blocks are dealt to the eight XCDs in
        // turn: block b runs on XCD b % 8): wave j of an XCD asks for one dword of each of the lines 64*j .. 64*j+63,
        // straight into the first 256 bytes of its own staging buffer, with no register and no wait involved; the
        // wave waits for it before it stages its first results there (by then the loads are long done: they were
        // issued before the activations the first unit has just used).
        const uint32_t n_lines = ((uint32_t)(p.cout * kFilterWords * 8) + 127u) >> 7;
        const uint32_t first = (uint32_t)((blockIdx.x >> 3) * kWavesPerBlock + wib) * 64u;
        if (first < n_lines) {
            const uint32_t line = first + lane < n_lines ? first + lane : n_lines - 1;
            const uint32_t last_byte = (uint32_t)(p.cout * kFilterWords * 8) - 4u;
            const uint32_t byte = line * 128u < last_byte ? line * 128u : last_byte;
            __builtin_amdgcn_global_load_lds(
                (const void __attribute__((address_space(1))) *)(reinterpret_cast<const unsigned char *>(p.w) + byte),
                (void __attribute__((address_space(3))) *)stage, 4, 0, 0);
        }
    }
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(p.x, p.x_bytes);
    int tile = (int)p.div_groups.div((uint32_t)u0);
    int cg = u0 - tile * p.n_groups;
    int ch_lo = (cg % WU) * Q;  // first staged channel of the current window
    bool need_load = true;
    uint32_t a[K32];

    auto flush = [&](auto group, int cg_now, int slot) {
        constexpr int G = decltype(group)::value;
        if constexpr (MODE == kModeAffineAddSign) {
            EpiAffineAddSign epi;
            epi.a = p.epi_a, epi.b = p.epi_b, epi.shortcut = p.epi_shortcut;
            epi.bits = p.epi_bits, epi.bits_ld = p.cout >> 3;
            stage_flush<WCH, G>(stage, lane, p.out, p.cout, tile, p.total, (cg_now - slot) * Q, ch_lo >> 2,
                                (slot * Q + Q - 1) >> 2, epi);
        } else if constexpr (MODE == kModeAccumulate) {
            EpiAccumulate epi;
            epi.shortcut = p.out;
            stage_flush<WCH, G>(stage, lane, p.out, p.cout, tile, p.total, (cg_now - slot) * Q, ch_lo >> 2,
                                (slot * Q + Q - 1) >> 2, epi);
        } else if constexpr (MODE == kModeAffineAdd) {
            EpiAffineAdd epi;
            epi.a = p.epi_a, epi.b = p.epi_b, epi.shortcut = p.epi_shortcut;
            stage_flush<WCH, G>(stage, lane, p.out, p.cout, tile, p.total, (cg_now - slot) * Q, ch_lo >> 2,
                                (slot * Q + Q - 1) >> 2, epi);
        } else {
            EpiStore epi;
            epi.through = p.through;
            stage_flush<WCH, G>(stage, lane, p.out, p.cout, tile, p.total, (cg_now - slot) * Q, ch_lo >> 2,
                                (slot * Q + Q - 1) >> 2, epi);
        }
    };

    for (int u = u0;; ++u) {
        if (need_load) {
            need_load = false;
            int pix = tile * 64 + lane;
            pix = pix < p.total ? pix : p.total - 1;
            const uint32_t t = p.div_ow.div(pix);
            const int ox = pix - t * p.OW;
            const uint32_t n = p.div_oh.div(t);
            const int oy = t - n * p.OH;
            const int y0 = oy * p.stride - p.pad, x0 = ox * p.stride - p.pad;
            // byte offset of tap (0,0); may be negative
            const int base = ((n * p.H + y0) * p.W + x0) * kPixelBytes + (HALF ? p.half * 64 : 0);
#pragma unroll
            for (int kh = 0; kh < 3; ++kh) {
                const bool row_ok = (unsigned)(y0 + kh) < (unsigned)p.H;
#pragma unroll
                for (int kw = 0; kw < 3; ++kw) {
                    const bool ok = row_ok && (unsigned)(x0 + kw) < (unsigned)p.W;
                    // an offset beyond the descriptor's range reads as zero
                    const int off = ok ? base + (kh * p.W + kw) * kPixelBytes : (int)0x80000000;
                    uint32_t *dst = a + (kh * 3 + kw) * CW * 2;
                    if constexpr (CW == 1) {
                        const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, off, 0, 0);
                        dst[0] = v.x, dst[1] = v.y;
                    } else {
#pragma unroll
                        for (int c = 0; c < CW / 2; ++c) {
                            const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, c * 16, 0);
                            dst[4 * c] = v.x, dst[4 * c + 1] = v.y, dst[4 * c + 2] = v.z, dst[4 * c + 3] = v.w;
                        }
                    }
                }
            }
        }

        // The SIMD issues from its oldest wave first, so with equal priorities the waves of a SIMD finish one after
        // the other and the last one runs alone at the single-wave issue rate.  Priority by remaining work keeps
        // them level: they reach their last units together.  (No gain measured with 7-8 resident waves.)
        const int left = Residency<CW, NARROW>::priorities ? u1 - u - 1 : 0;
        if (left >= 3) {
            __builtin_amdgcn_s_setprio(3);
        } else if (left == 2) {
            __builtin_amdgcn_s_setprio(2);
        } else if (left == 1) {
            __builtin_amdgcn_s_setprio(1);
        } else {
            __builtin_amdgcn_s_setprio(0);
        }
        uint32_t acc[Q];
        // One vector of filters per wait: the launch has put the filters into its XCD's L2 (above), so a scalar-cache
        // miss is short, and the second vector's 32 SGPRs are worth more elsewhere (seven batch-64 shapes in a step:
        // 95.7 us against 98.8 with two vectors per wait, 117 with one vector and filters that start cold).  With an
        // epilogue and 256 or 512 input channels the memory pipes are busy with the shortcut and the filters are
        // large: there two vectors per wait win at batch 256 (51 against 59 us, 54 against 55; 0.4-0.7 us lost at
        // batch 64).
        unit_rowmajor<K32, Q, ((MODE != kModeCounts && CW >= 4) ? 2 : 1), false, (HALF ? 128 : 0)>(
            p.w + (size_t)cg * Q * kFilterWords + (HALF ? p.half * 8 : 0), a, acc);
        const int slot = cg % WU;
        if constexpr (kPrefetchFilters) {
            if (u == u0) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the filter prefetch wrote into the staging buffer
        }
        stage_put<WCH, Q>(stage, lane, slot * Q, acc);

        // The window goes out when it is full or the tile ends.  The last unit of the wave leaves the loop first:
        // its flush runs where the activation registers are dead, so it can keep all of the window's shortcut loads
        // in flight at once -- every wave of a launch reaches that flush at about the same time, with no other
        // wave's arithmetic to hide the memory latency behind.
        if (u == u1 - 1) break;
        const bool last_in_tile = cg == p.n_groups - 1;
        if (slot == WU - 1 || last_in_tile) {
            flush(std::integral_constant<int, kFlushGroup>{}, cg, slot);
            ch_lo = 0;
        }
        if (last_in_tile) {
            cg = 0;
            ++tile;
            need_load = true;
        } else {
            ++cg;
        }
    }
    flush(std::integral_constant<int, 8>{}, cg, cg % WU);
}

// The row-split form (bconv3x3_rows.h): a block of three waves, wave r counting kernel row r of every output channel
// of the block's segment; partial counts meet in LDS.
template <int CW, int MODE>
__global__ __launch_bounds__(192) void bconv3x3_rows_kernel(const BconvArgs p) {
    typedef RowSplit<CW> RS;
    constexpr int DWR = RS::row_dwords, VEC = RS::vec, PIECES = RS::pieces, GROUP = RS::group, SEG = RS::segment, ROW = RS::row;
    constexpr int kFilterBytes = 9 * CW * 8;  // one output channel's weights
    constexpr int kPixelBytes = CW * 8;
    __shared__ __attribute__((aligned(16))) unsigned char plane[64 * ROW];
    const int tid = threadIdx.x, lane = tid & 63;
    const int r = __builtin_amdgcn_readfirstlane(tid >> 6);  // this wave's kernel row

    int i0, i1;
    item_range((int)blockIdx.x, p.items_per_wave, p.items_extra, i0, i1);  // the block's items of p.gran channels
    if (i0 >= i1) return;
    int tile = (int)p.div_groups.div((uint32_t)i0);  // n_groups = items per tile
    int ch = (i0 - tile * p.n_groups) * p.gran;
    int left = (i1 - i0) * p.gran;
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(p.x, p.x_bytes);

    {
        // Every wave walks the filters with scalar loads.  When other kernels have run in between they are in no L2
        // any more, and the first wave of an XCD to need a row would wait for memory in the middle of its pass.  So
        // the launch first touches every 128-byte line of the filters once per XCD (blocks are dealt to the eight
        // XCDs in turn: block b runs on XCD b % 8): wave j of an XCD asks for one dword of each of the lines
        // 64*j .. 64*j+63, straight into a sink in LDS, with no register involved.  The loads are done before the
        // wave's first activations are (vector loads complete in order).
        __shared__ uint32_t sink[RS::threads];
        const uint32_t filter_bytes = (uint32_t)(p.cout * kFilterBytes);
        const uint32_t n_lines = (filter_bytes + 127u) >> 7;
        const uint32_t first = (uint32_t)((blockIdx.x >> 3) * 3 + r) * 64u;
        if (first < n_lines) {
            const uint32_t line = first + lane < n_lines ? first + lane : n_lines - 1;
            const uint32_t byte = line * 128u < filter_bytes - 4u ? line * 128u : filter_bytes - 4u;
            __builtin_amdgcn_global_load_lds(
                (const void __attribute__((address_space(1))) *)(reinterpret_cast<const unsigned char *>(p.w) + byte),
                (void __attribute__((address_space(3))) *)(sink + r * 64), 4, 0, 0);
        }
    }
    uint32_t a[DWR];
    int loaded_tile = -1;
    bool plane_ready = false;
    while (left > 0) {
        int seg = p.cout - ch < SEG ? p.cout - ch : SEG;
        seg = seg < left ? seg : left;
        const int cbase = ch;  // first channel of the segment
        if (tile != loaded_tile) {
            loaded_tile = tile;
            int pix = tile * 64 + lane;
            pix = pix < p.total ? pix : p.total - 1;
            const uint32_t t = p.div_ow.div(pix);
            const int ox = pix - t * p.OW;
            const uint32_t nimg = p.div_oh.div(t);
            const int oy = t - nimg * p.OH;
            const int y = oy * p.stride - p.pad + r, x0 = ox * p.stride - p.pad;
            const int base = ((nimg * p.H + y) * p.W + x0) * kPixelBytes;  // byte offset of tap (r, 0); may be negative
            const bool row_ok = (unsigned)y < (unsigned)p.H;
#pragma unroll
            for (int kw = 0; kw < 3; ++kw) {
                const bool ok = row_ok && (unsigned)(x0 + kw) < (unsigned)p.W;
                // an offset beyond the descriptor's range reads as zero: the reference's padding word
                const int off = ok ? base + kw * kPixelBytes : (int)0x80000000;
#pragma unroll
                for (int c = 0; c < CW / 2; ++c) {
                    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, c * 16, 0);
                    uint32_t *dst = a + kw * CW * 2 + 4 * c;
                    dst[0] = v.x, dst[1] = v.y, dst[2] = v.z, dst[3] = v.w;
                }
            }
        }

        if (!plane_ready) {
            // the plane starts at zero (every store pass leaves it so); cleared behind the first loads, not before them
            plane_ready = true;
            for (int i = tid; i < 64 * ROW / 16; i += RS::threads) reinterpret_cast<u32x4 *>(plane)[i] = u32x4{0u, 0u, 0u, 0u};
            __syncthreads();
        }

        {
            // this wave's weights: row r of the segment's channels, GROUP channels per pass.  The scalar-load batches
            // form one sequence (channel by channel, PIECES per channel) and batch j lives in wv[j & 1]: the one a body
            // consumes was asked for by the body before it, also across passes (a pass is an even number of batches).
            const unsigned char *wseg = reinterpret_cast<const unsigned char *>(p.w) + (size_t)cbase * kFilterBytes + r * (DWR * 4);
            uint32_t *my = reinterpret_cast<uint32_t *>(plane + lane * ROW);
            WVec<VEC> wv[2];
            static_assert((GROUP * PIECES) % 2 == 0, "a pass starts with wv[0]");
            const int groups = seg / GROUP;
            uint32_t goff = 0;  // byte offset of the pass's first channel
            wv[0].template load_off<0>(wseg, goff);
            wv[0].wait();
#pragma unroll 1
            for (int g = 0; g < groups; ++g) {
                uint32_t acc[GROUP];
                const bool more = g + 1 < groups;
                // (Wave priorities by remaining work, which help the unit kernel at three and four waves per SIMD, cost
                // 0.3 us here: 16.8 against 16.4 us for 7 x 7 x 512 -> 512 at batch 64.)
                static_for<GROUP * PIECES>([&](auto j_) {
                    constexpr int j = j_, c = j / PIECES, piece = j % PIECES;
                    constexpr int jn = j + 1, cn = jn / PIECES, pn = jn % PIECES;
                    if constexpr (jn < GROUP * PIECES) {
                        wv[jn & 1].template load_off<cn * kFilterBytes + pn * VEC * 4>(wseg, goff);
                    } else {
                        if (more) wv[0].template load_off<GROUP * kFilterBytes>(wseg, goff);
                    }
                    rows_count<VEC, piece == 0>(acc[c], wv[j & 1], a + piece * VEC);
                    wv[jn & 1].wait();
                });
#pragma unroll
                for (int c = 0; c < GROUP; ++c) atomicAdd(my + g * GROUP + c, acc[c]);
                goff += GROUP * kFilterBytes;
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): nothing of this wave is on its way into LDS any more
        __syncthreads();
        if constexpr (MODE == kModeAffineAddSign) {
            EpiAffineAddSign epi;
            epi.a = p.epi_a, epi.b = p.epi_b, epi.shortcut = p.epi_shortcut;
            epi.bits = p.epi_bits, epi.bits_ld = p.cout >> 3;
            rows_flush<SEG, ROW, RS::threads>(plane, tid, p.out, p.cout, tile, p.total, cbase, seg, epi);
        } else if constexpr (MODE == kModeAffineAdd) {
            EpiAffineAdd epi;
            epi.a = p.epi_a, epi.b = p.epi_b, epi.shortcut = p.epi_shortcut;
            rows_flush<SEG, ROW, RS::threads>(plane, tid, p.out, p.cout, tile, p.total, cbase, seg, epi);
        } else {
            EpiStore epi;
            rows_flush<SEG, ROW, RS::threads>(plane, tid, p.out, p.cout, tile, p.total, cbase, seg, epi);
        }
        left -= seg, ch += seg;
        if (ch == p.cout) ch = 0, ++tile;
        if (left > 0) __syncthreads();  // the plane is zero again
    }
}

// A few tiles only (small batches): the kernel above would leave most SIMDs without a
// wave, each of the few waves grinding through all 4 or 8 input words of 9 taps.  Here a block is one work item of 64
// pixels x 8 output channels and its four waves split the depth: a channel's 18*CW weight dwords (9 taps x CW words,
// contiguous) are 36 chunks of CW*2 bytes, four per tap, and wave w takes chunks [9w, 9w + 9) -- of the weights and
// of every pixel's activations alike.  The block first copies the item's weights to LDS with coalesced loads (a
// wave's share of a channel is too short and too strided for the scalar-load stream of the big kernel), the four
// partial counts meet in LDS and the first wave applies the epilogue.  Eight channels are one byte of sign bits, so
// the packed copy needs no coordination between blocks.
template <int CW, int MODE>
__global__ __launch_bounds__(256) void bconv3x3_ksplit_kernel(const BconvArgs p) {
    constexpr int K32 = 18 * CW;       // weight dwords per channel
    constexpr int CD = CW / 2;         // dwords per chunk (1, 2 or 4)
    // dwords per wave and channel; with 64 input channels the 18 dwords of a channel go 5, 5, 4, 4 to the waves
    constexpr int WD = CW == 1 ? 5 : 9 * CD;
    __shared__ __attribute__((aligned(16))) uint32_t wlds[8 * K32];
    __shared__ uint32_t part[4][8][64];  // [wave][channel][pixel]
    const int lane = threadIdx.x & 63;
    const int wib = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tile = (int)p.div_groups.div(blockIdx.x);  // n_groups = cout / 8 here
    const int cg = (int)blockIdx.x - tile * p.n_groups;

    // The first wave will need the epilogue's operands at the very end; asked for now, they arrive while the counts
    // are made instead of adding a round trip to memory behind them.
    const int real_pix = tile * 64 + lane;
    const size_t out_off = (size_t)(real_pix < p.total ? real_pix : p.total - 1) * p.cout + cg * 8;
    float ea[8], eb[8];
    float4 s0 = make_float4(0.f, 0.f, 0.f, 0.f), s1 = s0;
    if constexpr (MODE != kModeCounts) {
        if (wib == 0) {
#pragma unroll
            for (int ch = 0; ch < 8; ++ch) ea[ch] = p.epi_a[cg * 8 + ch], eb[ch] = p.epi_b[cg * 8 + ch];
            if (p.epi_shortcut != nullptr) {
                s0 = *reinterpret_cast<const float4 *>(p.epi_shortcut + out_off);
                s1 = *reinterpret_cast<const float4 *>(p.epi_shortcut + out_off + 4);
            }
        }
    }

    // the item's weights: 8 channels x K32 dwords, contiguous in memory
    {
        const uint64_t *wsrc = p.w + (size_t)cg * 8 * 9 * CW;
        uint64_t *wdst = reinterpret_cast<uint64_t *>(wlds);
        for (int i = threadIdx.x; i < 8 * 9 * CW; i += 256) wdst[i] = wsrc[i];
    }

    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(p.x, p.x_bytes);
    const int pix = real_pix < p.total ? real_pix : p.total - 1;
    const uint32_t t = p.div_ow.div(pix);
    const int ox = pix - t * p.OW;
    const uint32_t n = p.div_oh.div(t);
    const int oy = t - n * p.OH;
    const int y0 = oy * p.stride - p.pad, x0 = ox * p.stride - p.pad;
    const int base = ((n * p.H + y0) * p.W + x0) * (CW * 8);  // byte offset of tap (0,0); may be negative
    uint32_t a[WD];
    const int first = CW == 1 ? wib * 5 - (wib > 2 ? wib - 2 : 0) : wib * WD;  // this wave's first dword of a channel
    const int count = CW == 1 ? (wib < 2 ? 5 : 4) : WD;                         // and how many it takes
    if constexpr (CW == 1) {
#pragma unroll
        for (int j = 0; j < WD; ++j) {
            const int d = first + j;  // wave-uniform; two dwords per tap
            const int tap = d >> 1, kh = tap / 3, kw = tap - kh * 3;
            const bool ok = j < count && (unsigned)(y0 + kh) < (unsigned)p.H && (unsigned)(x0 + kw) < (unsigned)p.W;
            // beyond the descriptor's range a load returns zero: the reference's padding word
            a[j] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, ok ? base + (kh * p.W + kw) * 8 + (d & 1) * 4 : (int)0x80000000, 0, 0);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 9; ++j) {
            const int chunk = wib * 9 + j;  // wave-uniform
            const int tap = chunk >> 2, kh = tap / 3, kw = tap - kh * 3;
            const bool ok = (unsigned)(y0 + kh) < (unsigned)p.H && (unsigned)(x0 + kw) < (unsigned)p.W;
            const int off = ok ? base + (kh * p.W + kw) * (CW * 8) + (chunk & 3) * (CD * 4) : (int)0x80000000;
            if constexpr (CD == 1) {
                a[j] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, off, 0, 0);
            } else if constexpr (CD == 2) {
                const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, off, 0, 0);
                a[j * 2] = v.x, a[j * 2 + 1] = v.y;
            } else {
                const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, 0);
                a[j * 4] = v.x, a[j * 4 + 1] = v.y, a[j * 4 + 2] = v.z, a[j * 4 + 3] = v.w;
            }
        }
    }
    __syncthreads();  // weights in LDS
    const uint32_t *wq = wlds + first;  // this wave's share of channel 0; every lane reads the same words
#pragma unroll
    for (int ch = 0; ch < 8; ++ch) {
        uint32_t c = 0;
#pragma unroll
        for (int d = 0; d < WD; ++d) {
            const uint32_t wd = (CW > 1 || d < count) ? wq[ch * K32 + d] : 0u;  // a[d] is zero where the share ends
            c += __builtin_popcount(wd ^ a[d]);
        }
        part[wib][ch][lane] = c;
    }
    __syncthreads();
    if (wib != 0 || real_pix >= p.total) return;

    float v[8];
#pragma unroll
    for (int ch = 0; ch < 8; ++ch)
        v[ch] = (float)(part[0][ch][lane] + part[1][ch][lane] + part[2][ch][lane] + part[3][ch][lane]);
    if constexpr (MODE != kModeCounts) {
#pragma clang fp contract(off)
        // a*cnt + b (+ shortcut), each operation rounded on its own like the separate layers
#pragma unroll
        for (int ch = 0; ch < 8; ++ch) {
            const float prod = ea[ch] * v[ch];
            v[ch] = prod + eb[ch];
        }
        if (p.epi_shortcut != nullptr) {
            v[0] = v[0] + s0.x, v[1] = v[1] + s0.y, v[2] = v[2] + s0.z, v[3] = v[3] + s0.w;
            v[4] = v[4] + s1.x, v[5] = v[5] + s1.y, v[6] = v[6] + s1.z, v[7] = v[7] + s1.w;
        }
    }
    *reinterpret_cast<float4 *>(p.out + out_off) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4 *>(p.out + out_off + 4) = make_float4(v[4], v[5], v[6], v[7]);
    if constexpr (MODE == kModeAffineAddSign) {
        uint32_t bits = 0;
#pragma unroll
        for (int ch = 0; ch < 8; ++ch) bits |= (v[ch] > 0.f ? 1u : 0u) << ch;
        p.epi_bits[(size_t)real_pix * (p.cout >> 3) + cg] = (unsigned char)bits;
    }
}

// So few work items (64 pixels x 8 channels) that splitting each over four waves gives a SIMD four waves at most
// (measured on Bi-Real-18 at batch 1 to 16: faster than the unit kernel up to there).
static bool splits_depth(long long tiles, int cin, int cout) {
    // 512 input channels: a unit there is 72 scalar loads of filters per channel, and the kernel that keeps an item's
    // filters in LDS stays ahead up to eight waves per SIMD (7x7 512->512 at batch 24 and 32: 4-6 % of the whole net)
    return tiles * (cout / 8) <= (long long)simd_count() * (cin >= 512 ? 2 : 1);
}

template <int CW, int MODE>
static int launch_ksplit(BconvArgs &a, long long tiles, hipStream_t stream) {
    a.n_groups = a.cout / 8;
    a.div_groups = FastDiv((uint32_t)a.n_groups);
    hipLaunchKernelGGL((bconv3x3_ksplit_kernel<CW, MODE>), dim3((unsigned)(tiles * a.n_groups)), dim3(256), 0, stream, a);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

// Raw counts are written through the L2 (stage_flush, stage_flush_window) when the output is larger than this: 9 MB
// for the builds with 16-channel windows, 6 MB for those with 32-channel windows; below it the whole windows are
// streaming stores and the pieces ordinary ones (0.2-0.6 us less per launch at 1.6-6 MB).  All stores of a launch go
// one way: a line that one wave finishes with one kind of store and another wave with another is written back twice,
// and written-through windows beside ordinary pieces took up to 1.6x as long from 38 MB up.  Measured on the seven
// stage shapes at batches 8 to 256 against streaming windows + ordinary pieces: 28x28 128->128 13.3 against 14.5 us at
// batch 64, 24.2 against 26.5 at batch 128; 56x56 64->64 14.6 against 16.2 at batch 64; 14x14 256->256 13.8 against
// 15.1; 56x56 64->128 at stride 2 8.7 against 9.6; 28x28 128->256 at stride 2 24.5 against 27.2 at batch 256; the
// seven-shape step 84.0 against 93.1 us at batch 64 and 261 against 267 at batch 256.
constexpr long long kThroughMinBytes16 = 9ll << 20, kThroughMinBytes32 = 6ll << 20;

template <int CW, int MODE, bool NARROW, bool HALF = false>
static int launch_variant(BconvArgs &a, long long tiles, hipStream_t stream) {
    constexpr int Q = UnitChannels<CW, NARROW>::value;
    constexpr int S = ItemUnits<Q, MODE == kModeAffineAddSign>::value;
    a.n_groups = a.cout / Q;
    const long long items = tiles * (a.n_groups / S);
    if (items >= (1ll << 31) / S) return fail(DAB_EUNSUPPORTED, "dab_bconv3x3: too many work units");
    static const int resident = resident_blocks_per_cu(bconv3x3_kernel<CW, MODE, NARROW, HALF>, 64 * kWavesPerBlock);
    int blocks_per_cu = resident;
    if constexpr (CW == 1 && !NARROW) {
        // 64 input channels: a unit is short (144 xor/popcount pairs) and a wave's fixed cost (arguments, pixel
        // decode, nine taps, the store pass) weighs as much as a unit, so fewer, longer-lived waves are ahead as long
        // as a wave's share still fits one 16-channel staging window (two units, one whole-window store pass): the
        // fewest waves per SIMD that keep every share at two units or less.  56 x 56 x 64 -> 128 at stride 2, batch
        // 64 (12 544 units): 9.5-9.8 us with 6 or 7 waves per SIMD against 10.3 with 8; 56 x 56 x 64 -> 64 at batch
        // 24-36: 0.4-0.9 us less than with 8 (measured for every count from 4 to 8 at eight batch sizes each).
        const long long per_simd = (items * S + 2ll * simd_count() - 1) / (2ll * simd_count());
        if (items * S >= (long long)simd_count() * resident && per_simd < blocks_per_cu) blocks_per_cu = (int)per_simd;
    }
    if constexpr (MODE == kModeCounts) {
        const long long out_bytes = 4ll * a.total * a.cout;
        a.through = 0;
        if (out_bytes >= (Residency<CW, NARROW>::window == 16 ? kThroughMinBytes16 : kThroughMinBytes32)) a.through = 1;
    }
    const int n_waves = pick_wave_count((int)items, blocks_per_cu, kWavesPerBlock, S);
    a.items_per_wave = (int)(items / n_waves);
    a.items_extra = (int)(items % n_waves);
    a.div_groups = FastDiv((uint32_t)a.n_groups);
    hipLaunchKernelGGL((bconv3x3_kernel<CW, MODE, NARROW, HALF>), dim3(n_waves / kWavesPerBlock), dim3(64 * kWavesPerBlock), 0, stream, a);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

// Blocks per CU of the row-split kernel: six (18 waves) at least (7 x 7 x 512 -> 512 at batch 64: 16.8 us with 4,
// 16.6 with 5, 15.7 with 6); launch_rows may take more for raw counts.
constexpr int kRowsBlocksPerCu = 6;

template <int CW, int MODE>
static int launch_rows(BconvArgs &a, long long tiles, hipStream_t stream) {
    a.gran = MODE == kModeAffineAddSign ? 8 : 4;
    a.n_groups = a.cout / a.gran;
    const long long items = tiles * a.n_groups;
    if (items >= (1ll << 31) / a.gran) return fail(DAB_EUNSUPPORTED, "dab_bconv3x3: too many work units");
    static const int blocks_per_cu = resident_blocks_per_cu(bconv3x3_rows_kernel<CW, MODE>, RowSplit<CW>::threads);
    // Blocks per CU.  A launch is one round of resident blocks, and it ends with its most loaded SIMD: the waves a
    // SIMD holds (three per block over four SIMDs) times the items of the largest block plus one (what a block does
    // before its first item -- activations, the plane -- is about an item's worth).  Raw counts take the count
    // between six per CU (fewer waves issue their pairs more slowly) and what is resident (ten at most) with the
    // smallest such product, the larger among equals (more waves hide more latency), as long as a block keeps two
    // items.  Against a fixed six: 7x7 512->512 14.6 against 15.7 us at batch 64 (nine blocks per CU), 11.9 against
    // 13.0 at batch 48; 14x14 256->512 at stride 2 7.6 against 8.2 at batch 48; level up to batch 28.  With an
    // epilogue the same rule gained and lost up to 1.5 us from size to size: six.
    const long long cus = simd_count() / 4;
    int per_cu = blocks_per_cu < kRowsBlocksPerCu ? blocks_per_cu : kRowsBlocksPerCu;
    if (MODE == kModeCounts) {
        long long best = -1;
        const int hi = blocks_per_cu < 10 ? blocks_per_cu : 10;
        for (int c = kRowsBlocksPerCu < hi ? kRowsBlocksPerCu : hi; c <= hi; ++c) {
            const long long b = cus * c < items ? cus * c : items;
            if (c > kRowsBlocksPerCu && (items + b - 1) / b < 2) break;
            const long long load = ((3 * b + simd_count() - 1) / simd_count()) * ((items + b - 1) / b + 1);
            if (best < 0 || load <= best) best = load, per_cu = c;
        }
    }
    long long blocks = cus * per_cu;
    if (blocks > items) blocks = items;
    a.items_per_wave = (int)(items / blocks);
    a.items_extra = (int)(items % blocks);
    a.div_groups = FastDiv((uint32_t)a.n_groups);
    hipLaunchKernelGGL((bconv3x3_rows_kernel<CW, MODE>), dim3((unsigned)blocks), dim3(RowSplit<CW>::threads), 0, stream, a);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

// 56 x 56 x 64 -> 64 with Affine, Add and sign bits inside Bi-Real-18: batch 128 (24 tiles per CU) level with the unit
// kernel, batch 64 behind it, batch 256 (49): 87-91 us a launch against 87-100, the net 1.619 against 1.631 ms
constexpr int kTile64MinTilesPerCu = 32;

// 64 input channels with an epilogue at large batch (the first stage of a residual net): the launch is bound by the
// fp32 shortcut it reads and the fp32 result it writes, and the unit kernel's waves, each storing 8 KB windows of a
// tile of its own, move them at 4.7-5.3 TB/s where a copy whose blocks take contiguous 16 KB chunks in turn reaches
// 6.0.  Here a block's four waves share a tile of 64 pixels x 64 output channels: every wave counts 16 channels for
// all 64 pixels (the tile's activations are 144 bytes per lane, fetched by each wave), the counts meet in LDS, and the
// block reads the tile's shortcut, applies the epilogue and writes the result as one contiguous piece (256 bytes per
// pixel; with more than 64 output channels a pixel's 64-channel part), 16 lanes to a pixel, so the sign bits of a
// pixel are one row of lanes.  Tiles are dealt to the resident blocks in turn.
constexpr int kTileRow = 64 * 4 + 16;  // bytes per pixel row of the staged tile: 16-byte writes of 16 lanes hit 64 banks once
template <int MODE>
__global__ __launch_bounds__(256, 6) void bconv3x3_tile64_kernel(const BconvArgs p) {
    static_assert(MODE == kModeAffineAdd || MODE == kModeAffineAddSign, "the tile kernel is for launches with an epilogue");
    constexpr int K32 = 18, Q = 8;
    __shared__ __attribute__((aligned(16))) unsigned char tile_lds[64 * kTileRow];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wib = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int column_tiles = p.cout >> 6;
    const int tiles = (p.total + 63) >> 6;
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(p.x, p.x_bytes);
    const int c4 = tid & 15;  // the thread's four channels of a pixel in the store pass

    uint32_t a[K32];
    auto fetch_tile = [&](int tile) {
        {
            int pix = tile * 64 + lane;
            pix = pix < p.total ? pix : p.total - 1;
            const uint32_t t = p.div_ow.div(pix);
            const int ox = pix - t * p.OW;
            const uint32_t n = p.div_oh.div(t);
            const int oy = t - n * p.OH;
            const int y0 = oy * p.stride - p.pad, x0 = ox * p.stride - p.pad;
            const int base = ((n * p.H + y0) * p.W + x0) * 8;  // byte offset of tap (0,0); may be negative
#pragma unroll
            for (int kh = 0; kh < 3; ++kh) {
                const bool row_ok = (unsigned)(y0 + kh) < (unsigned)p.H;
#pragma unroll
                for (int kw = 0; kw < 3; ++kw) {
                    const bool ok = row_ok && (unsigned)(x0 + kw) < (unsigned)p.W;
                    // an offset beyond the descriptor's range reads as zero: the reference's padding word
                    const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, ok ? base + (kh * p.W + kw) * 8 : (int)0x80000000, 0, 0);
                    a[(kh * 3 + kw) * 2] = v.x, a[(kh * 3 + kw) * 2 + 1] = v.y;
                }
            }
        }
    };
    if ((int)blockIdx.x < tiles) fetch_tile((int)blockIdx.x);
    for (int tile = (int)blockIdx.x; tile < tiles; tile += (int)gridDim.x) {
        for (int ct = 0; ct < column_tiles; ++ct) {
            // the store pass's shortcut values, asked for before the counting so that they arrive behind it:
            // thread t has pixels t / 16 + 16 * j, j = 0..3, channels 4 * (t % 16) ..
            const int pixel0 = tid >> 4;
            const size_t out_off = ((size_t)tile * 64 + pixel0) * p.cout + ct * 64 + c4 * 4;
            const size_t step = (size_t)16 * p.cout;  // 16 pixels on
            float4 sc[4];
            const bool with_shortcut = p.epi_shortcut != nullptr;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bool ok = with_shortcut && tile * 64 + pixel0 + 16 * j < p.total;
                sc[j] = ok ? *reinterpret_cast<const float4 *>(p.epi_shortcut + out_off + j * step) : make_float4(0.f, 0.f, 0.f, 0.f);
            }
            EpiAffineAdd epi;
            epi.a = p.epi_a, epi.b = p.epi_b, epi.shortcut = p.epi_shortcut;
            epi.prepare(ct * 64 + c4 * 4);

            // the wave's 16 channels of the lane's pixel, eight at a time (unrolled, the two units' registers keep the
            // kernel from six waves per SIMD)
#pragma unroll 1
            for (int u = 0; u < 2; ++u) {
                uint32_t acc[Q];
                const int cg = ct * 8 + wib * 2 + u;  // group of eight output channels
                unit_rowmajor<K32, Q>(p.w + (size_t)cg * Q * 9, a, acc);
                float f[Q];
#pragma unroll
                for (int q = 0; q < Q; ++q) f[q] = __uint_as_float(acc[q]) - kAccBias;
                unsigned char *row = tile_lds + lane * kTileRow + (wib * 16 + u * 8) * 4;
                *reinterpret_cast<float4 *>(row) = make_float4(f[0], f[1], f[2], f[3]);
                *reinterpret_cast<float4 *>(row + 16) = make_float4(f[4], f[5], f[6], f[7]);
            }
            // the tile's activations are dead: the next tile's come while this one is written
            if (ct == column_tiles - 1 && tile + (int)gridDim.x < tiles) fetch_tile(tile + (int)gridDim.x);
            __syncthreads();
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int pixel = pixel0 + 16 * j;
                const float4 v = *reinterpret_cast<const float4 *>(tile_lds + pixel * kTileRow + c4 * 16);
                const float4 r = with_shortcut ? epi.template apply<true>(v, sc[j]) : epi.template apply<false>(v, sc[j]);
                const bool ok = tile * 64 + pixel < p.total;
                if (ok) {
                    typedef float f32x4 __attribute__((ext_vector_type(4)));
                    __builtin_nontemporal_store(f32x4{r.x, r.y, r.z, r.w}, reinterpret_cast<f32x4 *>(p.out + out_off + j * step));
                }
                if constexpr (MODE == kModeAffineAddSign) {
                    // the 16 lanes of a pixel are one row of lanes
                    const uint32_t nib = sign_nibble(r);
                    uint32_t lo = c4 < 8 ? nib << (4 * c4) : 0u, hi = c4 >= 8 ? nib << (4 * (c4 - 8)) : 0u;
                    lo = or_from_lane_above<1>(lo), hi = or_from_lane_above<1>(hi);
                    lo = or_from_lane_above<2>(lo), hi = or_from_lane_above<2>(hi);
                    lo = or_from_lane_above<4>(lo), hi = or_from_lane_above<4>(hi);
                    lo = or_from_lane_above<8>(lo), hi = or_from_lane_above<8>(hi);
                    if (ok && c4 == 0)
                        *reinterpret_cast<uint64_t *>(p.epi_bits + ((size_t)tile * 64 + pixel) * (p.cout >> 3) + ct * 8) = ((uint64_t)hi << 32) | lo;
                }
            }
            __syncthreads();  // the staged tile is dead
        }
    }
}

// Whether the tile kernel takes a launch: 64 input channels, an epilogue, whole 64-channel tiles of output, and enough
// tiles that every resident block gets several (below that the unit kernel's finer split of the work is ahead).
static bool takes_tile64(long long tiles, int cin, int cout, int mode) {
    return cin == 64 && cout % 64 == 0 && (mode == kModeAffineAdd || mode == kModeAffineAddSign) &&
           tiles >= kTile64MinTilesPerCu * (long long)(simd_count() / 4);
}

template <int MODE>
static int launch_tile64(BconvArgs &a, long long tiles, hipStream_t stream) {
    static const int blocks_per_cu = resident_blocks_per_cu(bconv3x3_tile64_kernel<MODE>, 256);
    const long long resident = (long long)(simd_count() / 4) * blocks_per_cu;
    hipLaunchKernelGGL((bconv3x3_tile64_kernel<MODE>), dim3((unsigned)(tiles < resident ? tiles : resident)), dim3(256), 0, stream, a);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

// Which kernel runs a problem of `tiles` 64-pixel tiles: 0 = the small-problem kernel (blocks split the depth),
// 1 = the unit kernel at its wide residency, 2 = its second build: four waves per SIMD and whole-line stores for 64
// and 128 input channels, units of twice the channels for 256 and 512; 3 = the row-split kernel (raw counts only).
constexpr int kBuildSplitDepth = 0, kBuildWide = 1, kBuildNarrow = 2, kBuildRows = 3;

// The row-split kernel takes the raw counts of deep inputs whose activation fetch is what the other kernels wait for,
// from one tile up to 28 channel-tiles per SIMD with 512 input channels and with 256 at stride 2 (whose taps lie on
// twice as many cache lines), and up to 16 with 256 channels at stride 1.  Against the small-problem kernel (batch 1
// to 16) and the unit kernel: 7 x 7 x 512 -> 512: 3.9 against 4.6 us at batch 1, 6.8 against 7.6 at batch 16, 9.7
// against 11.4 at batch 32, 15.7 against 17.0 at batch 64, 19.2 against 18.6 at batch 80, 30.0 against 27.7 at batch
// 128; 14 x 14 x 256 -> 512 at stride 2: 3.1 against 3.8 us at batch 1, 4.7 against 6.1 at batch 16, 6.2 against 8.0 at
// batch 32, 9.3 against 10.1 at batch 64, 11.4 against 11.1 at batch 80; 14 x 14 x 256 -> 256: 3.1 against 3.8 us at
// batch 1, 6.0 against 7.0 at batch 16, 8.2 against 8.3 at batch 24, 11.4 against 9.9 at batch 40.  The entry points
// with an epilogue take it in a narrower window (below).
static bool takes_rows(long long tiles, int cin, int cout, int stride, int mode) {
    if (cout % 8 != 0 || !(cin == 512 || cin == 256)) return false;
    const bool deep = cin == 512 || stride >= 2;  // 512 input channels, or 256 at stride 2
    const long long work = tiles * cout, simds = simd_count();
    if (mode == kModeCounts) return work <= (deep ? 28 : 16) * simds;
    // With an epilogue the small-problem kernel stays ahead at small batches (its work items are whole bytes of sign
    // bits and its first wave has the shortcut in flight from the start) and the unit kernel from mid-sized ones on;
    // between them, measured at batches 1 to 64 of the three deep stage shapes: Affine + Add 7.8 against 8.2 us at
    // batch 16 and 18.3 against 19.1 at batch 64 (7x7 512->512), 6.8 against 8.5 at batch 16 (14x14 256->256); with
    // sign bits 14.3 against 19.9 us at batch 48 and 17.4 against 25.4 at batch 64 (7x7 512->512, where the unit
    // kernel's work items of four units are coarse), 8.8 against 10.6 at batch 24 (14x14 256->256), 7.8 against 9.8 at
    // batch 32 (14x14 256->512 at stride 2).
    // (without sign bits its work items are four channels, twice as many blocks as the small-problem kernel has: ahead
    // again on one or two tiles, 4.6 against 5.1 us for one image of 7x7 512->512)
    if (mode == kModeAffineAdd) return work <= simds || (work >= 6 * simds && work <= (deep ? 28 : 16) * simds);
    if (mode == kModeAffineAddSign) return cout % 64 == 0 && work >= (cin == 512 ? 8 : 6) * simds && work <= 28 * simds;
    return false;
}

static int pick_build(long long tiles, int cin, int cout, int stride = 1, int mode = kModeCounts) {
    if (takes_rows(tiles, cin, cout, stride, mode)) return kBuildRows;
    if (splits_depth(tiles, cin, cout)) return kBuildSplitDepth;
    const long long simds = simd_count();
    if (cin <= 128) {
        const long long units = tiles * (cout / 8);
        if (mode != kModeCounts) {
            // with an epilogue: four (eight) units or more per wave at four waves per SIMD
            if (units >= (cin == 64 ? 4ll : 8ll) * simds * 4) return kBuildNarrow;
        } else if (cin == 64) {
            // Raw counts, whose stores are written through and whose 64-byte runs then cost nothing extra: the
            // four-wave build is ahead only at stride 1 between 24 and 44 units per SIMD (56x56 64->64: 12.5 against
            // 11.4 us at batch 48, 14.7 against 15.1 at batch 64, 20.0 against 20.5 at batch 96; 27.9 against 26.5 at batch 128, 52.2 against 49.8
            // at batch 256; 56x56 64->128 at stride 2: 12.4 against 11.5 at batch 96, 27.8 against 26.1 at batch 256)
            if (stride == 1 && units >= 24 * simds && units < 44 * simds) return kBuildNarrow;
        } else {
            // 128 input channels: from 16 units per SIMD at stride 1 (28x28 128->128: 18.4 against 20.1 us at batch
            // 96, 22.9 against 24.2 at batch 128, level at batch 64), from 4 at stride 2 (28x28 128->256: 7.6
            // against 8.7 us at batch 48, 23.0 against 24.6 at batch 256)
            if (units >= (stride >= 2 ? 4 : 16) * simds) return kBuildNarrow;
        }
    } else {
        // large units: six or more per wave; raw counts with 512 input channels from three (7x7 512->512: 21.3 against
        // 21.9 us at batch 96, 26.4 against 27.8 at batch 128)
        const long long big_units = tiles * (cout / (cin == 256 ? 8 : 4));
        const long long per_wave = (mode == kModeCounts && cin == 512) ? 3 : 6;
        if (cout % 8 == 0 && big_units >= per_wave * simds * (cin == 256 ? 4 : 3)) return kBuildNarrow;
    }
    return kBuildWide;
}

template <int CW, int MODE>
static int launch_bconv3x3(BconvArgs &a, long long tiles, hipStream_t stream) {
    if constexpr (CW == 1 && (MODE == kModeAffineAdd || MODE == kModeAffineAddSign)) {
        if (takes_tile64(tiles, 64, a.cout, MODE)) return launch_tile64<MODE>(a, tiles, stream);
    }
    const int build = pick_build(tiles, CW * 64, a.cout, a.stride, MODE);
    if (build == kBuildSplitDepth) return launch_ksplit<CW, MODE>(a, tiles, stream);
    if constexpr (CW >= 4) {
        if (build == kBuildRows) return launch_rows<CW, MODE>(a, tiles, stream);
    }
    if (build == kBuildNarrow) return launch_variant<CW, MODE, true>(a, tiles, stream);
    return launch_variant<CW, MODE, false>(a, tiles, stream);
}

}  // namespace dab

static int bconv3x3_impl(const char *fn, const uint64_t *x, int n, int h, int w, int cin, const uint64_t *wgt, int cout,
                         int stride, int pad, const float *a_coef, const float *b_coef, const float *shortcut, int mode,
                         float *out, uint64_t *out_packed, dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(x && wgt && out, "%s: null pointer", fn);
    DAB_REQUIRE(n > 0 && h > 0 && w > 0 && cin > 0 && cout > 0, "%s: non-positive dimension", fn);
    DAB_REQUIRE(stride > 0 && pad >= 0, "%s: stride %d pad %d", fn, stride, pad);
    DAB_REQUIRE(cin % 64 == 0, "%s: cin %d is not a multiple of 64", fn, cin);
    DAB_REQUIRE(h + 2 * pad >= 3 && w + 2 * pad >= 3, "%s: input smaller than the kernel", fn);
    const bool two_halves = cin == 1024 && mode == kModeCounts;  // no fused epilogue for 1024 input channels
    if (!(cin == 64 || cin == 128 || cin == 256 || cin == 512 || two_halves) || cout % 8 != 0)
        return fail(DAB_EUNSUPPORTED, "%s: cin %d / cout %d not covered by the direct kernel", fn, cin, cout);
    DAB_REQUIRE((reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(wgt) & 7) == 0 &&
                    (reinterpret_cast<uintptr_t>(out) & 15) == 0,
                "%s: buffers must be 16-byte aligned", fn);
    const bool fused = mode != kModeCounts;
    if (mode == kModeAffineAddSign) {
        DAB_REQUIRE(out_packed, "%s: null pointer", fn);
        DAB_REQUIRE((reinterpret_cast<uintptr_t>(out_packed) & 7) == 0, "%s: buffers must be 16-byte aligned", fn);
        if (cout % 64 != 0) return fail(DAB_EUNSUPPORTED, "%s: cout %d is not a multiple of 64", fn, cout);
    }
    if (fused) {
        DAB_REQUIRE(a_coef && b_coef, "%s: null affine coefficients", fn);
        DAB_REQUIRE((reinterpret_cast<uintptr_t>(a_coef) & 15) == 0 && (reinterpret_cast<uintptr_t>(b_coef) & 15) == 0 &&
                        (reinterpret_cast<uintptr_t>(shortcut) & 15) == 0,
                    "%s: coefficient and shortcut buffers must be 16-byte aligned", fn);
    }

    BconvArgs a;
    a.x = x, a.w = wgt, a.out = out;
    a.epi_a = a_coef, a.epi_b = b_coef, a.epi_shortcut = shortcut;
    a.epi_bits = reinterpret_cast<unsigned char *>(out_packed);
    a.H = h, a.W = w;
    a.OH = out_dim(h, pad, 3, 1, stride), a.OW = out_dim(w, pad, 3, 1, stride);
    const long long total = (long long)n * a.OH * a.OW;
    const long long x_bytes = (long long)n * h * w * (cin / 64) * 8;
    if (total >= (1ll << 31) - 64 || x_bytes >= (1ll << 31) || total * cout >= (1ll << 40))
        return fail(DAB_EUNSUPPORTED, "%s: tensor too large for 32-bit pixel indexing", fn);
    a.total = (int)total;
    a.cout = cout, a.stride = stride, a.pad = pad;
    a.x_bytes = (uint32_t)x_bytes;
    a.div_ow = FastDiv((uint32_t)a.OW), a.div_oh = FastDiv((uint32_t)a.OH);
    const long long tiles = (total + 63) / 64;
    hipStream_t s = as_stream(stream);
    a.half = 0;
    a.through = 0;
    if (two_halves) {
        // the 512-channel unit kernel on words 0..7 of every pixel and tap, then on words 8..15 adding to the result
        // (the builds as for 512 channels; small problems take the unit kernel too)
        const bool big = pick_build(tiles, 512, cout) == kBuildNarrow;
        int rc = big ? launch_variant<8, kModeCounts, true, true>(a, tiles, s) : launch_variant<8, kModeCounts, false, true>(a, tiles, s);
        if (rc != DAB_OK) return rc;
        a.half = 1;
        return big ? launch_variant<8, kModeAccumulate, true, true>(a, tiles, s)
                   : launch_variant<8, kModeAccumulate, false, true>(a, tiles, s);
    }
    switch (mode * 16 + cin / 64) {
        case kModeCounts * 16 + 1: return launch_bconv3x3<1, kModeCounts>(a, tiles, s);
        case kModeCounts * 16 + 2: return launch_bconv3x3<2, kModeCounts>(a, tiles, s);
        case kModeCounts * 16 + 4: return launch_bconv3x3<4, kModeCounts>(a, tiles, s);
        case kModeCounts * 16 + 8: return launch_bconv3x3<8, kModeCounts>(a, tiles, s);
        case kModeAffineAdd * 16 + 1: return launch_bconv3x3<1, kModeAffineAdd>(a, tiles, s);
        case kModeAffineAdd * 16 + 2: return launch_bconv3x3<2, kModeAffineAdd>(a, tiles, s);
        case kModeAffineAdd * 16 + 4: return launch_bconv3x3<4, kModeAffineAdd>(a, tiles, s);
        case kModeAffineAdd * 16 + 8: return launch_bconv3x3<8, kModeAffineAdd>(a, tiles, s);
        case kModeAffineAddSign * 16 + 1: return launch_bconv3x3<1, kModeAffineAddSign>(a, tiles, s);
        case kModeAffineAddSign * 16 + 2: return launch_bconv3x3<2, kModeAffineAddSign>(a, tiles, s);
        case kModeAffineAddSign * 16 + 4: return launch_bconv3x3<4, kModeAffineAddSign>(a, tiles, s);
        case kModeAffineAddSign * 16 + 8: return launch_bconv3x3<8, kModeAffineAddSign>(a, tiles, s);
    }
    return fail(DAB_EINVAL, "%s: bad mode", fn);
}

extern "C" int dab_bconv3x3(const uint64_t *x, int n, int h, int w, int cin, const uint64_t *wgt, int cout, int stride,
                            int pad, float *out, dab_stream_t stream) {
    return bconv3x3_impl("dab_bconv3x3", x, n, h, w, cin, wgt, cout, stride, pad, nullptr, nullptr, nullptr, dab::kModeCounts,
                         out, nullptr, stream);
}

extern "C" int dab_bconv3x3_affine_add(const uint64_t *x, int n, int h, int w, int cin, const uint64_t *wgt, int cout,
                                       int stride, int pad, const float *a, const float *b, const float *shortcut,
                                       float *out, dab_stream_t stream) {
    return bconv3x3_impl("dab_bconv3x3_affine_add", x, n, h, w, cin, wgt, cout, stride, pad, a, b, shortcut,
                         dab::kModeAffineAdd, out, nullptr, stream);
}

extern "C" int dab_bconv3x3_affine_add_sign(const uint64_t *x, int n, int h, int w, int cin, const uint64_t *wgt, int cout,
                                            int stride, int pad, const float *a, const float *b, const float *shortcut,
                                            float *out, uint64_t *out_packed, dab_stream_t stream) {
    return bconv3x3_impl("dab_bconv3x3_affine_add_sign", x, n, h, w, cin, wgt, cout, stride, pad, a, b, shortcut,
                         dab::kModeAffineAddSign, out, out_packed, stream);
}

extern "C" int dab_bconv3x3_splits_depth(int64_t n_out_pixels, int cin, int cout) {
    if (n_out_pixels <= 0 || cout <= 0 || cout % 8 != 0 || !(cin == 64 || cin == 128 || cin == 256 || cin == 512)) return 0;
    return dab::splits_depth((n_out_pixels + 63) / 64, cin, cout) ? 1 : 0;
}

extern "C" int dab_bconv3x3_fused_shares_tiles(int64_t n_out_pixels, int cin, int cout) {
    if (n_out_pixels <= 0 || cout <= 0) return 0;
    return dab::takes_tile64((n_out_pixels + 63) / 64, cin, cout, dab::kModeAffineAdd) ? 1 : 0;
}

extern "C" int dab_bconv3x3_build(int64_t n_out_pixels, int cin, int cout) {
    if (n_out_pixels <= 0 || cout <= 0 || cout % 8 != 0 || !(cin == 64 || cin == 128 || cin == 256 || cin == 512)) return -1;
    // the builds of the entry points with an epilogue; dab_bconv3x3_counts_build answers for dab_bconv3x3 itself
    return dab::pick_build((n_out_pixels + 63) / 64, cin, cout, 1, dab::kModeAffineAdd);
}

extern "C" int dab_bconv3x3_epilogue_build(int64_t n_out_pixels, int cin, int cout, int stride, int with_sign) {
    if (n_out_pixels <= 0 || cout <= 0 || cout % 8 != 0 || stride <= 0 || !(cin == 64 || cin == 128 || cin == 256 || cin == 512)) return -1;
    if (with_sign && cout % 64 != 0) return -1;
    return dab::pick_build((n_out_pixels + 63) / 64, cin, cout, stride, with_sign ? dab::kModeAffineAddSign : dab::kModeAffineAdd);
}

extern "C" int dab_bconv3x3_counts_build(int64_t n_out_pixels, int cin, int cout, int stride) {
    if (n_out_pixels <= 0 || cout <= 0 || cout % 8 != 0 || stride <= 0 || !(cin == 64 || cin == 128 || cin == 256 || cin == 512)) return -1;
    return dab::pick_build((n_out_pixels + 63) / 64, cin, cout, stride, dab::kModeCounts);
}

