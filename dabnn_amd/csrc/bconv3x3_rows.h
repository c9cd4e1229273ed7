// Direct 3x3 binary convolution for 256 and 512 input channels, depth split by kernel row over the waves of a block.
//
// In the unit kernel (bconv3x3.hip) a lane holds all nine taps of its pixel, 72 or 144 VGPRs, which bounds the CU at
// four or three waves per SIMD, and every wave fetches them with 18 or 36 vector loads whose 64 lanes touch 32
// different cache lines each: at batch 64 that fetch is 0.5-2.8 us of a 10-17 us launch (measured by leaving loads
// out), with the vector ALUs waiting.  Here a block is three waves and wave r counts kernel row r only -- the three
// taps (r, 0..2), a third of the depth -- for ALL output channels of the block's segment: a third of the loads and of
// the activation registers per wave (48 VGPRs with 512 input channels: seven to eight waves per SIMD instead of
// three), and three times as many channels per fetched tap.  A channel's weights for one kernel row are contiguous
// (48 or 24 dwords) and reach v_xor_b32 as SGPR operands from scalar loads, as in the unit kernel: per 32 bits of
// depth and per output one v_xor_b32 and one v_bcnt_u32_b32.  The three partial counts of an output meet in LDS
// (ds_add_u32 on a plane of 64 pixels x 32 channels that starts at zero and that the store pass leaves at zero), and
// the block writes the plane out in 16-byte parts through the epilogue: whole 128-byte lines per pixel for a full
// segment.
//
// Work split: a block owns a contiguous range of output channels over the tiles of 64 pixels, cut at multiples of
// four channels (eight when sign bits are written), and walks it in segments of at most 32 channels of one tile.
// The three waves of a block always have the same amount of work.
#pragma once

#include "xnor_core.h"

namespace dab {

template <int CW>
struct RowSplit {
    static constexpr int row_dwords = 6 * CW;          // one channel's weights for one kernel row = a lane's activations
    static constexpr int vec = CW == 8 ? 16 : 24;      // dwords per scalar-load batch, one wait each
    static constexpr int pieces = row_dwords / vec;    // batches per channel: 3 or 1
    static constexpr int group = 4;                    // channels per pass of the accumulators
    static constexpr int segment = 32;                 // channels per store pass
    static constexpr int row = (segment + 4) * 4;      // bytes per pixel row of the plane (+16: conflict-free 16-byte reads)
    static constexpr int threads = 192;
};

// DW consecutive weight dwords as one or two scalar-load vectors, from p + off + OFF (off a wave-uniform byte offset
// in a register, OFF an immediate).
template <int DW>
struct WVec;
template <>
struct WVec<16> {
    u32x16 a;
    template <int OFF>
    __device__ __forceinline__ void load_off(const void *p, uint32_t off) {
        asm volatile("s_load_dwordx16 %0, %1, %2 offset:%3" : "=s"(a) : "s"(p), "s"(off), "n"(OFF));
    }
    // scalar loads return out of order: the only usable wait is "all of them"; tying the vector to the statement
    // keeps its consumers behind the wait
    __device__ __forceinline__ void wait() { asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(a)); }
    template <int I>
    __device__ __forceinline__ uint32_t get() const {
        return a[I];
    }
};
template <>
struct WVec<24> {
    u32x16 a;
    u32x8 b;
    template <int OFF>
    __device__ __forceinline__ void load_off(const void *p, uint32_t off) {
        asm volatile("s_load_dwordx16 %0, %1, %2 offset:%3" : "=s"(a) : "s"(p), "s"(off), "n"(OFF));
        asm volatile("s_load_dwordx8 %0, %1, %2 offset:%3" : "=s"(b) : "s"(p), "s"(off), "n"(OFF + 64));
    }
    __device__ __forceinline__ void wait() { asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(a), "+s"(b)); }
    template <int I>
    __device__ __forceinline__ uint32_t get() const {
        if constexpr (I < 16)
            return a[I];
        else
            return b[I - 16];
    }
};

// acc (+)= popcount(w ^ a) over DW dwords; FIRST: the accumulator is written, starting from zero.
template <int DW, bool FIRST>
__device__ __forceinline__ void rows_count(uint32_t &acc, const WVec<DW> &w, const uint32_t *a) {
    const uint32_t zero = 0;
    static_for<DW / 2>([&](auto e_) {
        constexpr int e = e_;
        if constexpr (FIRST && e == 0)
            xp2_first(acc, zero, w.template get<0>(), w.template get<1>(), a[0], a[1]);
        else
            xp2(acc, w.template get<2 * e>(), w.template get<2 * e + 1>(), a[2 * e], a[2 * e + 1]);
    });
}

// The store pass of a block: the plane's channels [0, seg) of a tile of 64 pixels go to out[pixel][cbase + ...]
// through the epilogue, and the plane is left at zero.  seg is a multiple of 4 (of 8 when sign bits are written).
// sc_pre: the shortcut values of the whole-segment pass, fetched by the caller before it counted.
template <int SEG, int ROW, int THREADS, class Epi>
__device__ __forceinline__ void rows_flush(unsigned char *plane, int tid, float *__restrict__ out, int ld, int tile, int total,
                                           int cbase, int seg, Epi epi, const float4 (&sc_pre)[3], bool pre_ok) {
    constexpr int NP = SEG / 4;  // 16-byte parts per pixel row of a whole segment
    static_assert(NP == 8 && THREADS % NP == 0, "eight lanes to a pixel");
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    // per-thread offsets of the pass are loop invariants of the caller: derived from an index the compiler cannot see
    // through they are made here and do not live across the counting
    asm volatile("" : "+v"(tid));
    const bool has_sc = Epi::kShortcut && epi.shortcut != nullptr;
    const u32x4 zero4 = {0u, 0u, 0u, 0u};
    auto to_float = [](u32x4 c) { return make_float4((float)c.x, (float)c.y, (float)c.z, (float)c.w); };
    if (seg == SEG && (tile + 1) * 64 <= total) {
        const int part = tid & (NP - 1);
        epi.prepare(cbase + part * 4);
        auto round = [&](int j, const float4 &sc_j) {
            const int pr = tid / NP + j * (THREADS / NP);  // 24 pixels per round: 24, 24, 16
            uint32_t w = 0;
            if (pr < 64) {
                u32x4 *src = reinterpret_cast<u32x4 *>(plane + pr * ROW + part * 16);
                const float4 v = to_float(*src);
                *src = zero4;
                const size_t off = ((size_t)tile * 64 + pr) * ld + cbase + part * 4;
                float4 r;
                if (has_sc) {
                    const float4 sc = pre_ok ? sc_j
                                             : *reinterpret_cast<const float4 *>((Epi::kReadsOut ? const_cast<const float *>(out) : epi.shortcut) + off);
                    r = epi.template apply<Epi::kShortcut>(v, sc);
                } else {
                    r = epi.template apply<false>(v, make_float4(0.f, 0.f, 0.f, 0.f));
                }
                // streaming store: the output is not read again by this kernel
                __builtin_nontemporal_store(f32x4{r.x, r.y, r.z, r.w}, reinterpret_cast<f32x4 *>(out + off));
                if constexpr (Epi::kEmit) w = sign_nibble(r) << (4 * part);
            }
            if constexpr (Epi::kEmit) {
                // the eight lanes of a pixel hold its segment's sign bits, four each: gather them in the first lane
                w = or_from_lane_above<1>(w);
                w = or_from_lane_above<2>(w);
                w = or_from_lane_above<4>(w);
                if (pr < 64 && part == 0)
                    *reinterpret_cast<uint32_t *>(epi.bits + ((size_t)tile * 64 + pr) * epi.bits_ld + (cbase >> 3)) = w;
            }
        };
        if constexpr (Epi::kShortcut) {
            round(0, sc_pre[0]);
            round(1, sc_pre[1]);
            round(2, sc_pre[2]);
        } else {
            // rolled: the rounds' temporaries would otherwise all live beside the activation registers
            const float4 none = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll 1
            for (int j = 0; j < 3; ++j) round(j, none);
        }
    } else {
        const int np = seg >> 2;                  // 16-byte parts per pixel row
        const int magic = (65536 + np - 1) / np;  // c / np for c < 512
        const int rounds = (64 * np + THREADS - 1) / THREADS;
        // every thread makes the same number of rounds (the sign bytes are gathered across lanes)
        for (int i = 0; i < rounds; ++i) {
            const int c = tid + i * THREADS;
            const int pr = (c * magic) >> 16;
            const int part = c - pr * np;
            const int pix = tile * 64 + pr;
            const bool in_plane = c < 64 * np;
            uint32_t nib = 0;
            if (in_plane) {
                u32x4 *src = reinterpret_cast<u32x4 *>(plane + pr * ROW + part * 16);
                const float4 v = to_float(*src);
                *src = zero4;
                if (pix < total) {
                    const size_t off = (size_t)pix * ld + cbase + part * 4;
                    epi.prepare(cbase + part * 4);
                    float4 r;
                    if (has_sc)
                        r = epi.template apply<Epi::kShortcut>(
                            v, *reinterpret_cast<const float4 *>((Epi::kReadsOut ? const_cast<const float *>(out) : epi.shortcut) + off));
                    else
                        r = epi.template apply<false>(v, make_float4(0.f, 0.f, 0.f, 0.f));
                    // Written through the L2 at device scope.  A block's share is 16 or 20 channels, so this is the
                    // path nearly all of the kernel's output takes, in pieces of a line; as ordinary or streaming
                    // stores the pieces wait in the L2 for the rest of their line, which another block writes at
                    // another time.  14x14 256->512 at stride 2: 6.1 against 7.9 us at batch 32, 9.15 against 9.7 at
                    // batch 64; 7x7 512->512 at batch 64: 15.7 against 16.6.
                    store_through(reinterpret_cast<f32x4 *>(out + off), f32x4{r.x, r.y, r.z, r.w});
                    if constexpr (Epi::kEmit) nib = sign_nibble(r);
                }
            }
            if constexpr (Epi::kEmit) {
                // np is even here and so are THREADS and 64 * np: the two halves of a byte sit in lanes 2k and 2k+1
                uint32_t w = nib << (4 * (part & 1));
                w = or_from_lane_above<1>(w);
                if (in_plane && pix < total && !(part & 1)) epi.bits[(size_t)pix * epi.bits_ld + ((cbase + part * 4) >> 3)] = (unsigned char)w;
            }
        }
    }
}

}  // namespace dab
