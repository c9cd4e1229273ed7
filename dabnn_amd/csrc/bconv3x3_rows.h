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
// the block writes the plane out in 16-byte parts through the epilogue.
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
// through the epilogue, in 16-byte parts (four channels), and the plane is left at zero.  seg is a multiple of 4 (of 8
// when sign bits are written).  A block's share is at most 24 channels wherever the launcher takes this kernel (at most
// 28 channel-tiles per SIMD over six blocks per CU), so the parts of a pixel are a piece of a line whose rest another
// block writes at another time: they are written through the L2 at device scope.  As ordinary or streaming stores
// the pieces wait in the L2 for the rest of their line; 14x14 256->512 at stride 2: 6.1 against 7.9 us at batch 32,
// 9.15 against 9.7 at batch 64; 7x7 512->512 at batch 64: 15.7 against 16.6.
template <int SEG, int ROW, int THREADS, class Epi>
__device__ __forceinline__ void rows_flush(unsigned char *plane, int tid, float *__restrict__ out, int ld, int tile, int total,
                                           int cbase, int seg, Epi epi) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    // per-thread offsets of the pass are loop invariants of the caller: derived from an index the compiler cannot see
    // through they are made here and do not live across the counting
    asm volatile("" : "+v"(tid));
    const bool has_sc = Epi::kShortcut && epi.shortcut != nullptr;
    const u32x4 zero4 = {0u, 0u, 0u, 0u};
    auto to_float = [](u32x4 c) { return make_float4((float)c.x, (float)c.y, (float)c.z, (float)c.w); };
    const int np = seg >> 2;                  // 16-byte parts per pixel row
    const int magic = (65536 + np - 1) / np;  // c / np for c < 512
    const int rounds = (64 * np + THREADS - 1) / THREADS;
    static_assert(SEG <= 32, "64 * SEG / 4 part indices stay below 512");
    // every thread makes the same number of rounds (the sign bytes are gathered across lanes)
    for (int i = 0; i < rounds; ++i) {
        const int c = tid + i * THREADS;
        const bool in_plane = c < 64 * np;
        const int pr = in_plane ? (c * magic) >> 16 : 0;
        const int part = in_plane ? c - pr * np : 0;
        const int pix = tile * 64 + pr;
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

}  // namespace dab
