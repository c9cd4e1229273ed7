// Device building blocks of the xor/popcount kernels (bconv3x3 and bgemm).
//
// Work decomposition shared by both kernels
// -----------------------------------------
// A "unit" is 64 output pixels (one per lane of a wave) times Q output
// channels (Q = 8, 4 or 2).  A lane keeps the packed activations of its pixel in VGPRs for as
// long as the wave stays on the same 64-pixel tile; the weights of the Q
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

// N dwords (4, 8 or 16) of weights through the scalar cache.
template <int N>
struct SVec;
template <>
struct SVec<4> {
    typedef u32x4 type;
};
template <>
struct SVec<8> {
    typedef u32x8 type;
};
template <>
struct SVec<16> {
    typedef u32x16 type;
};

// Immediate byte offset.
template <int N, int OFF>
__device__ __forceinline__ void sload(typename SVec<N>::type &v, const void *p) {
    if constexpr (N == 16) asm volatile("s_load_dwordx16 %0, %1, %2" : "=s"(v) : "s"(p), "n"(OFF));
    if constexpr (N == 8) asm volatile("s_load_dwordx8 %0, %1, %2" : "=s"(v) : "s"(p), "n"(OFF));
    if constexpr (N == 4) asm volatile("s_load_dwordx4 %0, %1, %2" : "=s"(v) : "s"(p), "n"(OFF));
}
// Wave-uniform register byte offset.
template <int N>
__device__ __forceinline__ void sload_off(typename SVec<N>::type &v, const void *p, uint32_t off) {
    if constexpr (N == 16) asm volatile("s_load_dwordx16 %0, %1, %2" : "=s"(v) : "s"(p), "s"(off));
    if constexpr (N == 8) asm volatile("s_load_dwordx8 %0, %1, %2" : "=s"(v) : "s"(p), "s"(off));
    if constexpr (N == 4) asm volatile("s_load_dwordx4 %0, %1, %2" : "=s"(v) : "s"(p), "s"(off));
}
// Scalar loads return out of order: the only usable wait is "all of them".
// Tying the vector to the statement keeps its consumers behind the wait.
template <class V>
__device__ __forceinline__ void swait(V &v) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(v));
}

// acc += popcount(w0 ^ a0) + popcount(w1 ^ a1), weights in SGPRs.
// Every instruction is an asm statement of its own and the two kinds alternate strictly.  Measured on the unit body
// (cycles per xor/bcnt pair and SIMD, 8 / 4 waves per SIMD): xor, bcnt, xor, bcnt as separate statements 7.0 / 7.3;
// the same four in one statement 7.35 / 7.7 (the compiler then puts its wait state for a possible DPP read behind
// the group instead of between an xor and the bcnt that needs its result); xor, xor, bcnt, bcnt 7.3 / 7.7.  With all
// operands in registers and no scalar loads in the loop the alternating order issues in 6.4 cycles per pair, the sum
// of the two issue times (v_xor_b32 2.3, v_bcnt_u32_b32 4.1), and 7.6 when instructions of a kind follow each other.
// GROUPED: xor xor bcnt bcnt in one statement -- only where it measured faster, the binary GEMM with 72 resident
// words per lane at three waves per SIMD (17.35 against 18.1 us for m512 k72 n3136).
template <bool GROUPED = false>
__device__ __forceinline__ void xp2(uint32_t &acc, uint32_t w0, uint32_t w1, uint32_t a0, uint32_t a1) {
    uint32_t t0, t1;
    if constexpr (GROUPED) {
        asm volatile(
            "v_xor_b32 %1, %3, %5\n\t"
            "v_xor_b32 %2, %4, %6\n\t"
            "v_bcnt_u32_b32 %0, %1, %0\n\t"
            "v_bcnt_u32_b32 %0, %2, %0"
            : "+v"(acc), "=&v"(t0), "=&v"(t1)
            : "s"(w0), "s"(w1), "v"(a0), "v"(a1));
        return;
    }
    asm volatile("v_xor_b32 %0, %1, %2" : "=v"(t0) : "s"(w0), "v"(a0));
    asm volatile("v_bcnt_u32_b32 %0, %1, %0" : "+v"(acc) : "v"(t0));
    asm volatile("v_xor_b32 %0, %1, %2" : "=v"(t1) : "s"(w1), "v"(a1));
    asm volatile("v_bcnt_u32_b32 %0, %1, %0" : "+v"(acc) : "v"(t1));
}

// The same for the first dword pair of a channel: acc = init + popcount(..) + popcount(..), init in an SGPR, so the
// accumulator needs no separate initialisation.
__device__ __forceinline__ void xp2_first(uint32_t &acc, uint32_t init, uint32_t w0, uint32_t w1, uint32_t a0, uint32_t a1) {
    uint32_t t0, t1;
    asm volatile("v_xor_b32 %0, %1, %2" : "=v"(t0) : "s"(w0), "v"(a0));
    asm volatile("v_bcnt_u32_b32 %0, %1, %2" : "=v"(acc) : "v"(t0), "s"(init));
    asm volatile("v_xor_b32 %0, %1, %2" : "=v"(t1) : "s"(w1), "v"(a1));
    asm volatile("v_bcnt_u32_b32 %0, %1, %0" : "+v"(acc) : "v"(t1));
}

// Accumulators start at the bit pattern of 2^23: adding an integer count
// c < 2^23 to that pattern yields the float 2^23 + c exactly, so one
// subtraction replaces the integer-to-float conversion.
constexpr uint32_t kAccInit = 0x4B000000u;
constexpr float kAccBias = 8388608.0f;
constexpr int kMaxCount = (1 << 23) - 1;

// ---------------------------------------------------------------- unit bodies
// A unit is 64 pixels x Q channels, Q in {8, 4, 2}.  Small Q keeps the unit
// short when the channel count is large: the tail of a launch is one unit
// executed by a lone wave, and a lone wave issues one VALU instruction per
// ~6 cycles, so a unit should stay near 600 instructions.

// Q channels whose K32 weight dwords each lie contiguously ([channel][K32],
// the reference's weight layout): Q*K32 dwords read as vectors of 16 (or 8).
// BV = vectors per wait.  A wait can only be "all outstanding scalar loads",
// so the latency cover of a batch is the vector work of the previous one: one
// vector (32 vector instructions, times the other waves of the SIMD) covers a
// scalar-cache miss that hits the L2; two ride out a miss to memory, at the
// price of 32 more SGPRs.
// acc is an output: acc[q] = 2^23 pattern + mismatch count of channel q.
// (Tried and dropped: loading the first batch of a wave's next unit behind the last batch of the current one, so
// that no unit starts with a wait.  7.07 -> 6.88 cycles per pair for the bare unit body at four waves per SIMD, but
// in the kernel the 16-32 SGPRs that then live across the store pass cost more than the wait: 97.9 against 95.7 us
// for the seven batch-64 shapes.)
// VEC_BYTES: distance between consecutive vectors in memory when they are not contiguous (one half of a filter row
// that is twice as deep: every other 64 bytes); 0 = contiguous.
template <int K32, int Q, int BV_WANTED = 1, bool GROUPED = false, int VEC_BYTES = 0>
__device__ __forceinline__ void unit_rowmajor(const void *wbase, const uint32_t (&a)[K32], uint32_t (&acc)[Q]) {
    constexpr int D = Q * K32;
    constexpr int VW = D % 16 == 0 ? 16 : 8;
    constexpr int VB = VEC_BYTES ? VEC_BYTES : VW * 4;
    constexpr int NV = D / VW;
    constexpr int BV = (NV % BV_WANTED == 0) ? BV_WANTED : 1;
    constexpr int NB = NV / BV;
    static_assert(K32 % 2 == 0 && D % VW == 0, "a dword pair never straddles two channels");
    typename SVec<VW>::type buf[2][BV];
    const uint32_t acc_init = kAccInit;  // the accumulators are written, not updated, by each channel's first pair
    static_for<BV>([&](auto b_) { sload<VW, b_ * VB>(buf[0][b_], wbase); });
    static_for<BV>([&](auto b_) { swait(buf[0][b_]); });
    static_for<NB>([&](auto j_) {
        constexpr int j = j_;
        if constexpr (j + 1 < NB)
            static_for<BV>([&](auto b_) { sload<VW, ((j + 1) * BV + b_) * VB>(buf[(j + 1) & 1][b_], wbase); });
        static_for<BV>([&](auto b_) {
            static_for<VW / 2>([&](auto e_) {
                constexpr int d = (j * BV + b_) * VW + e_ * 2;  // dword index within the Q-channel block
                constexpr int q = d / K32, k = d % K32;
                if constexpr (k == 0)
                    xp2_first(acc[q], acc_init, buf[j & 1][b_][e_ * 2], buf[j & 1][b_][e_ * 2 + 1], a[k], a[k + 1]);
                else
                    xp2<GROUPED>(acc[q], buf[j & 1][b_][e_ * 2], buf[j & 1][b_][e_ * 2 + 1], a[k], a[k + 1]);
            });
        });
        if constexpr (j + 1 < NB) static_for<BV>([&](auto b_) { swait(buf[(j + 1) & 1][b_]); });
    });
}

// Q channels stored channel-minor ([k word][channel], bgemm's column-major A):
// one scalar load holds word h of channels 0..Q-1; consecutive words are
// `stride` bytes apart.  Loads are issued in batches of B = 8/Q words (16
// dwords per batch, like unit_rowmajor) so that each wait is covered by 32
// vector instructions.
template <int K64, int Q>
__device__ __forceinline__ void unit_colmajor(const void *wbase, uint32_t stride, const uint32_t *a, uint32_t (&acc)[Q]) {
    constexpr int VW = 2 * Q;
    constexpr int B = (K64 % (8 / Q) == 0) ? 8 / Q : 1;
    constexpr int NB = K64 / B;
    typename SVec<VW>::type buf[2][B];
    uint32_t off = 0;
    static_for<B>([&](auto b_) {
        sload_off<VW>(buf[0][b_], wbase, off);
        off += stride;
    });
    static_for<B>([&](auto b_) { swait(buf[0][b_]); });
    static_for<NB>([&](auto j_) {
        constexpr int j = j_;
        if constexpr (j + 1 < NB) {
            static_for<B>([&](auto b_) {
                sload_off<VW>(buf[(j + 1) & 1][b_], wbase, off);
                off += stride;
            });
        }
        static_for<B>([&](auto b_) {
            constexpr int h = j * B + b_;
            static_for<Q>([&](auto q_) {
                xp2(acc[q_], buf[j & 1][b_][q_ * 2], buf[j & 1][b_][q_ * 2 + 1], a[2 * h], a[2 * h + 1]);
            });
        });
        if constexpr (j + 1 < NB) static_for<B>([&](auto b_) { swait(buf[(j + 1) & 1][b_]); });
    });
}

// ---------------------------------------------------------------- output staging
// A wave parks a window of WCH channels (32 or 16) of its 64 pixels in LDS, one
// row per pixel, and writes them out transposed: WCH/4 consecutive lanes cover
// the WCH*4 contiguous bytes of one pixel, so every store instruction writes
// whole or half cache lines instead of 64 scattered 16-byte pieces.  The narrow
// window halves the LDS a wave holds, which is what bounds the resident waves
// of the kernels with few activation registers.
template <int WCH>
struct Stage {
    static constexpr int row = WCH * 4 + 16;  // + 16 B pad: conflict-free 16-byte writes of one lane per row
    static constexpr int bytes = 64 * row;    // per wave
    static constexpr int parts = WCH / 4;     // 16-byte parts per pixel row
};

// Parks the Q results of a lane at channel offset ch_off (multiple of Q) of its row.
template <int WCH, int Q>
__device__ __forceinline__ void stage_put(unsigned char *stage, int lane, int ch_off, const uint32_t (&acc)[Q]) {
    float f[Q];
#pragma unroll
    for (int q = 0; q < Q; ++q) f[q] = __uint_as_float(acc[q]) - kAccBias;
    unsigned char *row = stage + lane * Stage<WCH>::row + ch_off * 4;
    if constexpr (Q == 2) {
        *reinterpret_cast<float2 *>(row) = make_float2(f[0], f[1]);
    } else {
#pragma unroll
        for (int q = 0; q < Q; q += 4) *reinterpret_cast<float4 *>(row + q * 4) = make_float4(f[q], f[q + 1], f[q + 2], f[q + 3]);
    }
}

// What happens to four consecutive channels of one pixel on their way out.
//   EpiStore          out = cnt                                  (the reference's BinConv output)
//   EpiAffineAdd      out = a[ch]*cnt + b[ch] (+ shortcut)       (BinConv -> Affine -> Add of a residual block in one
//                     pass; multiply, add and add are rounded separately, exactly like the three layers)
//   EpiAffineAddSign  the same, and bit (out > 0) of every result goes to a packed copy of the output, the words the
//                     next binary convolution would otherwise make by reading the fp32 blob again
//                     (pack_mat, dabnn/bitpack.h:277-293)
struct EpiStore {
    static constexpr bool kEmit = false;
    static constexpr bool kReadsOut = false;
    static constexpr bool kShortcut = false;  // the epilogue never reads a second tensor
    static constexpr bool kPolicy = true;     // the launch chooses how the stores go through the L2
    const float *shortcut = nullptr;
    int through = 0;  // write-through stores (see stage_flush_window)
    __device__ __forceinline__ void prepare(int) {}
    template <bool SC>
    __device__ __forceinline__ float4 apply(float4 v, float4) const {
        return v;
    }
};
struct EpiAffineAdd {
    static constexpr bool kPolicy = false;
    static constexpr bool kEmit = false;
    static constexpr bool kReadsOut = false;  // the shortcut is a tensor of its own
    static constexpr bool kShortcut = true;
    const float *a;
    const float *b;
    const float *shortcut;  // may be null; same layout as out
    float4 av, bv;
    __device__ __forceinline__ void prepare(int ch) {
        av = *reinterpret_cast<const float4 *>(a + ch);
        bv = *reinterpret_cast<const float4 *>(b + ch);
    }
    template <bool SC>
    __device__ __forceinline__ float4 apply(float4 v, float4 sc) const {
#pragma clang fp contract(off)
        float4 r;
        r.x = av.x * v.x, r.y = av.y * v.y, r.z = av.z * v.z, r.w = av.w * v.w;
        r.x = r.x + bv.x, r.y = r.y + bv.y, r.z = r.z + bv.z, r.w = r.w + bv.w;
        if constexpr (SC) r.x = r.x + sc.x, r.y = r.y + sc.y, r.z = r.z + sc.z, r.w = r.w + sc.w;
        return r;
    }
};
// out = cnt + what out holds: the second half of a convolution whose depth is counted in two passes (counts are
// integers far below 2^24, their float sum is exact)
struct EpiAccumulate {
    static constexpr bool kPolicy = false;
    static constexpr bool kEmit = false;
    static constexpr bool kReadsOut = true;  // the second operand is what `out` holds: read through `out` itself
    static constexpr bool kShortcut = true;
    const float *shortcut;  // non-null marker only; the store pass reads through its own `out` pointer
    __device__ __forceinline__ void prepare(int) {}
    template <bool SC>
    __device__ __forceinline__ float4 apply(float4 v, float4 sc) const {
        if constexpr (SC) v.x = v.x + sc.x, v.y = v.y + sc.y, v.z = v.z + sc.z, v.w = v.w + sc.w;
        return v;
    }
};
struct EpiAffineAddSign : EpiAffineAdd {
    static constexpr bool kEmit = true;
    unsigned char *bits;  // packed output, [pixel][bits_ld] bytes, bit c%8 of byte c/8 = (out[pixel][c] > 0)
    int bits_ld;          // cout / 8
};

// The whole-window store pass of stage_flush: lane = (pixel row pr0, 16-byte part), NP store instructions of
// 64/NP pixels each.  The shortcut values of G stores are fetched together before the first of them is used, so a
// flush waits for memory NP/G times and not once per store (the loads of one store cannot move above the previous
// store by themselves: the compiler has to assume the two tensors overlap).
//
// THROUGH: the stores are write-through at device scope (sc1) instead of streaming (nt).  A kernel's end waits until
// every dirty line it left in the L2s is written back, and the halves of a line that two store instructions fill
// (64-byte runs of a 16-channel window) or two waves (the pieces at the ends of their ranges) wait there for each
// other; part of them is written back twice (the write counter read 9-17 % above the output).  Written through,
// every piece leaves the L2 once, as it arrives: the counter reads the output size, a launch ends 0.3-1.6 us earlier
// at batch 64 and the next one starts on an L2 with nothing left to write.  Small outputs stay in the L2s either
// way and are 0.2-0.6 us faster with the streaming stores, so the launcher asks for this above a size.
template <int WCH, int G, bool SC, bool THROUGH, class Epi>
__device__ __forceinline__ void stage_flush_window(const unsigned char *stage, int lane, float *__restrict__ out, int ld,
                                                   int tile, int cbase, Epi &epi) {
    constexpr int NP = Stage<WCH>::parts, ROW = Stage<WCH>::row, PPI = 64 / NP;  // PPI pixels per store instruction
    static_assert(NP % G == 0, "group size must divide the number of stores");
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const int pr0 = lane / NP, part = lane % NP;
    const unsigned char *src = stage + pr0 * ROW + part * 16;
    const size_t off0 = ((size_t)tile * 64 + pr0) * ld + cbase + part * 4;
    epi.prepare(cbase + part * 4);
#pragma unroll
    for (int i0 = 0; i0 < NP; i0 += G) {
        float4 sc[G];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            if constexpr (SC && Epi::kReadsOut)
                sc[g] = *reinterpret_cast<const float4 *>(out + off0 + (size_t)(i0 + g) * PPI * ld);
            else if constexpr (SC)
                sc[g] = *reinterpret_cast<const float4 *>(epi.shortcut + off0 + (size_t)(i0 + g) * PPI * ld);
            else
                sc[g] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const int i = i0 + g;
            const float4 v = *reinterpret_cast<const float4 *>(src + i * PPI * ROW);
            const float4 r = epi.template apply<SC>(v, sc[g]);
            const f32x4 rv = {r.x, r.y, r.z, r.w};
            f32x4 *dst = reinterpret_cast<f32x4 *>(out + off0 + (size_t)i * PPI * ld);
            if constexpr (THROUGH)
                store_through(dst, rv);
            else
                // streaming store: the output is not read again by this kernel, and lines that leave the L2 early
                // do not have to be written back when the kernel ends
                __builtin_nontemporal_store(rv, dst);
            if constexpr (Epi::kEmit) {
                // the NP lanes of a pixel hold its window's sign bits, four each: gather them in the first lane
                uint32_t w = sign_nibble(r) << (4 * part);
                w = or_from_lane_above<1>(w);
                w = or_from_lane_above<2>(w);
                if constexpr (NP == 8) w = or_from_lane_above<4>(w);
                unsigned char *bd = epi.bits + ((size_t)tile * 64 + pr0 + i * PPI) * epi.bits_ld + (cbase >> 3);
                if (part == 0) {
                    if constexpr (NP == 8)
                        *reinterpret_cast<uint32_t *>(bd) = w;
                    else
                        *reinterpret_cast<uint16_t *>(bd) = (uint16_t)w;
                }
            }
        }
    }
}

// Writes the staged 16-byte parts [p_lo, p_hi] (4 channels each) of the
// WCH-channel window that starts at channel cbase.  out is [pixel][ld] floats;
// pixels >= total are skipped.  G: shortcut loads kept in flight in the whole-window pass.
template <int WCH, int G, class Epi>
__device__ __forceinline__ void stage_flush(const unsigned char *stage, int lane, float *__restrict__ out, int ld,
                                            int tile, int total, int cbase, int p_lo, int p_hi, Epi epi) {
    __builtin_amdgcn_wave_barrier();
    const int np = p_hi - p_lo + 1;  // 16-byte parts per pixel row
    constexpr int NP = Stage<WCH>::parts, ROW = Stage<WCH>::row;
    constexpr int GG = G < NP ? G : NP;
    const bool has_sc = Epi::kShortcut && epi.shortcut != nullptr;
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    // how the stores go through the L2 is the launch's choice (EpiStore), one way for all of them
    bool through = false;
    if constexpr (Epi::kPolicy) through = epi.through != 0;
    const bool parts_through = through;
    if (np == NP && (tile + 1) * 64 <= total) {
        if (has_sc)
            stage_flush_window<WCH, GG, Epi::kShortcut, false>(stage, lane, out, ld, tile, cbase, epi);
        else if (through)
            stage_flush_window<WCH, GG, false, Epi::kPolicy>(stage, lane, out, ld, tile, cbase, epi);
        else
            stage_flush_window<WCH, GG, false, false>(stage, lane, out, ld, tile, cbase, epi);
    } else {
        const int magic = (65536 + np - 1) / np;  // c / np for c < 512
        for (int i = 0; i < np; ++i) {
            const int c = lane + 64 * i;
            const int pr = (c * magic) >> 16;
            const int part = p_lo + (c - pr * np);
            const int pix = tile * 64 + pr;
            uint32_t nib = 0;
            if (pix < total) {
                const float4 v = *reinterpret_cast<const float4 *>(stage + pr * ROW + part * 16);
                const size_t off = (size_t)pix * ld + cbase + part * 4;
                epi.prepare(cbase + part * 4);
                float4 r;
                if (has_sc)
                    r = epi.template apply<Epi::kShortcut>(
                        v, *reinterpret_cast<const float4 *>((Epi::kReadsOut ? const_cast<const float *>(out) : epi.shortcut) + off));
                else
                    r = epi.template apply<false>(v, make_float4(0.f, 0.f, 0.f, 0.f));
                f32x4 *dst = reinterpret_cast<f32x4 *>(out + off);
                const f32x4 rv = {r.x, r.y, r.z, r.w};
                if (parts_through)
                    store_through(dst, rv);
                else
                    *dst = rv;
                if constexpr (Epi::kEmit) nib = sign_nibble(r);
            }
            if constexpr (Epi::kEmit) {
                // p_lo and np are even here (a wave's share of a pixel row is whole bytes of sign bits), so the two
                // halves of a byte sit in lanes 2k and 2k+1
                uint32_t w = nib << (4 * (part & 1));
                w = or_from_lane_above<1>(w);
                if (pix < total && !(part & 1)) epi.bits[(size_t)pix * epi.bits_ld + ((cbase + part * 4) >> 3)] = (unsigned char)w;
            }
        }
    }
    __builtin_amdgcn_wave_barrier();
}

// Contiguous item range [i0, i1) of wave `wv`: every wave gets `per` items and
// the first `extra` waves one more (per = n_items / n_waves, extra = the rest).
__device__ __forceinline__ void item_range(int wv, int per, int extra, int &i0, int &i1) {
    i0 = wv * per + (wv < extra ? wv : extra);
    i1 = i0 + per + (wv < extra ? 1 : 0);
}

// Host side: how many waves to launch for n_items work items.  All of them
// must be resident at once (a second round of waves would start when the
// first is nearly done and unbalance the SIMDs), so the count follows the
// kernel's real occupancy: blocks per CU as limited by VGPRs and LDS.
template <class Kernel>
inline int resident_blocks_per_cu(Kernel kernel, int block_threads) {
    int blocks = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, kernel, block_threads, 0) != hipSuccess || blocks < 1) blocks = 1;
    return blocks;
}

inline int pick_wave_count(int n_items, int blocks_per_cu, int waves_per_block, int units_per_item = 1) {
    long long w = (long long)(simd_count() / 4) * blocks_per_cu * waves_per_block;
    // Fewer items than resident waves: one item per wave.  When that still fills more than half of the machine,
    // two items per wave are faster, because a wave fetches its lane-resident operand once for both (items that are
    // two units or more already share it); smaller problems are latency-bound and keep one item per wave.
    if (w >= n_items) {
        w = (2ll * n_items > w && units_per_item < 2) ? (n_items + 1) / 2 : n_items;
        // the same number of waves on every SIMD where that costs few waves: a few more than a multiple of the SIMD count give some
        // SIMDs one wave, and its items, more than the others get (3136 waves of two items: the SIMDs with four waves
        // hold the launch until their eight items are done, the others have six)
        if (w > simd_count() && (w % simd_count()) * 8 < simd_count()) w -= w % simd_count();
    }
    if (w < 1) w = 1;
    return (int)((w + waves_per_block - 1) / waves_per_block * waves_per_block);
}

}  // namespace dab
