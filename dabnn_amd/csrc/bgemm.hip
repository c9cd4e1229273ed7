// Binary GEMM: C(i,j) += popcount(A(i,h) ^ B(h,j)), all operands column-major
// as in the reference (dabnn/bgemm.h:22-24,46-66,587-597):
//   A(i,h) = a[h*lda + i]   m x k words, the transposed filter bank
//   B(h,j) = b[j*ldb + h]   k x n words, one contiguous K-row per output pixel
//   C(i,j) = c[j*ldc + i]   m x n floats, i.e. NHWC output
//
// A lane owns one column j (output pixel) and holds its K-row in VGPRs; the 8
// rows i..i+7 of a unit are one 64-byte scalar load per K word, because A is
// stored channel-minor.  Two variants:
//   K64R > 0  the whole K-row (K64R words) stays resident across the units of
//             a tile (the network shapes: 18, 36, 72 words)
//   K64R == 0 any k: K is walked in chunks of 8 words whose activations are
//             re-read per unit (they stay in L1/L2), plus a word-by-word tail
#include "xnor_core.h"

namespace dab {

struct BgemmArgs {
    const uint64_t *a;
    const uint64_t *b;
    float *c;
    int m, n, k;
    int lda, ldb, ldc;
    int n_groups;  // ceil(m / 8)
    int n_units;
    int n_waves;
};

constexpr int kGemmWavesPerBlock = 4;
constexpr int kChunk = 8;  // K words per chunk of the generic variant

// DIRECT: every lane writes its own 8 results with scalar accesses (any ldc,
// any alignment); otherwise results go through the staging transpose.
template <int K64R, bool DIRECT>
__global__ __launch_bounds__(64 * kGemmWavesPerBlock) void bgemm_kernel(const BgemmArgs p) {
    __shared__ __attribute__((aligned(16))) unsigned char stage_all[DIRECT ? 16 : kGemmWavesPerBlock * kStageBytes];
    const int lane = threadIdx.x & 63;
    const int wib = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    unsigned char *stage = stage_all + (DIRECT ? 0 : wib * kStageBytes);
    const int wv = blockIdx.x * kGemmWavesPerBlock + wib;

    int u0, u1;
    unit_range(wv, p.n_waves, p.n_units, u0, u1);
    if (u0 >= u1) return;

    int tile = u0 / p.n_groups;
    int cg = u0 - tile * p.n_groups;
    int g_lo = cg & 3;
    bool need_load = true;
    constexpr int NA = K64R > 0 ? 2 * K64R : 2 * kChunk;
    uint32_t act[NA];
    const uint64_t *brow = nullptr;
    const uint32_t stride = (uint32_t)p.lda * 8u;

    for (int u = u0; u < u1; ++u) {
        if (need_load) {
            need_load = false;
            int col = tile * 64 + lane;
            col = col < p.n ? col : p.n - 1;
            brow = p.b + (size_t)col * p.ldb;
            if constexpr (K64R > 0) {
#pragma unroll
                for (int h = 0; h < K64R; ++h) {
                    const uint64_t v = brow[h];
                    act[2 * h] = (uint32_t)v, act[2 * h + 1] = (uint32_t)(v >> 32);
                }
            }
        }

        // The last group of a ragged m is shifted back to end at m, so that its
        // 64-byte weight loads stay inside A; rows below `first` were already
        // produced by the previous group and are not written again.
        const int first = cg * 8;
        const int i0 = first + 8 <= p.m ? first : p.m - 8;
        const uint64_t *wbase = p.a + i0;

        uint32_t acc[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) acc[q] = kAccInit;
        if constexpr (K64R > 0) {
            unit_colmajor<K64R>(wbase, stride, act, acc);
        } else {
            int h0 = 0;
            for (; h0 + kChunk <= p.k; h0 += kChunk) {
#pragma unroll
                for (int h = 0; h < kChunk; ++h) {
                    const uint64_t v = brow[h0 + h];
                    act[2 * h] = (uint32_t)v, act[2 * h + 1] = (uint32_t)(v >> 32);
                }
                unit_colmajor<kChunk>(wbase + (size_t)h0 * p.lda, stride, act, acc);
            }
            for (; h0 < p.k; ++h0) {
                const uint64_t v = brow[h0];
                act[0] = (uint32_t)v, act[1] = (uint32_t)(v >> 32);
                unit_colmajor<1>(wbase + (size_t)h0 * p.lda, stride, act, acc);
            }
        }

        const bool last_in_tile = cg == p.n_groups - 1;
        const bool ragged = i0 != first;
        if (DIRECT || ragged) {
            const int col = tile * 64 + lane;
            if (col < p.n) {
                float *crow = p.c + (size_t)col * p.ldc;
#pragma unroll
                for (int q = 0; q < 8; ++q)
                    if (i0 + q >= first) crow[i0 + q] += __uint_as_float(acc[q]) - kAccBias;
            }
        } else {
            stage_put(stage, lane, cg & 3, acc);
        }
        if (!DIRECT) {
            // a ragged last group is never staged: flush what precedes it in the window
            const int g_hi = ragged ? (cg & 3) - 1 : (cg & 3);
            if (((cg & 3) == 3 || last_in_tile || u == u1 - 1)) {
                if (g_hi >= g_lo) stage_flush<true>(stage, lane, p.c, p.ldc, tile, p.n, (cg & ~3) * 8, g_lo, g_hi);
                g_lo = 0;
            }
        }
        if (last_in_tile) {
            cg = 0;
            ++tile;
            need_load = true;
        } else {
            ++cg;
        }
    }
}

// One thread per output element; for m < 8, where the 8-row units do not apply.
__global__ void bgemm_small_m_kernel(const BgemmArgs p) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long long)p.m * p.n) return;
    const int i = (int)(idx % p.m);
    const long long j = idx / p.m;
    uint32_t cnt = 0;
    for (int h = 0; h < p.k; ++h) cnt += __popcll(p.a[(size_t)h * p.lda + i] ^ p.b[(size_t)j * p.ldb + h]);
    p.c[(size_t)j * p.ldc + i] += (float)cnt;
}

template <int K64R, bool DIRECT>
static int launch_bgemm(const BgemmArgs &args, hipStream_t stream) {
    hipLaunchKernelGGL((bgemm_kernel<K64R, DIRECT>), dim3(args.n_waves / kGemmWavesPerBlock),
                       dim3(64 * kGemmWavesPerBlock), 0, stream, args);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

}  // namespace dab

extern "C" int dab_bgemm(int m, int n, int k, const uint64_t *a, int lda, const uint64_t *b, int ldb, float *c, int ldc,
                         dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(a && b && c, "dab_bgemm: null pointer");
    DAB_REQUIRE(m > 0 && n > 0 && k > 0, "dab_bgemm: m %d n %d k %d", m, n, k);
    DAB_REQUIRE(lda >= m && ldb >= k && ldc >= m, "dab_bgemm: leading dimension smaller than the matrix (lda %d ldb %d ldc %d)",
                lda, ldb, ldc);
    DAB_REQUIRE((reinterpret_cast<uintptr_t>(a) & 7) == 0 && (reinterpret_cast<uintptr_t>(b) & 7) == 0 &&
                    (reinterpret_cast<uintptr_t>(c) & 3) == 0,
                "dab_bgemm: misaligned pointer");
    if ((long long)k * 64 > kMaxCount) return fail(DAB_EUNSUPPORTED, "dab_bgemm: k %d words exceeds the exact-count range", k);
    if ((long long)lda * 8 * k >= (1ll << 32)) return fail(DAB_EUNSUPPORTED, "dab_bgemm: A larger than 4 GiB");

    BgemmArgs g;
    g.a = a, g.b = b, g.c = c;
    g.m = m, g.n = n, g.k = k;
    g.lda = lda, g.ldb = ldb, g.ldc = ldc;
    hipStream_t s = as_stream(stream);
    if (m < 8) {
        const long long total = (long long)m * n;
        hipLaunchKernelGGL(bgemm_small_m_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, g);
        DAB_LAUNCH_CHECK();
        return DAB_OK;
    }
    g.n_groups = (m + 7) / 8;
    const long long units = (((long long)n + 63) / 64) * g.n_groups;
    if (units >= (1ll << 31)) return fail(DAB_EUNSUPPORTED, "dab_bgemm: too many work units");
    g.n_units = (int)units;
    g.n_waves = pick_wave_count(g.n_units, 4, kGemmWavesPerBlock);
    const bool direct = (ldc % 4 != 0) || (reinterpret_cast<uintptr_t>(c) & 15) != 0;
    if (direct) return launch_bgemm<0, true>(g, s);
    switch (k) {
        case 18: return launch_bgemm<18, false>(g, s);
        case 36: return launch_bgemm<36, false>(g, s);
        case 72: return launch_bgemm<72, false>(g, s);
        default: return launch_bgemm<0, false>(g, s);
    }
}
