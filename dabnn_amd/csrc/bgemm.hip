// Binary GEMM: C(i,j) += popcount(A(i,h) ^ B(h,j)), all operands column-major
// as in the reference (dabnn/bgemm.h:22-24,46-66,587-597):
//   A(i,h) = a[h*lda + i]   m x k words, the transposed filter bank
//   B(h,j) = b[j*ldb + h]   k x n words, one contiguous K-row per output pixel
//   C(i,j) = c[j*ldc + i]   m x n floats, i.e. NHWC output
//
// Mapping: a lane owns one ROW i of A (an output channel).  For a fixed K word
// the 64 rows of a tile are 512 contiguous bytes of A, so the lane-resident
// operand is fetched with fully coalesced loads; the K-row of a column j is
// contiguous in B and wave-uniform, so it comes through scalar loads and
// enters v_xor_b32 as SGPR operands; and for a fixed column the 64 results are
// 256 contiguous bytes of C, so the read-modify-write of C is coalesced
// without any transposition.
//
// A unit is 64 rows x Q columns.  Waves own contiguous ranges of units ordered
// row-tile major, so the A operand is reloaded only when a range crosses into
// the next row tile.
//   K64R > 0  k == K64R and ldb == k: the lane keeps its whole A row resident
//             (the network shapes: 18, 36, 72 words with Q = 8, 4, 2) and the
//             Q*k words of B of a unit are one contiguous run
//   K64R == 0 any k, any ldb: K is walked in chunks of 8 words; per chunk the
//             lane reloads 8 words of A (coalesced, L1/L2 resident)
#include "xnor_core.h"

namespace dab {

struct BgemmArgs {
    const uint64_t *a;
    const uint64_t *b;
    float *c;
    int m, n, k;
    int lda, ldb, ldc;
    int n_runs;  // ceil(n / Q) column runs per row tile
    int items_per_wave, items_extra;
    FastDiv div_runs;
    int overwrite;  // C = counts instead of C += counts: what the reference's fill(0) + bgemm pair leaves in C
};

constexpr int kGemmWavesPerBlock = 4;
constexpr int kChunk = 8;  // K words per chunk of the generic variant

// C(row, j) += counts of a unit.  Columns below j_first belong to the previous
// (shifted) run and are skipped; the test is wave-uniform.
template <int Q>
__device__ __forceinline__ void add_to_c(float *__restrict__ c, int ldc, int row, bool row_ok, int j0, int j_first,
                                         const uint32_t (&acc)[Q], bool overwrite) {
#pragma unroll
    for (int q = 0; q < Q; ++q) {
        const int j = j0 + q;
        if (j >= j_first && row_ok) {
            float *d = c + (size_t)j * ldc + row;
            const float cnt = __uint_as_float(acc[q]) - kAccBias;
            // 0.f + cnt == cnt: the store alone is the fill + accumulate pair.  The accumulating form reads C when
            // the count is done and wants it in the L2, where ordinary stores of an earlier launch leave it
            if (overwrite)
                store_through(d, cnt);
            else
                *d = *d + cnt;
        }
    }
}

// The same with the old values of C fetched by the caller before it counted (fetch_c), so that the round trip to
// memory lies behind the unit's arithmetic instead of after it.
template <int Q>
__device__ __forceinline__ void fetch_c(const float *__restrict__ c, int ldc, int row, bool row_ok, int j0, int j_first,
                                        float (&old)[Q], bool overwrite) {
#pragma unroll
    for (int q = 0; q < Q; ++q) {
        const int j = j0 + q;
        old[q] = (!overwrite && j >= j_first && row_ok) ? c[(size_t)j * ldc + row] : 0.f;
    }
}
template <int Q>
__device__ __forceinline__ void store_c(float *__restrict__ c, int ldc, int row, bool row_ok, int j0, int j_first,
                                        const uint32_t (&acc)[Q], const float (&old)[Q]) {
#pragma unroll
    for (int q = 0; q < Q; ++q) {
        const int j = j0 + q;
        if (j >= j_first && row_ok) {
            const float cnt = __uint_as_float(acc[q]) - kAccBias;
            store_through(c + (size_t)j * ldc + row, old[q] + cnt);  // 0.f + cnt == cnt: the overwriting form never read C
        }
    }
}

template <int K64R, int Q>
__global__ __launch_bounds__(64 * kGemmWavesPerBlock, K64R >= 72 ? 3 : (K64R >= 36 ? 5 : 6)) void bgemm_resident_kernel(const BgemmArgs p) {
    constexpr int K32 = 2 * K64R;
    const int lane = threadIdx.x & 63;
    const int wib = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wv = blockIdx.x * kGemmWavesPerBlock + wib;
    int i0, i1;
    item_range(wv, p.items_per_wave, p.items_extra, i0, i1);
    if (i0 >= i1) return;

    int mt = (int)p.div_runs.div((uint32_t)i0);
    int run = i0 - mt * p.n_runs;
    bool need_load = true;
    uint32_t w[K32];
    int row = 0;
    bool row_ok = false;
    for (int it = i0; it < i1; ++it) {
        if (need_load) {
            need_load = false;
            row = mt * 64 + lane;
            row_ok = row < p.m;
            const uint64_t *col = p.a + (row_ok ? row : p.m - 1);
#pragma unroll
            for (int h = 0; h < K64R; ++h) {
                const uint64_t v = col[(size_t)h * p.lda];
                w[2 * h] = (uint32_t)v, w[2 * h + 1] = (uint32_t)(v >> 32);
            }
        }
        // Priority by remaining work: the SIMD issues from its oldest wave first, so with equal priorities its few
        // resident waves finish one after the other and the last one runs alone at the single-wave issue rate.
        const int left = K64R >= 36 ? i1 - it - 1 : 0;  // 3-5 resident waves per SIMD; no effect measured with 6
        if (left >= 3) {
            __builtin_amdgcn_s_setprio(3);
        } else if (left == 2) {
            __builtin_amdgcn_s_setprio(2);
        } else if (left == 1) {
            __builtin_amdgcn_s_setprio(1);
        } else {
            __builtin_amdgcn_s_setprio(0);
        }
        // the last run of a ragged n is shifted back so its scalar loads stay inside B
        const int j_first = run * Q;
        const int j0 = j_first + Q <= p.n ? j_first : p.n - Q;
        uint32_t acc[Q];
        // B streams through the scalar cache: two vectors per wait.  The accumulating form asks for the old values of
        // C before it counts (cfg m512 k72 n3136: 16.8 instead of 17.2 us, four times the columns 59.7 instead of 65);
        // the overwriting form keeps the registers (two code paths, the test is wave-uniform).
        if (p.overwrite) {
            unit_rowmajor<K32, Q, 2, (K64R >= 72)>(p.b + (size_t)j0 * K64R, w, acc);
            add_to_c<Q>(p.c, p.ldc, row, row_ok, j0, j_first, acc, true);
        } else {
            float old[Q];
            fetch_c<Q>(p.c, p.ldc, row, row_ok, j0, j_first, old, false);
            unit_rowmajor<K32, Q, 2, (K64R >= 72)>(p.b + (size_t)j0 * K64R, w, acc);
            store_c<Q>(p.c, p.ldc, row, row_ok, j0, j_first, acc, old);
        }
        if (++run == p.n_runs) {
            run = 0;
            ++mt;
            need_load = true;
        }
    }
}

// Any k and ldb; Q = 8 columns per unit, two columns per scalar-load batch.
__global__ __launch_bounds__(64 * kGemmWavesPerBlock) void bgemm_chunked_kernel(const BgemmArgs p) {
    constexpr int Q = 8;
    const int lane = threadIdx.x & 63;
    const int wib = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wv = blockIdx.x * kGemmWavesPerBlock + wib;
    int i0, i1;
    item_range(wv, p.items_per_wave, p.items_extra, i0, i1);
    if (i0 >= i1) return;

    int mt = (int)p.div_runs.div((uint32_t)i0);
    int run = i0 - mt * p.n_runs;
    for (int it = i0; it < i1; ++it) {
        const int row = mt * 64 + lane;
        const bool row_ok = row < p.m;
        const uint64_t *acol = p.a + (row_ok ? row : p.m - 1);
        const int j_first = run * Q;
        const int j0 = j_first + Q <= p.n ? j_first : p.n - Q;
        uint32_t acc[Q];
#pragma unroll
        for (int q = 0; q < Q; ++q) acc[q] = kAccInit;

        int h0 = 0;
        for (; h0 + kChunk <= p.k; h0 += kChunk) {
            uint32_t w[2 * kChunk];
#pragma unroll
            for (int h = 0; h < kChunk; ++h) {
                const uint64_t v = acol[(size_t)(h0 + h) * p.lda];
                w[2 * h] = (uint32_t)v, w[2 * h + 1] = (uint32_t)(v >> 32);
            }
            // column j0+q contributes the 16 dwords b[(j0+q)*ldb + h0 .. +8)
            const uint64_t *bbase = p.b + (size_t)j0 * p.ldb + h0;
            const uint32_t bstride = (uint32_t)p.ldb * 8u;
            u32x16 buf[2][2];
            sload_off<16>(buf[0][0], bbase, 0u);
            sload_off<16>(buf[0][1], bbase, bstride);
            swait(buf[0][0]);
            swait(buf[0][1]);
            uint32_t off = bstride;
            static_for<Q / 2>([&](auto s_) {
                constexpr int s = s_;
                if constexpr (s + 1 < Q / 2) {
                    off += bstride;
                    sload_off<16>(buf[(s + 1) & 1][0], bbase, off);
                    off += bstride;
                    sload_off<16>(buf[(s + 1) & 1][1], bbase, off);
                }
                static_for<2>([&](auto c_) {
                    static_for<kChunk>([&](auto h_) {
                        xp2(acc[2 * s + c_], buf[s & 1][c_][2 * h_], buf[s & 1][c_][2 * h_ + 1], w[2 * h_], w[2 * h_ + 1]);
                    });
                });
                if constexpr (s + 1 < Q / 2) {
                    swait(buf[(s + 1) & 1][0]);
                    swait(buf[(s + 1) & 1][1]);
                }
            });
        }
        for (; h0 < p.k; ++h0) {  // K tail, one word at a time
            const uint64_t v = acol[(size_t)h0 * p.lda];
            const uint32_t wlo = (uint32_t)v, whi = (uint32_t)(v >> 32);
#pragma unroll
            for (int q = 0; q < Q; ++q) {
                const uint64_t bw = p.b[(size_t)(j0 + q) * p.ldb + h0];  // wave-uniform address
                acc[q] += __builtin_popcount(wlo ^ (uint32_t)bw) + __builtin_popcount(whi ^ (uint32_t)(bw >> 32));
            }
        }
        add_to_c<Q>(p.c, p.ldc, row, row_ok, j0, j_first, acc, p.overwrite != 0);
        if (++run == p.n_runs) {
            run = 0;
            ++mt;
        }
    }
}

// One thread per output element; for n < 8, where the column runs do not apply.
__global__ void bgemm_small_n_kernel(const BgemmArgs p) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long long)p.m * p.n) return;
    const int i = (int)(idx % p.m);
    const long long j = idx / p.m;
    uint32_t cnt = 0;
    for (int h = 0; h < p.k; ++h) cnt += __popcll(p.a[(size_t)h * p.lda + i] ^ p.b[(size_t)j * p.ldb + h]);
    float *d = p.c + (size_t)j * p.ldc + i;
    *d = p.overwrite ? (float)cnt : *d + (float)cnt;
}

template <int Q, class Kernel>
static bool plan_items(BgemmArgs &g, Kernel kernel, int &n_waves) {
    static const int blocks_per_cu = resident_blocks_per_cu(kernel, 64 * kGemmWavesPerBlock);
    g.n_runs = (g.n + Q - 1) / Q;
    const long long items = (((long long)g.m + 63) / 64) * g.n_runs;
    if (items >= (1ll << 31)) return false;
    n_waves = pick_wave_count((int)items, blocks_per_cu, kGemmWavesPerBlock);
    g.items_per_wave = (int)(items / n_waves);
    g.items_extra = (int)(items % n_waves);
    g.div_runs = FastDiv((uint32_t)g.n_runs);
    return true;
}

template <int K64R, int Q>
static int launch_resident(BgemmArgs &g, hipStream_t stream) {
    int n_waves = 0;
    if (!plan_items<Q>(g, bgemm_resident_kernel<K64R, Q>, n_waves)) return fail(DAB_EUNSUPPORTED, "dab_bgemm: too many work units");
    hipLaunchKernelGGL((bgemm_resident_kernel<K64R, Q>), dim3(n_waves / kGemmWavesPerBlock), dim3(64 * kGemmWavesPerBlock), 0,
                       stream, g);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

}  // namespace dab

static int bgemm_impl(int m, int n, int k, const uint64_t *a, int lda, const uint64_t *b, int ldb, float *c, int ldc,
                      bool overwrite, dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(a && b && c, "dab_bgemm: null pointer");
    DAB_REQUIRE(m > 0 && n > 0 && k > 0, "dab_bgemm: m %d n %d k %d", m, n, k);
    DAB_REQUIRE(lda >= m && ldb >= k && ldc >= m, "dab_bgemm: leading dimension smaller than the matrix (lda %d ldb %d ldc %d)",
                lda, ldb, ldc);
    DAB_REQUIRE((reinterpret_cast<uintptr_t>(a) & 7) == 0 && (reinterpret_cast<uintptr_t>(b) & 7) == 0 &&
                    (reinterpret_cast<uintptr_t>(c) & 3) == 0,
                "dab_bgemm: misaligned pointer");
    if ((long long)k * 64 > kMaxCount) return fail(DAB_EUNSUPPORTED, "dab_bgemm: k %d words exceeds the exact-count range", k);
    if ((long long)ldb * 8 * 8 >= (1ll << 32)) return fail(DAB_EUNSUPPORTED, "dab_bgemm: ldb too large");

    BgemmArgs g;
    g.a = a, g.b = b, g.c = c;
    g.m = m, g.n = n, g.k = k;
    g.lda = lda, g.ldb = ldb, g.ldc = ldc;
    g.overwrite = overwrite ? 1 : 0;
    hipStream_t s = as_stream(stream);
    if (n < 8) {
        const long long total = (long long)m * n;
        hipLaunchKernelGGL(bgemm_small_n_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, g);
        DAB_LAUNCH_CHECK();
        return DAB_OK;
    }
    if (ldb == k) {
        switch (k) {
            case 18: return launch_resident<18, 8>(g, s);
            case 36: return launch_resident<36, 4>(g, s);
            case 72: return launch_resident<72, 2>(g, s);
            default: break;
        }
    }
    int n_waves = 0;
    if (!plan_items<8>(g, bgemm_chunked_kernel, n_waves)) return fail(DAB_EUNSUPPORTED, "dab_bgemm: too many work units");
    hipLaunchKernelGGL(bgemm_chunked_kernel, dim3(n_waves / kGemmWavesPerBlock), dim3(64 * kGemmWavesPerBlock), 0, s, g);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

extern "C" int dab_bgemm(int m, int n, int k, const uint64_t *a, int lda, const uint64_t *b, int ldb, float *c, int ldc,
                         dab_stream_t stream) {
    return bgemm_impl(m, n, k, a, lda, b, ldb, c, ldc, false, stream);
}

extern "C" int dab_bgemm_overwrite(int m, int n, int k, const uint64_t *a, int lda, const uint64_t *b, int ldb, float *c,
                                   int ldc, dab_stream_t stream) {
    return bgemm_impl(m, n, k, a, lda, b, ldb, c, ldc, true, stream);
}
