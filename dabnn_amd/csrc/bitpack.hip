// Sign bit-packing and the small data-movement helpers around it.
//
// Packing rule (common/common_bitpack.h:26,110-174): bit j of word i is 1 iff
// x[64*i + j] > 0 (so +0, -0, NaN and negatives give 0).  On a 64-lane wave
// that is exactly one v_cmp_gt_f32: the lane mask it produces IS the word.
// A wave therefore reads 64 consecutive floats per instruction (256 coalesced
// bytes), keeps the 16 masks of a 4 KiB chunk in lanes 0-15 of a register pair
// and writes them with one 128-byte store.  HBM-bound: 4 bytes read and 1/16
// byte written per element.  Every float is read once, so the loads are
// non-temporal (411 MB: 69 instead of 78 us); the words are stored the ordinary
// way, the next kernel reads them.  Chunks of 16 words, not 64: four times as
// many waves in flight for the tensors of a single layer (25.7 MB: 3.8 instead
// of 5.2 us, 6.6 MB: 2.2 instead of 3.0 us; 411 MB: 67 against 68 us; 8 words:
// 64-byte stores, slower again from 13 MB up).
#include "common.h"

namespace dab {

constexpr int kPackWavesPerBlock = 4;

constexpr int kPackWords = 16;  // words per chunk of a wave

__global__ __launch_bounds__(64 * kPackWavesPerBlock) void bitpack_nhwc_kernel(const float *__restrict__ x,
                                                                              uint64_t *__restrict__ out,
                                                                              long long n_words) {
    const int lane = threadIdx.x & 63;
    const long long wave = (long long)blockIdx.x * kPackWavesPerBlock + (threadIdx.x >> 6);
    const long long n_chunks = (n_words + kPackWords - 1) / kPackWords;
    const long long stride = (long long)gridDim.x * kPackWavesPerBlock;
    for (long long chunk = wave; chunk < n_chunks; chunk += stride) {
        const long long w0 = chunk * kPackWords;
        const float *src = x + w0 * 64 + lane;
        uint64_t mine = 0;
        if (w0 + kPackWords <= n_words) {
#pragma unroll
            for (int i = 0; i < kPackWords; ++i) {
                const uint64_t word = __ballot(__builtin_nontemporal_load(src + (long long)i * 64) > 0.0f);
                mine = (lane == i) ? word : mine;
            }
            if (lane < kPackWords) store_through(out + w0 + lane, mine);
        } else {
            const int rem = (int)(n_words - w0);
            for (int i = 0; i < rem; ++i) {
                const uint64_t word = __ballot(src[(long long)i * 64] > 0.0f);
                mine = (lane == i) ? word : mine;
            }
            if (lane < rem) out[w0 + lane] = mine;
        }
    }
}

// NCHW input: a lane owns one pixel and walks the 64 channels of a word, so
// the loads of a wave are 64 consecutive floats of one channel plane.
__global__ __launch_bounds__(256) void bitpack_nchw_kernel(const float *__restrict__ x, uint64_t *__restrict__ out,
                                                           int n, int cw, long long hw) {
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;  // over n * cw * hw, pixel fastest
    const long long total = (long long)n * cw * hw;
    if (idx >= total) return;
    const long long pix = idx % hw;
    const long long t = idx / hw;
    const int k = (int)(t % cw);
    const long long img = t / cw;
    const float *src = x + ((img * cw + k) * 64) * hw + pix;
    uint32_t lo = 0, hi = 0;
#pragma unroll 8
    for (int j = 0; j < 32; ++j) lo |= (__builtin_nontemporal_load(src + (long long)j * hw) > 0.0f ? 1u : 0u) << j;
#pragma unroll 8
    for (int j = 0; j < 32; ++j) hi |= (__builtin_nontemporal_load(src + (long long)(j + 32) * hw) > 0.0f ? 1u : 0u) << j;
    out[(img * hw + pix) * cw + k] = ((uint64_t)hi << 32) | lo;
}

__global__ __launch_bounds__(256) void pad_bit_kernel(const uint64_t *__restrict__ x, uint64_t *__restrict__ out, int n,
                                                      int h, int w, int cw, int pad_h, int pad_w) {
    const int oh = h + 2 * pad_h, ow = w + 2 * pad_w;
    const long long total = (long long)n * oh * ow * cw;
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int c = (int)(idx % cw);
    long long t = idx / cw;
    const int xo = (int)(t % ow);
    t /= ow;
    const int yo = (int)(t % oh);
    const long long img = t / oh;
    const int yi = yo - pad_h, xi = xo - pad_w;
    uint64_t v = 0;
    if (yi >= 0 && yi < h && xi >= 0 && xi < w) v = x[((img * h + yi) * w + xi) * cw + c];
    out[idx] = v;
}

__global__ __launch_bounds__(256) void weight_transpose_kernel(const uint64_t *__restrict__ w, uint64_t *__restrict__ wt,
                                                               int m, int k) {
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;  // over k*m, m fastest (coalesced writes)
    if (idx >= (long long)m * k) return;
    const int j = (int)(idx % m);
    const int i = (int)(idx / m);
    wt[idx] = w[(size_t)j * k + i];
}

// Split::forward_impl (dabnn/layers/Split.cpp:6-21): word j of pixel p goes to out1[p][j] for j < cw/2, else to
// out2[p][j - cw/2].  One thread per input word, coalesced reads.
__global__ __launch_bounds__(256) void split_bit_kernel(const uint64_t *__restrict__ x, uint64_t *__restrict__ out1,
                                                        uint64_t *__restrict__ out2, long long n_pix, int cw) {
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n_pix * cw) return;
    const long long pix = idx / cw;
    const int j = (int)(idx - pix * cw), half = cw / 2;
    const uint64_t v = x[idx];
    if (j < half)
        out1[pix * half + j] = v;
    else
        out2[pix * half + j - half] = v;
}

// Shuffle::forward_impl (dabnn/layers/Shuffle.cpp:6-43), one thread per pixel, in place:
//   128 channels: the pixel's four 32-bit quarters a b c d become a c b d
//   256 channels: words 1 and 2 change places;  512 channels: words 2,3 change places with words 4,5
//   any other channel count is left as it is, as in the reference
__global__ __launch_bounds__(256) void shuffle_bit_kernel(uint64_t *__restrict__ x, long long n_pix, int elem_c) {
    const long long pix = (long long)blockIdx.x * 256 + threadIdx.x;
    if (pix >= n_pix) return;
    if (elem_c == 128) {
        uint64_t *p = x + pix * 2;
        const uint64_t w0 = p[0], w1 = p[1];
        p[0] = (w0 & 0xffffffffull) | (w1 << 32);
        p[1] = (w0 >> 32) | (w1 & 0xffffffff00000000ull);
    } else if (elem_c == 256) {
        uint64_t *p = x + pix * 4;
        const uint64_t t = p[1];
        p[1] = p[2];
        p[2] = t;
    } else if (elem_c == 512) {
        uint64_t *p = x + pix * 8;
        const uint64_t t2 = p[2], t3 = p[3];
        p[2] = p[4], p[3] = p[5];
        p[4] = t2, p[5] = t3;
    }
}

static unsigned blocks_for(long long total, int per_block) {
    long long b = (total + per_block - 1) / per_block;
    return (unsigned)(b < 1 ? 1 : b);
}

}  // namespace dab

extern "C" int dab_bitpack_nhwc(const float *x, uint64_t *out, int64_t n_pix, int c, dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(x && out, "dab_bitpack_nhwc: null pointer");
    DAB_REQUIRE(n_pix > 0 && c > 0, "dab_bitpack_nhwc: n_pix %lld c %d", (long long)n_pix, c);
    DAB_REQUIRE(c % 64 == 0, "dab_bitpack_nhwc: c %d is not a multiple of 64", c);
    const long long n_words = (long long)n_pix * (c / 64);
    const long long chunks = (n_words + kPackWords - 1) / kPackWords;
    long long blocks = (chunks + kPackWavesPerBlock - 1) / kPackWavesPerBlock;
    const long long cap = (long long)simd_count() * 8;  // grid-stride beyond 8 waves per SIMD
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(bitpack_nhwc_kernel, dim3((unsigned)blocks), dim3(64 * kPackWavesPerBlock), 0, as_stream(stream), x,
                       out, n_words);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

extern "C" int dab_bitpack_nchw(const float *x, uint64_t *out, int n, int c, int h, int w, dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(x && out, "dab_bitpack_nchw: null pointer");
    DAB_REQUIRE(n > 0 && c > 0 && h > 0 && w > 0, "dab_bitpack_nchw: non-positive dimension");
    DAB_REQUIRE(c % 64 == 0, "dab_bitpack_nchw: c %d is not a multiple of 64", c);
    const long long total = (long long)n * (c / 64) * h * w;
    hipLaunchKernelGGL(bitpack_nchw_kernel, dim3(blocks_for(total, 256)), dim3(256), 0, as_stream(stream), x, out, n,
                       c / 64, (long long)h * w);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

extern "C" int dab_pad_bit(const uint64_t *x, int n, int h, int w, int cw, int pad_h, int pad_w, uint64_t *out,
                           dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(x && out, "dab_pad_bit: null pointer");
    DAB_REQUIRE(n > 0 && h > 0 && w > 0 && cw > 0 && pad_h >= 0 && pad_w >= 0, "dab_pad_bit: bad dimension");
    const long long total = (long long)n * (h + 2 * pad_h) * (w + 2 * pad_w) * cw;
    hipLaunchKernelGGL(pad_bit_kernel, dim3(blocks_for(total, 256)), dim3(256), 0, as_stream(stream), x, out, n, h, w, cw,
                       pad_h, pad_w);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

extern "C" int dab_weight_transpose(const uint64_t *w, int m, int k, uint64_t *wt, dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(w && wt, "dab_weight_transpose: null pointer");
    DAB_REQUIRE(m > 0 && k > 0, "dab_weight_transpose: m %d k %d", m, k);
    hipLaunchKernelGGL(weight_transpose_kernel, dim3(blocks_for((long long)m * k, 256)), dim3(256), 0, as_stream(stream),
                       w, wt, m, k);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

extern "C" int dab_split_bit(const uint64_t *x, int64_t n_pix, int cw, uint64_t *out1, uint64_t *out2, dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(x && out1 && out2, "dab_split_bit: null pointer");
    DAB_REQUIRE(n_pix > 0 && cw > 0, "dab_split_bit: n_pix %lld cw %d", (long long)n_pix, cw);
    // the reference asserts elem_c % 128 == 0 && elem_c <= 512 (dabnn/layers/Split.h:22-23)
    DAB_REQUIRE(cw % 2 == 0 && cw <= 8, "Split: %d channels", cw * 64);
    if (n_pix * cw >= (1ll << 40)) return fail(DAB_EUNSUPPORTED, "dab_split_bit: tensor too large");
    hipLaunchKernelGGL(split_bit_kernel, dim3(blocks_for((long long)n_pix * cw, 256)), dim3(256), 0, as_stream(stream), x, out1,
                       out2, (long long)n_pix, cw);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}

extern "C" int dab_shuffle_bit_inplace(uint64_t *x, int64_t n_pix, int elem_c, dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(x, "dab_shuffle_bit_inplace: null pointer");
    DAB_REQUIRE(n_pix > 0, "dab_shuffle_bit_inplace: n_pix %lld", (long long)n_pix);
    // dabnn/layers/Shuffle.h:19-20
    DAB_REQUIRE(elem_c > 0 && elem_c % 128 == 0 && elem_c <= 512, "Shuffle: %d channels", elem_c);
    if (n_pix >= (1ll << 40)) return fail(DAB_EUNSUPPORTED, "dab_shuffle_bit_inplace: tensor too large");
    hipLaunchKernelGGL(shuffle_bit_kernel, dim3(blocks_for((long long)n_pix, 256)), dim3(256), 0, as_stream(stream), x,
                       (long long)n_pix, elem_c);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}
