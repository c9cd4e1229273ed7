// fused_binarize_im2col (dabnn/fused_binarize_im2col.h:6-68) on the GPU.
//
// Output: one row per output pixel, each row = the kh*kw*c gathered floats
// (zeros where a tap falls outside the image) zero-extended to a multiple of
// 128 and sign-packed; row_words = ceil(kh*kw*c/128)*2 words.
//
// A wave produces one word per compare: lane l looks at 64 consecutive
// floats and the lane mask of (value > 0) is the word.  When c is a multiple
// of 64 a word never straddles two taps, so binarising and gathering commute:
// a block packs the input rows that its output rows touch into LDS once
// (every float is read about once, not kh*kw times) and then writes its col
// rows by copying words out of LDS.  The general path resolves tap and
// channel per lane for every output word.
// HBM-bound: 4 bytes per input element read (plus the halo rows shared by
// neighbouring blocks), 8 bytes per output word written.
#include "common.h"

namespace dab {

struct Im2colArgs {
    const float *x;
    uint64_t *col;
    int n, h, w, c;
    int kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w;
    int oh, ow;
    int row_words;
    int len;  // kh*kw*c
    long long n_words;
    FastDiv div_row_words, div_ow, div_oh, div_c, div_kw, div_cw;
    int rows_per_block, blocks_per_image;  // tiled kernel only
    int packed_words;                      // tiled kernel: words of packed input rows a block holds in LDS
    int step_wi, step_ox, step_oy;         // tiled kernel: what 512 words further on means for (index in row, ox, oy)
};

constexpr int kIm2colWavesPerBlock = 4;

// c % 64 == 0, one block per (image, run of rows_per_block output rows).  Phase 1 packs the input rows
// [y_lo, y_hi) that the run's windows reach (contiguous in memory) into LDS, one 256-byte load and one compare per
// word, every wave an equal share of the words; phase 2 writes the run's col rows, which are contiguous too, one word
// per lane from LDS or zero.
template <int THREADS>
__global__ __launch_bounds__(THREADS) void fused_binarize_im2col_tiled_kernel(const Im2colArgs p) {
    extern __shared__ uint64_t packed[];
    constexpr int WAVES = THREADS / 64;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wib = __builtin_amdgcn_readfirstlane(tid >> 6);
    // neighbouring runs of an image share their halo rows: consecutive runs go to the same XCD, where the second
    // reader of a row finds it in the L2 (64x28x28x128: 7.0 us against 8.2 with the runs dealt to the XCDs in turn)
    const int run_id = (int)xcd_contiguous_block(blockIdx.x, gridDim.x);
    const int img = run_id / p.blocks_per_image, rb = run_id - img * p.blocks_per_image;
    const int cw = p.c >> 6;
    const int oy0 = rb * p.rows_per_block;
    const int oy1 = oy0 + p.rows_per_block < p.oh ? oy0 + p.rows_per_block : p.oh;
    int y_lo = oy0 * p.stride_h - p.pad_h;
    int y_hi = (oy1 - 1) * p.stride_h - p.pad_h + (p.kh - 1) * p.dil_h + 1;
    y_lo = y_lo < 0 ? 0 : y_lo;
    y_hi = y_hi > p.h ? p.h : y_hi;
    const int n_in = y_hi > y_lo ? (y_hi - y_lo) * p.w * cw : 0;  // words to pack
    const float *src = p.x + ((size_t)img * p.h + y_lo) * p.w * p.c;
    const int per = (n_in + WAVES - 1) / WAVES;
    const int j_end = (wib + 1) * per < n_in ? (wib + 1) * per : n_in;
    for (int j0 = wib * per; j0 < j_end; j0 += 64) {
        const int cnt = j_end - j0 < 64 ? j_end - j0 : 64;
        uint64_t mine = 0;
        // up to 64 independent loads in flight, asked for in groups of eight (the words past cnt in the last group
        // repeat the last one and are not stored)
        float v[64];
#pragma unroll
        for (int g8 = 0; g8 < 64; g8 += 8) {
            if (g8 < cnt) {
#pragma unroll
                for (int i = g8; i < g8 + 8; ++i) v[i] = src[(size_t)(j0 + (i < cnt ? i : cnt - 1)) * 64 + lane];
            }
        }
#pragma unroll
        for (int g8 = 0; g8 < 64; g8 += 8) {
            if (g8 < cnt) {
#pragma unroll
                for (int i = g8; i < g8 + 8; ++i) {
                    const uint64_t word = __ballot(v[i] > 0.0f);
                    mine = (lane == i) ? word : mine;
                }
            }
        }
        if (lane < cnt) packed[j0 + lane] = mine;
    }
    // What a word of a col row gathers depends on its index in the row alone: tap (row and column offset of the
    // window) and channel word, decoded once per block into a table behind the packed rows.  Entry: x = the tap's row
    // offset (far outside every image for the zero padding word), y = column offset * 4096 + channel word.
    int2 *word_tab = reinterpret_cast<int2 *>(packed + p.packed_words);
    for (int wi = tid; wi < p.row_words; wi += THREADS) {
        const uint32_t tap = p.div_cw.div((uint32_t)wi);  // >= kh*kw for the zero padding word
        const int k = wi - tap * cw;
        const uint32_t a = p.div_kw.div(tap);
        const int b = tap - a * p.kw;
        word_tab[wi] = make_int2((int)tap < p.kh * p.kw ? (int)a * p.dil_h - p.pad_h : -(1 << 20), (b * p.dil_w - p.pad_w) * 4096 + k);
    }
    __syncthreads();
    uint64_t *dst = p.col + ((size_t)img * p.oh + oy0) * p.ow * p.row_words;
    const int n_out = (oy1 - oy0) * p.ow * p.row_words;
    // word g = tid + i * THREADS of the run: pixel and index in the row advance by constants, no division in the loop
    uint32_t pix0 = p.div_row_words.div((uint32_t)tid);
    int wi = tid - (int)pix0 * p.row_words;
    int oyl = (int)p.div_ow.div(pix0);
    int ox = (int)pix0 - oyl * p.ow;
    for (int g = tid; g < n_out; g += THREADS) {
        const int2 e = word_tab[wi];
        const int y = (oy0 + oyl) * p.stride_h + e.x;
        const int xx = ox * p.stride_w + (e.y >> 12);
        // a row inside the image is inside [y_lo, y_hi): the run's windows span exactly that range
        const bool ok = y >= 0 && y < p.h && xx >= 0 && xx < p.w;
        store_through(dst + g, ok ? packed[((y - y_lo) * p.w + xx) * cw + (e.y & 4095)] : 0ull);
        wi += p.step_wi;
        const int carry = wi >= p.row_words ? 1 : 0;
        wi -= carry ? p.row_words : 0;
        ox += p.step_ox + carry;
        oyl += p.step_oy;
        if (ox >= p.ow) ox -= p.ow, ++oyl;
    }
}

// c % 64 == 0, for images whose rows do not fit the tiled kernel's LDS budget.
// Lane l first decodes output word g0 + l of the chunk (row ->
// image/oy/ox, word -> tap/channel word, bounds test) with ordinary vector
// arithmetic, 64 words at once; the 64 element offsets are then broadcast one
// by one (v_readlane) and every word becomes one coalesced 256-byte load, one
// compare and a select into the owning lane.  All 64 loads are independent.
__global__ __launch_bounds__(64 * kIm2colWavesPerBlock) void fused_binarize_im2col_aligned_kernel(const Im2colArgs p) {
    const int lane = threadIdx.x & 63;
    const int wib = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const long long wave = (long long)blockIdx.x * kIm2colWavesPerBlock + wib;
    const long long n_chunks = (p.n_words + 63) / 64;
    const long long stride = (long long)gridDim.x * kIm2colWavesPerBlock;
    const int cw = p.c >> 6;
    for (long long chunk = wave; chunk < n_chunks; chunk += stride) {
        const long long g0 = chunk * 64;
        const uint32_t g = (uint32_t)(g0 + lane);
        bool ok = (long long)g < p.n_words;
        const uint32_t row = p.div_row_words.div(ok ? g : 0u);
        const int wi = (ok ? g : 0u) - row * p.row_words;
        const uint32_t t = p.div_ow.div(row);
        const int ox = row - t * p.ow;
        const uint32_t img = p.div_oh.div(t);
        const int oy = t - img * p.oh;
        const uint32_t tap = p.div_cw.div((uint32_t)wi);  // >= kh*kw for the zero padding word
        const int k = wi - tap * cw;
        const uint32_t a = p.div_kw.div(tap);
        const int b = tap - a * p.kw;
        const int y = oy * p.stride_h - p.pad_h + (int)a * p.dil_h;
        const int xx = ox * p.stride_w - p.pad_w + b * p.dil_w;
        ok = ok && (int)tap < p.kh * p.kw && y >= 0 && y < p.h && xx >= 0 && xx < p.w;
        // element offset of the word's first float (numel < 2^31 checked on the host); 0 when masked
        const uint32_t off = ok ? (((img * p.h + y) * p.w + xx) * p.c + k * 64) : 0u;
        const uint64_t okmask = __ballot(ok);
        uint64_t mine = 0;
#pragma unroll 16
        for (int i = 0; i < 64; ++i) {
            const uint32_t o = __builtin_amdgcn_readlane(off, i);
            const float v = p.x[o + lane];
            uint64_t word = __ballot(v > 0.0f);
            word = ((okmask >> i) & 1) ? word : 0ull;
            mine = (lane == i) ? word : mine;
        }
        if (g0 + lane < p.n_words) p.col[g0 + lane] = mine;
    }
}

// Any c: tap and channel are resolved per lane for every word.
__global__ __launch_bounds__(64 * kIm2colWavesPerBlock) void fused_binarize_im2col_generic_kernel(const Im2colArgs p) {
    const int lane = threadIdx.x & 63;
    const int wib = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const long long wave = (long long)blockIdx.x * kIm2colWavesPerBlock + wib;
    const long long n_chunks = (p.n_words + 63) / 64;
    const long long stride = (long long)gridDim.x * kIm2colWavesPerBlock;
    for (long long chunk = wave; chunk < n_chunks; chunk += stride) {
        const long long g0 = chunk * 64;
        const int count = (int)(p.n_words - g0 < 64 ? p.n_words - g0 : 64);
        uint64_t mine = 0;
        for (int i = 0; i < count; ++i) {
            const uint32_t g = (uint32_t)(g0 + i);  // global word index (n_words < 2^31 checked on the host)
            const uint32_t row = p.div_row_words.div(g);
            const int wi = g - row * p.row_words;
            const uint32_t t = p.div_ow.div(row);
            const int ox = row - t * p.ow;
            const uint32_t img = p.div_oh.div(t);
            const int oy = t - img * p.oh;
            const int e = wi * 64 + lane;
            float v = 0.0f;
            if (e < p.len) {
                const uint32_t tap = p.div_c.div((uint32_t)e);
                const int ch = e - tap * p.c;
                const uint32_t a = p.div_kw.div(tap);
                const int b = tap - a * p.kw;
                const int y = oy * p.stride_h - p.pad_h + (int)a * p.dil_h;
                const int xx = ox * p.stride_w - p.pad_w + b * p.dil_w;
                if (y >= 0 && y < p.h && xx >= 0 && xx < p.w) v = p.x[(((size_t)img * p.h + y) * p.w + xx) * p.c + ch];
            }
            const uint64_t word = __ballot(v > 0.0f);
            mine = (lane == i) ? word : mine;
        }
        if (lane < count) p.col[g0 + lane] = mine;
    }
}

}  // namespace dab

extern "C" int dab_col_row_words(int kh, int kw, int c) { return (kh * kw * c + 127) / 128 * 2; }

extern "C" int dab_fused_binarize_im2col(const float *x, int n, int h, int w, int c, int kh, int kw, int pad_h, int pad_w,
                                         int stride_h, int stride_w, int dil_h, int dil_w, uint64_t *col,
                                         dab_stream_t stream) {
    using namespace dab;
    DAB_REQUIRE(x && col, "dab_fused_binarize_im2col: null pointer");
    DAB_REQUIRE(n > 0 && h > 0 && w > 0 && c > 0 && kh > 0 && kw > 0, "dab_fused_binarize_im2col: non-positive dimension");
    DAB_REQUIRE(pad_h >= 0 && pad_w >= 0 && stride_h > 0 && stride_w > 0 && dil_h > 0 && dil_w > 0,
                "dab_fused_binarize_im2col: bad pad/stride/dilation");
    DAB_REQUIRE((long long)kh * kw * c < 60000, "kernel_h * kernel_w * im.c must be smaller than 60000");
    Im2colArgs a;
    a.x = x, a.col = col;
    a.n = n, a.h = h, a.w = w, a.c = c;
    a.kh = kh, a.kw = kw, a.pad_h = pad_h, a.pad_w = pad_w;
    a.stride_h = stride_h, a.stride_w = stride_w, a.dil_h = dil_h, a.dil_w = dil_w;
    a.oh = out_dim(h, pad_h, kh, dil_h, stride_h), a.ow = out_dim(w, pad_w, kw, dil_w, stride_w);
    DAB_REQUIRE(a.oh > 0 && a.ow > 0, "dab_fused_binarize_im2col: empty output");
    a.len = kh * kw * c;
    a.row_words = dab_col_row_words(kh, kw, c);
    a.n_words = (long long)n * a.oh * a.ow * a.row_words;
    if (a.n_words >= (1ll << 31)) return fail(DAB_EUNSUPPORTED, "dab_fused_binarize_im2col: more than 2^31 output words");
    if ((long long)n * h * w * c >= (1ll << 31)) return fail(DAB_EUNSUPPORTED, "dab_fused_binarize_im2col: more than 2^31 input elements");
    a.div_row_words = FastDiv((uint32_t)a.row_words);
    a.div_ow = FastDiv((uint32_t)a.ow), a.div_oh = FastDiv((uint32_t)a.oh);
    a.div_c = FastDiv((uint32_t)c), a.div_kw = FastDiv((uint32_t)kw);
    a.div_cw = FastDiv((uint32_t)(c >= 64 ? c / 64 : 1));
    a.rows_per_block = 0, a.blocks_per_image = 0;
    const long long chunks = (a.n_words + 63) / 64;
    long long blocks = (chunks + kIm2colWavesPerBlock - 1) / kIm2colWavesPerBlock;
    const long long cap = (long long)simd_count() * 8;
    if (blocks > cap) blocks = cap;
    if (c % 64 == 0) {
        // Rows per block.  A block's time goes with the input rows it packs, rows + halo; a CU holds one block, so a
        // launch takes ceil(blocks / CUs) rounds of them, and from the second round on the loads of one block run
        // beside the stores of another (measured: 15 % less than the rounds' sum).  The candidate with the smallest
        // estimate wins, among those whose packed rows fit 48 KB; measured at 64 and 256 images of 28x28x128,
        // 14x14x256 and 7x7x512 with every candidate: the estimate picks the fastest or one within 3 % of it.
        const int cw = c / 64;
        auto in_rows = [&](int r) { return (long long)(r - 1) * stride_h + (long long)(kh - 1) * dil_h + 1; };
        auto lds_bytes = [&](int r) { return (in_rows(r) * w * cw + a.row_words) * 8; };  // packed rows + the word table
        const long long cus = simd_count() / 4;
        int r = 1;
        double best = 0.0;
        for (int cand = 1; cand <= a.oh; ++cand) {
            if (lds_bytes(cand) > 48 * 1024) break;
            const long long rounds = ((long long)n * ((a.oh + cand - 1) / cand) + cus - 1) / cus;
            const double est = (double)rounds * (double)in_rows(cand) * (rounds > 1 ? 0.85 : 1.0);
            if (cand == 1 || est <= best) best = est, r = cand;
        }
        if (lds_bytes(r) <= 48 * 1024) {
            a.rows_per_block = r;
            a.blocks_per_image = (a.oh + r - 1) / r;
            a.packed_words = (int)(in_rows(r) * w * cw);
            const int step_pix = 512 / a.row_words;
            a.step_wi = 512 % a.row_words, a.step_ox = step_pix % a.ow, a.step_oy = step_pix / a.ow;
            hipLaunchKernelGGL(fused_binarize_im2col_tiled_kernel<512>, dim3((unsigned)(n * a.blocks_per_image)), dim3(512),
                               (size_t)lds_bytes(r), as_stream(stream), a);
            DAB_LAUNCH_CHECK();
            return DAB_OK;
        }
    }
    if (c % 64 == 0)
        hipLaunchKernelGGL(fused_binarize_im2col_aligned_kernel, dim3((unsigned)blocks), dim3(64 * kIm2colWavesPerBlock), 0,
                           as_stream(stream), a);
    else
        hipLaunchKernelGGL(fused_binarize_im2col_generic_kernel, dim3((unsigned)blocks), dim3(64 * kIm2colWavesPerBlock),
                           0, as_stream(stream), a);
    DAB_LAUNCH_CHECK();
    return DAB_OK;
}
