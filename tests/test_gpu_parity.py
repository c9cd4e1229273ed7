"""GPU parity: HIP kernels (through the C ABI) vs the CPU oracle, bit-exact.

Same seeded inputs go to both sides.  Sizes are chosen so the oracle finishes
in seconds; the benchmark's full shapes at batch 64 are checked through
size-independent properties in test_gpu_properties.py.
"""
import numpy as np
import pytest
import torch

import oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dab():
    import dabnn_amd
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return dabnn_amd


def rng(seed):
    return np.random.default_rng(seed)


def dev_f(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


def dev_u(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.uint64).view(np.int64)).cuda()


def host_u(t):
    return t.cpu().numpy().view(np.uint64)


def special_floats(shape, seed):
    x = rng(seed).standard_normal(shape).astype(np.float32)
    x.flat[::7] = 0.0
    x.flat[3::11] = -0.0
    x.flat[5::13] = np.nan
    x.flat[1::17] = np.float32(1e-45)
    x.flat[2::19] = -np.float32(1e-45)
    x.flat[4::23] = np.inf
    x.flat[6::29] = -np.inf
    return x


# ---------------------------------------------------------------- bitpack
@pytest.mark.parametrize("shape", [
    (1, 8, 8, 128), (1, 1, 1, 64), (2, 5, 3, 192), (1, 56, 56, 64), (1, 56, 56, 512), (3, 7, 7, 512), (1, 9, 7, 64),
    (1, 64, 64, 256),  # the shape of tests/bitpack_test.cpp:38-60
])
def test_pack_mat(dab, shape):
    x = special_floats(shape, 1)
    got = host_u(dab.pack_mat(dev_f(x)))
    want = np.stack([orc.pack_mat(img) for img in x])
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("shape", [(1, 64, 4, 5), (2, 128, 7, 9), (1, 512, 56, 56), (3, 192, 1, 1)])
def test_bitpack_nchw(dab, shape):
    x = special_floats(shape, 2)
    got = host_u(dab.bitpack_nchw(dev_f(x)))
    want = np.stack([orc.pack_nchw(img) for img in x])
    np.testing.assert_array_equal(got, want)
    # and it is pack_mat of the NHWC permutation
    nhwc = np.ascontiguousarray(np.transpose(x, (0, 2, 3, 1)))
    np.testing.assert_array_equal(got, host_u(dab.pack_mat(dev_f(nhwc))))


def test_pack_mat_rejects_bad_channels(dab):
    with pytest.raises(RuntimeError, match="multiple of 64"):
        dab.pack_mat(torch.zeros((1, 2, 2, 100), device="cuda"))


@pytest.mark.parametrize("n,h,w,cw,ph,pw", [(1, 4, 6, 2, 1, 2), (3, 7, 7, 8, 1, 1), (1, 5, 5, 1, 0, 0)])
def test_pad_bit(dab, n, h, w, cw, ph, pw):
    x = rng(3).integers(0, 2**64, size=(n, h, w, cw), dtype=np.uint64)
    got = host_u(dab.pad(dev_u(x), ph, pw))
    want = np.stack([orc.pad_bit(img, ph, pw) for img in x])
    np.testing.assert_array_equal(got, want)


# ---------------------------------------------------------------- Split / Shuffle on packed words
@pytest.mark.parametrize("shape", [(1, 4, 6, 2), (3, 7, 7, 4), (2, 5, 3, 6), (5, 14, 14, 8), (64, 28, 28, 4)])
def test_split_and_shuffle_bit(dab, shape):
    x = rng(5).integers(0, 2**64, size=shape, dtype=np.uint64)
    o1, o2 = dab.split_bit(dev_u(x))
    w1, w2 = orc.split_bit(x)
    np.testing.assert_array_equal(host_u(o1), w1)
    np.testing.assert_array_equal(host_u(o2), w2)
    np.testing.assert_array_equal(host_u(dab.shuffle_bit_inplace(dev_u(x))), orc.shuffle_bit(x.copy()))


def test_split_and_shuffle_reject_other_channel_counts(dab):
    for cw in (1, 3, 10):
        x = torch.zeros((1, 2, 2, cw), dtype=torch.int64, device="cuda")
        with pytest.raises(RuntimeError, match="Split: %d channels" % (cw * 64)):
            dab.split_bit(x)
        with pytest.raises(RuntimeError, match="Shuffle: %d channels" % (cw * 64)):
            dab.shuffle_bit_inplace(x)


# ---------------------------------------------------------------- fused_binarize_im2col
@pytest.mark.parametrize("n,h,w,c,k,pad,stride,dil", [
    (1, 8, 8, 128, 3, 1, 1, 1), (2, 8, 8, 64, 3, 1, 2, 1), (1, 7, 9, 192, 3, 1, 1, 1), (1, 6, 6, 128, 5, 2, 2, 1),
    (2, 5, 5, 3, 3, 1, 1, 1), (1, 4, 4, 100, 1, 0, 1, 1), (1, 10, 10, 64, 3, 2, 1, 2), (1, 28, 28, 128, 3, 1, 1, 1),
    (1, 14, 14, 256, 3, 1, 2, 1), (2, 7, 7, 512, 3, 1, 1, 1), (1, 3, 3, 128, 3, 0, 2, 1),
    # enough images that a block of the row-tiled kernel takes several output rows (2, 8 = whole image, 2 with a
    # ragged last block, 1 under stride 2)
    (40, 14, 14, 64, 3, 1, 1, 1), (300, 8, 8, 64, 3, 1, 1, 1), (150, 9, 9, 64, 5, 2, 2, 2), (70, 12, 10, 128, 3, 1, 2, 1),
])
def test_fused_binarize_im2col(dab, n, h, w, c, k, pad, stride, dil):
    x = special_floats((n, h, w, c), 4)
    got = host_u(dab.fused_binarize_im2col(dev_f(x), k, k, pad, pad, stride, stride, dil, dil))
    want = np.concatenate([orc.fused_binarize_im2col(img, k, k, pad, pad, stride, stride, dil, dil) for img in x])
    np.testing.assert_array_equal(got, want)


def test_fused_binarize_im2col_size_limit(dab):
    with pytest.raises(RuntimeError, match="smaller than 60000"):
        dab.fused_binarize_im2col(torch.zeros((1, 1, 1, 60000), device="cuda"), 1, 1, 0, 0, 1, 1)


# ---------------------------------------------------------------- bgemm
@pytest.mark.parametrize("m,n,k", [
    (159, 253, 68),  # tests/bgemm_test.cpp:12-27
    (128, 784, 18), (256, 196, 36), (512, 49, 72),  # tests/bgemm_test.cpp:132-181
    (33, 17, 10), (8, 64, 1), (16, 1, 9), (5, 70, 3), (1, 1, 1), (64, 130, 8), (72, 65, 25),
    (512, 3136, 72),  # the benchmark's standalone bgemm
])
def test_bgemm_matches_naive(dab, m, n, k):
    a = rng(10).integers(0, 2**64, size=(k, m), dtype=np.uint64)
    b = rng(11).integers(0, 2**64, size=(n, k), dtype=np.uint64)
    c0 = rng(12).integers(0, 1000, size=(n, m)).astype(np.float32)  # C is accumulated into
    want = c0.copy()
    orc.bgemm_naive(m, n, k, a, m, b, k, want, m)
    c = dev_f(c0)
    dab.bgemm(m, n, k, dev_u(a), m, dev_u(b), k, c, m)
    np.testing.assert_array_equal(c.cpu().numpy(), want)


@pytest.mark.parametrize("m,n,k,lda,ldb,ldc", [(24, 70, 5, 31, 9, 28), (24, 70, 18, 24, 20, 27), (40, 64, 36, 48, 36, 40),
                                               (7, 9, 3, 8, 4, 11)])
def test_bgemm_leading_dimensions(dab, m, n, k, lda, ldb, ldc):
    a = rng(13).integers(0, 2**64, size=(k, lda), dtype=np.uint64)
    b = rng(14).integers(0, 2**64, size=(n, ldb), dtype=np.uint64)
    c0 = rng(15).integers(0, 50, size=(n, ldc)).astype(np.float32)
    want = c0.copy()
    orc.bgemm_naive(m, n, k, a, lda, b, ldb, want, ldc)
    c = dev_f(c0)
    dab.bgemm(m, n, k, dev_u(a), lda, dev_u(b), ldb, c, ldc)
    np.testing.assert_array_equal(c.cpu().numpy(), want)


@pytest.mark.parametrize("m,n,k,lda,ldb,ldc", [(512, 49, 72, 512, 72, 512), (128, 784, 18, 128, 18, 128), (24, 70, 5, 31, 9, 28),
                                               (72, 65, 25, 72, 25, 72), (16, 3, 9, 16, 9, 16), (40, 64, 36, 48, 36, 40)])
def test_bgemm_overwrite_is_fill_then_bgemm(dab, m, n, k, lda, ldb, ldc):
    """The pair output_mat->fill(0) + bgemm of dabnn/layers/BinConv.cpp:153-165 as one store: whatever C held before
    (NaN included) is gone, elements outside the m x n window (leading-dimension padding) are untouched."""
    a = rng(13).integers(0, 2**64, size=(k, lda), dtype=np.uint64)
    b = rng(14).integers(0, 2**64, size=(n, ldb), dtype=np.uint64)
    c0 = rng(15).standard_normal((n, ldc)).astype(np.float32)
    c0[::3, ::5] = np.nan
    want = c0.copy()
    want[:, :m] = 0.0
    orc.bgemm_naive(m, n, k, a, lda, b, ldb, want, ldc)
    c = dev_f(c0)
    dab.bgemm_overwrite(m, n, k, dev_u(a), lda, dev_u(b), ldb, c, ldc)
    np.testing.assert_array_equal(c.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_bgemm_rejects_bad_arguments(dab):
    a = torch.zeros(16, dtype=torch.int64, device="cuda")
    c = torch.zeros(16, dtype=torch.float32, device="cuda")
    with pytest.raises(RuntimeError, match="leading dimension"):
        dab.bgemm(4, 2, 2, a, 3, a, 2, c, 4)
    with pytest.raises(RuntimeError):
        dab.bgemm(0, 2, 2, a, 4, a, 2, c, 4)


def test_weight_transpose(dab):
    w = rng(16).integers(0, 2**64, size=(24, 18), dtype=np.uint64)
    np.testing.assert_array_equal(host_u(dab.weight_transpose(dev_u(w))), orc.weight_transpose(w))


def test_im2col_transpose_bgemm_equals_baseline_bconv(dab):
    """The chain asserted by tests/bgemm_test.cpp:32-130 (3x3 stride 2 -> 1x1 output; 5x5 pad 2 stride 2)."""
    for (h, c, cout, k, pad, stride) in [(3, 128, 128, 3, 0, 2), (9, 128, 16, 5, 2, 2)]:
        x = rng(17).standard_normal((1, h, h, c)).astype(np.float32)
        wgt = rng(18).integers(0, 2**64, size=(cout, k * k * c // 64), dtype=np.uint64)
        want = orc.baseline_bconv(orc.pack_mat(x[0]), wgt, k, k, pad, pad, stride, stride)
        col = dab.fused_binarize_im2col(dev_f(x), k, k, pad, pad, stride, stride)
        nrow, kk = col.shape
        c_out = torch.zeros((nrow, cout), dtype=torch.float32, device="cuda")
        dab.bgemm(cout, nrow, kk, dab.weight_transpose(dev_u(wgt)), cout, col, kk, c_out, cout)
        np.testing.assert_array_equal(c_out.cpu().numpy().reshape(want.shape), want)


# ---------------------------------------------------------------- direct 3x3 bconv
@pytest.mark.parametrize("n,h,w,cin,cout,stride,pad", [
    (1, 8, 8, 64, 64, 1, 1), (1, 8, 8, 128, 128, 1, 1), (1, 8, 8, 256, 64, 1, 1), (1, 8, 8, 512, 32, 1, 1),
    (2, 9, 7, 64, 8, 1, 1), (3, 7, 10, 128, 24, 2, 1), (1, 6, 6, 64, 40, 1, 0), (2, 5, 5, 256, 16, 2, 0),
    (1, 3, 3, 128, 128, 2, 0),  # 1x1 output
    (5, 13, 13, 64, 72, 1, 1),  # pixel count not a multiple of 64, channel groups not a multiple of 4
    (1, 64, 64, 64, 64, 1, 1), (1, 64, 64, 64, 64, 2, 1),  # tests/bconv_test.cpp:164-250
    (1, 64, 64, 128, 128, 1, 1),  # tests/bconv_test.cpp bconv_test_3x3_128
    (1, 32, 32, 256, 256, 1, 1), (1, 16, 16, 512, 256, 1, 1), (1, 16, 16, 512, 1024, 2, 1),
    (1, 56, 56, 64, 64, 1, 1), (1, 28, 28, 128, 128, 1, 1), (1, 14, 14, 256, 256, 1, 1), (1, 7, 7, 512, 512, 1, 1),
    (1, 56, 56, 64, 128, 2, 1), (1, 28, 28, 128, 256, 2, 1), (1, 14, 14, 256, 512, 2, 1),  # the seven ResNet-18 stage shapes of the benchmark, batch 1
    # more than 1024 work items of 64 pixels x 8 channels (2048 with 512 input channels): the unit kernel (everything above runs the small-problem
    # kernel), every channel count at stride 1 and 2, ragged last tiles, no padding, and the two narrow builds
    (6, 56, 56, 64, 64, 1, 1), (9, 28, 28, 128, 128, 1, 1), (17, 14, 14, 256, 256, 1, 1), (25, 7, 7, 512, 512, 1, 1),
    (10, 56, 56, 64, 128, 2, 1), (20, 28, 28, 128, 256, 2, 1), (30, 14, 14, 256, 512, 2, 1), (40, 9, 9, 64, 272, 1, 0), (48, 7, 7, 512, 512, 1, 1),
    (64, 56, 56, 64, 64, 1, 1), (200, 28, 28, 128, 128, 1, 1),
    # 1024 input channels (dabnn/layers/BinConv.cpp:118 lists them): two passes over 512 channels each, the second
    # adding to the first; a single tile, ragged tiles at stride 1 and 2, no padding, and enough work for the
    # large-unit build
    (1, 7, 7, 1024, 64, 1, 1), (3, 9, 11, 1024, 24, 2, 1), (2, 6, 6, 1024, 1024, 1, 0), (100, 7, 7, 1024, 1024, 1, 1),
])
def test_bconv_3x3_matches_baseline_bconv(dab, n, h, w, cin, cout, stride, pad):
    cw = cin // 64
    x = rng(20).integers(0, 2**64, size=(n, h, w, cw), dtype=np.uint64)
    wgt = rng(21).integers(0, 2**64, size=(cout, 9 * cw), dtype=np.uint64)
    got = dab.bconv_3x3(dev_u(x), dev_u(wgt), stride, pad).cpu().numpy()
    want = np.stack([orc.baseline_bconv(img, wgt, 3, 3, pad, pad, stride, stride) for img in x])
    np.testing.assert_array_equal(got, want)


def test_bconv_3x3_equals_pad_then_bconv_on_padded(dab):
    """bconv_3x3(pad(x)) of the reference == the unpadded entry point with pad 1."""
    x = rng(22).integers(0, 2**64, size=(2, 10, 10, 2), dtype=np.uint64)
    wgt = rng(23).integers(0, 2**64, size=(16, 18), dtype=np.uint64)
    a = dab.bconv_3x3(dev_u(x), dev_u(wgt), 1, 1)
    b = dab.bconv_3x3(dab.pad(dev_u(x), 1, 1), dev_u(wgt), 1, 0)
    assert torch.equal(a, b)
    want = np.stack([orc.bconv_3x3_padded(orc.pad_bit(img, 1, 1), wgt, 1) for img in x])
    np.testing.assert_array_equal(a.cpu().numpy(), want)


@pytest.mark.parametrize("n,h,w,cin,cout,stride,with_shortcut", [
    (2, 9, 7, 64, 64, 1, True), (1, 14, 14, 256, 256, 1, True), (3, 8, 8, 128, 24, 2, True), (1, 7, 7, 512, 64, 1, False),
    (5, 13, 13, 64, 72, 1, True), (1, 56, 56, 64, 64, 1, True),
    # the unit kernel (more than 1024 work items)
    (6, 56, 56, 64, 64, 1, True), (9, 28, 28, 128, 72, 1, True), (17, 14, 14, 256, 256, 1, False), (25, 7, 7, 512, 512, 1, True), (48, 7, 7, 512, 512, 1, True),
    (20, 28, 28, 128, 256, 2, True),
])
def test_bconv_affine_add_equals_three_reference_layers(dab, n, h, w, cin, cout, stride, with_shortcut):
    r = rng(24)
    cw = cin // 64
    x = r.integers(0, 2**64, size=(n, h, w, cw), dtype=np.uint64)
    wgt = r.integers(0, 2**64, size=(cout, 9 * cw), dtype=np.uint64)
    a = (r.standard_normal(cout) / 50).astype(np.float32)
    b = r.standard_normal(cout).astype(np.float32)
    want = np.stack([orc.baseline_bconv(img, wgt, 3, 3, 1, 1, stride, stride) for img in x])
    sc = r.standard_normal(want.shape).astype(np.float32) if with_shortcut else None
    for img in want:
        orc.affine_inplace(img, a, b)
    if with_shortcut:
        want = want + sc  # add_inplace: one rounding per element, as numpy
    got = dab.bconv_3x3_affine_add(dev_u(x), dev_u(wgt), dev_f(a), dev_f(b), dev_f(sc) if with_shortcut else None, stride, 1)
    np.testing.assert_array_equal(got.cpu().numpy(), want)


@pytest.mark.parametrize("n,h,w,cin,cout,stride,with_shortcut", [
    (2, 9, 7, 64, 64, 1, True), (1, 14, 14, 256, 256, 1, True), (3, 8, 8, 128, 128, 2, True), (1, 7, 7, 512, 64, 1, False),
    (5, 13, 13, 64, 192, 1, True), (1, 56, 56, 64, 64, 1, True), (4, 7, 7, 512, 512, 1, True), (2, 14, 14, 256, 512, 2, True),
    (3, 28, 28, 128, 128, 1, True), (70, 5, 5, 256, 64, 1, False),
    # the unit kernel (more than 1024 work items)
    (6, 56, 56, 64, 64, 1, True), (9, 28, 28, 128, 128, 1, True), (17, 14, 14, 256, 256, 1, True), (25, 7, 7, 512, 512, 1, True),
    (30, 14, 14, 256, 512, 2, False), (10, 56, 56, 64, 128, 2, True), (48, 7, 7, 512, 512, 1, True),
])
def test_bconv_affine_add_sign_packs_its_own_output(dab, n, h, w, cin, cout, stride, with_shortcut):
    """The fp32 result equals the three reference layers, and the packed copy is pack_mat of that result, bit for bit
    (zeros, negatives and the exact-zero sums of the shortcut included)."""
    r = rng(25)
    cw = cin // 64
    x = r.integers(0, 2**64, size=(n, h, w, cw), dtype=np.uint64)
    wgt = r.integers(0, 2**64, size=(cout, 9 * cw), dtype=np.uint64)
    a = (r.standard_normal(cout) / 50).astype(np.float32)
    b = r.standard_normal(cout).astype(np.float32)
    a[::5] = 0.0  # a*cnt + b == b: constant channels, some of them exactly zero
    b[::10] = 0.0
    want = np.stack([orc.baseline_bconv(img, wgt, 3, 3, 1, 1, stride, stride) for img in x])
    sc = r.standard_normal(want.shape).astype(np.float32) if with_shortcut else None
    for img in want:
        orc.affine_inplace(img, a, b)
    if with_shortcut:
        sc[:, :, :, ::10] = 0.0
        want = want + sc
    got, packed = dab.bconv_3x3_affine_add_sign(dev_u(x), dev_u(wgt), dev_f(a), dev_f(b),
                                                dev_f(sc) if with_shortcut else None, stride, 1)
    np.testing.assert_array_equal(got.cpu().numpy(), want)
    np.testing.assert_array_equal(host_u(packed), np.stack([orc.pack_mat(img) for img in want]))


@pytest.mark.parametrize("n,h,w,cin,cout,stride,pad", [
    # the shapes the row-split kernel is there for: 7 x 7 x 512 and the stride-2 layer into it, at batch 64 and 40
    (64, 7, 7, 512, 512, 1, 1), (64, 14, 14, 256, 512, 2, 1), (44, 7, 7, 512, 512, 1, 1),
    # a pixel count that is no multiple of 64, channel counts that are no multiple of a 32-channel segment, ranges
    # of work that cross tiles in the middle of a segment
    (200, 9, 7, 512, 88, 1, 1), (900, 7, 7, 512, 24, 1, 1), (130, 13, 11, 256, 104, 2, 1), (360, 5, 9, 512, 200, 2, 1),
    # no padding, and a stride of 3
    (340, 9, 9, 512, 64, 1, 0), (300, 15, 15, 256, 72, 3, 1),
    # small batches, where it runs in place of the small-problem kernel: one image of the three deep stage shapes,
    # a single tile that is not full, eight output channels, 256 input channels at stride 1 up to its bound
    (1, 7, 7, 512, 512, 1, 1), (1, 14, 14, 256, 256, 1, 1), (1, 14, 14, 256, 512, 2, 1), (3, 7, 7, 512, 40, 1, 1),
    (2, 5, 5, 256, 8, 1, 1), (16, 14, 14, 256, 256, 1, 1), (20, 14, 14, 256, 256, 1, 1),
])
def test_row_split_kernel_counts(dab, n, h, w, cin, cout, stride, pad):
    """dab_bconv3x3 through its row-split build (blocks of three waves, one kernel row each, partial counts added in
    LDS), named by the library so that the case cannot drift to another kernel: the whole batch against
    baseline_bconv bit for bit."""
    from dabnn_amd import capi
    oh, ow = (h + 2 * pad - 3) // stride + 1, (w + 2 * pad - 3) // stride + 1
    assert capi.lib.dab_bconv3x3_counts_build(n * oh * ow, cin, cout, stride) == 3
    r = rng(31)
    cw = cin // 64
    x = r.integers(0, 2**64, size=(n, h, w, cw), dtype=np.uint64)
    wgt = r.integers(0, 2**64, size=(cout, 9 * cw), dtype=np.uint64)
    got = dab.bconv_3x3(dev_u(x), dev_u(wgt), stride, pad).cpu().numpy()
    want = np.stack([orc.baseline_bconv(img, wgt, 3, 3, pad, pad, stride, stride) for img in x])
    np.testing.assert_array_equal(got, want)
    # the entry point with an epilogue (on whichever build it takes at this size) agrees with it
    a = (r.standard_normal(cout) / 50).astype(np.float32)
    b = r.standard_normal(cout).astype(np.float32)
    fused = dab.bconv_3x3_affine_add(dev_u(x), dev_u(wgt), dev_f(a), dev_f(b), None, stride, pad)
    sep = dev_f(want.copy())
    dab.affine_inplace(sep, dev_f(a), dev_f(b))
    assert torch.equal(fused, sep)


@pytest.mark.parametrize("n,h,w,cin,cout,stride,with_shortcut", [
    # the sizes between the small and the mid-sized problems at which the entry points with an epilogue take the
    # row-split kernel: the deep stage shapes of Bi-Real-18 at batch 16 to 64, a ragged pixel count, no shortcut
    (32, 7, 7, 512, 512, 1, True), (64, 7, 7, 512, 512, 1, True), (16, 14, 14, 256, 256, 1, True),
    (24, 14, 14, 256, 512, 2, True), (50, 9, 7, 512, 192, 1, False), (21, 13, 15, 256, 320, 1, True),
])
def test_fused_epilogues_through_the_row_split_kernel(dab, n, h, w, cin, cout, stride, with_shortcut):
    """BinConv + Affine + Add (+ sign) through the row-split kernel, named by the library: the fp32 result against the
    three reference layers and the packed copy against pack_mat of it, bit for bit, whole batch."""
    from dabnn_amd import capi
    oh, ow = (h + 2 - 3) // stride + 1, (w + 2 - 3) // stride + 1
    assert capi.lib.dab_bconv3x3_epilogue_build(n * oh * ow, cin, cout, stride, 1) == 3
    r = rng(41)
    cw = cin // 64
    x = r.integers(0, 2**64, size=(n, h, w, cw), dtype=np.uint64)
    wgt = r.integers(0, 2**64, size=(cout, 9 * cw), dtype=np.uint64)
    a = (r.standard_normal(cout) / 50).astype(np.float32)
    b = r.standard_normal(cout).astype(np.float32)
    a[::5] = 0.0
    b[::10] = 0.0
    want = np.stack([orc.baseline_bconv(img, wgt, 3, 3, 1, 1, stride, stride) for img in x])
    sc = r.standard_normal(want.shape).astype(np.float32) if with_shortcut else None
    for img in want:
        orc.affine_inplace(img, a, b)
    if with_shortcut:
        sc[:, :, :, ::10] = 0.0
        want = want + sc
    got, packed = dab.bconv_3x3_affine_add_sign(dev_u(x), dev_u(wgt), dev_f(a), dev_f(b),
                                                dev_f(sc) if with_shortcut else None, stride, 1)
    np.testing.assert_array_equal(got.cpu().numpy(), want)
    np.testing.assert_array_equal(host_u(packed), np.stack([orc.pack_mat(img) for img in want]))
    if capi.lib.dab_bconv3x3_epilogue_build(n * oh * ow, cin, cout, stride, 0) == 3:
        plain = dab.bconv_3x3_affine_add(dev_u(x), dev_u(wgt), dev_f(a), dev_f(b), dev_f(sc) if with_shortcut else None, stride, 1)
        np.testing.assert_array_equal(plain.cpu().numpy(), want)


@pytest.mark.parametrize("n,h,w,cin,cout,stride,build", [
    # the four-waves-per-SIMD build of the unit kernel (many units per wave): 128 input channels from 8 units per wave
    # on, 64 input channels from 4 -- the stage-2 and stage-1 blocks of Bi-Real-18 at batch 256
    (170, 28, 28, 128, 128, 1, 2), (44, 56, 56, 64, 64, 1, 2),
    # just below the switch: the wide build on nearly the same problem
    (160, 28, 28, 128, 128, 1, 1),
    # 256 and 512 input channels: the builds with units of twice the channels, taken from six such units per wave on
    (256, 14, 14, 256, 256, 1, 2), (200, 7, 7, 512, 512, 1, 2), (190, 14, 14, 256, 512, 2, 1),
])
def test_fused_epilogues_of_the_named_build(dab, n, h, w, cin, cout, stride, build):
    """BinConv + Affine + Add (+ sign) through the build the test names (asked from the library, so the case cannot
    drift to another kernel unnoticed): images 0, the middle one and the last against the three reference layers
    bit for bit, the whole batch against the counts-only kernel followed by the separate Affine, Add and pack_mat."""
    from dabnn_amd import capi
    oh = (h + 2 - 3) // stride + 1
    assert capi.lib.dab_bconv3x3_build(n * oh * oh, cin, cout) == build
    r = rng(26)
    cw = cin // 64
    x = r.integers(0, 2**64, size=(n, h, w, cw), dtype=np.uint64)
    wgt = r.integers(0, 2**64, size=(cout, 9 * cw), dtype=np.uint64)
    a = (r.standard_normal(cout) / 50).astype(np.float32)
    b = r.standard_normal(cout).astype(np.float32)
    a[::5] = 0.0
    b[::10] = 0.0
    sc = r.standard_normal((n, oh, oh, cout)).astype(np.float32)
    sc[:, :, :, ::10] = 0.0
    xd, wd, ad, bd, scd = dev_u(x), dev_u(wgt), dev_f(a), dev_f(b), dev_f(sc)
    sep = dab.bconv_3x3(xd, wd, stride, 1)
    dab.affine_inplace(sep, ad, bd)
    dab.add_inplace(sep, scd)
    got1 = dab.bconv_3x3_affine_add(xd, wd, ad, bd, scd, stride, 1)
    got2, packed = dab.bconv_3x3_affine_add_sign(xd, wd, ad, bd, scd, stride, 1)
    assert torch.equal(got1, sep)
    assert torch.equal(got2, sep)
    assert torch.equal(packed, dab.pack_mat(sep))
    nosc = dab.bconv_3x3_affine_add(xd, wd, ad, bd, None, stride, 1)
    for i in (0, n // 2 - 2, n - 1):
        want = orc.baseline_bconv(x[i], wgt, 3, 3, 1, 1, stride, stride)
        orc.affine_inplace(want, a, b)
        np.testing.assert_array_equal(nosc[i].cpu().numpy(), want)
        want = want + sc[i]
        np.testing.assert_array_equal(got1[i].cpu().numpy(), want)
        np.testing.assert_array_equal(got2[i].cpu().numpy(), want)
        np.testing.assert_array_equal(host_u(packed[i]), orc.pack_mat(want))


@pytest.mark.parametrize("n,h,w,cout,stride", [
    (168, 56, 56, 64, 1),    # a stage-1 block of Bi-Real-18 at batch 168: 8232 tiles
    (180, 55, 55, 64, 1),    # a last tile that is not full
    (170, 112, 112, 128, 2),  # two 64-channel tiles per pixel, stride 2
])
def test_fused_epilogues_of_the_shared_tile_kernel(dab, n, h, w, cout, stride):
    """BinConv + Affine + Add (+ sign) over 64 input channels at a batch where a block's waves share a tile (asked
    from the library): bit for bit the unit kernel's result on the two halves of the batch, which are below the
    switch; three images against the three reference layers."""
    from dabnn_amd import capi
    oh = (h + 2 - 3) // stride + 1
    assert capi.lib.dab_bconv3x3_fused_shares_tiles(n * oh * oh, 64, cout) == 1
    assert capi.lib.dab_bconv3x3_fused_shares_tiles((n // 2 + 1) * oh * oh, 64, cout) == 0
    r = rng(27)
    x = r.integers(0, 2**64, size=(n, h, w, 1), dtype=np.uint64)
    wgt = r.integers(0, 2**64, size=(cout, 9), dtype=np.uint64)
    a = (r.standard_normal(cout) / 50).astype(np.float32)
    b = r.standard_normal(cout).astype(np.float32)
    a[::5] = 0.0
    sc = r.standard_normal((n, oh, oh, cout)).astype(np.float32)
    sc[:, :, :, ::10] = 0.0
    xd, wd, ad, bd, scd = dev_u(x), dev_u(wgt), dev_f(a), dev_f(b), dev_f(sc)
    got1 = dab.bconv_3x3_affine_add(xd, wd, ad, bd, scd, stride, 1)
    got2, packed = dab.bconv_3x3_affine_add_sign(xd, wd, ad, bd, scd, stride, 1)
    nosc = dab.bconv_3x3_affine_add(xd, wd, ad, bd, None, stride, 1)
    half = n // 2
    for lo, hi in ((0, half), (half, n)):
        want, want_bits = dab.bconv_3x3_affine_add_sign(xd[lo:hi].contiguous(), wd, ad, bd, scd[lo:hi].contiguous(), stride, 1)
        assert torch.equal(got1[lo:hi], want)
        assert torch.equal(got2[lo:hi], want)
        assert torch.equal(packed[lo:hi], want_bits)
        assert torch.equal(nosc[lo:hi], dab.bconv_3x3_affine_add(xd[lo:hi].contiguous(), wd, ad, bd, None, stride, 1))
    for i in (0, half - 1, n - 1):
        want = orc.baseline_bconv(x[i], wgt, 3, 3, 1, 1, stride, stride)
        orc.affine_inplace(want, a, b)
        np.testing.assert_array_equal(nosc[i].cpu().numpy(), want)
        want = want + sc[i]
        np.testing.assert_array_equal(got2[i].cpu().numpy(), want)
        np.testing.assert_array_equal(host_u(packed[i]), orc.pack_mat(want))


def test_bconv_3x3_unsupported_and_invalid(dab):
    from dabnn_amd.capi import DabUnsupported
    x = torch.zeros((1, 4, 4, 3), dtype=torch.int64, device="cuda")  # 192 channels
    w = torch.zeros((8, 27), dtype=torch.int64, device="cuda")
    with pytest.raises(DabUnsupported):
        dab.bconv_3x3(x, w)
    x = torch.zeros((1, 4, 4, 1), dtype=torch.int64, device="cuda")
    with pytest.raises(DabUnsupported):  # cout not a multiple of 8
        dab.bconv_3x3(x, torch.zeros((5, 9), dtype=torch.int64, device="cuda"))
    # 1024 input channels: counts only, no fused epilogue
    x16 = torch.zeros((1, 4, 4, 16), dtype=torch.int64, device="cuda")
    w16 = torch.zeros((8, 144), dtype=torch.int64, device="cuda")
    ab = torch.zeros(8, device="cuda")
    assert dab.bconv_3x3(x16, w16, 1, 1).shape == (1, 4, 4, 8)
    with pytest.raises(DabUnsupported):
        dab.bconv_3x3_affine_add(x16, w16, ab, ab, None, 1, 1)
    with pytest.raises(RuntimeError, match="smaller than the kernel"):
        dab.bconv_3x3(torch.zeros((1, 2, 2, 1), dtype=torch.int64, device="cuda"),
                      torch.zeros((8, 9), dtype=torch.int64, device="cuda"), 1, 0)


# ---------------------------------------------------------------- BinConv layer
@pytest.mark.parametrize("n,h,w,c,cout,k,pad,stride,method", [
    (1, 56, 56, 64, 64, 3, 1, 1, 0),  # the benchmark's single layer
    (2, 8, 8, 64, 32, 3, 1, 2, 0), (2, 8, 8, 128, 64, 3, 1, 1, 0), (1, 7, 7, 512, 16, 3, 1, 1, 0),
    (1, 6, 10, 192, 8, 3, 1, 1, 1),  # 192 channels -> im2col + bgemm
    (2, 9, 9, 128, 16, 5, 2, 2, 1),  # 5x5
    (1, 6, 6, 256, 32, 1, 0, 1, 1),  # 1x1
    (1, 6, 6, 64, 12, 1, 0, 1, 1),  # 64 channels, not 3x3: unpadded filters against padded rows
    (1, 8, 8, 128, 20, 3, 1, 1, 1),  # cout not a multiple of 8 -> bgemm with a ragged last group
    (2, 7, 7, 1024, 32, 3, 1, 1, 0),  # 1024 channels: direct, in two passes
])
def test_binconv_layer_matches_reference_dispatch(dab, n, h, w, c, cout, k, pad, stride, method):
    x = rng(30).standard_normal((n, h, w, c)).astype(np.float32)
    wf = rng(31).standard_normal((cout, k, k, c)).astype(np.float32)
    wp = orc.pack_weight(wf)
    layer = dab.BinConv(dev_u(wp), k, k, pad, pad, stride, stride)
    got = layer(dev_f(x)).cpu().numpy()
    assert layer.method == method
    if c == 64 and k != 3:
        want = np.stack([orc.baseline_bconv(orc.pack_mat(img), wp, k, k, pad, pad, stride, stride) for img in x])
    else:
        want = np.stack([orc.binconv_forward(img, wp, k, k, pad, pad, stride, stride)[0] for img in x])
    np.testing.assert_array_equal(got, want)


def test_binconv_config1_k_minus_2cnt(dab):
    """The benchmark's single 56x56x64 layer: counts, then K - 2*cnt through the folded affine, vs a float convolution."""
    r = rng(32)
    x = r.standard_normal((1, 56, 56, 64)).astype(np.float32)
    wf = r.standard_normal((64, 3, 3, 64)).astype(np.float32)
    layer = dab.BinConv(dev_u(orc.pack_weight(wf)), 3, 3, 1, 1, 1, 1)
    cnt = layer(dev_f(x))
    a, b = orc.bn_fold(np.ones(64), np.zeros(64), np.zeros(64), np.ones(64), 0.0, 576)  # identity BN after a bconv
    y = dab.affine_inplace(cnt.clone(), dev_f(a), dev_f(b)).cpu().numpy()[0]
    xs = torch.from_numpy(np.where(x[0] > 0, 1.0, -1.0)).permute(2, 0, 1)[None]
    ws = torch.from_numpy(np.where(wf > 0, 1.0, -1.0)).permute(0, 3, 1, 2)
    conv = torch.nn.functional.conv2d(torch.nn.functional.pad(xs, (1, 1, 1, 1), value=-1.0), ws)[0].permute(1, 2, 0)
    np.testing.assert_array_equal(y, conv.numpy().astype(np.float32))


# ---------------------------------------------------------------- float glue (1e-4 relative)
RTOL = 1e-4


@pytest.mark.parametrize("n,h,c,cout,k,pad,stride,dil,bias", [
    (1, 4, 2, 2, 3, 1, 1, 1, False), (1, 8, 2, 2, 5, 2, 2, 1, False), (2, 9, 3, 4, 3, 2, 1, 2, True),
    (1, 32, 3, 64, 7, 3, 2, 1, False), (2, 7, 64, 128, 1, 0, 1, 1, False), (3, 1, 512, 1000, 1, 0, 1, 1, True),
    (1, 17, 5, 70, 3, 1, 2, 1, True), (2, 9, 3, 32, 3, 1, 2, 1, False), (1, 23, 16, 20, 3, 1, 1, 1, True),
    (1, 12, 7, 200, 5, 2, 1, 1, True), (130, 1, 33, 65, 1, 0, 1, 1, False), (1, 40, 8, 8, 3, 1, 1, 1, False),
    # three-channel images large enough for the big-tile kernels: ragged pixel and channel tiles, with and without
    # padding, stride 1 and 2, dilation (the 7x7 cases take the one-load-per-tap loader)
    (5, 180, 3, 40, 7, 3, 2, 1, True), (5, 181, 3, 64, 7, 0, 2, 1, False), (2, 150, 3, 33, 7, 3, 1, 1, False),
    (4, 200, 3, 64, 7, 6, 2, 2, True), (4, 190, 3, 24, 3, 1, 2, 1, True),
    # a handful of pixels through a 1x1 convolution: the matrix-vector kernel (ragged channel count, 1 to 8 pixels)
    (1, 1, 512, 1000, 1, 0, 1, 1, True), (8, 1, 64, 70, 1, 0, 1, 1, False), (2, 2, 256, 65, 1, 0, 1, 1, True),
    (5, 1, 1024, 64, 1, 0, 1, 1, False),
    # too few 128-row tiles for the CUs but plenty of 64 x 64 ones: ragged in both directions, padded and not
    (3, 40, 32, 96, 3, 1, 1, 1, True), (2, 61, 8, 130, 1, 0, 1, 1, False),
])
def test_fconv(dab, n, h, c, cout, k, pad, stride, dil, bias):
    r = rng(40)
    x = r.standard_normal((n, h, h, c)).astype(np.float32)
    wgt = r.standard_normal((cout, k, k, c)).astype(np.float32)
    bv = r.standard_normal(cout).astype(np.float32) if bias else None
    got = dab.fconv(dev_f(x), dev_f(wgt), dev_f(bv) if bias else None, k, k, pad, pad, stride, stride, dil,
                    dil).cpu().numpy()
    want = np.stack([orc.fconv(img, wgt, bv, k, k, pad, pad, stride, stride, dil, dil) for img in x])
    scale = np.abs(want).max()
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=RTOL * scale)


@pytest.mark.parametrize("affine,relu,bias", [(True, True, False), (True, False, True), (False, True, True)])
def test_fconv_affine_relu_equals_separate_layers(dab, affine, relu, bias):
    """One pass gives what FpConv2D, Affine and Relu give one after the other, bit for bit against the separate GPU
    layers and within the float tolerance against the CPU restatement."""
    r = rng(43)
    n, h, c, cout, k = 2, 19, 3, 32, 3
    x = r.standard_normal((n, h, h, c)).astype(np.float32)
    wgt = r.standard_normal((cout, k, k, c)).astype(np.float32)
    bv = r.standard_normal(cout).astype(np.float32) if bias else None
    a, b = r.standard_normal(cout).astype(np.float32), r.standard_normal(cout).astype(np.float32)
    got = dab.fconv_affine_relu(dev_f(x), dev_f(wgt), dev_f(bv) if bias else None, dev_f(a) if affine else None,
                                dev_f(b) if affine else None, relu, k, k, 1, 1, 2, 2).cpu().numpy()
    sep = dab.fconv(dev_f(x), dev_f(wgt), dev_f(bv) if bias else None, k, k, 1, 1, 2, 2)
    if affine:
        dab.affine_inplace(sep, dev_f(a), dev_f(b))
    sep = sep.cpu().numpy()
    want = np.stack([orc.fconv(img, wgt, bv, k, k, 1, 1, 2, 2) for img in x])
    if affine:
        want = np.stack([orc.affine_inplace(img.copy(), a, b) for img in want])
    if relu:
        sep, want = np.maximum(sep, 0), np.maximum(want, 0)
    np.testing.assert_array_equal(got, sep)
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=RTOL * np.abs(want).max())


@pytest.mark.parametrize("n,h,w,pad,cout,bias,affine,relu", [
    (24, 112, 112, 1, 32, False, True, True),   # the three-convolution stem's second convolution
    (22, 112, 112, 1, 64, True, False, False),  # its third
    (99, 59, 46, 2, 32, True, True, False),     # 61 output rows: the last column of four tiles is one row high; pad 2
    (25, 114, 114, 0, 64, False, False, True),  # no padding
    (520, 30, 16, 1, 32, True, False, True),    # one tile per row: both pixels beside it are padding; last column two rows high
    (1400, 3, 48, 1, 64, False, True, False),   # three output rows: every column of tiles is cut short
    (1100, 14, 14, 2, 32, False, False, False), # 16 x 16 output of a 14 x 14 image: two rows and columns of padding all round
])
def test_fconv_3x3_over_32_channels_on_split_operands(dab, n, h, w, pad, cout, bias, affine, relu):
    """3x3, stride 1 convolutions over 32 channels that are large enough take the kernel that multiplies on the bf16
    matrix cores with operands split in three (fp32 accuracy): within the float tolerance of the CPU layers on a sample
    of images and of a float64 convolution on all of them, exact on small integers, and an infinity or a NaN in the
    image comes out where IEEE arithmetic puts it (zero times infinity included: a zero weight)."""
    # with a MaxPool behind them these shapes take one pass at either size: the band kernel at batch 18, this kernel's
    # pooled form where it is large enough
    if cout == 64 and pad == 1 and h == 112:
        assert dab.fconv_maxpool_pays(n, h, w, 32, 3, 3, pad, pad, 1, 1, 1, 1, cout)
        assert dab.fconv_maxpool_pays(18, h, w, 32, 3, 3, pad, pad, 1, 1, 1, 1, cout)
    r = rng(61)
    x = r.standard_normal((n, h, w, 32)).astype(np.float32)
    wgt = (r.standard_normal((cout, 3, 3, 32)) / 17).astype(np.float32)
    bv = r.standard_normal(cout).astype(np.float32) if bias else None
    a, b = r.standard_normal(cout).astype(np.float32), r.standard_normal(cout).astype(np.float32)

    def gpu(x, wgt):
        return dab.fconv_affine_relu(dev_f(x), dev_f(wgt), dev_f(bv) if bias else None, dev_f(a) if affine else None,
                                     dev_f(b) if affine else None, relu, 3, 3, pad, pad, 1, 1)

    def cpu(img, wgt):
        y = orc.fconv(img, wgt, bv, 3, 3, pad, pad, 1, 1)
        if affine:
            y = orc.affine_inplace(y.copy(), a, b)
        return np.maximum(y, 0) if relu else y

    def f64(x, wgt):
        y = torch.nn.functional.conv2d(torch.from_numpy(x).cuda().double().permute(0, 3, 1, 2),
                                       torch.from_numpy(wgt).cuda().double().permute(0, 3, 1, 2), padding=pad)
        if bias:
            y = y + torch.from_numpy(bv).cuda().double().view(1, -1, 1, 1)
        if affine:
            y = y * torch.from_numpy(a).cuda().double().view(1, -1, 1, 1) + torch.from_numpy(b).cuda().double().view(1, -1, 1, 1)
        if relu:
            y = torch.where(y < 0, torch.zeros_like(y), y)  # std::max(v, 0.f): a NaN stays
        return y.permute(0, 2, 3, 1).cpu().numpy()

    got = gpu(x, wgt).cpu().numpy()
    want = f64(x, wgt)
    assert got.shape == want.shape
    scale = np.abs(want).max()
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=RTOL * scale)
    # much closer than the tolerance asks: the split loses nothing an fp32 loop keeps
    assert np.abs(got - want).max() <= 4e-6 * scale
    for i in (0, n // 2, n - 1):
        np.testing.assert_allclose(got[i], cpu(x[i], wgt), rtol=RTOL, atol=RTOL * scale)
    # small integers: every product and partial sum is exact
    xi = r.integers(-3, 4, x.shape).astype(np.float32)
    wi = r.integers(-2, 3, wgt.shape).astype(np.float32)
    if affine:
        a, b = r.integers(-2, 3, cout).astype(np.float32), r.integers(-9, 10, cout).astype(np.float32)
    if bias:
        bv = r.integers(-5, 6, cout).astype(np.float32)
    goti = gpu(xi, wi).cpu().numpy()
    for i in (0, n - 1):
        np.testing.assert_array_equal(goti[i], cpu(xi[i], wi))
    # a NaN pixel and an infinity in one channel (the work items they touch are made again the slow way, the others are
    # not: one pixel beside a tile and one in a corner among them), then also an infinity in a weight (its products with
    # the image's zeros are NaN; every work item the slow way)
    xi[0, h // 2, w // 3, :] = np.nan
    xi[-1, h // 3, w // 2, 5] = np.inf
    xi[1, 0, 0, 7] = -np.inf
    xi[2, min(5, h - 1), min(16 - pad, w - 1), 3] = np.inf  # the first pixel right of the first tile's sixteen: that tile sees it through its halo only
    for weight_too in (False, True):
        if weight_too:
            wi[3, 1, 1, 9] = np.inf
        with np.errstate(invalid="ignore"):
            want = f64(xi, wi)
        goti = gpu(xi, wi).cpu().numpy()
        np.testing.assert_array_equal(np.isnan(goti), np.isnan(want))
        np.testing.assert_array_equal(goti[~np.isnan(want)], want[~np.isnan(want)].astype(np.float32))


def test_fconv_ramp_cases_of_reference_tests(dab):
    """tests/fconv_test.cpp:14-41 and :43-70: ramp image and ramp weights, exact in fp32."""
    for (h, k, pad, stride) in [(4, 3, 1, 1), (8, 5, 2, 2)]:
        x = np.arange(h * h * 2, dtype=np.float32).reshape(1, h, h, 2)
        wgt = np.arange(k * k * 2 * 2, dtype=np.float32).reshape(2, k, k, 2)
        got = dab.fconv(dev_f(x), dev_f(wgt), None, k, k, pad, pad, stride, stride).cpu().numpy()[0]
        np.testing.assert_array_equal(got, orc.baseline_fconv(x[0], wgt, k, k, pad, pad, stride, stride))


@pytest.mark.parametrize("n,h,w,c,k,pad,stride", [(1, 9, 6, 64, 3, 1, 2), (2, 112, 112, 64, 3, 1, 2), (3, 7, 7, 192, 2, 0, 2),
                                                  (1, 5, 5, 128, 3, 1, 1)])
def test_max_pool_sign_packs_its_own_output(dab, n, h, w, c, k, pad, stride):
    x = special_floats((n, h, w, c), 44)
    x[np.isnan(x)] = 0.0  # the reference's max over NaN depends on the tap order; zeros and infinities stay
    got, packed = dab.max_pool_sign(dev_f(x), k, k, pad, pad, stride, stride)
    want = np.stack([orc.max_pool(img, k, k, pad, pad, stride, stride) for img in x])
    np.testing.assert_array_equal(got.cpu().numpy(), want)
    np.testing.assert_array_equal(host_u(packed), np.stack([orc.pack_mat(img) for img in want]))
    with pytest.raises(RuntimeError):
        dab.max_pool_sign(torch.zeros((1, 4, 4, 32), device="cuda"), 2, 2, 0, 0, 2, 2)


def test_affine_add_bit_exact(dab):
    r = rng(41)
    x = r.standard_normal((2, 5, 7, 64)).astype(np.float32)
    a, b = r.standard_normal(64).astype(np.float32), r.standard_normal(64).astype(np.float32)
    y = r.standard_normal(x.shape).astype(np.float32)
    got = dab.affine_inplace(dev_f(x), dev_f(a), dev_f(b))
    want = np.stack([orc.affine_inplace(img.copy(), a, b) for img in x])
    np.testing.assert_array_equal(got.cpu().numpy(), want)
    got2 = dab.add_inplace(got, dev_f(y)).cpu().numpy()
    np.testing.assert_array_equal(got2, want + y)


@pytest.mark.parametrize("n,h,w,c,cout,affine", [(1, 56, 56, 64, 128, True), (2, 9, 7, 8, 5, False), (3, 28, 28, 128, 256, True),
                                                 (1, 14, 14, 256, 512, True), (40, 56, 56, 64, 128, True), (1, 2, 2, 4, 8, False),
                                                 # enough pixels for the large tiles: one column tile (128 rows, 32-deep
                                                 # slices), more than 128 output channels (64 rows x 256 columns), the
                                                 # latter with a ragged last tile both ways
                                                 (48, 56, 56, 64, 128, True), (170, 28, 28, 128, 256, False),
                                                 (97, 30, 30, 64, 200, True), (256, 14, 14, 256, 512, True),
                                                 # eight pooled pixels or fewer and 64 output channels or more: the
                                                 # convolution alone would be the matrix-vector kernel's
                                                 (1, 4, 9, 20, 242, False), (2, 2, 5, 64, 64, True)])
def test_ave_pool2_fconv1x1_equals_the_two_layers(dab, n, h, w, c, cout, affine):
    """The shortcut branch of a down-sampling block in one launch: the pooled tensor is bit for bit what ave_pool
    writes (and what the CPU restatement computes), the convolution bit for bit what fconv_affine_relu makes of it."""
    r = rng(46)
    x = r.standard_normal((n, h, w, c)).astype(np.float32)
    x[0, 0, 0, :4] = [0.0, -0.0, 1e-40, -1e-40]
    wgt = (r.standard_normal((cout, 1, 1, c)) / np.sqrt(c)).astype(np.float32)
    a, b = r.standard_normal(cout).astype(np.float32), r.standard_normal(cout).astype(np.float32)
    pooled, out = dab.ave_pool2_fconv1x1(dev_f(x), dev_f(wgt), None, dev_f(a) if affine else None,
                                         dev_f(b) if affine else None, False)
    want_pooled = dab.ave_pool(dev_f(x), 2, 2, 0, 0, 2, 2)
    want_out = dab.fconv_affine_relu(want_pooled, dev_f(wgt), None, dev_f(a) if affine else None,
                                     dev_f(b) if affine else None, False, 1, 1, 0, 0, 1, 1)
    np.testing.assert_array_equal(pooled.cpu().numpy(), want_pooled.cpu().numpy())
    np.testing.assert_array_equal(out.cpu().numpy(), want_out.cpu().numpy())
    cpu_pooled = np.stack([orc.ave_pool(img, 2, 2, 0, 0, 2, 2) for img in x[:2]])
    np.testing.assert_array_equal(pooled.cpu().numpy()[:2], cpu_pooled)
    with pytest.raises(RuntimeError):
        dab.ave_pool2_fconv1x1(dev_f(x[..., :3].copy()), dev_f(wgt[..., :3].copy()), None, None, None, False)


@pytest.mark.parametrize("n,h,w,c,cout,bias,affine,relu", [
    (8, 56, 56, 64, 128, False, True, False),    # the first shortcut branch of Bi-Real-18, whole tiles
    (9, 30, 27, 64, 200, True, True, True),      # odd sizes: a ragged last pixel tile, a ragged second column tile
    (11, 28, 28, 64, 72, True, False, True),     # one column tile, mostly empty
    (2, 112, 112, 64, 384, False, False, False),  # three column tiles
    (3, 28, 28, 128, 256, True, True, False)])   # 128 channels: the tile kernel, without the pooled tensor too
def test_ave_pool2_fconv1x1_with_the_pooled_tile_in_lds(dab, n, h, w, c, cout, bias, affine, relu):
    """64 input channels and enough pixels: a block pools its pixels once into LDS and walks the column tiles over
    them.  Same bits as the two layers, with infinities, NaNs, signed zeros and denormals in the input, with every
    epilogue, and the same convolution when the pooled tensor is not asked for."""
    r = rng(47)
    x = r.standard_normal((n, h, w, c)).astype(np.float32)
    x.flat[::7] = 0.0
    x.flat[3::11] = -0.0
    x.flat[1::17] = np.float32(1e-45)
    x.flat[2::19] = -np.float32(1e-45)
    x.flat[::9973] = np.nan
    x.flat[5::10007] = np.inf
    x.flat[7::10009] = -np.inf

    def same_bits(got, want):
        got, want = got.cpu().numpy(), want.cpu().numpy()
        np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
        np.testing.assert_array_equal(np.where(np.isnan(got), 0, got.view(np.uint32)), np.where(np.isnan(want), 0, want.view(np.uint32)))

    wgt = (r.standard_normal((cout, 1, 1, c)) / np.sqrt(c)).astype(np.float32)
    bv = r.standard_normal(cout).astype(np.float32)
    a, b = r.standard_normal(cout).astype(np.float32), r.standard_normal(cout).astype(np.float32)
    args = (dev_f(wgt), dev_f(bv) if bias else None, dev_f(a) if affine else None, dev_f(b) if affine else None, relu)
    pooled, out = dab.ave_pool2_fconv1x1(dev_f(x), *args)
    want_pooled = dab.ave_pool(dev_f(x), 2, 2, 0, 0, 2, 2)
    want_out = dab.fconv_affine_relu(want_pooled, *args, 1, 1, 0, 0, 1, 1)
    same_bits(pooled, want_pooled)
    same_bits(out, want_out)
    assert np.isfinite(want_out.cpu().numpy()).mean() > 0.3
    none, out2 = dab.ave_pool2_fconv1x1(dev_f(x), *args, want_pooled=False)
    assert none is None
    same_bits(out2, want_out)
    # against the CPU layers on finite data (sums of other orders: the tolerance of the float layers)
    xf = r.standard_normal((2, h, w, c)).astype(np.float32)
    _, got = dab.ave_pool2_fconv1x1(dev_f(xf), *args)
    for i in range(2):
        want = orc.fconv(orc.ave_pool(xf[i], 2, 2, 0, 0, 2, 2), wgt, bv if bias else None, 1, 1, 0, 0, 1, 1)
        if affine:
            want = orc.affine_inplace(want, a, b)
        if relu:
            want = orc.relu_inplace(want)
        np.testing.assert_allclose(got[i].cpu().numpy(), want, rtol=1e-4, atol=1e-4 * np.abs(want).max())


def test_ave_pool2_fconv1x1_needs_the_pooled_buffer_for_a_handful_of_pixels(dab):
    x = torch.zeros((1, 4, 4, 64), device="cuda")
    w = torch.zeros((64, 1, 1, 64), device="cuda")
    with pytest.raises(RuntimeError):
        dab.ave_pool2_fconv1x1(x, w, None, None, None, False, want_pooled=False)
    dab.ave_pool2_fconv1x1(x, w, None, None, None, False)


@pytest.mark.parametrize("n,h,w,c,cout,bias,affine,relu", [
    (1, 7, 7, 512, 1000, True, False, False),   # the end of Bi-Real-18 at batch 1
    (8, 7, 7, 512, 1000, False, False, False),  # the most images it takes
    (3, 8, 8, 1024, 64, True, True, True),      # the deepest and the largest window it takes, the fewest channels
    (2, 1, 1, 4, 77, False, True, False),       # no pooling to speak of; a ragged last block
    (5, 5, 3, 36, 100, True, False, True),      # a depth that leaves most lanes idle
])
def test_global_ave_pool_fconv1x1_equals_the_two_layers(dab, n, h, w, c, cout, bias, affine, relu):
    """A global AvePool and the classifier behind it in one launch (small batch): the pooled tensor is bit for bit what
    ave_pool writes and what the CPU restatement computes, the result bit for bit what fconv_affine_relu makes of it
    and within the float tolerance of the CPU layers."""
    assert dab.global_ave_pool_fconv1x1_takes(n, h, w, c, cout)
    r = rng(47)
    x = r.standard_normal((n, h, w, c)).astype(np.float32)
    x[0, 0, 0, :4] = [0.0, -0.0, 1e-40, -1e-40]
    wgt = (r.standard_normal((cout, 1, 1, c)) / np.sqrt(c)).astype(np.float32)
    bv = r.standard_normal(cout).astype(np.float32)
    a, b = r.standard_normal(cout).astype(np.float32), r.standard_normal(cout).astype(np.float32)
    args = (dev_f(bv) if bias else None, dev_f(a) if affine else None, dev_f(b) if affine else None, relu)
    pooled, out = dab.global_ave_pool_fconv1x1(dev_f(x), dev_f(wgt), *args)
    want_pooled = dab.ave_pool(dev_f(x), h, w, 0, 0, 1, 1)
    want_out = dab.fconv_affine_relu(want_pooled, dev_f(wgt), *args, 1, 1, 0, 0, 1, 1)
    assert pooled.shape == (n, 1, 1, c) and out.shape == (n, 1, 1, cout)
    np.testing.assert_array_equal(pooled.cpu().numpy(), want_pooled.cpu().numpy())
    np.testing.assert_array_equal(out.cpu().numpy(), want_out.cpu().numpy())
    cpu_pooled = np.stack([orc.ave_pool(img, h, w, 0, 0, 1, 1) for img in x])
    np.testing.assert_array_equal(pooled.cpu().numpy(), cpu_pooled)
    for i in (0, n - 1):
        y = orc.fconv(cpu_pooled[i], wgt, bv if bias else None, 1, 1, 0, 0, 1, 1)
        if affine:
            y = orc.affine_inplace(y.copy(), a, b)
        if relu:
            y = np.maximum(y, 0)
        np.testing.assert_allclose(out.cpu().numpy()[i], y, rtol=RTOL, atol=RTOL * np.abs(y).max())
    # shapes it leaves to the two separate calls
    for shape in [(9, 7, 7, 512, 1000), (1, 9, 8, 512, 1000), (1, 7, 7, 510, 1000), (1, 7, 7, 2048, 1000), (1, 7, 7, 512, 10)]:
        assert not dab.global_ave_pool_fconv1x1_takes(*shape)
    with pytest.raises(RuntimeError):
        dab.global_ave_pool_fconv1x1(dev_f(np.zeros((9, h, w, c), np.float32)), dev_f(wgt), None, None, None, False)


@pytest.mark.parametrize("n,h,w,c,k,pad,stride,dil,cout,bias,affine,relu", [
    # output width 28, 56, 112 (bands of 16, 8, 4 rows), one band per image and several, three-channel images and
    # multiples of four channels, a depth that is no multiple of the slice, two channel tiles, a ragged channel tile
    (2, 64, 56, 3, 7, 3, 2, 1, 64, False, True, False), (3, 16, 112, 3, 7, 3, 2, 1, 64, True, False, True),
    (1, 224, 224, 3, 7, 3, 2, 1, 64, False, True, False), (2, 32, 56, 32, 3, 1, 1, 1, 64, False, True, True),
    (2, 16, 28, 8, 3, 1, 1, 1, 128, True, True, False), (1, 16, 28, 4, 5, 2, 1, 1, 20, False, False, False),
    (1, 36, 60, 3, 3, 0, 1, 2, 64, True, True, True),
    # the 7x7 stride-2 stem at output width 112 has a kernel of its own: odd image sizes, two channel tiles on one
    # block, a ragged channel tile, a single band
    (2, 31, 223, 3, 7, 3, 2, 1, 128, True, True, True), (1, 8, 224, 3, 7, 3, 2, 1, 20, False, False, False),
    # more bands than blocks: a block makes consecutive bands and hands the last row of one to the next in registers
    # (ranges of one and two bands here, some across two images)
    (12, 224, 224, 3, 7, 3, 2, 1, 64, False, True, False), (100, 32, 56, 4, 3, 1, 1, 1, 64, True, True, True),
    (90, 16, 224, 4, 3, 1, 1, 1, 8, False, False, True),
])
def test_fconv_maxpool_one_pass(dab, n, h, w, c, k, pad, stride, dil, cout, bias, affine, relu):
    """FpConv2D (+ Affine + Relu) + MaxPool 3x3 stride 2 pad 1 without the convolution's output in memory: within
    the float tolerance of the CPU layers, bit for bit what max_pool makes of the separate float convolution on
    the device when the data make fp32 sums exact, and the packed copy is pack_mat of the pooled tensor it wrote."""
    r = rng(47)
    x = r.standard_normal((n, h, w, c)).astype(np.float32)
    wgt = (r.standard_normal((cout, k, k, c)) / np.sqrt(k * k * c)).astype(np.float32)
    bv = r.standard_normal(cout).astype(np.float32) if bias else None
    a, b = r.standard_normal(cout).astype(np.float32), r.standard_normal(cout).astype(np.float32)
    sign = cout % 64 == 0

    def cpu(x, wgt, bv, a, b):
        out = []
        for img in x:
            y = orc.fconv(img, wgt, bv, k, k, pad, pad, stride, stride, dil, dil)
            if affine:
                y = orc.affine_inplace(y.copy(), a, b)
            if relu:
                y = np.maximum(y, 0)
            out.append(orc.max_pool(y, 3, 3, 1, 1, 2, 2))
        return np.stack(out)

    def gpu(x, wgt, bv, a, b):
        return dab.fconv_maxpool(dev_f(x), dev_f(wgt), dev_f(bv) if bias else None, dev_f(a) if affine else None,
                                 dev_f(b) if affine else None, relu, k, k, pad, pad, stride, stride, dil, dil, want_sign=sign)

    pooled, packed = gpu(x, wgt, bv, a, b)
    got, want = pooled.cpu().numpy(), cpu(x, wgt, bv, a, b)
    assert got.shape == want.shape
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=RTOL * np.abs(want).max())
    if sign:
        np.testing.assert_array_equal(host_u(packed), np.stack([orc.pack_mat(img) for img in got]))
    # small integers: every product and partial sum is exact in fp32, whatever the order of the additions
    xi = r.integers(-3, 4, x.shape).astype(np.float32)
    wi = r.integers(-2, 3, wgt.shape).astype(np.float32)
    bi = r.integers(-5, 6, cout).astype(np.float32) if bias else None
    ai, ci = r.integers(-2, 3, cout).astype(np.float32), r.integers(-9, 10, cout).astype(np.float32)
    pooled, packed = gpu(xi, wi, bi, ai, ci)
    want = cpu(xi, wi, bi, ai, ci)
    np.testing.assert_array_equal(pooled.cpu().numpy(), want)
    if sign:
        np.testing.assert_array_equal(host_u(packed), np.stack([orc.pack_mat(img) for img in want]))
    sep = dab.fconv_affine_relu(dev_f(xi), dev_f(wi), dev_f(bi) if bias else None, dev_f(ai) if affine else None,
                                dev_f(ci) if affine else None, relu, k, k, pad, pad, stride, stride, dil, dil)
    np.testing.assert_array_equal(pooled.cpu().numpy(), dab.max_pool(sep, 3, 3, 1, 1, 2, 2).cpu().numpy())
    # a NaN and an infinity in the image: the windows they reach are NaN (or infinite) after the convolution, and the
    # pool passes over NaN as max_pool_fallback's comparison does
    xi[0, h // 2, w // 3, :] = np.nan
    xi[-1, h // 3, w // 2, 0] = np.inf
    with np.errstate(invalid="ignore"):
        want = cpu(xi, wi, bi, ai, ci)
    pooled, packed = gpu(xi, wi, bi, ai, ci)
    np.testing.assert_array_equal(pooled.cpu().numpy(), want)
    if sign:
        np.testing.assert_array_equal(host_u(packed), np.stack([orc.pack_mat(img) for img in want]))
    # the largest float in the image (its leading bf16 part would round up to an infinity) under filters of -1, 0, 1:
    # every sum it takes part in is exact, and no window may turn infinite or NaN because of the split
    xl = r.integers(-3, 4, x.shape).astype(np.float32)
    xl[0, h // 2, w // 2, 0] = np.finfo(np.float32).max
    xl[-1, h // 3, w // 3, c - 1] = -np.finfo(np.float32).max
    wl = r.integers(-1, 2, wgt.shape).astype(np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        want = cpu(xl, wl, bi, ai, ci)
    pooled, packed = gpu(xl, wl, bi, ai, ci)
    np.testing.assert_array_equal(pooled.cpu().numpy(), want)
    # an infinite filter value: its channel is infinite where the tap meets a non-zero pixel and NaN where it meets a
    # zero (padding included), as in the reference's product of the im2col matrix
    xf = r.integers(-3, 4, x.shape).astype(np.float32)
    wf = wi.copy()
    wf[cout // 2, k // 2, 0, 0] = np.inf
    with np.errstate(over="ignore", invalid="ignore"):
        want = cpu(xf, wf, bi, ai, ci)
    pooled, packed = gpu(xf, wf, bi, ai, ci)
    np.testing.assert_array_equal(pooled.cpu().numpy(), want)
    if sign:
        np.testing.assert_array_equal(host_u(packed), np.stack([orc.pack_mat(img) for img in want]))


@pytest.mark.parametrize("n,h,w,pad,cout,bias,affine,relu", [
    (22, 112, 112, 1, 64, False, True, True),   # the three-convolution stem's last convolution and its MaxPool
    (24, 112, 112, 1, 32, True, False, False),  # 32 output channels: no sign bits
    (600, 28, 16, 1, 64, True, True, False),    # one tile per row: no tile to the left anywhere
    (300, 28, 32, 1, 64, False, False, True),   # two tiles per row
    (70, 110, 110, 2, 64, False, True, True),   # pad 2: a 112 x 112 output of a 110 x 110 image
])
def test_fconv_maxpool_over_32_channels_pools_in_registers(dab, n, h, w, pad, cout, bias, affine, relu):
    """3x3 stride-1 convolutions over 32 channels that are large enough take the split-operand kernel also with a
    MaxPool 3x3 stride 2 pad 1 behind them: a tile column pools what it holds and a second pass completes the cells
    that need the row above or the pixel to the left.  Equal to max_pool_sign of the separate convolution on the
    device (the same products, the same maxima), within the float tolerance of the CPU layers, exact on small
    integers, and infinities and NaNs come out as the CPU layers put them."""
    assert dab.fconv_maxpool_pays(n, h, w, 32, 3, 3, pad, pad, 1, 1, 1, 1, cout)
    r = rng(63)
    x = r.standard_normal((n, h, w, 32)).astype(np.float32)
    wgt = (r.standard_normal((cout, 3, 3, 32)) / 17).astype(np.float32)
    bv = r.standard_normal(cout).astype(np.float32) if bias else None
    a, b = r.standard_normal(cout).astype(np.float32), r.standard_normal(cout).astype(np.float32)
    sign = cout % 64 == 0

    def both(x, wgt, bv, a, b):
        args = (dev_f(bv) if bias else None, dev_f(a) if affine else None, dev_f(b) if affine else None, relu)
        pooled, packed = dab.fconv_maxpool(dev_f(x), dev_f(wgt), *args, 3, 3, pad, pad, 1, 1, 1, 1, want_sign=sign)
        conv = dab.fconv_affine_relu(dev_f(x), dev_f(wgt), *args, 3, 3, pad, pad, 1, 1)
        if sign:
            want, want_packed = dab.max_pool_sign(conv, 3, 3, 1, 1, 2, 2)
            assert torch.equal(packed, want_packed)
            assert torch.equal(packed, dab.pack_mat(pooled))
        else:
            want = dab.max_pool(conv, 3, 3, 1, 1, 2, 2)
        return pooled.cpu().numpy(), want.cpu().numpy()

    def cpu(img, wgt, bv, a, b):
        y = orc.fconv(img, wgt, bv, 3, 3, pad, pad, 1, 1)
        if affine:
            y = orc.affine_inplace(y.copy(), a, b)
        if relu:
            y = np.maximum(y, 0)
        return orc.max_pool(y, 3, 3, 1, 1, 2, 2)

    got, want = both(x, wgt, bv, a, b)
    assert got.shape == (n, (h + 2 * pad - 2) // 2, (w + 2 * pad - 2) // 2, cout)
    np.testing.assert_array_equal(got, want)
    for i in (0, n - 1):
        ref = cpu(x[i], wgt, bv, a, b)
        np.testing.assert_allclose(got[i], ref, rtol=RTOL, atol=RTOL * np.abs(ref).max())
    # small integers: exact; then an infinity, a NaN pixel and a NaN at a tile's edge
    xi = r.integers(-3, 4, x.shape).astype(np.float32)
    wi = r.integers(-2, 3, wgt.shape).astype(np.float32)
    bi = r.integers(-5, 6, cout).astype(np.float32) if bias else None
    ai, ci = r.integers(-2, 3, cout).astype(np.float32), r.integers(-9, 10, cout).astype(np.float32)
    got, want = both(xi, wi, bi, ai, ci)
    np.testing.assert_array_equal(got, want)
    for i in (0, n - 1):
        np.testing.assert_array_equal(got[i], cpu(xi[i], wi, bi, ai, ci))
    xi[0, h // 2, w // 3, :] = np.nan
    xi[-1, h // 3, w // 2, 5] = np.inf
    xi[1, min(3, h - 1), min(15, w - 1), 7] = -np.inf
    xi[2, min(4, h - 1), min(16 - pad, w - 1), 3] = np.nan
    got, want = both(xi, wi, bi, ai, ci)
    np.testing.assert_array_equal(got, want)
    with np.errstate(invalid="ignore"):
        for i in (0, 1, 2, n - 1):
            np.testing.assert_array_equal(got[i], cpu(xi[i], wi, bi, ai, ci))


def test_fconv_maxpool_rejects_other_shapes(dab):
    x = torch.zeros((1, 60, 60, 3), device="cuda")
    wgt = torch.zeros((64, 7, 7, 3), device="cuda")
    with pytest.raises(RuntimeError, match="output width"):
        dab.fconv_maxpool(x, wgt, None, None, None, False, 7, 7, 3, 3, 2, 2)  # 30 x 30 output
    with pytest.raises(RuntimeError, match="output width"):
        dab.fconv_maxpool(torch.zeros((1, 58, 56, 3), device="cuda"), wgt, None, None, None, False, 7, 7, 3, 3, 2, 2)  # 29 rows
    with pytest.raises(RuntimeError, match="sign bits"):
        dab.fconv_maxpool(torch.zeros((1, 64, 56, 3), device="cuda"), torch.zeros((32, 7, 7, 3), device="cuda"), None, None,
                          None, False, 7, 7, 3, 3, 2, 2, want_sign=True)


def test_relu_bit_exact_including_nan_and_negative_zero(dab):
    """std::max(x, 0.f) of the reference keeps a NaN and a negative zero; so do the stand-alone kernel and the fused
    epilogue of the float convolution."""
    x = special_floats((2, 9, 7, 64), 52)
    want = orc.relu_inplace(x.copy())
    got = dab.relu_inplace(dev_f(x)).cpu().numpy()
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    # a 1x1 convolution with the identity as weights leaves the values as they are; zeros elsewhere in a row do not
    # disturb a NaN or an infinity of the same pixel here, because every row of the identity has one non-zero entry
    # and 0 * finite = 0 -- so take finite inputs plus NaN only
    y = rng(53).standard_normal((1, 4, 4, 8)).astype(np.float32)
    y[0, 1, 2, :] = np.nan
    y[0, 0, 0, 0] = -0.0
    eye = np.eye(8, dtype=np.float32).reshape(8, 1, 1, 8)
    fused = dab.fconv_affine_relu(dev_f(y), dev_f(eye), None, None, None, True, 1, 1, 0, 0, 1, 1).cpu().numpy()
    np.testing.assert_array_equal(np.isnan(fused), np.isnan(y))
    np.testing.assert_array_equal(fused[~np.isnan(y)], np.maximum(y[~np.isnan(y)], 0))


@pytest.mark.parametrize("shape", [(2, 5, 7, 64), (1, 3, 3, 5), (3, 16, 16, 192), (1, 1, 1, 1)])
def test_prelu_bit_exact(dab, shape):
    r = rng(44)
    x = r.standard_normal(shape).astype(np.float32)
    x.ravel()[:2] = [0.0, -0.0][:x.size]
    for slope in (np.array([0.25], np.float32), r.uniform(-0.5, 0.5, shape[-1]).astype(np.float32)):
        got = dab.prelu_inplace(dev_f(x), dev_f(slope)).cpu().numpy()
        want = np.stack([orc.prelu_inplace(img.copy(), slope) for img in x])
        np.testing.assert_array_equal(got, want)
    if shape[-1] > 2:
        with pytest.raises(RuntimeError, match="slope must have size 1 or c"):
            dab.prelu_inplace(dev_f(x), dev_f(np.ones(2, np.float32)))


@pytest.mark.parametrize("n,h,w,ca,cb", [(2, 5, 7, 64, 64), (1, 3, 3, 5, 2), (3, 16, 16, 128, 64), (1, 1, 1, 1, 1)])
def test_concat_bit_exact(dab, n, h, w, ca, cb):
    r = rng(45)
    a = r.standard_normal((n, h, w, ca)).astype(np.float32)
    b = r.standard_normal((n, h, w, cb)).astype(np.float32)
    got = dab.concat(dev_f(a), dev_f(b)).cpu().numpy()
    np.testing.assert_array_equal(got, np.stack([orc.concat(x, y) for x, y in zip(a, b)]))
    with pytest.raises(RuntimeError, match="shapes differ"):
        dab.concat(dev_f(a), dev_f(b[:, :, :-1] if w > 1 else np.zeros((n, h, w + 1, cb), np.float32)))


@pytest.mark.parametrize("n,h,w,c,k,pad,stride", [(1, 8, 8, 4, 2, 0, 2), (2, 7, 7, 512, 7, 0, 1), (1, 9, 6, 4, 3, 1, 2),
                                                  (1, 112, 112, 64, 3, 1, 2), (2, 56, 56, 64, 2, 0, 2),
                                                  # windows of up to 49 taps cut by the border, few enough outputs for the
                                                  # all-taps-in-flight kernel; a 6x6 window; many outputs of a 7x7 one
                                                  (1, 9, 9, 64, 7, 3, 2), (3, 12, 12, 32, 6, 2, 3), (8, 28, 28, 128, 7, 3, 1)])
def test_pools(dab, n, h, w, c, k, pad, stride):
    x = rng(42).standard_normal((n, h, w, c)).astype(np.float32)
    avg = dab.ave_pool(dev_f(x), k, k, pad, pad, stride, stride).cpu().numpy()
    mx = dab.max_pool(dev_f(x), k, k, pad, pad, stride, stride).cpu().numpy()
    want_avg = np.stack([orc.ave_pool(img, k, k, pad, pad, stride, stride) for img in x])
    want_max = np.stack([orc.max_pool(img, k, k, pad, pad, stride, stride) for img in x])
    np.testing.assert_allclose(avg, want_avg, rtol=RTOL, atol=1e-6)
    np.testing.assert_array_equal(mx, want_max)
