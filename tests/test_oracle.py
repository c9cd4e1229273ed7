"""Pins the CPU oracle against independent evidence (runs without a GPU).

Each oracle function is checked against something that is not a retyping of
its own loop: the golden vector held by the reference's own tests, closed
forms (numpy packbits, integer matmul over unpacked bits), textbook float
convolution / pooling from torch on +-1 data, brute force on tiny inputs, and
invariants.  The GPU parity tests then compare the HIP kernels with this
oracle.
"""
import json
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle as orc


def rng(seed):
    return np.random.default_rng(seed)


def unpack_bits(words):
    """uint64 [..., n] -> uint8 [..., n*64], bit j of word i at index i*64+j."""
    w = np.ascontiguousarray(words, dtype="<u8")
    return np.unpackbits(w.view(np.uint8).reshape(w.shape + (8,)), axis=-1, bitorder="little").reshape(
        w.shape[:-1] + (w.shape[-1] * 64,))


def np_pack(x):
    """Independent sign pack: numpy packbits, little bit order, viewed as <u8."""
    bits = (np.asarray(x, dtype=np.float32) > 0)
    return np.packbits(bits, axis=-1, bitorder="little").view("<u8")


def float_conv_counts(xbits_pm1, wbits_pm1, kh, kw, pad, stride, dil=1):
    """Textbook oracle: cnt = (K - conv(sign x, sign w, padding = -1)) / 2."""
    x = torch.from_numpy(xbits_pm1).double().permute(2, 0, 1)[None]  # 1,C,H,W
    w = torch.from_numpy(wbits_pm1).double().permute(0, 3, 1, 2)  # Cout,C,KH,KW
    xp = F.pad(x, (pad[1], pad[1], pad[0], pad[0]), value=-1.0)
    y = F.conv2d(xp, w, stride=stride, dilation=dil)[0].permute(1, 2, 0)
    K = kh * kw * xbits_pm1.shape[2]
    return ((K - y) / 2).numpy()


# ---------------------------------------------------------------- bit packing
def test_pack64_known_answers(golden_dir):
    for case in json.load(open(os.path.join(golden_dir, "pack64_known_answers.json"))):
        vals = np.array([float(v) for v in case["values"]], dtype=np.float32)
        assert orc.pack_64(vals) == int(case["word"], 16), case["name"]


def test_pack64_eff_bits():
    v = np.ones(64, dtype=np.float32)
    assert orc.pack_64(v, 64) == 2**64 - 1
    assert orc.pack_64(v, 10) == 2**10 - 1
    assert orc.pack_64(v, 0) == 0


@pytest.mark.parametrize("shape", [(8, 8, 128), (5, 4, 64), (3, 2, 192), (56, 56, 64)])
def test_pack_mat_matches_numpy_packbits(shape):
    x = rng(1).standard_normal(shape).astype(np.float32)
    x.flat[::7] = 0.0
    x.flat[3::11] = -0.0
    x.flat[5::13] = np.nan
    got = orc.pack_mat(x)
    assert got.shape == shape[:2] + (shape[2] // 64,)
    np.testing.assert_array_equal(got, np_pack(x).reshape(got.shape))


def test_pack_nchw_is_pack_of_permuted_input():
    x = rng(2).standard_normal((128, 5, 6)).astype(np.float32)
    np.testing.assert_array_equal(orc.pack_nchw(x), np_pack(np.transpose(x, (1, 2, 0))).reshape(5, 6, 2))


def test_pad_bit_is_zero_word_border():
    x = rng(3).integers(0, 2**64, size=(4, 6, 2), dtype=np.uint64)
    got = orc.pad_bit(x, 1, 2)
    np.testing.assert_array_equal(got, np.pad(x, ((1, 1), (2, 2), (0, 0))))


# ---------------------------------------------------------------- im2col
def test_im2col_reference_golden_vector(golden_dir):
    g = json.load(open(os.path.join(golden_dir, "im2col_4x4x2_k3p1.json")))
    im = np.array(g["input"], dtype=np.float32).reshape(g["h"], g["w"], g["c"])
    col = orc.im2col(im, g["kh"], g["kw"], g["pad"], g["pad"], g["stride"], g["stride"])
    np.testing.assert_array_equal(col.ravel(), np.array(g["expected"], dtype=np.float32))


def np_im2col(im, kh, kw, pad, stride, dil):
    h, w, c = im.shape
    p = np.pad(im, ((pad[0], pad[0]), (pad[1], pad[1]), (0, 0)))
    oh = orc.out_dim(h, pad[0], kh, stride[0], dil[0])
    ow = orc.out_dim(w, pad[1], kw, stride[1], dil[1])
    rows = []
    for oy in range(oh):
        for ox in range(ow):
            taps = [p[oy * stride[0] + a * dil[0], ox * stride[1] + b * dil[1]] for a in range(kh) for b in range(kw)]
            rows.append(np.concatenate(taps))
    return np.stack(rows)


@pytest.mark.parametrize("h,w,c,k,pad,stride,dil", [
    (7, 5, 3, 3, (1, 1), (1, 1), (1, 1)),
    (9, 8, 4, 5, (2, 2), (2, 2), (1, 1)),
    (8, 8, 2, 3, (2, 1), (1, 2), (2, 1)),
    (6, 6, 64, 1, (0, 0), (1, 1), (1, 1)),
])
def test_im2col_matches_numpy_gather(h, w, c, k, pad, stride, dil):
    im = rng(4).standard_normal((h, w, c)).astype(np.float32)
    got = orc.im2col(im, k, k, pad[0], pad[1], stride[0], stride[1], dil[0], dil[1])
    np.testing.assert_array_equal(got, np_im2col(im, k, k, pad, stride, dil))


def test_im2col_on_packed_words():
    x = rng(5).integers(0, 2**64, size=(5, 6, 2), dtype=np.uint64)
    got = orc.im2col(x, 3, 3, 1, 1, 2, 2)
    np.testing.assert_array_equal(got, np_im2col(x, 3, 3, (1, 1), (2, 2), (1, 1)))


@pytest.mark.parametrize("h,w,c,k,pad,stride", [
    (8, 8, 128, 3, 1, 1), (8, 8, 64, 3, 1, 2), (7, 9, 192, 3, 1, 1), (6, 6, 128, 5, 2, 2), (5, 5, 3, 3, 1, 1),
    (4, 4, 100, 1, 0, 1),
])
def test_fused_binarize_im2col_is_pack_of_float_im2col(h, w, c, k, pad, stride):
    im = rng(6).standard_normal((h, w, c)).astype(np.float32)
    im.flat[::5] = 0.0
    col_f = np_im2col(im, k, k, (pad, pad), (stride, stride), (1, 1))
    row = k * k * c
    row128 = (row + 127) // 128 * 128
    col_f = np.pad(col_f, ((0, 0), (0, row128 - row)))
    want = np_pack(col_f)
    got = orc.fused_binarize_im2col(im, k, k, pad, pad, stride, stride)
    assert got.shape == (col_f.shape[0], row128 // 64) == (col_f.shape[0], orc.col_row_words(k, k, c))
    np.testing.assert_array_equal(got, want)


def test_fused_binarize_im2col_size_limit():
    im = np.zeros((1, 1, 60000), dtype=np.float32)
    with pytest.raises(RuntimeError):
        orc.fused_binarize_im2col(im, 1, 1, 0, 0, 1, 1)


# ---------------------------------------------------------------- binary conv
def random_pm1(shape, seed):
    return np.where(rng(seed).standard_normal(shape) > 0, 1.0, -1.0).astype(np.float32)


@pytest.mark.parametrize("h,w,c,cout,k,pad,stride,dil", [
    (8, 8, 64, 64, 3, 1, 1, 1),
    (8, 8, 128, 128, 3, 1, 2, 1),
    (7, 10, 64, 16, 3, 1, 1, 1),  # non-square
    (9, 9, 128, 8, 5, 2, 2, 1),  # the 5x5 case of tests/bgemm_test.cpp:82-130
    (3, 3, 128, 128, 3, 0, 2, 1),  # 1x1 output, tests/bgemm_test.cpp:32-80
    (10, 10, 64, 4, 3, 2, 1, 2),  # dilation
    (6, 6, 256, 32, 1, 0, 1, 1),
])
def test_baseline_bconv_vs_float_convolution(h, w, c, cout, k, pad, stride, dil):
    x = random_pm1((h, w, c), 10)
    wgt = random_pm1((cout, k, k, c), 11)
    want = float_conv_counts(x, wgt, k, k, (pad, pad), stride, dil)
    got = orc.baseline_bconv(np_pack(x).reshape(h, w, c // 64), np_pack(wgt.reshape(cout, -1)), k, k, pad, pad,
                             stride, stride, dil, dil)
    np.testing.assert_array_equal(got, want.astype(np.float32))


def test_baseline_bconv_brute_force_tiny():
    x = rng(12).integers(0, 2**64, size=(3, 4, 1), dtype=np.uint64)
    wgt = rng(13).integers(0, 2**64, size=(2, 9), dtype=np.uint64)
    got = orc.baseline_bconv(x, wgt, 3, 3, 1, 1, 1, 1)
    for oy in range(3):
        for ox in range(4):
            for co in range(2):
                cnt = 0
                for a in range(3):
                    for b in range(3):
                        y, xx = oy - 1 + a, ox - 1 + b
                        word = int(x[y, xx, 0]) if 0 <= y < 3 and 0 <= xx < 4 else 0
                        cnt += bin(word ^ int(wgt[co, a * 3 + b])).count("1")
                assert got[oy, ox, co] == cnt


def test_baseline_bconv_invariants():
    h = w = 6
    x = rng(14).integers(0, 2**64, size=(h, w, 2), dtype=np.uint64)
    wgt = rng(15).integers(0, 2**64, size=(5, 18), dtype=np.uint64)
    base = orc.baseline_bconv(x, wgt, 3, 3, 1, 1, 1, 1)
    comp = orc.baseline_bconv(~x, wgt, 3, 3, 1, 1, 1, 1)
    # interior pixels: complementing the input turns cnt into K - cnt
    np.testing.assert_array_equal(base[1:-1, 1:-1] + comp[1:-1, 1:-1], np.full((h - 2, w - 2, 5), 9 * 128.0))
    # input equal to the filter everywhere -> zero mismatches in the interior
    same = np.tile(wgt[0].reshape(3, 3, 2)[1, 1], (h, w, 1))
    wsame = np.tile(same[0, 0], (1, 9))
    assert (orc.baseline_bconv(same, wsame, 3, 3, 1, 1, 1, 1)[1:-1, 1:-1] == 0).all()
    # corner: out-of-range taps read a zero word, so they contribute popcount(w)
    oob_taps = [0, 1, 2, 3, 6]
    inb_taps = [4, 5, 7, 8]
    for co in range(5):
        wt = wgt[co].reshape(9, 2)
        cnt = sum(bin(int(v)).count("1") for t in oob_taps for v in wt[t])
        for t in inb_taps:
            yy, xx = t // 3 - 1, t % 3 - 1
            cnt += sum(bin(int(a) ^ int(b)).count("1") for a, b in zip(wt[t], x[yy, xx]))
        assert base[0, 0, co] == cnt


def test_bconv_3x3_padded_equals_baseline_with_padding():
    for stride in (1, 2):
        x = rng(16).integers(0, 2**64, size=(8, 8, 2), dtype=np.uint64)
        wgt = rng(17).integers(0, 2**64, size=(16, 18), dtype=np.uint64)
        a = orc.bconv_3x3_padded(orc.pad_bit(x, 1, 1), wgt, stride)
        b = orc.baseline_bconv(x, wgt, 3, 3, 1, 1, stride, stride)
        np.testing.assert_array_equal(a, b)


def test_popcount_fast_equals_bitwise_count():
    a = rng(18).integers(0, 2**64, size=257, dtype=np.uint64)
    b = rng(19).integers(0, 2**64, size=257, dtype=np.uint64)
    slow = orc.lib().orc_xor_popcount_slow(a.ctypes.data_as(orc._c_u64_p), b.ctypes.data_as(orc._c_u64_p), a.size)
    assert slow == int(unpack_bits(a ^ b).sum())
    x = a[:250].reshape(5, 5, 10)
    w = b[:90].reshape(1, 90)
    assert orc.baseline_bconv(x, w, 3, 3, 0, 0, 1, 1)[1, 1, 0] == int(
        unpack_bits(x[1:4, 1:4].reshape(1, 90) ^ w).sum())


# ---------------------------------------------------------------- bgemm
@pytest.mark.parametrize("m,n,k", [(159, 253, 68), (128, 784, 18), (256, 196, 36), (512, 49, 72), (33, 17, 10),
                                   (1, 1, 1)])
def test_bgemm_naive_vs_integer_matmul(m, n, k):
    a = rng(20).integers(0, 2**64, size=(k, m), dtype=np.uint64)  # A(i,h) = a[h*lda+i]
    b = rng(21).integers(0, 2**64, size=(n, k), dtype=np.uint64)  # B(h,j) = b[j*ldb+h]
    c0 = rng(22).integers(0, 1000, size=(n, m)).astype(np.float32)  # C(i,j) = c[j*ldc+i]
    c = c0.copy()
    orc.bgemm_naive(m, n, k, a, m, b, k, c, m)
    abits = unpack_bits(a.T.copy()).astype(np.int64)  # m, k*64
    bbits = unpack_bits(b).astype(np.int64)  # n, k*64
    # popcount(a^b) = sum a + sum b - 2 a.b
    want = abits.sum(1)[None, :] + bbits.sum(1)[:, None] - 2 * (bbits @ abits.T)
    np.testing.assert_array_equal(c, c0 + want.astype(np.float32))


def test_bgemm_leading_dimensions():
    m, n, k, lda, ldb, ldc = 5, 4, 3, 7, 6, 9
    a = rng(23).integers(0, 2**64, size=(k, lda), dtype=np.uint64)
    b = rng(24).integers(0, 2**64, size=(n, ldb), dtype=np.uint64)
    c = np.zeros((n, ldc), dtype=np.float32)
    orc.bgemm_naive(m, n, k, a, lda, b, ldb, c, ldc)
    for i in range(m):
        for j in range(n):
            assert c[j, i] == sum(bin(int(a[h, i]) ^ int(b[j, h])).count("1") for h in range(k))
    assert (c[:, m:] == 0).all()


def test_weight_transpose_construction():
    w = rng(25).integers(0, 2**64, size=(6, 4), dtype=np.uint64)
    np.testing.assert_array_equal(orc.weight_transpose(w), w.T)


def test_im2col_plus_bgemm_equals_baseline_bconv():
    """The equality the reference asserts in tests/bgemm_test.cpp:32-130."""
    for (h, c, cout, k, pad, stride) in [(3, 128, 128, 3, 0, 2), (9, 128, 16, 5, 2, 2)]:
        x = rng(26).integers(0, 2**64, size=(h, h, c // 64), dtype=np.uint64)
        wgt = rng(27).integers(0, 2**64, size=(cout, k * k * c // 64), dtype=np.uint64)
        want = orc.baseline_bconv(x, wgt, k, k, pad, pad, stride, stride)
        col = orc.im2col(x, k, k, pad, pad, stride, stride)
        n, kk = col.shape
        cmat = np.zeros((n, cout), dtype=np.float32)
        orc.bgemm_naive(cout, n, kk, orc.weight_transpose(wgt), cout, col, kk, cmat, cout)
        np.testing.assert_array_equal(cmat.reshape(want.shape), want)


# ---------------------------------------------------------------- BinConv layer
@pytest.mark.parametrize("h,w,c,cout,stride", [(8, 8, 64, 32, 1), (8, 8, 64, 64, 2), (8, 8, 128, 64, 1),
                                               (7, 7, 256, 16, 2), (6, 10, 192, 8, 1)])
def test_binconv_forward_both_arms_vs_float_convolution(h, w, c, cout, stride):
    x = rng(30).standard_normal((h, w, c)).astype(np.float32)
    wf = rng(31).standard_normal((cout, 3, 3, c)).astype(np.float32)
    wp = orc.pack_weight(wf)
    out, method = orc.binconv_forward(x, wp, 3, 3, 1, 1, stride, stride)
    assert method == (2 if c == 64 else 3)
    want = float_conv_counts(np.where(x > 0, 1.0, -1.0), np.where(wf > 0, 1.0, -1.0), 3, 3, (1, 1), stride)
    np.testing.assert_array_equal(out, want.astype(np.float32))


def test_pack_weight_alignment_rule():
    # c == 64: no padding, 9 words per 3x3 filter; c == 192: 27 words padded to 28
    assert orc.pack_weight(np.ones((2, 3, 3, 64), dtype=np.float32)).shape == (2, 9)
    w = orc.pack_weight(np.ones((2, 3, 3, 192), dtype=np.float32))
    assert w.shape == (2, 28)
    assert (w[:, :27] == 2**64 - 1).all() and (w[:, 27] == 0).all()
    # c == 3 (float stem shapes never reach here, but the rule is general): 27 bits -> 2 words
    w = orc.pack_weight(np.ones((1, 3, 3, 3), dtype=np.float32))
    assert w.shape == (1, 2) and w[0, 0] == 2**27 - 1 and w[0, 1] == 0


def test_bn_fold_gives_k_minus_2cnt():
    """Affine(folded BN)(cnt) == BN(conv(sign x, sign w)) (docs/onnx2bnn.md step 2)."""
    h = w = 6
    c, cout = 128, 16
    r = rng(32)
    x = r.standard_normal((h, w, c)).astype(np.float32)
    wf = r.standard_normal((cout, 3, 3, c)).astype(np.float32)
    scale, bias, mean = (r.standard_normal(cout).astype(np.float32) for _ in range(3))
    var = r.uniform(0.5, 2.0, cout).astype(np.float32)
    cb = r.standard_normal(cout).astype(np.float32)
    cnt, _ = orc.binconv_forward(x, orc.pack_weight(wf), 3, 3, 1, 1, 1, 1)
    a, b = orc.bn_fold(scale, bias, mean, var, 1e-5, 3 * 3 * c, cb)
    got = orc.affine_inplace(cnt.copy(), a, b)
    conv = 9 * c - 2 * cnt.astype(np.float64) + cb
    want = scale * (conv - mean) / np.sqrt(var.astype(np.float64) + 1e-5) + bias
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-3)
    a0, b0 = orc.bn_fold(scale, bias, mean, var, 1e-5, 0, None)
    np.testing.assert_allclose(a0, scale / np.sqrt(var + 1e-5), rtol=1e-6)
    np.testing.assert_allclose(b0, bias - scale * mean / np.sqrt(var + 1e-5), rtol=1e-5, atol=1e-6)


# ---------------------------------------------------------------- float glue
def torch_conv_nhwc(x, wgt, bias, stride, pad, dil=1):
    xt = torch.from_numpy(x).double().permute(2, 0, 1)[None]
    wt = torch.from_numpy(wgt).double().permute(0, 3, 1, 2)
    bt = None if bias is None else torch.from_numpy(bias).double()
    return F.conv2d(xt, wt, bt, stride=stride, padding=pad, dilation=dil)[0].permute(1, 2, 0).numpy()


@pytest.mark.parametrize("h,c,cout,k,pad,stride,dil", [
    (4, 2, 2, 3, 1, 1, 1),  # tests/fconv_test.cpp:14-41
    (8, 2, 2, 5, 2, 2, 1),  # tests/fconv_test.cpp:43-
    (9, 3, 4, 3, 2, 1, 2),
    (14, 3, 8, 7, 3, 2, 1),
    (5, 16, 10, 1, 0, 1, 1),
])
def test_fconv_and_baseline_fconv_on_ramp_and_random(h, c, cout, k, pad, stride, dil):
    ramp = np.arange(h * h * c, dtype=np.float32).reshape(h, h, c)
    wramp = np.arange(cout * k * k * c, dtype=np.float32).reshape(cout, k, k, c)
    want = torch_conv_nhwc(ramp, wramp, None, stride, pad, dil)
    np.testing.assert_allclose(orc.baseline_fconv(ramp, wramp, k, k, pad, pad, stride, stride, dil, dil), want,
                               rtol=1e-5)
    np.testing.assert_allclose(orc.fconv(ramp, wramp, None, k, k, pad, pad, stride, stride, dil, dil), want,
                               rtol=1e-5)
    x = rng(40).standard_normal((h, h, c)).astype(np.float32)
    wgt = rng(41).standard_normal((cout, k, k, c)).astype(np.float32)
    bias = rng(42).standard_normal(cout).astype(np.float32)
    want = torch_conv_nhwc(x, wgt, bias, stride, pad, dil)
    np.testing.assert_allclose(orc.fconv(x, wgt, bias, k, k, pad, pad, stride, stride, dil, dil), want, rtol=1e-4,
                               atol=1e-4)


def test_affine_and_add():
    x = rng(43).standard_normal((3, 4, 8)).astype(np.float32)
    a = rng(44).standard_normal(8).astype(np.float32)
    b = rng(45).standard_normal(8).astype(np.float32)
    np.testing.assert_array_equal(orc.affine_inplace(x.copy(), a, b), a * x + b)
    y = rng(46).standard_normal((3, 4, 8)).astype(np.float32)
    np.testing.assert_array_equal(orc.add_inplace(x.copy(), y), x + y)


def test_relu_known_answers():
    """dabnn/layers/Relu.cpp:22-26 is std::max(x, 0.f) = (x < 0) ? 0 : x: negatives and -inf become +0, while -0, NaN,
    denormals and +inf pass through bit for bit."""
    x = np.array([-1.0, -0.0, 0.0, 1.0, np.nan, -np.inf, np.inf, -1e-40, 1e-40], np.float32)
    want = np.array([0.0, -0.0, 0.0, 1.0, np.nan, 0.0, np.inf, 0.0, 1e-40], np.float32)
    got = orc.relu_inplace(x.copy())
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    y = rng(51).standard_normal((3, 5, 8)).astype(np.float32)
    np.testing.assert_array_equal(orc.relu_inplace(y.copy()), torch.relu(torch.from_numpy(y)).numpy())


def test_prelu_vs_torch_and_concat_vs_numpy():
    """dabnn/layers/PRelu.cpp:6-30 against torch.nn.functional.prelu (NCHW, so the slope indexes dim 1) for one slope
    and for one slope per channel; dabnn/layers/Concat.cpp:7-21 against numpy.concatenate on the channel axis."""
    x = rng(48).standard_normal((5, 4, 8)).astype(np.float32)
    x[0, 0, :3] = [0.0, -0.0, -1.0]
    xt = torch.from_numpy(x).permute(2, 0, 1)[None]
    for slope in (np.array([0.25], np.float32), rng(49).uniform(-0.5, 0.5, 8).astype(np.float32)):
        want = F.prelu(xt, torch.from_numpy(slope))[0].permute(1, 2, 0).numpy()
        np.testing.assert_array_equal(orc.prelu_inplace(x.copy(), slope), want)
    with pytest.raises(RuntimeError, match="slope must have size 1 or input.channels"):
        orc.prelu_inplace(x.copy(), np.ones(3, np.float32))
    y = rng(50).standard_normal((5, 4, 3)).astype(np.float32)
    np.testing.assert_array_equal(orc.concat(x, y), np.concatenate([x, y], axis=-1))
    np.testing.assert_array_equal(orc.concat(y, x), np.concatenate([y, x], axis=-1))


@pytest.mark.parametrize("h,w,c,k,pad,stride", [(8, 8, 4, 2, 0, 2), (7, 7, 8, 7, 0, 1), (9, 6, 4, 3, 1, 2),
                                                (112, 112, 4, 3, 1, 2)])
def test_pools_vs_torch(h, w, c, k, pad, stride):
    x = rng(47).standard_normal((h, w, c)).astype(np.float32)
    xt = torch.from_numpy(x).permute(2, 0, 1)[None]
    avg = F.avg_pool2d(xt, k, stride, pad, count_include_pad=False)[0].permute(1, 2, 0).numpy()
    mx = F.max_pool2d(xt, k, stride, pad)[0].permute(1, 2, 0).numpy()
    np.testing.assert_allclose(orc.ave_pool(x, k, k, pad, pad, stride, stride), avg, rtol=1e-5, atol=1e-6)
    np.testing.assert_array_equal(orc.max_pool(x, k, k, pad, pad, stride, stride), mx)


def test_run_segments_fed_with_its_own_blobs_reproduces_the_layer_loop():
    """The segment-wise evaluation used to check a device run layer by layer, given the CPU run's own final blobs,
    must return exactly those blobs: in-place layers join the segment of the blob they rewrite, also when other
    layers (the shortcut of a down-sampling block) sit in between."""
    from dabnn_amd import models
    from oracle import net as orc_net
    for layers, inits, hw in (models.small_bnn(1, hw=16, width=64) [:2] + (16,), models.bireal18(3, stem=True)[:2] + (64,)):
        x = np.random.default_rng(5).standard_normal((hw, hw, 3)).astype(np.float32)
        if hw == 64:  # Bi-Real-18 graph on a 64 x 64 image: the 7 x 7 pool before the classifier becomes 2 x 2
            layers = [dict(l, kernel_shape=[2, 2]) if l["name"] == "pool5" else l for l in layers]
        cpu = orc_net.run_model(layers, inits, x)
        count = 0
        for name, _, want in orc_net.run_segments(layers, inits, lambda b: cpu[b]):
            np.testing.assert_array_equal(want, cpu[name])
            count += 1
        assert count == (7 if hw == 16 else 28)


# ---------------------------------------------------------------- Split / Shuffle on packed words
def _unpack_bits(words, c):
    """uint64 [..., cw] -> uint8 bits [..., c], bit j of word i = channel 64*i + j."""
    b = np.unpackbits(words[..., None].view(np.uint8), axis=-1, bitorder="little")
    return b.reshape(words.shape[:-1] + (c,))


@pytest.mark.parametrize("c", [128, 256, 384, 512])
def test_split_bit_is_a_slice_of_the_channel_axis(c):
    """dabnn/layers/Split.cpp:6-21: output 1 holds channels [0, c/2), output 2 channels [c/2, c), checked on the
    unpacked bits (numpy slicing), so that a mixed-up half or word order fails."""
    r = np.random.default_rng(60)
    x = r.integers(0, 2**64, size=(3, 5, c // 64), dtype=np.uint64)
    o1, o2 = orc.split_bit(x)
    bits = _unpack_bits(x, c)
    np.testing.assert_array_equal(_unpack_bits(o1, c // 2), bits[..., :c // 2])
    np.testing.assert_array_equal(_unpack_bits(o2, c // 2), bits[..., c // 2:])


def test_split_bit_rejects_other_channel_counts():
    for cw in (1, 3, 10):
        with pytest.raises(RuntimeError, match="Split"):
            orc.split_bit(np.zeros((2, 2, cw), dtype=np.uint64))


@pytest.mark.parametrize("c,group", [(128, 32), (256, 64), (512, 128)])
def test_shuffle_bit_is_a_channel_permutation(c, group):
    """dabnn/layers/Shuffle.cpp:6-43 read as a permutation of channels: the channels form four runs of `group`
    (a b c d) and come out as a c b d -- the two-group channel shuffle at that granularity; applying it twice
    is the identity."""
    r = np.random.default_rng(61)
    x = r.integers(0, 2**64, size=(4, 3, c // 64), dtype=np.uint64)
    bits = _unpack_bits(x, c)
    y = orc.shuffle_bit(x.copy())
    if c == 512:
        # the reference swaps words 2,3 with words 4,5 of the eight: runs of 128 channels, 1 and 2 change places
        want = np.concatenate([bits[..., :128], bits[..., 256:384], bits[..., 128:256], bits[..., 384:]], axis=-1)
    else:
        q = bits.reshape(bits.shape[:-1] + (4, group))
        want = q[..., [0, 2, 1, 3], :].reshape(bits.shape)
    np.testing.assert_array_equal(_unpack_bits(y, c), want)
    np.testing.assert_array_equal(orc.shuffle_bit(y.copy()), x)


def test_shuffle_bit_leaves_384_channels_alone_and_rejects_the_rest():
    x = np.random.default_rng(62).integers(0, 2**64, size=(2, 2, 6), dtype=np.uint64)
    np.testing.assert_array_equal(orc.shuffle_bit(x.copy()), x)  # no branch for 384 in the reference
    for cw in (1, 3, 10):
        with pytest.raises(RuntimeError, match="Shuffle"):
            orc.shuffle_bit(np.zeros((1, 1, cw), dtype=np.uint64))
