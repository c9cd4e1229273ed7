"""GPU: the benchmark's shapes at full batch size, checked through properties that do
not need the CPU oracle to chew through billions of bit operations:

* an independent textbook computation on the GPU itself: for +-1 tensors the
  mismatch count equals (K - conv2d(sign x, sign w, padding value -1)) / 2,
  with conv2d from torch (exact in fp32: |sums| <= 4608 < 2^24);
* complement symmetry: cnt(~x, w) + cnt(x, w) == 9*Cin on interior pixels;
* batch consistency: every image of a batch equals the batch-1 result;
* bgemm linearity in C: running twice adds the counts twice.
A sample of outputs is also compared with the CPU oracle.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle as orc

pytestmark = pytest.mark.gpu

STAGE_SHAPES = [(56, 64, 64, 1), (28, 128, 128, 1), (14, 256, 256, 1), (7, 512, 512, 1), (56, 64, 128, 2),
                (28, 128, 256, 2), (14, 256, 512, 2)]


@pytest.fixture(scope="module")
def dab():
    import dabnn_amd
    assert torch.cuda.is_available()
    return dabnn_amd


def unpack_pm1(words, c):
    """int64 [..., cw] -> float +-1 [..., c] on the GPU."""
    shifts = torch.arange(64, device=words.device, dtype=torch.int64)
    bits = (words.unsqueeze(-1) >> shifts) & 1
    return (bits.reshape(words.shape[:-1] + (c,)).to(torch.float32) * 2 - 1)


def rand_words(gen, *shape):
    return torch.randint(-2**63, 2**63 - 1, shape, dtype=torch.int64, generator=gen).cuda()


@pytest.mark.parametrize("hw,cin,cout,stride", STAGE_SHAPES)
def test_bconv_batch64_equals_float_convolution(dab, hw, cin, cout, stride):
    gen = torch.Generator().manual_seed(hw * 1000 + cin + stride)
    n = 64
    x = rand_words(gen, n, hw, hw, cin // 64)
    w = rand_words(gen, cout, 9 * cin // 64)
    cnt = dab.bconv_3x3(x, w, stride, 1)
    xs = unpack_pm1(x, cin).permute(0, 3, 1, 2)  # N,C,H,W
    ws = unpack_pm1(w.reshape(cout, 3, 3, cin // 64), cin).permute(0, 3, 1, 2)
    torch.backends.cudnn.allow_tf32 = False
    torch.backends.cuda.matmul.allow_tf32 = False
    conv = F.conv2d(F.pad(xs, (1, 1, 1, 1), value=-1.0), ws, stride=stride).permute(0, 2, 3, 1)
    want = (9 * cin - conv) / 2
    assert torch.equal(cnt, want), (cnt - want).abs().max().item()
    # batch consistency with the batch-1 launch and a CPU-oracle sample (image 17)
    one = dab.bconv_3x3(x[17:18].contiguous(), w, stride, 1)
    assert torch.equal(one[0], cnt[17])
    xi = x[17].cpu().numpy().view(np.uint64)
    wi = w.cpu().numpy().view(np.uint64)
    cpu = orc.baseline_bconv(xi, wi, 3, 3, 1, 1, stride, stride)
    np.testing.assert_array_equal(cnt[17].cpu().numpy(), cpu)


@pytest.mark.parametrize("n,h,w,cin,cout,stride", [
    # outputs on both sides of the sizes at which a launch of raw counts starts to write through the L2 (6 MB with
    # 32-channel staging windows, 9 MB with 16-channel ones), ragged pixel counts, channel counts that are no
    # multiple of a window, every channel depth, both strides
    (23, 31, 29, 64, 72, 1), (37, 30, 27, 64, 104, 1), (90, 41, 39, 64, 64, 2), (150, 29, 31, 64, 136, 2),
    (21, 27, 25, 128, 136, 1), (35, 26, 29, 128, 152, 1), (61, 33, 31, 128, 200, 2),
    (70, 15, 13, 256, 120, 1), (100, 14, 15, 256, 264, 1), (170, 17, 15, 256, 520, 2),
    (111, 9, 7, 512, 232, 1), (190, 8, 9, 512, 520, 1), (45, 56, 56, 64, 64, 1),
])
def test_bconv_sizes_around_the_store_policy_switch(dab, n, h, w, cin, cout, stride):
    """dab_bconv3x3 against the float convolution of the +-1 tensors (exact in fp32), whole tensor, at sizes where
    the launcher changes the way the stores go through the L2 and where waves' ranges cut staging windows apart."""
    gen = torch.Generator().manual_seed(n * 7 + h * 3 + cout)
    x = rand_words(gen, n, h, w, cin // 64)
    wt = rand_words(gen, cout, 9 * cin // 64)
    cnt = dab.bconv_3x3(x, wt, stride, 1)
    xs = unpack_pm1(x, cin).permute(0, 3, 1, 2)
    ws = unpack_pm1(wt.reshape(cout, 3, 3, cin // 64), cin).permute(0, 3, 1, 2)
    torch.backends.cudnn.allow_tf32 = False
    torch.backends.cuda.matmul.allow_tf32 = False
    conv = F.conv2d(F.pad(xs, (1, 1, 1, 1), value=-1.0), ws, stride=stride).permute(0, 2, 3, 1)
    want = (9 * cin - conv) / 2
    assert torch.equal(cnt, want), (cnt - want).abs().max().item()


@pytest.mark.parametrize("hw,cin,cout,stride", [(56, 64, 64, 1), (14, 256, 256, 1), (28, 128, 256, 2)])
def test_bconv_complement_symmetry(dab, hw, cin, cout, stride):
    gen = torch.Generator().manual_seed(99)
    x = rand_words(gen, 8, hw, hw, cin // 64)
    w = rand_words(gen, cout, 9 * cin // 64)
    a = dab.bconv_3x3(x, w, stride, 1)
    b = dab.bconv_3x3(~x, w, stride, 1)
    s = (a + b)
    interior = s[:, 1:-1, 1:-1] if stride == 1 else s[:, 1:, 1:][:, :-1, :-1]
    assert (interior == 9 * cin).all()


def test_bgemm_config2_linearity_and_float_reference(dab):
    m, n, k = 512, 3136, 72
    gen = torch.Generator().manual_seed(5)
    a = rand_words(gen, k, m)
    b = rand_words(gen, n, k)
    c = torch.zeros((n, m), dtype=torch.float32, device="cuda")
    dab.bgemm(m, n, k, a, m, b, k, c, m)
    first = c.clone()
    dab.bgemm(m, n, k, a, m, b, k, c, m)
    assert torch.equal(c, 2 * first)  # C is accumulated into
    av = unpack_pm1(a.t().contiguous(), k * 64)  # m, K
    bv = unpack_pm1(b, k * 64)  # n, K
    want = (k * 64 - bv @ av.t()) / 2
    assert torch.equal(first, want)


def test_bitpack_config2_roundtrip(dab):
    gen = torch.Generator().manual_seed(6)
    x = torch.randn((1, 512, 56, 56), generator=gen).cuda()  # NCHW
    words = dab.bitpack_nchw(x)
    assert words.shape == (1, 56, 56, 8)
    back = unpack_pm1(words, 512)  # NHWC +-1
    want = torch.where(x > 0, 1.0, -1.0).permute(0, 2, 3, 1)
    assert torch.equal(back, want)
    nhwc = x.permute(0, 2, 3, 1).contiguous()
    assert torch.equal(dab.pack_mat(nhwc), words)
    # batch 64 of the same shape
    xb = torch.randn((64, 56, 56, 512), generator=gen).cuda()
    assert torch.equal(unpack_pm1(dab.pack_mat(xb), 512), torch.where(xb > 0, 1.0, -1.0))


def test_fused_im2col_batch64_equals_pack_of_unfold(dab):
    gen = torch.Generator().manual_seed(7)
    x = torch.randn((64, 28, 28, 128), generator=gen).cuda()
    col = dab.fused_binarize_im2col(x, 3, 3, 1, 1, 1, 1)
    assert col.shape == (64 * 28 * 28, 18)
    # independent gather: zero-pad, take the 9 taps in (kh, kw) order, sign-pack with pack_mat
    xp = F.pad(x, (0, 0, 1, 1, 1, 1))
    taps = [xp[:, a:a + 28, b:b + 28, :] for a in range(3) for b in range(3)]
    gathered = torch.cat(taps, dim=-1).reshape(-1, 9 * 128).contiguous()
    assert torch.equal(dab.pack_mat(gathered), col)


@pytest.mark.parametrize("hw,cin,cout,stride", STAGE_SHAPES)
def test_fused_epilogue_batch64_equals_separate_layers(dab, hw, cin, cout, stride):
    """At full batch the one-pass BinConv + Affine + Add (+ sign) equals the separate kernels of the library bit for bit:
    counts, then affine_inplace, add_inplace, and pack_mat of the result."""
    gen = torch.Generator().manual_seed(7 * hw + cin + stride)
    n = 64
    x = rand_words(gen, n, hw, hw, cin // 64)
    w = rand_words(gen, cout, 9 * cin // 64)
    a = (torch.randn(cout, generator=gen) / 40).cuda()
    b = torch.randn(cout, generator=gen).cuda()
    a[::7] = 0.0
    b[::14] = 0.0  # exact zeros in the result: their sign bit must be 0
    want = dab.bconv_3x3(x, w, stride, 1)
    sc = torch.randn(want.shape, generator=gen).cuda()
    sc[..., ::14] = 0.0
    dab.affine_inplace(want, a, b)
    dab.add_inplace(want, sc)
    got1 = dab.bconv_3x3_affine_add(x, w, a, b, sc, stride, 1)
    assert torch.equal(got1, want)
    got2, packed = dab.bconv_3x3_affine_add_sign(x, w, a, b, sc, stride, 1)
    assert torch.equal(got2, want)
    assert torch.equal(packed, dab.pack_mat(want))
    assert (want == 0).any()


@pytest.mark.parametrize("n,hw,c,cout,k,pad,stride", [(32, 224, 3, 64, 7, 3, 2), (16, 112, 32, 64, 3, 1, 1), (64, 28, 64, 128, 1, 0, 1),
                                                       (256, 1, 512, 1000, 1, 0, 1), (1, 224, 3, 64, 7, 3, 2)])
def test_fconv_full_size_against_torch(dab, n, hw, c, cout, k, pad, stride):
    """The float convolutions of Bi-Real-18 at their real sizes against torch's fp32 convolution on the GPU, 1e-4
    relative (the tolerance of the float layers), with and without the fused Affine + Relu."""
    gen = torch.Generator().manual_seed(n + hw + c)
    x = torch.randn((n, hw, hw, c), generator=gen).cuda()
    w = (torch.randn((cout, k, k, c), generator=gen) / (k * k * c) ** 0.5).cuda()
    bias = torch.randn(cout, generator=gen).cuda()
    a, b = torch.randn(cout, generator=gen).cuda(), torch.randn(cout, generator=gen).cuda()
    torch.backends.cudnn.allow_tf32 = False
    torch.backends.cuda.matmul.allow_tf32 = False
    ref = F.conv2d(x.permute(0, 3, 1, 2), w.permute(0, 3, 1, 2), bias, stride=stride, padding=pad).permute(0, 2, 3, 1)
    got = dab.fconv(x, w, bias, k, k, pad, pad, stride, stride)
    scale = ref.abs().max().item()
    assert (got - ref).abs().max().item() <= 1e-4 * scale
    fused = dab.fconv_affine_relu(x, w, bias, a, b, True, k, k, pad, pad, stride, stride)
    ref2 = torch.relu(ref * a + b)
    assert (fused - ref2).abs().max().item() <= 1e-4 * max(ref2.abs().max().item(), scale * a.abs().max().item())


@pytest.mark.parametrize("n,hw,c,cout,k,pad,stride,relu", [(256, 224, 3, 64, 7, 3, 2, False), (64, 112, 32, 64, 3, 1, 1, True),
                                                            (7, 224, 3, 64, 7, 3, 2, True)])
def test_fconv_maxpool_full_size_against_torch(dab, n, hw, c, cout, k, pad, stride, relu):
    """The last convolution of either Bi-Real-18 stem with its MaxPool 3x3 stride 2 inside, at the real sizes (every
    persistent block walks many bands), against torch's fp32 convolution and max pooling on the GPU, 1e-4 relative;
    the packed copy is pack_mat of the pooled tensor the launch wrote."""
    gen = torch.Generator().manual_seed(n + hw + c)
    x = torch.randn((n, hw, hw, c), generator=gen).cuda()
    w = (torch.randn((cout, k, k, c), generator=gen) / (k * k * c) ** 0.5).cuda()
    a, b = torch.randn(cout, generator=gen).cuda(), torch.randn(cout, generator=gen).cuda()
    torch.backends.cudnn.allow_tf32 = False
    torch.backends.cuda.matmul.allow_tf32 = False
    # the Net takes this pass for both stems: the band kernel for the 7x7 stem, the pooled form of the split-operand
    # kernel for the 3x3 convolution over 32 channels at this size
    assert dab.fconv_maxpool_pays(n, hw, hw, c, k, k, pad, pad, stride, stride, 1, 1, cout)
    ref = F.conv2d(x.permute(0, 3, 1, 2), w.permute(0, 3, 1, 2), None, stride=stride, padding=pad)
    ref = ref * a.view(1, -1, 1, 1) + b.view(1, -1, 1, 1)
    scale = ref.abs().max().item()
    if relu:
        ref = torch.relu(ref)
    ref = F.max_pool2d(ref, 3, 2, 1).permute(0, 2, 3, 1)
    pooled, packed = dab.fconv_maxpool(x, w, None, a, b, relu, k, k, pad, pad, stride, stride, want_sign=True)
    assert pooled.shape == ref.shape
    assert (pooled - ref).abs().max().item() <= 1e-4 * scale
    assert torch.equal(packed, dab.pack_mat(pooled))
