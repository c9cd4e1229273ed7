"""GPU parity on seeded random shapes: the kernels against the CPU oracle over shapes nobody picked by hand.

Every case is bit-exact for the binary path and the pools and within the float tolerance for the convolutions; the
shapes are small enough for the oracle to finish the whole file in seconds.
"""
import numpy as np
import pytest
import torch

import oracle as orc

pytestmark = pytest.mark.gpu

RTOL = 1e-4


@pytest.fixture(scope="module")
def dab():
    import dabnn_amd
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return dabnn_amd


def dev_f(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


def dev_u(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.uint64).view(np.int64)).cuda()


def host_u(t):
    return t.cpu().numpy().view(np.uint64)


@pytest.mark.parametrize("seed", range(4))
def test_bconv_3x3_all_modes_on_random_shapes(dab, seed):
    """bconv_3x3 (baseline_bconv, common/baseline.h:77-116), its fused Affine + Add and the packed copy of the result."""
    r = np.random.default_rng(100 + seed)
    for _ in range(12):
        cin = int(r.choice([64, 128, 256, 512, 1024]))
        cw = cin // 64
        n, h, w = int(r.integers(1, 30)), int(r.integers(3, 30)), int(r.integers(3, 30))
        if r.random() < 0.2:
            n = int(r.integers(30, 120))  # enough work items for the unit kernel
        cout, stride, pad = int(r.integers(1, 33)) * 8, int(r.integers(1, 3)), int(r.integers(0, 2))
        case = "n %d h %d w %d cin %d cout %d stride %d pad %d" % (n, h, w, cin, cout, stride, pad)
        x = r.integers(0, 2**64, size=(n, h, w, cw), dtype=np.uint64)
        wgt = r.integers(0, 2**64, size=(cout, 9 * cw), dtype=np.uint64)
        want = np.stack([orc.baseline_bconv(img, wgt, 3, 3, pad, pad, stride, stride) for img in x])
        got = dab.bconv_3x3(dev_u(x), dev_u(wgt), stride, pad).cpu().numpy()
        np.testing.assert_array_equal(got, want, err_msg=case)
        if cin > 512 or pad != 1:
            continue
        a = (r.standard_normal(cout) / 50).astype(np.float32)
        b = r.standard_normal(cout).astype(np.float32)
        sc = r.standard_normal(want.shape).astype(np.float32) if r.random() < 0.7 else None
        ref = want.copy()
        for img in ref:
            orc.affine_inplace(img, a, b)
        if sc is not None:
            ref = ref + sc
        shortcut = dev_f(sc) if sc is not None else None
        got = dab.bconv_3x3_affine_add(dev_u(x), dev_u(wgt), dev_f(a), dev_f(b), shortcut, stride, 1)
        np.testing.assert_array_equal(got.cpu().numpy(), ref, err_msg=case)
        if cout % 64 == 0:
            out, bits = dab.bconv_3x3_affine_add_sign(dev_u(x), dev_u(wgt), dev_f(a), dev_f(b), shortcut, stride, 1)
            np.testing.assert_array_equal(out.cpu().numpy(), ref, err_msg=case)
            assert torch.equal(bits, dab.pack_mat(out)), case


@pytest.mark.parametrize("seed", range(4))
def test_binconv_layer_on_random_shapes(dab, seed):
    """BinConv::forward_impl (dabnn/layers/BinConv.cpp:137-191) from fp32 input, whichever method the dispatch picks,
    with fused_binarize_im2col and pack_mat on the same input."""
    r = np.random.default_rng(200 + seed)
    for _ in range(16):
        c = 64 * int(r.integers(1, 9)) if r.random() < 0.8 else int(r.choice([64, 128, 192, 256, 320, 512, 1024]))
        k = int(r.choice([1, 3, 3, 3, 5]))
        pad, stride = int(r.integers(0, k // 2 + 1)), int(r.integers(1, 3))
        n, h, w, cout = int(r.integers(1, 6)), int(r.integers(k, 20)), int(r.integers(k, 20)), int(r.integers(1, 20)) * 8
        case = "n %d h %d w %d c %d cout %d k %d pad %d stride %d" % (n, h, w, c, cout, k, pad, stride)
        x = r.standard_normal((n, h, w, c)).astype(np.float32)
        x.flat[::13] = 0.0
        x.flat[5::17] = -0.0
        x.flat[3::29] = np.nan
        wp = orc.pack_weight(r.standard_normal((cout, k, k, c)).astype(np.float32))
        layer = dab.BinConv(dev_u(wp), k, k, pad, pad, stride, stride)
        got = layer(dev_f(x)).cpu().numpy()
        if c == 64 and k != 3:
            want = np.stack([orc.baseline_bconv(orc.pack_mat(img), wp, k, k, pad, pad, stride, stride) for img in x])
        else:
            want = np.stack([orc.binconv_forward(img, wp, k, k, pad, pad, stride, stride)[0] for img in x])
        np.testing.assert_array_equal(got, want, err_msg=case)
        got = host_u(dab.fused_binarize_im2col(dev_f(x), k, k, pad, pad, stride, stride))
        want = np.concatenate([orc.fused_binarize_im2col(img, k, k, pad, pad, stride, stride) for img in x])
        np.testing.assert_array_equal(got, want, err_msg=case)
        np.testing.assert_array_equal(host_u(dab.pack_mat(dev_f(x))), np.stack([orc.pack_mat(img) for img in x]), err_msg=case)


@pytest.mark.parametrize("seed", range(3))
def test_fconv_and_pools_on_random_shapes(dab, seed):
    """FpConv2D (dabnn/fconv.h:14-76) and the pools (dabnn/layers/AvePool.cpp:84-123, MaxPool.cpp:209-246)."""
    r = np.random.default_rng(300 + seed)
    for _ in range(14):
        c, k = int(r.choice([3, 4, 8, 32, 64, 128, 5])), int(r.choice([1, 3, 5, 7]))
        pad, stride, dil = int(r.integers(0, k // 2 + 1)), int(r.integers(1, 3)), 1 if r.random() < 0.8 else 2
        n, h, w = int(r.integers(1, 5)), int(r.integers((k - 1) * dil + 1, 40)), int(r.integers((k - 1) * dil + 1, 40))
        cout = int(r.integers(1, 140))
        case = "n %d h %d w %d c %d cout %d k %d pad %d stride %d dil %d" % (n, h, w, c, cout, k, pad, stride, dil)
        x = r.standard_normal((n, h, w, c)).astype(np.float32)
        wgt = (r.standard_normal((cout, k, k, c)) / np.sqrt(k * k * c)).astype(np.float32)
        bias = r.standard_normal(cout).astype(np.float32) if r.random() < 0.5 else None
        got = dab.fconv(dev_f(x), dev_f(wgt), dev_f(bias) if bias is not None else None, k, k, pad, pad, stride, stride,
                        dil, dil).cpu().numpy()
        want = np.stack([orc.fconv(img, wgt, bias, k, k, pad, pad, stride, stride, dil, dil) for img in x])
        np.testing.assert_allclose(got, want, rtol=RTOL, atol=RTOL * np.abs(want).max(), err_msg=case)
        kp = int(r.integers(1, 4))
        sp, pp = int(r.integers(1, 3)), int(r.integers(0, kp // 2 + 1))
        if h + 2 * pp >= kp and w + 2 * pp >= kp:
            for gpu_pool, cpu_pool in ((dab.ave_pool, orc.ave_pool), (dab.max_pool, orc.max_pool)):
                got = gpu_pool(dev_f(x), kp, kp, pp, pp, sp, sp).cpu().numpy()
                want = np.stack([cpu_pool(img, kp, kp, pp, pp, sp, sp) for img in x])
                np.testing.assert_array_equal(got, want, err_msg=case + " pool %d %d %d" % (kp, pp, sp))


def test_fconv_over_32_channels_on_random_shapes(dab):
    """The split-operand kernel for 3x3 stride-1 convolutions over 32 channels takes problems of 4096 columns of tiles
    and more: random image sizes and paddings at the smallest batch that gets there, against a float64 convolution."""
    r = np.random.default_rng(400)
    done = 0
    while done < 8:
        pad, ow = int(r.integers(0, 3)), 16 * int(r.integers(1, 5))
        w, h = ow + 2 - 2 * pad, int(r.integers(max(1, 3 - 2 * pad), 40))
        oh, cout = h + 2 * pad - 2, int(r.choice([32, 64]))
        n = -(-4096 // (-(-oh // 4) * (ow // 16))) + int(r.integers(0, 5))
        if n * h * w * 128 >= 2**30 or n * oh * ow * cout * 4 >= 2**30:
            continue
        done += 1
        case = "n %d h %d w %d pad %d cout %d" % (n, h, w, pad, cout)
        x = r.standard_normal((n, h, w, 32)).astype(np.float32)
        wgt = (r.standard_normal((cout, 3, 3, 32)) / 17).astype(np.float32)
        bias = r.standard_normal(cout).astype(np.float32) if r.random() < 0.5 else None
        affine, relu = bool(r.random() < 0.5), bool(r.random() < 0.5)
        a, b = r.standard_normal(cout).astype(np.float32), r.standard_normal(cout).astype(np.float32)
        got = dab.fconv_affine_relu(dev_f(x), dev_f(wgt), dev_f(bias) if bias is not None else None,
                                    dev_f(a) if affine else None, dev_f(b) if affine else None, relu, 3, 3, pad, pad, 1, 1)
        y = torch.nn.functional.conv2d(dev_f(x).double().permute(0, 3, 1, 2), dev_f(wgt).double().permute(0, 3, 1, 2), padding=pad)
        if bias is not None:
            y = y + dev_f(bias).double().view(1, -1, 1, 1)
        if affine:
            y = y * dev_f(a).double().view(1, -1, 1, 1) + dev_f(b).double().view(1, -1, 1, 1)
        if relu:
            y = torch.relu(y)
        y = y.permute(0, 2, 3, 1)
        assert got.shape == y.shape, case
        assert (got.double() - y).abs().max().item() <= 4e-6 * y.abs().max().item(), case


@pytest.mark.parametrize("seed", range(2))
def test_pooled_shortcut_convolution_on_random_shapes(dab, seed):
    """AvePool 2x2 stride 2 + 1x1 FpConv2D (+ bias, Affine, Relu) in one launch (dabnn/layers/AvePool.cpp:84-123,
    dabnn/fconv.h:14-76): over 64 channels with enough pixels the kernel that keeps a block's pooled pixels in LDS,
    otherwise the tile kernel with the pooling loader.  Pooled tensor and convolution bit for bit those of the two
    separate launches, the same convolution without the pooled tensor, and both within the float tolerance of the
    CPU layers."""
    r = np.random.default_rng(500 + seed)
    for case_no in range(12):
        if case_no < 7:  # 64 channels and thousands of pooled pixels: the pooled tile in LDS
            c, n, h, w = 64, int(r.integers(6, 25)), int(r.integers(30, 60)), int(r.integers(30, 60))
            cout = int(r.choice([65, 72, 128, 130, 200, 256, 384]))
        else:
            c = int(r.choice([64, 64, 128, 32, 8]))
            n, h, w = int(r.integers(1, 12)), int(r.integers(2, 60)), int(r.integers(2, 60))
            cout = int(r.choice([65, 72, 128, 130, 200, 256, 384, 17]))
        flags = [bool(r.random() < 0.5) for _ in range(3)]
        case = "n %d h %d w %d c %d cout %d bias %d affine %d relu %d" % (n, h, w, c, cout, *flags)
        x = r.standard_normal((n, h, w, c)).astype(np.float32)
        wgt = (r.standard_normal((cout, 1, 1, c)) / np.sqrt(c)).astype(np.float32)
        bias, a, b = (r.standard_normal(cout).astype(np.float32) for _ in range(3))
        args = (dev_f(wgt), dev_f(bias) if flags[0] else None, dev_f(a) if flags[1] else None,
                dev_f(b) if flags[1] else None, flags[2])
        pooled, out = dab.ave_pool2_fconv1x1(dev_f(x), *args)
        want_pooled = dab.ave_pool(dev_f(x), 2, 2, 0, 0, 2, 2)
        want_out = dab.fconv_affine_relu(want_pooled, *args, 1, 1, 0, 0, 1, 1)
        np.testing.assert_array_equal(pooled.cpu().numpy(), want_pooled.cpu().numpy(), err_msg=case)
        np.testing.assert_array_equal(out.cpu().numpy(), want_out.cpu().numpy(), err_msg=case)
        if n * (h // 2) * (w // 2) > 8 or cout < 64:
            _, out2 = dab.ave_pool2_fconv1x1(dev_f(x), *args, want_pooled=False)
            np.testing.assert_array_equal(out2.cpu().numpy(), want_out.cpu().numpy(), err_msg=case)
        for i in range(min(n, 2)):
            cpu_pooled = orc.ave_pool(x[i], 2, 2, 0, 0, 2, 2)
            np.testing.assert_array_equal(pooled[i].cpu().numpy(), cpu_pooled, err_msg=case)
            want = orc.fconv(cpu_pooled, wgt, bias if flags[0] else None, 1, 1, 0, 0, 1, 1)
            if flags[1]:
                want = orc.affine_inplace(want, a, b)
            if flags[2]:
                want = orc.relu_inplace(want)
            np.testing.assert_allclose(out[i].cpu().numpy(), want, rtol=RTOL, atol=RTOL * np.abs(want).max(), err_msg=case)
