"""CPU oracle for dabnn's binary-convolution path (test infrastructure only).

numpy-facing ctypes wrappers around ``libdab_oracle.so`` (built from
``dab_oracle.c`` by ``oracle/Makefile``).  Only tests, the smoke check and the
CPU-baseline leg of the benchmark may import this package; the shipped
library never does.

All image tensors are single images in the reference's layouts: fp32
``[H, W, C]`` and packed ``uint64`` ``[H, W, C/64]``.  ``*_batch`` helpers loop
over a leading image axis the way a caller of the reference (which has no
batch dimension, dabnn/net.cpp:64-65) would.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libdab_oracle.so")

_c_float_p = ctypes.POINTER(ctypes.c_float)
_c_u64_p = ctypes.POINTER(ctypes.c_uint64)


def build(force=False):
    """Compile the oracle with gcc (reference release flags, no -march)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libdab_oracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        i, sz, fp, up, vp = ctypes.c_int, ctypes.c_size_t, _c_float_p, _c_u64_p, ctypes.c_void_p
        L.orc_pack_64.restype = ctypes.c_uint64
        L.orc_pack_64.argtypes = [fp, sz]
        L.orc_pack_mat.restype = i
        L.orc_pack_mat.argtypes = [fp, sz, up]
        L.orc_pack_nchw.restype = i
        L.orc_pack_nchw.argtypes = [fp, i, i, i, up]
        L.orc_pad_bit.restype = None
        L.orc_pad_bit.argtypes = [up, i, i, i, i, i, up]
        L.orc_pad_float.restype = None
        L.orc_pad_float.argtypes = [fp, i, i, i, i, i, ctypes.c_float, fp]
        L.orc_baseline_bconv.restype = None
        L.orc_baseline_bconv.argtypes = [up, i, i, i, up, i, i, i, i, i, i, i, i, i, i, fp, i, i]
        L.orc_xor_popcount_slow.restype = ctypes.c_uint32
        L.orc_xor_popcount_slow.argtypes = [up, up, sz]
        L.orc_bconv_3x3_padded.restype = None
        L.orc_bconv_3x3_padded.argtypes = [up, i, i, i, up, i, i, i, fp]
        L.orc_im2col.restype = None
        L.orc_im2col.argtypes = [vp, i, i, i, i, i, i, i, i, i, i, i, i, vp]
        L.orc_col_row_words.restype = i
        L.orc_col_row_words.argtypes = [i, i, i]
        L.orc_fused_binarize_im2col.restype = i
        L.orc_fused_binarize_im2col.argtypes = [fp, i, i, i, i, i, i, i, i, i, i, i, up]
        L.orc_weight_transpose.restype = None
        L.orc_weight_transpose.argtypes = [up, i, i, up]
        L.orc_bgemm_naive.restype = None
        L.orc_bgemm_naive.argtypes = [i, i, i, up, i, up, i, fp, i]
        L.orc_binconv_forward.restype = i
        L.orc_binconv_forward.argtypes = [fp, i, i, i, up, i, i, i, i, i, i, i, i, fp]
        L.orc_pack_weight.restype = i
        L.orc_pack_weight.argtypes = [fp, i, i, i, up]
        L.orc_bn_fold.restype = None
        L.orc_bn_fold.argtypes = [fp, fp, fp, fp, ctypes.c_float, i, i, fp, fp, fp]
        L.orc_baseline_fconv.restype = None
        L.orc_baseline_fconv.argtypes = [fp, i, i, i, fp, i, i, i, i, i, i, i, i, i, fp, i, i]
        L.orc_fconv.restype = i
        L.orc_fconv.argtypes = [fp, i, i, i, fp, fp, i, i, i, i, i, i, i, i, i, fp]
        L.orc_affine_inplace.restype = None
        L.orc_affine_inplace.argtypes = [fp, sz, i, fp, fp]
        L.orc_add_inplace.restype = None
        L.orc_add_inplace.argtypes = [fp, fp, sz]
        L.orc_prelu_inplace.restype = i
        L.orc_prelu_inplace.argtypes = [fp, sz, i, fp, i]
        L.orc_concat.restype = None
        L.orc_concat.argtypes = [fp, i, fp, i, sz, fp]
        L.orc_split_bit.restype = None
        L.orc_split_bit.argtypes = [up, sz, i, up, up]
        L.orc_shuffle_bit.restype = None
        L.orc_shuffle_bit.argtypes = [up, sz, i]
        L.orc_ave_pool.restype = None
        L.orc_ave_pool.argtypes = [fp, i, i, i, i, i, i, i, i, i, fp]
        L.orc_max_pool.restype = None
        L.orc_max_pool.argtypes = [fp, i, i, i, i, i, i, i, i, i, fp]
        _lib = L
    return _lib


def _f(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(_c_float_p)


def _u(a):
    a = np.ascontiguousarray(a, dtype=np.uint64)
    return a, a.ctypes.data_as(_c_u64_p)


def out_dim(size, pad, k, stride, dil=1):
    """common/Shaper.cpp:34-54 output extent (integer division)."""
    return (size + 2 * pad - (dil * (k - 1) + 1)) // stride + 1


def pack_64(f, eff_bits=64):
    f, p = _f(f)
    assert f.size >= 64
    return int(lib().orc_pack_64(p, eff_bits))


def pack_mat(x):
    """fp32 [..., C] (C % 64 == 0) -> uint64 [..., C/64]."""
    x, p = _f(x)
    assert x.shape[-1] % 64 == 0
    out = np.empty(x.shape[:-1] + (x.shape[-1] // 64,), dtype=np.uint64)
    rc = lib().orc_pack_mat(p, x.size, out.ctypes.data_as(_c_u64_p))
    assert rc == 0
    return out


def pack_nchw(x):
    """fp32 [C, H, W] -> uint64 [H, W, C/64]."""
    x, p = _f(x)
    c, h, w = x.shape
    out = np.empty((h, w, c // 64), dtype=np.uint64)
    rc = lib().orc_pack_nchw(p, c, h, w, out.ctypes.data_as(_c_u64_p))
    assert rc == 0
    return out


def pad_bit(x, pad_h, pad_w):
    x, p = _u(x)
    h, w, cw = x.shape
    out = np.empty((h + 2 * pad_h, w + 2 * pad_w, cw), dtype=np.uint64)
    lib().orc_pad_bit(p, h, w, cw, pad_h, pad_w, out.ctypes.data_as(_c_u64_p))
    return out


def baseline_bconv(x, wgt, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h=1, dil_w=1, cout=None):
    """x uint64 [H, W, CW]; wgt uint64 [Cout, words_per_filter] -> fp32 [OH, OW, Cout]."""
    x, xp = _u(x)
    wgt, wp = _u(wgt)
    h, w, cw = x.shape
    cout = wgt.shape[0] if cout is None else cout
    hwc = wgt.size // wgt.shape[0]
    oh, ow = out_dim(h, pad_h, kh, stride_h, dil_h), out_dim(w, pad_w, kw, stride_w, dil_w)
    out = np.zeros((oh, ow, cout), dtype=np.float32)
    lib().orc_baseline_bconv(xp, h, w, cw, wp, hwc, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, cout,
                             out.ctypes.data_as(_c_float_p), oh, ow)
    return out


def bconv_3x3_padded(xp_, wgt, stride=1):
    xp_, p = _u(xp_)
    wgt, wp = _u(wgt)
    hp, wpd, cw = xp_.shape
    cout = wgt.shape[0]
    hwc = wgt.size // cout
    out = np.zeros((out_dim(hp, 0, 3, stride), out_dim(wpd, 0, 3, stride), cout), dtype=np.float32)
    lib().orc_bconv_3x3_padded(p, hp, wpd, cw, wp, hwc, stride, cout, out.ctypes.data_as(_c_float_p))
    return out


def im2col(im, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h=1, dil_w=1):
    """[H, W, C] of any 4- or 8-byte dtype -> [OH*OW, kh*kw*C]."""
    im = np.ascontiguousarray(im)
    h, w, c = im.shape
    oh, ow = out_dim(h, pad_h, kh, stride_h, dil_h), out_dim(w, pad_w, kw, stride_w, dil_w)
    col = np.empty((oh * ow, kh * kw * c), dtype=im.dtype)
    lib().orc_im2col(im.ctypes.data, h, w, c, im.itemsize, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w,
                     col.ctypes.data)
    return col


def col_row_words(kh, kw, c):
    return int(lib().orc_col_row_words(kh, kw, c))


def fused_binarize_im2col(im, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h=1, dil_w=1):
    im, p = _f(im)
    h, w, c = im.shape
    oh, ow = out_dim(h, pad_h, kh, stride_h, dil_h), out_dim(w, pad_w, kw, stride_w, dil_w)
    col = np.empty((oh * ow, col_row_words(kh, kw, c)), dtype=np.uint64)
    rc = lib().orc_fused_binarize_im2col(p, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w,
                                         col.ctypes.data_as(_c_u64_p))
    if rc != 0:
        raise RuntimeError("kernel_h * kernel_w * im.c must be smaller than 60000")
    return col


def weight_transpose(w):
    """[m, k] -> flat [k*m] column-major A operand."""
    w, p = _u(w)
    m, k = w.shape
    out = np.empty((k, m), dtype=np.uint64)
    lib().orc_weight_transpose(p, m, k, out.ctypes.data_as(_c_u64_p))
    return out


def bgemm_naive(m, n, k, a, lda, b, ldb, c, ldc):
    """In-place C += popcount(A ^ B); a, b uint64 flat, c fp32 flat."""
    a, ap = _u(a)
    b, bp = _u(b)
    assert c.dtype == np.float32 and c.flags["C_CONTIGUOUS"]
    lib().orc_bgemm_naive(m, n, k, ap, lda, bp, ldb, c.ctypes.data_as(_c_float_p), ldc)
    return c


def binconv_forward(x, wgt, kh, kw, pad_h, pad_w, stride_h, stride_w):
    """The BinConv layer on a non-ARM target. Returns (out [OH, OW, Cout], method)."""
    x, xp = _f(x)
    wgt, wp = _u(wgt)
    h, w, c = x.shape
    cout = wgt.shape[0]
    hwc = wgt.size // cout
    oh, ow = out_dim(h, pad_h, kh, stride_h), out_dim(w, pad_w, kw, stride_w)
    out = np.zeros((oh, ow, cout), dtype=np.float32)
    rc = lib().orc_binconv_forward(xp, h, w, c, wp, hwc, kh, kw, pad_h, pad_w, stride_h, stride_w, cout,
                                   out.ctypes.data_as(_c_float_p))
    if rc < 0:
        raise RuntimeError("orc_binconv_forward failed: %d" % rc)
    return out, rc


def pack_weight(wf):
    """fp32 [Cout, KH, KW, Cin] -> uint64 [Cout, words_per_filter] (converter rule)."""
    wf, p = _f(wf)
    n, kh, kw, c = wf.shape
    hwc = kh * kw * c
    per = hwc // 64 if c == 64 else (hwc + 127) // 128 * 2
    out = np.zeros((n, per), dtype=np.uint64)
    got = lib().orc_pack_weight(p, n, hwc, c, out.ctypes.data_as(_c_u64_p))
    assert got == per
    return out


def bn_fold(scale, bias, mean, var, eps=1e-5, k_bits=0, conv_bias=None):
    scale, sp = _f(scale)
    bias, bp = _f(bias)
    mean, mp = _f(mean)
    var, vp = _f(var)
    n = scale.size
    a = np.empty(n, dtype=np.float32)
    b = np.empty(n, dtype=np.float32)
    cb = None
    if conv_bias is not None:
        conv_bias, cb = _f(conv_bias)
    lib().orc_bn_fold(sp, bp, mp, vp, eps, n, k_bits, cb, a.ctypes.data_as(_c_float_p), b.ctypes.data_as(_c_float_p))
    return a, b


def baseline_fconv(x, wgt, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h=1, dil_w=1):
    x, xp = _f(x)
    wgt, wp = _f(wgt)
    h, w, c = x.shape
    cout = wgt.size // (kh * kw * c)
    oh, ow = out_dim(h, pad_h, kh, stride_h, dil_h), out_dim(w, pad_w, kw, stride_w, dil_w)
    out = np.zeros((oh, ow, cout), dtype=np.float32)
    lib().orc_baseline_fconv(xp, h, w, c, wp, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, cout,
                             out.ctypes.data_as(_c_float_p), oh, ow)
    return out


def fconv(x, wgt, bias, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h=1, dil_w=1):
    x, xp = _f(x)
    wgt, wp = _f(wgt)
    h, w, c = x.shape
    cout = wgt.size // (kh * kw * c)
    bp = None
    if bias is not None:
        bias, bp = _f(bias)
    oh, ow = out_dim(h, pad_h, kh, stride_h, dil_h), out_dim(w, pad_w, kw, stride_w, dil_w)
    out = np.empty((oh, ow, cout), dtype=np.float32)
    rc = lib().orc_fconv(xp, h, w, c, wp, bp, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, cout,
                         out.ctypes.data_as(_c_float_p))
    assert rc == 0
    return out


def affine_inplace(x, a, b):
    assert x.dtype == np.float32 and x.flags["C_CONTIGUOUS"]
    a, ap = _f(a)
    b, bp = _f(b)
    c = x.shape[-1]
    lib().orc_affine_inplace(x.ctypes.data_as(_c_float_p), x.size // c, c, ap, bp)
    return x


def add_inplace(a, b):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    b, bp = _f(b)
    lib().orc_add_inplace(a.ctypes.data_as(_c_float_p), bp, a.size)
    return a


def relu_inplace(x):
    """dabnn/layers/Relu.cpp:22-26: *ptr = std::max(*ptr, 0.f), i.e. (x < 0) ? 0 : x -- a NaN and a negative zero stay
    what they are (numpy.maximum would return +0 for -0 on some builds)."""
    assert x.dtype == np.float32
    np.copyto(x, np.float32(0), where=x < 0)
    return x


def prelu_inplace(x, slope):
    assert x.dtype == np.float32 and x.flags["C_CONTIGUOUS"]
    slope, sp = _f(slope)
    c = x.shape[-1]
    if lib().orc_prelu_inplace(x.ctypes.data_as(_c_float_p), x.size // c, c, sp, slope.size) != 0:
        raise RuntimeError("slope must have size 1 or input.channels")  # dabnn/layers/PRelu.cpp:7-9
    return x


def concat(a, b):
    a, ap = _f(a)
    b, bp = _f(b)
    assert a.shape[:-1] == b.shape[:-1]
    ca, cb = a.shape[-1], b.shape[-1]
    out = np.empty(a.shape[:-1] + (ca + cb,), dtype=np.float32)
    lib().orc_concat(ap, ca, bp, cb, a.size // ca, out.ctypes.data_as(_c_float_p))
    return out


def split_bit(x):
    """dabnn/layers/Split.cpp:6-21: packed [..., cw] -> two packed [..., cw/2]; the channel count must be a multiple
    of 128 and at most 512 (dabnn/layers/Split.h:22-23)."""
    x, xp = _u(x)
    cw = x.shape[-1]
    if (cw * 64) % 128 != 0 or cw * 64 > 512:
        raise RuntimeError("Split: %d channels" % (cw * 64))
    o1 = np.empty(x.shape[:-1] + (cw // 2,), dtype=np.uint64)
    o2 = np.empty_like(o1)
    lib().orc_split_bit(xp, x.size // cw, cw, o1.ctypes.data_as(_c_u64_p), o2.ctypes.data_as(_c_u64_p))
    return o1, o2


def shuffle_bit(x):
    """dabnn/layers/Shuffle.cpp:6-43 in place on packed [..., cw] (uint64, contiguous)."""
    assert x.dtype == np.uint64 and x.flags["C_CONTIGUOUS"]
    cw = x.shape[-1]
    if (cw * 64) % 128 != 0 or cw * 64 > 512:
        raise RuntimeError("Shuffle: %d channels" % (cw * 64))  # dabnn/layers/Shuffle.h:19-20
    lib().orc_shuffle_bit(x.ctypes.data_as(_c_u64_p), x.size // cw, cw * 64)
    return x


def ave_pool(x, kh, kw, pad_h, pad_w, stride_h, stride_w):
    x, xp = _f(x)
    h, w, c = x.shape
    out = np.empty((out_dim(h, pad_h, kh, stride_h), out_dim(w, pad_w, kw, stride_w), c), dtype=np.float32)
    lib().orc_ave_pool(xp, h, w, c, pad_h, pad_w, stride_h, stride_w, kh, kw, out.ctypes.data_as(_c_float_p))
    return out


def max_pool(x, kh, kw, pad_h, pad_w, stride_h, stride_w):
    x, xp = _f(x)
    h, w, c = x.shape
    out = np.empty((out_dim(h, pad_h, kh, stride_h), out_dim(w, pad_w, kw, stride_w), c), dtype=np.float32)
    lib().orc_max_pool(xp, h, w, c, pad_h, pad_w, stride_h, stride_w, kh, kw, out.ctypes.data_as(_c_float_p))
    return out
