"""Reference-named operators over torch CUDA tensors.

Function names and argument meaning follow the reference's free functions
(dabnn/bitpack.h, dabnn/fused_binarize_im2col.h, dabnn/bgemm.h, dabnn/bconv.h,
dabnn/pad.h, dabnn/fconv.h and the float layers), with a leading batch axis:
fp32 activations are ``[N, H, W, C]``, packed activations ``int64 [N, H, W, C/64]``
(torch has no uint64 arithmetic; the bit pattern is what matters).  torch only
supplies device memory and the current stream.
"""
import ctypes

import torch

from . import capi
from .capi import check, lib


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _need(t, dtype, name):
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == dtype and t.is_contiguous()):
        raise capi.DabError(capi.DAB_EINVAL, "%s must be a contiguous CUDA tensor of %s" % (name, dtype))


def _empty(shape, dtype, device):
    """Like torch.empty, but an empty result still owns memory, so the C ABI (not a null check) reports bad shapes."""
    numel = 1
    for d in shape:
        numel *= d
    if numel > 0:
        return torch.empty(shape, dtype=dtype, device=device)
    return torch.empty(1, dtype=dtype, device=device)


def out_dim(size, pad, k, stride, dil=1):
    return (size + 2 * pad - (dil * (k - 1) + 1)) // stride + 1


def col_row_words(kh, kw, c):
    return lib.dab_col_row_words(kh, kw, c)


def pack_mat(x):
    """pack_mat (dabnn/bitpack.h:277-293): fp32 [..., C] -> int64 [..., C/64]."""
    _need(x, torch.float32, "x")
    c = x.shape[-1]
    out = _empty(x.shape[:-1] + (max(c // 64, 0),), torch.int64, x.device)
    check(lib.dab_bitpack_nhwc(_ptr(x), _ptr(out), x.numel() // max(c, 1), c, _stream()))
    return out


def bitpack_nchw(x):
    """fp32 [N, C, H, W] -> int64 [N, H, W, C/64] (same words as pack_mat of the NHWC permutation)."""
    _need(x, torch.float32, "x")
    n, c, h, w = x.shape
    out = _empty((n, h, w, c // 64), torch.int64, x.device)
    check(lib.dab_bitpack_nchw(_ptr(x), _ptr(out), n, c, h, w, _stream()))
    return out


def pad(x, pad_h, pad_w):
    """pad, Bit branch (dabnn/pad.h:7-19)."""
    _need(x, torch.int64, "x")
    n, h, w, cw = x.shape
    out = _empty((n, h + 2 * pad_h, w + 2 * pad_w, cw), torch.int64, x.device)
    check(lib.dab_pad_bit(_ptr(x), n, h, w, cw, pad_h, pad_w, _ptr(out), _stream()))
    return out


def split_bit(x):
    """Split::forward_impl (dabnn/layers/Split.cpp:6-21): packed [..., CW] -> two packed [..., CW/2]."""
    _need(x, torch.int64, "x")
    cw = x.shape[-1]
    half = tuple(x.shape[:-1]) + (max(cw // 2, 1),)
    o1, o2 = _empty(half, torch.int64, x.device), _empty(half, torch.int64, x.device)
    check(lib.dab_split_bit(_ptr(x), x.numel() // max(cw, 1), cw, _ptr(o1), _ptr(o2), _stream()))
    return o1, o2


def shuffle_bit_inplace(x):
    """Shuffle::forward_impl (dabnn/layers/Shuffle.cpp:6-43), in place on packed [..., CW]."""
    _need(x, torch.int64, "x")
    cw = x.shape[-1]
    check(lib.dab_shuffle_bit_inplace(_ptr(x), x.numel() // max(cw, 1), cw * 64, _stream()))
    return x


def fused_binarize_im2col(x, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h=1, dil_w=1):
    """fused_binarize_im2col (dabnn/fused_binarize_im2col.h:6-68): -> int64 [N*OH*OW, row_words]."""
    _need(x, torch.float32, "x")
    n, h, w, c = x.shape
    oh, ow = out_dim(h, pad_h, kh, stride_h, dil_h), out_dim(w, pad_w, kw, stride_w, dil_w)
    col = _empty((max(n * oh * ow, 0), col_row_words(kh, kw, c)), torch.int64, x.device)
    check(lib.dab_fused_binarize_im2col(_ptr(x), n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w,
                                        _ptr(col), _stream()))
    return col


def weight_transpose(w):
    """BinConv constructor transpose (dabnn/layers/BinConv.cpp:59-76): [m, k] -> [k, m]."""
    _need(w, torch.int64, "w")
    m, k = w.shape
    wt = _empty((k, m), torch.int64, w.device)
    check(lib.dab_weight_transpose(_ptr(w), m, k, _ptr(wt), _stream()))
    return wt


def bgemm(m, n, k, a, lda, b, ldb, c, ldc):
    """bgemm (dabnn/bgemm.h:46-66): column-major C += popcount(A ^ B), in place on c."""
    _need(a, torch.int64, "a")
    _need(b, torch.int64, "b")
    _need(c, torch.float32, "c")
    if a.numel() < (k - 1) * lda + m or b.numel() < (n - 1) * ldb + k or c.numel() < (n - 1) * ldc + m:
        raise capi.DabError(capi.DAB_EINVAL, "bgemm: operand smaller than its m/n/k/ld description")
    check(lib.dab_bgemm(m, n, k, _ptr(a), lda, _ptr(b), ldb, _ptr(c), ldc, _stream()))
    return c


def bgemm_overwrite(m, n, k, a, lda, b, ldb, c, ldc):
    """fill(0) + bgemm (dabnn/layers/BinConv.cpp:153-165) as one launch: C = popcount(A ^ B), C is not read."""
    _need(a, torch.int64, "a")
    _need(b, torch.int64, "b")
    _need(c, torch.float32, "c")
    if a.numel() < (k - 1) * lda + m or b.numel() < (n - 1) * ldb + k or c.numel() < (n - 1) * ldc + m:
        raise capi.DabError(capi.DAB_EINVAL, "bgemm: operand smaller than its m/n/k/ld description")
    check(lib.dab_bgemm_overwrite(m, n, k, _ptr(a), lda, _ptr(b), ldb, _ptr(c), ldc, _stream()))
    return c


def bconv_3x3(x, weight, stride=1, pad=1):
    """pad + bconv_3x3 (dabnn/bconv.h:855-931): packed [N,H,W,CW], weight int64 [Cout, 9*CW] -> fp32 counts."""
    _need(x, torch.int64, "x")
    _need(weight, torch.int64, "weight")
    n, h, w, cw = x.shape
    cout = weight.shape[0]
    if weight.numel() != cout * 9 * cw:
        raise capi.DabError(capi.DAB_EINVAL, "bconv_3x3: weight has %d words, expected %d" % (weight.numel(), cout * 9 * cw))
    oh, ow = out_dim(h, pad, 3, stride), out_dim(w, pad, 3, stride)
    out = _empty((n, max(oh, 0), max(ow, 0), cout), torch.float32, x.device)
    check(lib.dab_bconv3x3(_ptr(x), n, h, w, cw * 64, _ptr(weight), cout, stride, pad, _ptr(out), _stream()))
    return out


def bconv_3x3_affine_add(x, weight, a, b, shortcut=None, stride=1, pad=1):
    """bconv_3x3, affine_inplace and add_inplace of a residual block in one pass: a*cnt + b (+ shortcut)."""
    _need(x, torch.int64, "x")
    _need(weight, torch.int64, "weight")
    _need(a, torch.float32, "a")
    _need(b, torch.float32, "b")
    n, h, w, cw = x.shape
    cout = weight.shape[0]
    if weight.numel() != cout * 9 * cw or a.numel() != cout or b.numel() != cout:
        raise capi.DabError(capi.DAB_EINVAL, "bconv_3x3_affine_add: operand sizes do not match")
    oh, ow = out_dim(h, pad, 3, stride), out_dim(w, pad, 3, stride)
    out = _empty((n, max(oh, 0), max(ow, 0), cout), torch.float32, x.device)
    if shortcut is not None:
        _need(shortcut, torch.float32, "shortcut")
        if shortcut.shape != out.shape:
            raise capi.DabError(capi.DAB_EINVAL, "bconv_3x3_affine_add: shortcut shape differs from the output")
    check(lib.dab_bconv3x3_affine_add(_ptr(x), n, h, w, cw * 64, _ptr(weight), cout, stride, pad, _ptr(a), _ptr(b),
                                      _ptr(shortcut) if shortcut is not None else None, _ptr(out), _stream()))
    return out


def bconv_3x3_affine_add_sign(x, weight, a, b, shortcut=None, stride=1, pad=1):
    """bconv_3x3_affine_add that also returns pack_mat of its result (the next BinConv's packed input):
    (fp32 [N,OH,OW,Cout], int64 [N,OH,OW,Cout/64])."""
    _need(x, torch.int64, "x")
    _need(weight, torch.int64, "weight")
    _need(a, torch.float32, "a")
    _need(b, torch.float32, "b")
    n, h, w, cw = x.shape
    cout = weight.shape[0]
    if weight.numel() != cout * 9 * cw or a.numel() != cout or b.numel() != cout:
        raise capi.DabError(capi.DAB_EINVAL, "bconv_3x3_affine_add_sign: operand sizes do not match")
    oh, ow = out_dim(h, pad, 3, stride), out_dim(w, pad, 3, stride)
    out = _empty((n, max(oh, 0), max(ow, 0), cout), torch.float32, x.device)
    packed = _empty((n, max(oh, 0), max(ow, 0), max(cout // 64, 1)), torch.int64, x.device)
    if shortcut is not None:
        _need(shortcut, torch.float32, "shortcut")
        if shortcut.shape != out.shape:
            raise capi.DabError(capi.DAB_EINVAL, "bconv_3x3_affine_add_sign: shortcut shape differs from the output")
    check(lib.dab_bconv3x3_affine_add_sign(_ptr(x), n, h, w, cw * 64, _ptr(weight), cout, stride, pad, _ptr(a), _ptr(b),
                                           _ptr(shortcut) if shortcut is not None else None, _ptr(out), _ptr(packed),
                                           _stream()))
    return out, packed


class BinConv:
    """The BinConv layer (dabnn/layers/BinConv.h:9-38, BinConv.cpp:17-191) over a batch.

    weight: int64 [Cout, words_per_filter] in the converter's layout
    (tools/onnx2bnn/OnnxConverter.cpp:121-156).  The constructor builds the
    transposed weights for the bgemm method, as the reference's does.
    """

    DIRECT_CONV, BGEMM = 0, 1

    def __init__(self, weight, kh, kw, pad_h, pad_w, stride_h, stride_w):
        _need(weight, torch.int64, "weight")
        self.weight = weight
        self.kh, self.kw = kh, kw
        self.pad_h, self.pad_w, self.stride_h, self.stride_w = pad_h, pad_w, stride_h, stride_w
        self.cout, self.hwc_words = weight.shape
        self.transposed_weight = weight_transpose(weight)
        self.method = None
        self._ws = None

    def forward(self, x):
        _need(x, torch.float32, "x")
        n, h, w, c = x.shape
        need = lib.dab_binconv_workspace_bytes(n, h, w, c, self.kh, self.kw, self.pad_h, self.pad_w, self.stride_h,
                                               self.stride_w)
        if self._ws is None or self._ws.numel() < need or self._ws.device != x.device:
            self._ws = torch.empty(max(need, 16), dtype=torch.uint8, device=x.device)
        oh = out_dim(h, self.pad_h, self.kh, self.stride_h)
        ow = out_dim(w, self.pad_w, self.kw, self.stride_w)
        out = _empty((n, max(oh, 0), max(ow, 0), self.cout), torch.float32, x.device)
        method = ctypes.c_int(-1)
        check(lib.dab_binconv_forward(_ptr(x), n, h, w, c, _ptr(self.weight), _ptr(self.transposed_weight),
                                      self.hwc_words, self.kh, self.kw, self.pad_h, self.pad_w, self.stride_h,
                                      self.stride_w, self.cout, _ptr(out), _ptr(self._ws), self._ws.numel(),
                                      ctypes.byref(method), _stream()))
        self.method = method.value
        return out

    __call__ = forward


def fconv(x, weight, bias, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h=1, dil_w=1):
    """fconv (dabnn/fconv.h:14-76): weight fp32 [Cout, kh, kw, C], optional bias."""
    _need(x, torch.float32, "x")
    _need(weight, torch.float32, "weight")
    n, h, w, c = x.shape
    cout = weight.numel() // (kh * kw * c)
    if bias is not None:
        _need(bias, torch.float32, "bias")
    oh, ow = out_dim(h, pad_h, kh, stride_h, dil_h), out_dim(w, pad_w, kw, stride_w, dil_w)
    out = _empty((n, max(oh, 0), max(ow, 0), cout), torch.float32, x.device)
    check(lib.dab_fconv(_ptr(x), n, h, w, c, _ptr(weight), _ptr(bias) if bias is not None else None, kh, kw, pad_h,
                        pad_w, stride_h, stride_w, dil_h, dil_w, cout, _ptr(out), _stream()))
    return out


def fconv_affine_relu(x, weight, bias, a, b, relu, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h=1, dil_w=1):
    """fconv with the Affine (a, b; None for none) and Relu layers that follow it applied in the same pass
    (dabnn/fconv.h:14-76, dabnn/layers/Affine.cpp:10-23, dabnn/layers/Relu.cpp)."""
    _need(x, torch.float32, "x")
    _need(weight, torch.float32, "weight")
    n, h, w, c = x.shape
    cout = weight.numel() // (kh * kw * c)
    for name, t in (("bias", bias), ("a", a), ("b", b)):
        if t is not None:
            _need(t, torch.float32, name)
            if t.numel() != cout:
                raise capi.DabError(capi.DAB_EINVAL, "fconv_affine_relu: %s does not match the channel count" % name)
    oh, ow = out_dim(h, pad_h, kh, stride_h, dil_h), out_dim(w, pad_w, kw, stride_w, dil_w)
    out = _empty((n, max(oh, 0), max(ow, 0), cout), torch.float32, x.device)
    opt = lambda t: _ptr(t) if t is not None else None
    check(lib.dab_fconv_affine_relu(_ptr(x), n, h, w, c, _ptr(weight), opt(bias), opt(a), opt(b), int(bool(relu)), kh, kw,
                                    pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, cout, _ptr(out), _stream()))
    return out


def ave_pool2_fconv1x1(x, weight, bias, a, b, relu, want_pooled=True):
    """AvePool 2x2 stride 2 + 1x1 FpConv2D (+ Affine + Relu) in one launch; returns (pooled, out), or (None, out)
    without writing the pooled tensor when want_pooled is false."""
    _need(x, torch.float32, "x")
    _need(weight, torch.float32, "weight")
    n, h, w, c = x.shape
    cout = weight.shape[0]
    if weight.numel() != cout * c:
        raise capi.DabError(capi.DAB_EINVAL, "ave_pool2_fconv1x1: weight must be [cout, 1, 1, c]")
    def opt(t, name):
        if t is None:
            return None
        _need(t, torch.float32, name)
        if t.numel() != cout:
            raise capi.DabError(capi.DAB_EINVAL, "ave_pool2_fconv1x1: %s does not match the channel count" % name)
        return _ptr(t)
    oh, ow = out_dim(h, 0, 2, 2), out_dim(w, 0, 2, 2)
    pooled = _empty((n, max(oh, 0), max(ow, 0), c), torch.float32, x.device) if want_pooled else None
    out = _empty((n, max(oh, 0), max(ow, 0), cout), torch.float32, x.device)
    check(lib.dab_ave_pool2_fconv1x1(_ptr(x), n, h, w, c, _ptr(weight), opt(bias, "bias"), opt(a, "a"), opt(b, "b"),
                                     int(bool(relu)), cout, _ptr(pooled) if want_pooled else None, _ptr(out), _stream()))
    return pooled, out


def global_ave_pool_fconv1x1(x, weight, bias, a, b, relu):
    """Global AvePool (one h x w window) + 1x1 FpConv2D (+ Affine + Relu) in one launch; returns (pooled, out)."""
    _need(x, torch.float32, "x")
    _need(weight, torch.float32, "weight")
    n, h, w, c = x.shape
    cout = weight.shape[0]
    if weight.numel() != cout * c:
        raise capi.DabError(capi.DAB_EINVAL, "global_ave_pool_fconv1x1: weight must be [cout, 1, 1, c]")
    def opt(t, name):
        if t is None:
            return None
        _need(t, torch.float32, name)
        if t.numel() != cout:
            raise capi.DabError(capi.DAB_EINVAL, "global_ave_pool_fconv1x1: %s does not match the channel count" % name)
        return _ptr(t)
    pooled = _empty((n, 1, 1, c), torch.float32, x.device)
    out = _empty((n, 1, 1, cout), torch.float32, x.device)
    check(lib.dab_global_ave_pool_fconv1x1(_ptr(x), n, h, w, c, _ptr(weight), opt(bias, "bias"), opt(a, "a"), opt(b, "b"),
                                           int(bool(relu)), cout, _ptr(pooled), _ptr(out), _stream()))
    return pooled, out


def global_ave_pool_fconv1x1_takes(n, h, w, c, cout):
    """Whether global_ave_pool_fconv1x1 covers the shapes (small batch, window and depth within the kernel's limits)."""
    return bool(lib.dab_global_ave_pool_fconv1x1_takes(n, h, w, c, cout))


def fconv_maxpool(x, weight, bias, a, b, relu, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h=1, dil_w=1, want_sign=False):
    """FpConv2D (+ Affine + Relu) and MaxPool 3x3 stride 2 pad 1 in one pass; returns (pooled, pack_mat of it or None)."""
    _need(x, torch.float32, "x")
    _need(weight, torch.float32, "weight")
    n, h, w, c = x.shape
    cout = weight.shape[0]
    if weight.numel() != cout * kh * kw * c:
        raise capi.DabError(capi.DAB_EINVAL, "fconv_maxpool: weight must be [cout, kh, kw, c]")
    def opt(t, name):
        if t is None:
            return None
        _need(t, torch.float32, name)
        if t.numel() != cout:
            raise capi.DabError(capi.DAB_EINVAL, "fconv_maxpool: %s does not match the channel count" % name)
        return _ptr(t)
    geom = (n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, cout)
    carry_floats = lib.dab_fconv_maxpool_carry_floats(*geom)
    oh, ow = out_dim(h, pad_h, kh, stride_h, dil_h), out_dim(w, pad_w, kw, stride_w, dil_w)
    ph, pw = max(oh, 0) // 2, max(ow, 0) // 2
    pooled = _empty((n, ph, pw, cout), torch.float32, x.device)
    carry = _empty((max(int(carry_floats), 4),), torch.float32, x.device)
    packed = _empty((n, ph, pw, max(cout // 64, 1)), torch.int64, x.device) if want_sign else None
    check(lib.dab_fconv_maxpool(_ptr(x), n, h, w, c, _ptr(weight), opt(bias, "bias"), opt(a, "a"), opt(b, "b"),
                                int(bool(relu)), kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, cout,
                                _ptr(pooled), _ptr(packed) if want_sign else None, _ptr(carry), _stream()))
    return pooled, packed


def fconv_maxpool_pays(n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, cout):
    """Whether the one-pass convolution + MaxPool takes these shapes and beats the two launches on this device."""
    return bool(lib.dab_fconv_maxpool_pays(n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, cout))


def affine_inplace(x, a, b):
    """affine_inplace (dabnn/layers/Affine.cpp:10-23)."""
    _need(x, torch.float32, "x")
    _need(a, torch.float32, "a")
    _need(b, torch.float32, "b")
    c = x.shape[-1]
    if a.numel() != c or b.numel() != c:
        raise capi.DabError(capi.DAB_EINVAL, "affine: coefficient length does not match the channel count")
    check(lib.dab_affine_inplace(_ptr(x), x.numel() // c, c, _ptr(a), _ptr(b), _stream()))
    return x


def add_inplace(a, b):
    """add_inplace (dabnn/layers/Add.cpp:7-17)."""
    _need(a, torch.float32, "a")
    _need(b, torch.float32, "b")
    if a.shape != b.shape:
        raise capi.DabError(capi.DAB_EINVAL, "add: shapes differ")
    check(lib.dab_add_inplace(_ptr(a), _ptr(b), a.numel(), _stream()))
    return a


def relu_inplace(x):
    """Relu::forward_impl (dabnn/layers/Relu.cpp)."""
    _need(x, torch.float32, "x")
    check(lib.dab_relu_inplace(_ptr(x), x.numel(), _stream()))
    return x


def prelu_inplace(x, slope):
    """PRelu::forward_impl (dabnn/layers/PRelu.cpp:6-30): slope holds one value or one per channel."""
    _need(x, torch.float32, "x")
    _need(slope, torch.float32, "slope")
    c = x.shape[-1]
    check(lib.dab_prelu_inplace(_ptr(x), x.numel() // c, c, _ptr(slope), slope.numel(), _stream()))
    return x


def concat(a, b):
    """Concat::forward_impl (dabnn/layers/Concat.cpp:7-21): two NHWC tensors joined along the channel axis."""
    _need(a, torch.float32, "a")
    _need(b, torch.float32, "b")
    if a.shape[:-1] != b.shape[:-1]:
        raise capi.DabError(capi.DAB_EINVAL, "concat: shapes differ outside the channel axis")
    ca, cb = a.shape[-1], b.shape[-1]
    out = _empty(tuple(a.shape[:-1]) + (ca + cb,), torch.float32, a.device)
    check(lib.dab_concat_channels(_ptr(a), ca, _ptr(b), cb, a.numel() // ca, _ptr(out), _stream()))
    return out


def _pool(fn, x, kh, kw, pad_h, pad_w, stride_h, stride_w):
    _need(x, torch.float32, "x")
    n, h, w, c = x.shape
    oh, ow = out_dim(h, pad_h, kh, stride_h), out_dim(w, pad_w, kw, stride_w)
    out = _empty((n, max(oh, 0), max(ow, 0), c), torch.float32, x.device)
    check(fn(_ptr(x), n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, _ptr(out), _stream()))
    return out


def ave_pool(x, kh, kw, pad_h, pad_w, stride_h, stride_w):
    """ave_pool_fallback (dabnn/layers/AvePool.cpp:84-123)."""
    return _pool(lib.dab_ave_pool, x, kh, kw, pad_h, pad_w, stride_h, stride_w)


def max_pool(x, kh, kw, pad_h, pad_w, stride_h, stride_w):
    """max_pool_fallback (dabnn/layers/MaxPool.cpp:209-246)."""
    return _pool(lib.dab_max_pool, x, kh, kw, pad_h, pad_w, stride_h, stride_w)


def max_pool_sign(x, kh, kw, pad_h, pad_w, stride_h, stride_w):
    """max_pool that also returns pack_mat of its result: (fp32 [N,OH,OW,C], int64 [N,OH,OW,C/64])."""
    _need(x, torch.float32, "x")
    n, h, w, c = x.shape
    oh, ow = out_dim(h, pad_h, kh, stride_h), out_dim(w, pad_w, kw, stride_w)
    out = _empty((n, max(oh, 0), max(ow, 0), c), torch.float32, x.device)
    packed = _empty((n, max(oh, 0), max(ow, 0), max(c // 64, 1)), torch.int64, x.device)
    check(lib.dab_max_pool_sign(_ptr(x), n, h, w, c, kh, kw, pad_h, pad_w, stride_h, stride_w, _ptr(out), _ptr(packed),
                                _stream()))
    return out, packed
