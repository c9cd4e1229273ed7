"""MI355X (gfx950) backend for the binary-convolution path of dabnn.

The compute lives in ``lib/libdabnn_hip.so`` (hand-written HIP kernels behind
the C ABI declared in ``include/dabnn_hip.h``).  This package is the thin
Python plumbing over it: it hands device pointers of torch tensors to the C
ABI and mirrors the reference's function names.  There is no CPU fallback:
importing :mod:`dabnn_amd.capi` raises when the library has not been built.
"""
from . import capi  # noqa: F401
from .ops import (  # noqa: F401
    BinConv,
    add_inplace,
    affine_inplace,
    ave_pool,
    ave_pool2_fconv1x1,
    global_ave_pool_fconv1x1,
    global_ave_pool_fconv1x1_takes,
    bconv_3x3,
    bconv_3x3_affine_add,
    bconv_3x3_affine_add_sign,
    bgemm,
    bgemm_overwrite,
    bitpack_nchw,
    col_row_words,
    concat,
    fconv,
    fconv_affine_relu,
    fconv_maxpool,
    fconv_maxpool_pays,
    fused_binarize_im2col,
    max_pool,
    max_pool_sign,
    pack_mat,
    pad,
    prelu_inplace,
    relu_inplace,
    shuffle_bit_inplace,
    split_bit,
    weight_transpose,
)
