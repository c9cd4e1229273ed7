"""ctypes binding of ``libdabnn_hip.so`` (the C ABI in ``include/dabnn_hip.h``)."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libdabnn_hip.so")

DAB_OK = 0
DAB_EINVAL = -1
DAB_EUNSUPPORTED = -2
DAB_EHIP = -3


class DabError(RuntimeError):
    """A C-ABI call failed; mirrors the std::runtime_error of BNN_ASSERT (common/helper.h:69-77)."""

    def __init__(self, code, message):
        super().__init__(message)
        self.code = code


class DabUnsupported(DabError):
    pass


def _load():
    # torch ships its own copy of the HIP runtime.  Import it first so that this library binds to the runtime that
    # owns torch's device context; two runtimes in one process do not see each other's devices.
    import torch  # noqa: F401
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "%s is missing: build it with `make -C dabnn_amd/csrc` (or __graft_entry__.build()); "
            "there is no CPU fallback" % LIB_PATH)
    return ctypes.CDLL(LIB_PATH)


lib = _load()

_i, _i64, _sz, _vp = ctypes.c_int, ctypes.c_int64, ctypes.c_size_t, ctypes.c_void_p

# name -> (restype, argtypes); every symbol the header declares
SIGNATURES = {
    "dab_last_error": (ctypes.c_char_p, []),
    "dab_version": (_i, []),
    "dab_device_info": (_i, [ctypes.POINTER(_i), ctypes.POINTER(_i)]),
    "dab_bitpack_nhwc": (_i, [_vp, _vp, _i64, _i, _vp]),
    "dab_bitpack_nchw": (_i, [_vp, _vp, _i, _i, _i, _i, _vp]),
    "dab_pad_bit": (_i, [_vp, _i, _i, _i, _i, _i, _i, _vp, _vp]),
    "dab_split_bit": (_i, [_vp, _i64, _i, _vp, _vp, _vp]),
    "dab_shuffle_bit_inplace": (_i, [_vp, _i64, _i, _vp]),
    "dab_fused_binarize_im2col": (_i, [_vp] + [_i] * 12 + [_vp, _vp]),
    "dab_col_row_words": (_i, [_i, _i, _i]),
    "dab_bgemm": (_i, [_i, _i, _i, _vp, _i, _vp, _i, _vp, _i, _vp]),
    "dab_bgemm_overwrite": (_i, [_i, _i, _i, _vp, _i, _vp, _i, _vp, _i, _vp]),
    "dab_weight_transpose": (_i, [_vp, _i, _i, _vp, _vp]),
    "dab_bconv3x3": (_i, [_vp, _i, _i, _i, _i, _vp, _i, _i, _i, _vp, _vp]),
    "dab_bconv3x3_affine_add": (_i, [_vp, _i, _i, _i, _i, _vp, _i, _i, _i, _vp, _vp, _vp, _vp, _vp]),
    "dab_bconv3x3_affine_add_sign": (_i, [_vp, _i, _i, _i, _i, _vp, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp]),
    "dab_binconv_workspace_bytes": (_sz, [_i] * 10),
    "dab_binconv_forward": (_i, [_vp, _i, _i, _i, _i, _vp, _vp] + [_i] * 8 + [_vp, _vp, _sz, ctypes.POINTER(_i), _vp]),
    "dab_binconv_forward_static": (_i, [_vp, _i, _i, _i, _i, _vp, _vp] + [_i] * 8 + [_vp, ctypes.POINTER(_i), _vp]),
    "dab_fconv": (_i, [_vp, _i, _i, _i, _i, _vp, _vp] + [_i] * 9 + [_vp, _vp]),
    "dab_fconv_affine_relu": (_i, [_vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp] + [_i] * 10 + [_vp, _vp]),
    "dab_ave_pool2_fconv1x1": (_i, [_vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp]),
    "dab_global_ave_pool_fconv1x1": (_i, [_vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp]),
    "dab_global_ave_pool_fconv1x1_takes": (_i, [_i] * 5),
    "dab_fconv_maxpool": (_i, [_vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp] + [_i] * 10 + [_vp, _vp, _vp, _vp]),
    "dab_fconv_maxpool_carry_floats": (_i64, [_i] * 13),
    "dab_fconv_maxpool_pays": (_i, [_i] * 13),
    "dab_affine_inplace": (_i, [_vp, _i64, _i, _vp, _vp, _vp]),
    "dab_add_inplace": (_i, [_vp, _vp, _i64, _vp]),
    "dab_relu_inplace": (_i, [_vp, _i64, _vp]),
    "dab_bconv3x3_splits_depth": (_i, [_i64, _i, _i]),
    "dab_bconv3x3_build": (_i, [_i64, _i, _i]),
    "dab_bconv3x3_counts_build": (_i, [_i64, _i, _i, _i]),
    "dab_bconv3x3_epilogue_build": (_i, [_i64, _i, _i, _i, _i]),
    "dab_bconv3x3_fused_shares_tiles": (_i, [_i64, _i, _i]),
    "dab_prelu_inplace": (_i, [_vp, _i64, _i, _vp, _i, _vp]),
    "dab_concat_channels": (_i, [_vp, _i, _vp, _i, _i64, _vp, _vp]),
    "dab_fill_f32": (_i, [_vp, _i64, ctypes.c_float, _vp]),
    "dab_ave_pool": (_i, [_vp] + [_i] * 10 + [_vp, _vp]),
    "dab_max_pool": (_i, [_vp] + [_i] * 10 + [_vp, _vp]),
    "dab_max_pool_sign": (_i, [_vp] + [_i] * 10 + [_vp, _vp, _vp]),
}

for _name, (_res, _args) in SIGNATURES.items():
    _fn = getattr(lib, _name)
    _fn.restype = _res
    _fn.argtypes = _args


def last_error():
    return lib.dab_last_error().decode()


def check(rc):
    if rc == DAB_OK:
        return
    msg = last_error()
    if rc == DAB_EUNSUPPORTED:
        raise DabUnsupported(rc, msg)
    raise DabError(rc, msg)


def device_info():
    cus, khz = _i(0), _i(0)
    check(lib.dab_device_info(ctypes.byref(cus), ctypes.byref(khz)))
    return cus.value, khz.value
