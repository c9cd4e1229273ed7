"""Host-side checks of the C ABI that need no GPU: the library loads, exports
every symbol the header declares, and rejects bad arguments before touching
the device."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(headers=("dabnn_hip.h", "dabnn_hip_tuning.h")):
    text = "".join(open(os.path.join(ROOT, "include", h)).read() for h in headers)
    return sorted(set(re.findall(r"^DAB_API [^;(]*?\b(dab_\w+)\(", text, flags=re.M)))


def test_dispatch_probes_live_in_the_tuning_header():
    """dabnn_hip.h is the reference's surface plus the documented extensions; the probes that only say which kernel
    would run are declared in dabnn_hip_tuning.h."""
    probes = declared_symbols(("dabnn_hip_tuning.h",))
    assert probes == sorted(["dab_bconv3x3_build", "dab_bconv3x3_counts_build", "dab_bconv3x3_epilogue_build", "dab_bconv3x3_splits_depth", "dab_bconv3x3_fused_shares_tiles",
                             "dab_global_ave_pool_fconv1x1_takes", "dab_fconv_maxpool_pays"])
    assert not set(probes) & set(declared_symbols(("dabnn_hip.h",)))


def test_header_declares_the_expected_entry_points():
    names = declared_symbols()
    for must in ["dab_bitpack_nhwc", "dab_bitpack_nchw", "dab_fused_binarize_im2col", "dab_bgemm", "dab_bconv3x3",
                 "dab_binconv_forward", "dab_last_error", "dab_fconv", "dab_affine_inplace", "dab_add_inplace",
                 "dab_ave_pool", "dab_max_pool", "dab_pad_bit", "dab_weight_transpose"]:
        assert must in names


def test_library_exports_every_declared_symbol():
    from dabnn_amd import capi
    for name in declared_symbols():
        assert hasattr(capi.lib, name), name
        assert name in capi.SIGNATURES, "no ctypes signature for " + name
    assert capi.lib.dab_version() >= 1


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    import importlib
    from dabnn_amd import capi
    monkeypatch.setattr(capi, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(ImportError, match="no CPU fallback"):
        capi._load()
    importlib.reload(capi)


def test_argument_validation_without_device():
    from dabnn_amd import capi
    lib = capi.lib
    null = ctypes.c_void_p(None)
    one = ctypes.c_void_p(16)  # never dereferenced: validation fails first
    assert lib.dab_bitpack_nhwc(null, null, 1, 64, null) == capi.DAB_EINVAL
    assert "null pointer" in capi.last_error()
    assert lib.dab_bitpack_nhwc(one, one, 4, 100, null) == capi.DAB_EINVAL
    assert "multiple of 64" in capi.last_error()
    assert lib.dab_bgemm(4, 4, 4, one, 2, one, 4, one, 4, null) == capi.DAB_EINVAL
    assert "leading dimension" in capi.last_error()
    assert lib.dab_bconv3x3(one, 1, 8, 8, 192, one, 8, 1, 1, one, null) == capi.DAB_EUNSUPPORTED
    assert lib.dab_bconv3x3(one, 1, 8, 8, 64, one, 5, 1, 1, one, null) == capi.DAB_EUNSUPPORTED
    assert lib.dab_bconv3x3(one, 1, 2, 2, 64, one, 8, 1, 0, one, null) == capi.DAB_EINVAL
    assert lib.dab_fused_binarize_im2col(one, 1, 1, 1, 60000, 1, 1, 0, 0, 1, 1, 1, 1, one, null) == capi.DAB_EINVAL
    assert "smaller than 60000" in capi.last_error()
    with pytest.raises(capi.DabUnsupported):
        capi.check(capi.DAB_EUNSUPPORTED)
    with pytest.raises(RuntimeError):
        capi.check(capi.DAB_EINVAL)


def test_workspace_and_row_words():
    from dabnn_amd import capi
    lib = capi.lib
    assert lib.dab_col_row_words(3, 3, 64) == 10  # 9 words rounded up to 128 bits
    assert lib.dab_col_row_words(3, 3, 128) == 18
    assert lib.dab_col_row_words(3, 3, 512) == 72
    assert lib.dab_col_row_words(5, 5, 128) == 50
    assert lib.dab_col_row_words(3, 3, 3) == 2
    # direct method needs the packed input, bgemm method the column matrix
    assert lib.dab_binconv_workspace_bytes(1, 56, 56, 64, 3, 3, 1, 1, 1, 1) == 56 * 56 * 10 * 8
    assert lib.dab_binconv_workspace_bytes(2, 7, 7, 512, 3, 3, 1, 1, 1, 1) == 2 * 49 * 72 * 8
