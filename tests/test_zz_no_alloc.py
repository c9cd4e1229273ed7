"""dab_binconv_forward_static, the entry point that allocates nothing on the device: its scratch is a buffer inside the
library's code object.  Checked through the C ABI against dab_binconv_forward (caller's workspace) bit for bit, on two
calls in a row, the second on a smaller input, for both arms (direct 3x3 and im2col + bgemm); sizes beyond the buffer
are refused."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 16 << 20  # DAB_BINCONV_STATIC_SCRATCH_BYTES of include/dabnn_hip.h


def _run_both(r, n, h, w, c, cout, k, pad, stride):
    from dabnn_amd import capi
    import oracle as orc
    lib = capi.lib
    x = torch.from_numpy(r.standard_normal((n, h, w, c)).astype(np.float32)).cuda()
    wp = orc.pack_weight(r.standard_normal((cout, k, k, c)).astype(np.float32))
    wgt = torch.from_numpy(wp.view(np.int64)).cuda()
    wgt_t = torch.from_numpy(np.ascontiguousarray(wp.T).view(np.int64)).cuda()
    oh, ow = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
    need = lib.dab_binconv_workspace_bytes(n, h, w, c, k, k, pad, pad, stride, stride)
    assert need <= SCRATCH_BYTES
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    want = torch.full((n, oh, ow, cout), -1.0, device="cuda")
    got = torch.full((n, oh, ow, cout), -2.0, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    m_want, m_got = ctypes.c_int(-1), ctypes.c_int(-1)
    capi.check(lib.dab_binconv_forward(p(x), n, h, w, c, p(wgt), p(wgt_t), wp.shape[1], k, k, pad, pad, stride, stride,
                                       cout, p(want), p(ws), need, ctypes.byref(m_want), stream))
    capi.check(lib.dab_binconv_forward_static(p(x), n, h, w, c, p(wgt), p(wgt_t), wp.shape[1], k, k, pad, pad, stride,
                                              stride, cout, p(got), ctypes.byref(m_got), stream))
    torch.cuda.synchronize()
    assert m_got.value == m_want.value
    assert torch.equal(got, want)
    # and against the CPU restatement on the first and last image
    for i in (0, n - 1):
        ref = orc.binconv_forward(x[i].cpu().numpy(), wp, k, k, pad, pad, stride, stride)[0]
        np.testing.assert_array_equal(got[i].cpu().numpy(), ref)
    return m_got.value


@pytest.mark.parametrize("first,second", [
    # direct arm: the scratch holds the packed activations; the second call is smaller and leaves stale words behind it
    ((8, 28, 28, 128, 64, 3, 1, 1), (2, 14, 14, 128, 32, 3, 1, 2)),
    # bgemm arm: the scratch holds the column matrix (192 channels, then a 5x5 filter on a smaller image)
    ((6, 12, 12, 192, 40, 3, 1, 1), (1, 9, 9, 128, 16, 5, 2, 2)),
    # one arm after the other
    ((4, 56, 56, 64, 64, 3, 1, 1), (3, 6, 6, 256, 24, 1, 0, 1)),
])
def test_static_scratch_equals_callers_workspace(first, second):
    r = np.random.default_rng(70)
    _run_both(r, *first)
    _run_both(r, *second)


def test_static_scratch_refuses_larger_problems():
    from dabnn_amd import capi
    lib = capi.lib
    one = ctypes.c_void_p(256)  # never dereferenced: the size check comes first
    # 512 x 56 x 56 x 64 channels packed = 12.8 MB fits; 1024 images do not
    n = 1024
    assert lib.dab_binconv_workspace_bytes(n, 56, 56, 64, 3, 3, 1, 1, 1, 1) > SCRATCH_BYTES
    rc = lib.dab_binconv_forward_static(one, n, 56, 56, 64, one, one, 9, 3, 3, 1, 1, 1, 1, 64, one, None, None)
    assert rc == capi.DAB_EUNSUPPORTED
    assert "static buffer holds" in capi.last_error()
