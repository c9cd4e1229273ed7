"""Python face of the C++ network runtime (``libdabnn_host.so``, C ABI in
``include/dabnn_net.h``): the bnn::Net surface of the reference
(dabnn/net.h:50-61) -- read / read_buf / run / get_blob and the flags
optimize / run_fconv / strict -- plus a batch size."""
import ctypes
import os

import numpy as np

from . import capi  # loads libdabnn_hip.so first (and fails loudly when it is missing)

_HERE = os.path.dirname(os.path.abspath(__file__))
HOST_LIB_PATH = os.path.join(_HERE, "lib", "libdabnn_host.so")

DABNET_OK, DABNET_ERUNTIME, DABNET_EINVALID, DABNET_EKEY = 0, -1, -2, -3


def _load():
    if not os.path.exists(HOST_LIB_PATH):
        raise ImportError("%s is missing: build it with `make -C dabnn_amd/host`" % HOST_LIB_PATH)
    return ctypes.CDLL(HOST_LIB_PATH)


hostlib = _load()
_i, _vp, _sz, _cp = ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_char_p

NET_SIGNATURES = {
    "dabnet_last_error": (_cp, []),
    "dabnet_create": (_vp, []),
    "dabnet_destroy": (None, [_vp]),
    "dabnet_set_batch": (_i, [_vp, _i]),
    "dabnet_set_flags": (_i, [_vp, _i, _i, _i]),
    "dabnet_set_use_graph": (_i, [_vp, _i]),
    "dabnet_set_profile": (_i, [_vp, _i]),
    "dabnet_time_report": (_cp, [_vp]),
    "dabnet_read_file": (_i, [_vp, _cp]),
    "dabnet_read_buf": (_i, [_vp, _vp, _sz]),
    "dabnet_check_model": (_i, [_vp, _sz, _i]),
    "dabnet_run": (_i, [_vp, _vp]),
    "dabnet_run_device": (_i, [_vp, _vp]),
    "dabnet_input_name": (_cp, [_vp]),
    "dabnet_blob_info": (_i, [_vp, _cp, ctypes.POINTER(_i * 4), ctypes.POINTER(_i), ctypes.POINTER(_sz)]),
    "dabnet_get_blob": (_i, [_vp, _cp, _vp, _sz]),
    "dabnet_num_layers": (_i, [_vp]),
    "dabnet_layer_desc": (_cp, [_vp, _i]),
}
for _name, (_res, _args) in NET_SIGNATURES.items():
    _fn = getattr(hostlib, _name)
    _fn.restype = _res
    _fn.argtypes = _args


def _check(rc):
    if rc == DABNET_OK:
        return
    msg = hostlib.dabnet_last_error().decode()
    if rc == DABNET_EINVALID:
        raise ValueError(msg)  # std::invalid_argument
    if rc == DABNET_EKEY:
        raise KeyError(msg)  # StrKeyMap::at
    raise RuntimeError(msg)  # std::runtime_error


def check_model(buf, run_fconv=True):
    """Parse and check a .dab model on the host (no GPU): raises what Net.read_buf would raise for it."""
    b = bytes(buf)
    _check(hostlib.dabnet_check_model(b, len(b), int(run_fconv)))


class Net:
    def __init__(self, batch=1, optimize=True, run_fconv=True, strict=True):
        self._h = hostlib.dabnet_create()
        if not self._h:
            raise RuntimeError(hostlib.dabnet_last_error().decode())
        self.batch = batch
        self._input_bytes = None  # of the input blob, asked for once
        _check(hostlib.dabnet_set_batch(self._h, batch))
        _check(hostlib.dabnet_set_flags(self._h, int(optimize), int(run_fconv), int(strict)))

    @classmethod
    def create(cls, **kw):
        return cls(**kw)

    def close(self):
        if self._h and hostlib is not None:  # at interpreter exit the module's globals may be gone already
            hostlib.dabnet_destroy(self._h)
        self._h = None

    def __del__(self):
        self.close()

    def read(self, path):
        _check(hostlib.dabnet_read_file(self._h, os.fsencode(path)))
        return self

    def read_buf(self, buf):
        b = bytes(buf)
        _check(hostlib.dabnet_read_buf(self._h, b, len(b)))
        return self

    def run(self, x):
        """x: host array of batch x H x W x C float32 (NHWC), or a CUDA torch tensor of that shape, which the layers
        read in place (reuse one tensor run after run: the net's HIP graph holds its address)."""
        if hasattr(x, "is_cuda") and x.is_cuda:
            import torch
            assert x.dtype == torch.float32 and x.is_contiguous()
            if self._input_bytes is None:
                self._input_bytes = self.blob_info(self.input_name)[2]
            if x.numel() * 4 != self._input_bytes:
                raise ValueError("input tensor does not match the model's input size")
            torch.cuda.current_stream().synchronize()
            _check(hostlib.dabnet_run_device(self._h, ctypes.c_void_p(x.data_ptr())))
            return self
        a = np.ascontiguousarray(x, dtype=np.float32)
        _, _, nbytes = self.blob_info(self.input_name)
        if a.nbytes != nbytes:
            raise ValueError("input has %d bytes, the model wants %d" % (a.nbytes, nbytes))
        _check(hostlib.dabnet_run(self._h, a.ctypes.data_as(ctypes.c_void_p)))
        return self

    @property
    def input_name(self):
        return hostlib.dabnet_input_name(self._h).decode()

    def blob_info(self, name):
        shape, is_bit, nbytes = (_i * 4)(), _i(0), _sz(0)
        _check(hostlib.dabnet_blob_info(self._h, name.encode(), ctypes.byref(shape), ctypes.byref(is_bit),
                                        ctypes.byref(nbytes)))
        return tuple(shape), bool(is_bit.value), nbytes.value

    def get_blob(self, name):
        shape, is_bit, nbytes = self.blob_info(name)
        out = np.empty(nbytes // (8 if is_bit else 4), dtype=np.uint64 if is_bit else np.float32)
        _check(hostlib.dabnet_get_blob(self._h, name.encode(), out.ctypes.data_as(ctypes.c_void_p), nbytes))
        if int(np.prod(shape)) == out.size:
            out = out.reshape(shape)
        return out

    def set_use_graph(self, on=True):
        _check(hostlib.dabnet_set_use_graph(self._h, int(on)))

    def set_profile(self, on=True):
        _check(hostlib.dabnet_set_profile(self._h, int(on)))

    def time_report(self):
        return hostlib.dabnet_time_report(self._h).decode()

    def layers(self):
        n = hostlib.dabnet_num_layers(self._h)
        return [hostlib.dabnet_layer_desc(self._h, i).decode() for i in range(n)]
