"""Helpers for the GPU parity tests: torch is used for device memory only; every compute call goes through the
C-ABI of libugache_hip.so / libcoll_cache.so."""
import ctypes as C

import numpy as np
import torch

from ugache_amd import hip

_TORCH_VIEW = {np.dtype(np.uint32): np.int32, np.dtype(np.uint64): np.int64, np.dtype(np.uint16): np.int16}


def to_dev(a):
    """numpy array -> torch tensor on cuda:0 holding the same bytes (unsigned types are viewed as signed)."""
    a = np.ascontiguousarray(a)
    if a.dtype.fields is not None:  # structured: ship as bytes
        a = a.view(np.uint8)
    v = _TORCH_VIEW.get(a.dtype)
    if v is not None:
        a = a.view(v)
    return torch.from_numpy(a).cuda()


def to_np(t, dtype=None, shape=None):
    a = t.detach().cpu().numpy()
    if dtype is not None:
        a = a.view(np.uint8).reshape(-1).view(dtype)
    if shape is not None:
        a = a.reshape(shape)
    return a


def dev_bytes(nbytes, fill=None):
    t = torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device="cuda")
    if fill is not None:
        t.fill_(fill)
    return t


def dev_zeros_u32(n):
    return torch.zeros(max(int(n), 1), dtype=torch.int32, device="cuda")


def ptr(t):
    return 0 if t is None else t.data_ptr()


def sync():
    torch.cuda.synchronize()


def status_value(st):
    sync()
    return int(st.cpu().numpy().view(np.uint32)[0])


class PinnedArray:
    """numpy array living in pinned, GPU-mapped host memory from ugk_host_malloc."""

    def __init__(self, shape, dtype):
        self.dtype = np.dtype(dtype)
        self.shape = tuple(shape)
        self.nbytes = int(np.prod(self.shape)) * self.dtype.itemsize
        p = C.c_void_p()
        hip.call("ugk_host_malloc", C.byref(p), max(self.nbytes, 16))
        self.ptr = p.value
        buf = (C.c_uint8 * max(self.nbytes, 16)).from_address(self.ptr)
        self.array = np.frombuffer(buf, dtype=self.dtype, count=int(np.prod(self.shape))).reshape(self.shape)

    def free(self):
        if self.ptr:
            self.array = None
            hip.call("ugk_host_free", self.ptr)
            self.ptr = 0


def pinned_from(a):
    a = np.ascontiguousarray(a)
    p = PinnedArray(a.shape, a.dtype)
    p.array[...] = a
    return p
