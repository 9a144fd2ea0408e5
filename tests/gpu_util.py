"""Helpers for the GPU parity tests: raw device / pinned buffers through the
library's own runtime services, moved to and from numpy with plain hipMemcpy
(mfrt_memcpy), which shares no code with the copy kernels under test."""

import ctypes

import numpy as np

from memfabric_hybrid_amd import native


class DeviceBuffer:
    def __init__(self, lib, nbytes):
        self.lib = lib
        self.nbytes = nbytes
        self.ptr = lib.mfrt_alloc_device(nbytes)
        if not self.ptr:
            raise MemoryError(f"device allocation of {nbytes} bytes failed")

    def upload(self, array, offset=0):
        a = np.ascontiguousarray(array)
        assert offset + a.nbytes <= self.nbytes
        err = self.lib.mfrt_memcpy(self.ptr + offset, a.ctypes.data, a.nbytes)
        assert err == 0, self.lib.mfrt_error_string(err)

    def download(self, offset=0, nbytes=None):
        nbytes = self.nbytes - offset if nbytes is None else nbytes
        out = np.empty(nbytes, dtype=np.uint8)
        err = self.lib.mfrt_memcpy(out.ctypes.data, self.ptr + offset, nbytes)
        assert err == 0, self.lib.mfrt_error_string(err)
        return out

    def fill(self, value):
        assert self.lib.mfrt_memset(self.ptr, value, self.nbytes) == 0

    def free(self):
        if self.ptr:
            self.lib.mfrt_free_device(self.ptr)
            self.ptr = None


class PinnedBuffer:
    """Pinned, device-mapped host memory viewed as a numpy uint8 array."""

    def __init__(self, lib, nbytes):
        self.lib = lib
        self.nbytes = nbytes
        self.ptr = lib.mfrt_alloc_host(nbytes)
        if not self.ptr:
            raise MemoryError(f"pinned allocation of {nbytes} bytes failed")
        self.array = np.ctypeslib.as_array((ctypes.c_uint8 * nbytes).from_address(self.ptr))

    def free(self):
        if self.ptr:
            self.array = None
            self.lib.mfrt_free_host(self.ptr)
            self.ptr = None


def host_view(ptr, nbytes):
    return np.ctypeslib.as_array((ctypes.c_uint8 * nbytes).from_address(ptr))


def xcopy(lib, src, dst, lens, route, stream=None, sync=True):
    n = len(lens)
    ret = lib.mf_xcopy_batch(native.u64_array(src), native.u64_array(dst), native.u64_array(lens), n, route, stream)
    assert ret == 0, native.last_error()
    if sync:
        err = lib.mfrt_stream_sync(stream) if stream else lib.mfrt_device_sync()
        assert err == 0, lib.mfrt_error_string(err)


def oracle_batch(oracle, src_arr, dst_arr, src_off, dst_off, lens):
    """dst_arr[dst_off[i]:+len] = src_arr[src_off[i]:+len] through the oracle's C loop."""
    from tests.oracle_lib import ptr_array, u64_array
    srcs = ptr_array([src_arr.ctypes.data + int(s) for s in src_off])
    dsts = ptr_array([dst_arr.ctypes.data + int(d) for d in dst_off])
    assert oracle.orc_batch_copy_fast(dsts, srcs, u64_array(lens), len(lens)) == 0
