"""Python face of the BM copy API with the names of the reference's pybind
module (``memfabric_hybrid.bm``: src/smem/csrc/python_wrapper/memfabric_hybrid/pymf_hybrid.cpp:151-175,
584-638): ``initialize``, ``create``, ``BigMemory.copy_data`` / ``copy_data_batch``
/ ``wait`` / ``peer_rank_ptr`` ...  Every call goes straight through ctypes to
the C ABI; addresses are plain integers as in the reference.
"""

import ctypes
from enum import IntEnum

from . import native


class BmCopyType(IntEnum):
    L2G = 0
    G2L = 1
    G2H = 2
    H2G = 3
    L2GH = 4
    GH2L = 5
    GH2H = 6
    H2GH = 7
    G2G = 8
    AUTO = 9


class BmMemType(IntEnum):
    LOCAL_DEVICE = 0
    LOCAL_HOST = 1
    DEVICE = 2
    HOST = 3


class BmDataOpType(IntEnum):
    SDMA = 1
    HOST_RDMA = 2
    HOST_TCP = 4
    DEVICE_RDMA = 8
    HOST_URMA = 16


class BmConfig:
    """Default-initialised smem_bm_config_t."""

    def __init__(self):
        self.c = native.SmemBmConfig()
        ret = native.lib().smem_bm_config_init(ctypes.byref(self.c))
        if ret != 0:
            raise RuntimeError(f"smem_bm_config_init failed: {ret}")


def initialize(store_url, world_size, device_id, config=None):
    config = config or BmConfig()
    return native.lib().smem_bm_init(store_url.encode(), world_size, device_id, ctypes.byref(config.c))


def uninitialize(flags=0):
    native.lib().smem_bm_uninit(flags)


def bm_rank_id():
    return native.lib().smem_bm_get_rank_id()


class BigMemory:
    def __init__(self, handle):
        self._h = handle

    @property
    def handle(self):
        return self._h

    def join(self, flags=0):
        return native.lib().smem_bm_join(self._h, flags)

    def leave(self, flags=0):
        return native.lib().smem_bm_leave(self._h, flags)

    def local_mem_size(self, mem_type=BmMemType.DEVICE):
        return native.lib().smem_bm_get_local_mem_size_by_mem_type(self._h, int(mem_type))

    def peer_rank_ptr(self, peer_rank, mem_type=BmMemType.DEVICE):
        ptr = native.lib().smem_bm_ptr_by_mem_type(self._h, int(mem_type), peer_rank)
        if not ptr:
            raise RuntimeError("get pointer by rank failed: " + native.last_error())
        return ptr

    def destroy(self):
        native.lib().smem_bm_destroy(self._h)
        self._h = None

    def get_rank_id_by_gva(self, gva):
        return native.lib().smem_bm_get_rank_id_by_gva(self._h, gva)

    def register(self, addr, size):
        return native.lib().smem_bm_register_user_mem(self._h, addr, size)

    def unregister(self, addr):
        return native.lib().smem_bm_unregister_user_mem(self._h, addr)

    def copy_data(self, src_ptr, dst_ptr, size, type, flags=0):  # noqa: A002 - the reference's argument name
        params = native.SmemCopyParams(src_ptr, dst_ptr, size)
        return native.lib().smem_bm_copy(self._h, ctypes.byref(params), int(type), flags)

    def copy_data_batch(self, src_addrs, dst_addrs, sizes, count, type, flags=0):  # noqa: A002
        srcs = native.ptr_array(src_addrs[:count])
        dsts = native.ptr_array(dst_addrs[:count])
        lens = native.u64_array(sizes[:count])
        params = native.BatchCopyParams(srcs, dsts, lens, count)
        return native.lib().smem_bm_copy_batch(self._h, ctypes.byref(params), int(type), flags)

    def wait(self):
        return native.lib().smem_bm_wait(self._h)


def create(id, local_dram_size, local_hbm_size, data_op_type=BmDataOpType.SDMA, flags=0):  # noqa: A002
    handle = native.lib().smem_bm_create(id, 1, int(data_op_type), local_dram_size, local_hbm_size, flags)
    if not handle:
        raise RuntimeError("create bm handle failed: " + native.last_error())
    return BigMemory(handle)
