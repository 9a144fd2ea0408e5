"""Python face of the transfer front-end with the names of the reference's transfer adapter
(``TransferEngine``: src/smem/csrc/python_wrapper/mk_transfer_adapter/csrc/pytransfer.cpp:40-360,
396-433).  Addresses are plain integers; every method returns the C ABI's code (0 on success).
Objects of one process see each other at once, so ``initialize`` and ``register_memory`` do not
wait the 10 and 8 seconds the reference spends on its config store.
"""

import ctypes
from enum import IntEnum

from . import native


class TransferOpcode(IntEnum):
    Read = 0
    Write = 1


class TransDataOpType(IntEnum):
    SDMA = 1
    DEVICE_RDMA = 8


_ROLES = {"Prefill": native.SMEM_TRANS_SENDER, "Decode": native.SMEM_TRANS_RECEIVER}


def _arrays(buffers, peer_buffers, lengths):
    if not (len(buffers) == len(peer_buffers) == len(lengths)) or len(buffers) > 0xFFFFFFFF:
        return None
    return native.ptr_array(buffers), native.ptr_array(peer_buffers), native.u64_array(lengths)


class TransferEngine:
    TransferOpcode = TransferOpcode
    TransDataOpType = TransDataOpType

    def __init__(self):
        self._lib = native.lib()
        self._handle = None

    def initialize(self, store_url, session_id, role, device_id, data_op_type=TransDataOpType.SDMA):
        if role not in _ROLES:
            return -1
        cfg = native.SmemTransConfig()
        ret = self._lib.smem_trans_config_init(ctypes.byref(cfg))
        if ret != 0:
            return ret
        cfg.role = _ROLES[role]
        cfg.deviceId = device_id
        cfg.dataOpType = int(data_op_type)
        ret = self._lib.smem_trans_init(ctypes.byref(cfg))
        if ret != 0:
            return ret
        self._handle = self._lib.smem_trans_create(store_url.encode(), session_id.encode(), ctypes.byref(cfg))
        return 0 if self._handle else -1

    def register_memory(self, buffer_addr, capacity):
        if not self._handle:
            return -1
        return self._lib.smem_trans_register_mem(self._handle, buffer_addr, capacity, 0)

    def unregister_memory(self, buffer_addr):
        if not self._handle:
            return -1
        return self._lib.smem_trans_deregister_mem(self._handle, buffer_addr)

    def batch_register_memory(self, buffer_addrs, capacities):
        if not self._handle or len(buffer_addrs) != len(capacities):
            return -1
        return self._lib.smem_trans_batch_register_mem(self._handle, native.ptr_array(buffer_addrs),
                                                       native.u64_array(capacities), len(buffer_addrs), 0)

    def transfer_sync_write(self, dest_session, buffer, peer_buffer, length, flags=0):
        if not self._handle:
            return -1
        return self._lib.smem_trans_write(self._handle, buffer, dest_session.encode(), peer_buffer, length, flags)

    def transfer_sync_read(self, dest_session, buffer, peer_buffer, length, flags=0):
        if not self._handle:
            return -1
        return self._lib.smem_trans_read(self._handle, buffer, dest_session.encode(), peer_buffer, length, flags)

    def transfer_async_write_submit(self, dest_session, buffer, peer_buffer, length, stream, flags=0):
        if not self._handle:
            return -1
        return self._lib.smem_trans_write_submit(self._handle, buffer, dest_session.encode(), peer_buffer, length,
                                                 stream, flags)

    def transfer_async_read_submit(self, dest_session, buffer, peer_buffer, length, stream, flags=0):
        if not self._handle:
            return -1
        return self._lib.smem_trans_read_submit(self._handle, buffer, dest_session.encode(), peer_buffer, length,
                                                stream, flags)

    def batch_transfer_sync_write(self, dest_session, buffers, peer_buffers, lengths, flags=0):
        arrays = _arrays(buffers, peer_buffers, lengths) if self._handle else None
        if arrays is None:
            return -1
        return self._lib.smem_trans_batch_write(self._handle, arrays[0], dest_session.encode(), arrays[1], arrays[2],
                                                len(buffers), flags)

    def batch_transfer_sync_read(self, dest_session, buffers, peer_buffers, lengths, flags=0):
        arrays = _arrays(buffers, peer_buffers, lengths) if self._handle else None
        if arrays is None:
            return -1
        return self._lib.smem_trans_batch_read(self._handle, arrays[0], dest_session.encode(), arrays[1], arrays[2],
                                               len(buffers), flags)

    def batch_transfer_async_write_submit(self, dest_session, buffers, peer_buffers, lengths, stream, flags=0):
        arrays = _arrays(buffers, peer_buffers, lengths) if self._handle else None
        if arrays is None:
            return -1
        return self._lib.smem_trans_batch_write_submit(self._handle, arrays[0], dest_session.encode(), arrays[1],
                                                       arrays[2], len(buffers), stream, flags)

    def batch_transfer_async_read_submit(self, dest_session, buffers, peer_buffers, lengths, stream, flags=0):
        arrays = _arrays(buffers, peer_buffers, lengths) if self._handle else None
        if arrays is None:
            return -1
        return self._lib.smem_trans_batch_read_submit(self._handle, arrays[0], dest_session.encode(), arrays[1],
                                                      arrays[2], len(buffers), stream, flags)

    def destroy(self):
        if self._handle:
            self._lib.smem_trans_destroy(self._handle, 0)
            self._handle = None

    def unInitialize(self):
        self._lib.smem_trans_uninit(0)
