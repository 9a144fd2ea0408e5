"""ctypes binding of the C ABI declared in ``include/*.h``.

There is no Python or CPU substitute behind these functions: if the shared
library is missing, ``lib()`` raises, and if no GPU is present the library's
own init calls fail with their error codes.
"""

import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(_HERE, "lib")
DATAPLANE_PATH = os.path.join(LIB_DIR, "libmf_hip_dataplane.so")
PLUGIN_PATH = os.path.join(LIB_DIR, "libmf_hybm_copy_extend.so")
YARDSTICK_PATH = os.path.join(LIB_DIR, "libmf_hip_yardstick.so")

# ---- enums (values pinned in include/mf_xcopy_types.h) ---------------------
BM_OK = 0
BM_ERROR = -1
BM_INVALID_PARAM = -2
BM_NOT_INITIALIZED = -9
SM_OK = 0
SM_ERROR = -1
SM_INVALID_PARAM = -2000
SM_NOT_INITIALIZED = -2008

MF_COPY_UNORDERED_FLAG = 1 << 16
ASYNC_COPY_FLAG = 1
COPY_EXTEND_FLAG = 2

HYBM_MEM_TYPE_DEVICE = 1
HYBM_MEM_TYPE_HOST = 2
HYBM_MEM_TYPE_BUTT = 3

HYBM_DIRECTIONS = [
    "LH2GH", "LH2GD", "LD2GH", "LD2GD", "GH2GH", "GH2GD", "GH2LH", "GH2LD",
    "GD2GH", "GD2GD", "GD2LH", "GD2LD", "AUTO", "BUTT",
]
HYBM_DIR = {name: i for i, name in enumerate(HYBM_DIRECTIONS)}

SMEM_MEM_TYPE_LOCAL_DEVICE = 0
SMEM_MEM_TYPE_LOCAL_HOST = 1
SMEM_MEM_TYPE_DEVICE = 2
SMEM_MEM_TYPE_HOST = 3
SMEM_MEM_TYPE_BUTT = 4

SMEMB_DATA_OP_SDMA = 1
SMEMB_DATA_OP_HOST_RDMA = 2
SMEMB_DATA_OP_HOST_TCP = 4
SMEMB_DATA_OP_DEVICE_RDMA = 8
SMEMB_DATA_OP_HOST_URMA = 16

SMEM_TRANS_SENDER = 1
SMEM_TRANS_RECEIVER = 2
SMEM_TRANS_BOTH = 3

SMEMB_COPY = {"L2G": 0, "G2L": 1, "G2H": 2, "H2G": 3, "L2GH": 4, "GH2L": 5, "GH2H": 6, "H2GH": 7, "G2G": 8,
              "AUTO": 9, "BUTT": 10}

ROUTE_HBM = 0
ROUTE_TO_HOST = 1
ROUTE_FROM_HOST = 2

PTR_PAGEABLE = 0
PTR_DEVICE = 1
PTR_PINNED_HOST = 2

u8p = ctypes.POINTER(ctypes.c_uint8)
u32 = ctypes.c_uint32
u64 = ctypes.c_uint64
i32 = ctypes.c_int32
i64 = ctypes.c_int64
vp = ctypes.c_void_p
u64p = ctypes.POINTER(ctypes.c_uint64)


class SmemTlsConfig(ctypes.Structure):
    _fields_ = [("tlsEnable", ctypes.c_bool)] + [
        (n, ctypes.c_char * 256)
        for n in ("caPath", "crlPath", "certPath", "keyPath", "keyPassPath", "packagePath", "decrypterLibPath")
    ]


class SmemBmConfig(ctypes.Structure):
    _fields_ = [
        ("initTimeout", u32), ("createTimeout", u32), ("controlOperationTimeout", u32),
        ("startConfigStoreServer", ctypes.c_bool), ("startConfigStoreOnly", ctypes.c_bool),
        ("dynamicWorldSize", ctypes.c_bool), ("unifiedAddressSpace", ctypes.c_bool),
        ("autoRanking", ctypes.c_bool), ("rankId", ctypes.c_uint16), ("flags", u32),
        ("hcomUrl", ctypes.c_char * 64), ("hcomTlsConfig", SmemTlsConfig), ("storeTlsConfig", SmemTlsConfig),
    ]


class SmemBmCreateOption(ctypes.Structure):
    _fields_ = [
        ("maxDramSize", u64), ("maxHbmSize", u64), ("localDRAMSize", u64), ("localHBMSize", u64),
        ("dataOpType", ctypes.c_int), ("flags", u32), ("tag", ctypes.c_char * 32),
        ("tagOpInfo", ctypes.c_char * 256), ("dramShmFd", ctypes.c_int),
    ]


class SmemCopyParams(ctypes.Structure):
    _fields_ = [("src", vp), ("dest", vp), ("dataSize", ctypes.c_size_t)]


class BatchCopyParams(ctypes.Structure):
    """Layout shared by smem_batch_copy_params and hybm_batch_copy_params."""
    _fields_ = [("sources", ctypes.POINTER(vp)), ("destinations", ctypes.POINTER(vp)),
                ("dataSizes", u64p), ("batchSize", u32)]


class Copy2dDesc(ctypes.Structure):
    _fields_ = [("src", u64), ("dst", u64), ("width", u64), ("height", u64), ("spitch", u64), ("dpitch", u64)]


class HybmCopyParams(ctypes.Structure):
    _fields_ = [("src", vp), ("dest", vp), ("dataSize", u64)]


class SmemTransConfig(ctypes.Structure):
    _fields_ = [("role", ctypes.c_int), ("initTimeout", u32), ("deviceId", u32), ("flags", u32),
                ("dataOpType", ctypes.c_int), ("startConfigServer", ctypes.c_bool)]


class HybmTlsConfig(SmemTlsConfig):
    pass


class HybmOptions(ctypes.Structure):
    _fields_ = [
        ("bmType", ctypes.c_int), ("memType", ctypes.c_int), ("bmDataOpType", ctypes.c_int),
        ("rankCount", ctypes.c_uint16), ("rankId", ctypes.c_uint16), ("devId", ctypes.c_uint16),
        ("maxHBMSize", u64), ("maxDRAMSize", u64), ("deviceVASpace", u64), ("hostVASpace", u64),
        ("scene", ctypes.c_int), ("globalUniqueAddress", ctypes.c_bool), ("role", ctypes.c_int), ("flags", u32),
        ("transUrl", ctypes.c_char * 64), ("tag", ctypes.c_char * 32), ("tagOpInfo", ctypes.c_char * 256),
        ("tlsOption", HybmTlsConfig), ("dramShmFd", ctypes.c_int),
    ]


# name -> (restype, argtypes); every symbol include/*.h declares for libmf_hip_dataplane.so
_SIGNATURES = {
    # mf_xcopy_api.h, hybm layer
    "hybm_init": (i32, [ctypes.c_uint16, u64]),
    "hybm_uninit": (None, []),
    "hybm_get_error_string": (ctypes.c_char_p, [i32]),
    "hybm_set_extern_logger": (None, [vp]),
    "hybm_set_log_level": (i32, [ctypes.c_int]),
    "hybm_create_entity": (vp, [ctypes.c_uint16, ctypes.POINTER(HybmOptions), u32]),
    "hybm_destroy_entity": (None, [vp, u32]),
    "hybm_reserve_mem_space": (i32, [vp, u32]),
    "hybm_unreserve_mem_space": (i32, [vp, u32]),
    "hybm_get_memory_ptr": (vp, [vp, ctypes.c_int]),
    "hybm_alloc_local_memory": (vp, [vp, ctypes.c_int, u64, u32]),
    "hybm_free_local_memory": (i32, [vp, vp, u32, u32]),
    "hybm_get_slice_va": (vp, [vp, vp]),
    "hybm_register_local_memory": (vp, [vp, vp, u64, u32]),
    "hybm_data_copy": (i32, [vp, ctypes.POINTER(HybmCopyParams), ctypes.c_int, vp, u32]),
    "hybm_data_batch_copy": (i32, [vp, ctypes.POINTER(BatchCopyParams), ctypes.c_int, vp, u32]),
    "hybm_wait": (i32, [vp]),
    # mf_xcopy_api.h, smem layer
    "smem_bm_config_init": (i32, [ctypes.POINTER(SmemBmConfig)]),
    "smem_bm_init": (i32, [ctypes.c_char_p, u32, ctypes.c_uint16, ctypes.POINTER(SmemBmConfig)]),
    "smem_bm_uninit": (None, [u32]),
    "smem_bm_get_rank_id": (u32, []),
    "smem_bm_create": (vp, [u32, u32, ctypes.c_int, u64, u64, u32]),
    "smem_bm_create2": (vp, [u32, ctypes.POINTER(SmemBmCreateOption)]),
    "smem_bm_destroy": (None, [vp]),
    "smem_bm_join": (i32, [vp, u32]),
    "smem_bm_leave": (i32, [vp, u32]),
    "smem_bm_get_local_mem_size_by_mem_type": (u64, [vp, ctypes.c_int]),
    "smem_bm_ptr_by_mem_type": (vp, [vp, ctypes.c_int, ctypes.c_uint16]),
    "smem_bm_copy": (i32, [vp, ctypes.POINTER(SmemCopyParams), ctypes.c_int, u32]),
    "smem_bm_copy_batch": (i32, [vp, ctypes.POINTER(BatchCopyParams), ctypes.c_int, u32]),
    "mf_bm_copy_batch_replay": (i32, [vp, ctypes.POINTER(ctypes.POINTER(BatchCopyParams)), u32, u32, ctypes.c_int, u32]),
    "mf_trans_batch_write_replay": (i32, [vp, ctypes.POINTER(ctypes.POINTER(BatchCopyParams)), u32, u32, ctypes.c_char_p, vp]),
    "mf_bm_copy_batch_replay_threads": (i32, [vp, ctypes.POINTER(ctypes.POINTER(BatchCopyParams)), u32, u32, ctypes.c_int, u32,
                                        ctypes.POINTER(ctypes.c_double)]),
    "smem_bm_wait": (i32, [vp]),
    "smem_bm_register_user_mem": (i32, [vp, u64, u64]),
    "smem_bm_unregister_user_mem": (i32, [vp, u64]),
    "smem_bm_get_rank_id_by_gva": (u32, [vp, vp]),
    "smem_set_extern_logger": (i32, [vp]),
    "smem_set_log_level": (i32, [ctypes.c_int]),
    "smem_get_last_err_msg": (ctypes.c_char_p, []),
    # mf_hip_dataplane.h and mf_hip_dataplane_internal.h
    "mf_xcopy_batch": (i32, [u64p, u64p, u64p, u32, i32, vp]),
    "mf_xcopy_device_table": (i32, [vp, u32, i32, vp]),
    "mf_xcopy_device_table_static": (i32, [vp, u32, i32, vp]),
    "mf_xcopy_2d_batch": (i32, [vp, u32, i32, vp]),
    "mf_copy2d_describe": (None, [u64, ctypes.POINTER(u32), ctypes.POINTER(u32)]),
    "mf_copy2d_rowcol_mismatches": (u32, [u32, u32, u32, u32]),
    "mf_xcopy_thread_stream": (vp, []),
    "mf_xcopy_tune": (i32, [u32, u32, u32]),
    "mf_xcopy_unordered_streams": (i32, [u32]),
    "mf_xcopy_stream_queues": (u32, [ctypes.POINTER(u32), u32]),
    "mf_xcopy_tune_table": (i32, [u32, u32]),
    "mf_xcopy_tune_hold": (i32, [u32, i32, u32]),
    "mf_xcopy_calibration": (i32, [ctypes.POINTER(i32), ctypes.POINTER(i32), ctypes.POINTER(u32), ctypes.POINTER(u32),
                                 ctypes.POINTER(u32), ctypes.POINTER(ctypes.c_float)]),
    "mf_xcopy_hold_stores": (i32, [i32]),
    "mf_xcopy_windows": (i32, [u32]),
    "mf_xcopy_choose_units": (u32, [u64, u32, i32]),
    "mf_xcopy_launch_count": (u64, []),
    "mf_xcopy_describe_plan": (i64, [u64p, u64p, u64p, u32, u32, u64p, u64, ctypes.POINTER(i32)]),
    "mf_host_launch_costs": (i32, [vp, vp, u32]),
    "mf_pin_thread_near_gpu": (i32, []),
    "mf_moe_workspace_bytes": (u64, [u32, u32, u32]),
    "mf_moe_dispatch": (i32, [vp, vp, u32, u32, u32, u32, vp, vp, vp, vp, vp, vp, u64, vp]),
    "mf_moe_combine": (i32, [vp, vp, vp, u32, u32, u32, vp, vp]),
    "mf_moe_combine_windows": (i32, [u32, u32]),
    "mf_moe_xcd_streams": (i32, []),
    "mfrt_init": (ctypes.c_int, [ctypes.c_int]),
    "mfrt_shutdown": (None, []),
    "mfrt_is_initialised": (ctypes.c_int, []),
    "mfrt_device_id": (ctypes.c_int, []),
    "mfrt_current_device": (ctypes.c_int, []),
    "mfrt_bind_thread": (ctypes.c_int, []),
    "mfrt_cu_count": (u32, []),
    "mfrt_error_string": (ctypes.c_char_p, [ctypes.c_int]),
    "mfrt_alloc_device": (vp, [u64]),
    "mfrt_free_device": (ctypes.c_int, [vp]),
    "mfrt_alloc_host": (vp, [u64]),
    "mfrt_free_host": (ctypes.c_int, [vp]),
    "mfrt_pointer_kind": (ctypes.c_int, [vp]),
    "mfrt_stream_create": (vp, []),
    "mfrt_stream_destroy": (ctypes.c_int, [vp]),
    "mfrt_stream_sync": (ctypes.c_int, [vp]),
    "mfrt_device_sync": (ctypes.c_int, []),
    "mfrt_event_create": (vp, []),
    "mfrt_event_destroy": (ctypes.c_int, [vp]),
    "mfrt_event_record": (ctypes.c_int, [vp, vp]),
    "mfrt_event_sync": (ctypes.c_int, [vp]),
    "mfrt_stream_wait_event": (ctypes.c_int, [vp, vp]),
    "mfrt_streams_share_queue": (ctypes.c_int, [vp, vp]),
    "mfrt_event_done": (ctypes.c_int, [vp]),
    "mfrt_event_elapsed_ms": (ctypes.c_float, [vp, vp]),
    "mfrt_memcpy": (ctypes.c_int, [vp, vp, u64]),
    "mfrt_memset": (ctypes.c_int, [vp, ctypes.c_int, u64]),
    "mfrt_memcpy_async": (ctypes.c_int, [vp, vp, u64, vp]),
    "mf_va_clear": (None, []),
    "mf_va_add": (i32, [u64, u64, i32, u64, u32]),
    "mf_va_add_external": (i32, [u64, u64, i32, u64, u32, u32]),
    "mf_va_remove": (None, [u64]),
    "mf_va_gva_of_lva": (u64, [u64]),
    "mf_va_lva_of_gva": (u64, [u64]),
    "mf_va_is_gva": (i32, [u64]),
    "mf_va_is_known": (i32, [u64]),
    "mf_va_mem_type": (i32, [u64]),
    "mf_va_rank": (i64, [u64]),
    "mf_va_infer_direction": (i32, [u64, u64]),
    "mf_va_reserve": (u64, [u32, u64, i32]),
    "mf_va_unreserve": (None, [u64]),
    "mf_va_range_count": (u64, []),
    "mf_va_reserved_count": (u64, []),
    "mf_dir_compose": (i32, [i32, i32, i32, i32]),
    "mf_dir_translate_smem": (i32, [i32, i32, i32]),
    "mf_dir_checks": (i32, [i32]),
    "mf_gva_contains": (i32, [u64, u64, u64, u64, u64]),
    "mf_gva_rank": (u32, [u64, u64, u64, u64, u64]),
    "mf_gva_mask48": (u64, [u64]),
    "mf_trans_combine": (u32, [u64p, u32, u64p]),
    "mf_trans_translate": (u64, [u64p, u32, u64, u64]),
    "mf_trans_parse_name": (i32, [ctypes.c_char_p, u8p]),
    # mf_xcopy_api.h, transfer front-end
    "smem_trans_config_init": (i32, [ctypes.POINTER(SmemTransConfig)]),
    "smem_trans_init": (i32, [ctypes.POINTER(SmemTransConfig)]),
    "smem_trans_uninit": (None, [u32]),
    "smem_trans_create": (vp, [ctypes.c_char_p, ctypes.c_char_p, ctypes.POINTER(SmemTransConfig)]),
    "smem_trans_destroy": (None, [vp, u32]),
    "smem_trans_malloc": (vp, [vp, ctypes.c_size_t]),
    "smem_trans_free": (i32, [vp, vp]),
    "smem_trans_register_mem": (i32, [vp, vp, ctypes.c_size_t, u32]),
    "smem_trans_batch_register_mem": (i32, [vp, ctypes.POINTER(vp), u64p, u32, u32]),
    "smem_trans_deregister_mem": (i32, [vp, vp]),
    "smem_trans_write": (i32, [vp, vp, ctypes.c_char_p, vp, ctypes.c_size_t, u32]),
    "smem_trans_batch_write": (i32, [vp, ctypes.POINTER(vp), ctypes.c_char_p, ctypes.POINTER(vp), u64p, u32, u32]),
    "smem_trans_read": (i32, [vp, vp, ctypes.c_char_p, vp, ctypes.c_size_t, u32]),
    "smem_trans_batch_read": (i32, [vp, ctypes.POINTER(vp), ctypes.c_char_p, ctypes.POINTER(vp), u64p, u32, u32]),
    "smem_trans_read_submit": (i32, [vp, vp, ctypes.c_char_p, vp, ctypes.c_size_t, vp, u32]),
    "smem_trans_write_submit": (i32, [vp, vp, ctypes.c_char_p, vp, ctypes.c_size_t, vp, u32]),
    "smem_trans_batch_read_submit": (i32, [vp, ctypes.POINTER(vp), ctypes.c_char_p, ctypes.POINTER(vp), u64p, u32,
                                           vp, u32]),
    "smem_trans_batch_write_submit": (i32, [vp, ctypes.POINTER(vp), ctypes.c_char_p, ctypes.POINTER(vp), u64p, u32,
                                            vp, u32]),
}

_PLUGIN_SIGNATURES = {
    "hybm_copy_extend": (None, [vp, vp, u64, u32, vp]),
    "hybm_batch_copy_extend": (None, [vp, u32, vp, u32, vp]),
    "mf_copy_extend_failures": (u64, []),
}

_YARDSTICK_SIGNATURES = {
    "mf_probe_hbm": (i32, [i32, vp, vp, u64, vp]),
}

_lock = threading.Lock()
_lib = None
_plugin = None
_yardstick = None


# pace of the combine's read and write parts the library starts with (MB/s), for callers that switch it and back
MOE_COMBINE_WINDOWS_DEFAULT = (6800000, 6200000)


def _bind(handle, table):
    for name, (restype, argtypes) in table.items():
        fn = getattr(handle, name)  # AttributeError names the missing symbol
        fn.restype = restype
        fn.argtypes = argtypes
    return handle


def lib():
    """The data-plane library; raises OSError if it has not been built."""
    global _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(DATAPLANE_PATH):
                raise OSError(
                    f"{DATAPLANE_PATH} is missing: build it with `make -C memfabric_hybrid_amd/csrc` "
                    "(or __graft_entry__.build()); there is no fallback path")
            _lib = _bind(ctypes.CDLL(DATAPLANE_PATH, mode=ctypes.RTLD_GLOBAL), _SIGNATURES)
        return _lib


def plugin():
    """The two-symbol copy plugin, loaded the way the reference loads it (dlopen by path)."""
    global _plugin
    with _lock:
        if _plugin is None:
            if not os.path.exists(PLUGIN_PATH):
                raise OSError(f"{PLUGIN_PATH} is missing: build it with `make -C memfabric_hybrid_amd/csrc`")
            _plugin = _bind(ctypes.CDLL(PLUGIN_PATH, mode=ctypes.RTLD_LOCAL), _PLUGIN_SIGNATURES)
        return _plugin


def yardstick():
    """The streaming yardstick kernels (measurement tooling of bench.py and the tests)."""
    global _yardstick
    with _lock:
        if _yardstick is None:
            if not os.path.exists(YARDSTICK_PATH):
                raise OSError(f"{YARDSTICK_PATH} is missing: build it with `make -C memfabric_hybrid_amd/csrc`")
            _yardstick = _bind(ctypes.CDLL(YARDSTICK_PATH, mode=ctypes.RTLD_LOCAL), _YARDSTICK_SIGNATURES)
        return _yardstick


def declared_symbols():
    return sorted(_SIGNATURES), sorted(_PLUGIN_SIGNATURES)


def last_error():
    return lib().smem_get_last_err_msg().decode("utf-8", "replace")


def u64_array(values):
    arr = (ctypes.c_uint64 * len(values))()
    for i, v in enumerate(values):
        arr[i] = int(v)
    return arr


def ptr_array(values):
    arr = (ctypes.c_void_p * len(values))()
    for i, v in enumerate(values):
        arr[i] = int(v)
    return arr
