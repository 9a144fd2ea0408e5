"""ctypes loader of the checkers under oracle/: the C restatement
(oracle/_build/libmf_oracle.so) and, when it was built, the reference-derived
library (oracle/_ref/libmf_ref.so).  Test infrastructure only."""

import ctypes
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_SO = os.path.join(ORACLE_DIR, "_build", "libmf_oracle.so")
REF_SO = os.path.join(ORACLE_DIR, "_ref", "libmf_ref.so")

u32 = ctypes.c_uint32
u64 = ctypes.c_uint64
i32 = ctypes.c_int32
i64 = ctypes.c_int64
vp = ctypes.c_void_p
u64p = ctypes.POINTER(ctypes.c_uint64)
vpp = ctypes.POINTER(ctypes.c_void_p)

_ORACLE_SIG = {
    "orc_copy": (i32, [vp, u64, vp, u64]),
    "orc_batch_copy": (i32, [vpp, vpp, u64p, u32]),
    "orc_batch_copy_fast": (i32, [vpp, vpp, u64p, u32]),
    "orc_copy_2d": (None, [vp, u64, vp, u64, u64, u64]),
    "orc_lcg_fill": (None, [vp, i32, u32]),
    "orc_lcg_mismatch": (i64, [vp, vp, u32]),
    "orc_direct_map": (i32, [i32, i32]),
    "orc_trans_direction": (i32, [i32, i32, i32]),
    "orc_infer_table": (i32, [i32, i32]),
    "orc_check_map": (i32, [i32, i32]),
    "orc_mask48": (u64, [u64]),
    "orc_gva_contains": (i32, [u64, u64, u64, u64, u64]),
    "orc_gva_rank": (u32, [u64, u64, u64, u64, u64]),
    "orc_gva_ptr_of_rank": (u64, [u64, u64, u32]),
    "orc_operator_rank": (u32, [u64, u64, u64, u64]),
    "orc_va_clear": (None, []),
    "orc_va_add": (i32, [u64, u64, i32, u64, u32, u32]),
    "orc_va_gva_of_lva": (u64, [u64]),
    "orc_va_lva_of_gva": (u64, [u64]),
    "orc_va_is_gva": (i32, [u64]),
    "orc_va_is_known": (i32, [u64]),
    "orc_va_mem_type": (i32, [u64]),
    "orc_va_rank": (i64, [u64]),
    "orc_va_remove": (None, [u64]),
    "orc_va_reserve": (u64, [u64, i32]),
    "orc_va_unreserve": (None, [u64]),
    "orc_va_classify": (i32, [u64]),
    "orc_va_infer_direction": (i32, [u64, u64]),
    "orc_coalesce": (u32, [u64p, u64p, u64p, u32, u64p]),
    "orc_trans_align": (None, [u64p, u64p]),
    "orc_trans_combine": (u32, [u64p, u32, u64p]),
    "orc_trans_translate": (u64, [u64p, u32, u64, u64]),
    "orc_ref_kernel_single_range": (None, [u64, u32, u32, u64p, u64p]),
    "orc_ref_kernel_batch_range": (None, [u32, u32, u32, ctypes.POINTER(u32), ctypes.POINTER(u32)]),
    "orc_moe_dispatch": (i32, [vp, vp, u32, u32, u32, u32, vp, vp, vp, vp, vp]),
    "orc_moe_combine": (None, [vp, vp, vp, u32, u32, u32, vp]),
    "orc_moe_route": (None, [vp, u32, u32, u32, vp, vp]),
    "orc_fill_random": (None, [vp, u64, u64]),
}

_REF_SIG = {
    "ref_va_clear": (None, []),
    "ref_va_add": (i32, [u64, u64, i32, u64, u32]),
    "ref_va_add_external": (i32, [u64, u64, i32, u64, u32, u32]),
    "ref_va_remove": (None, [u64]),
    "ref_va_gva_of_lva": (u64, [u64]),
    "ref_va_lva_of_gva": (u64, [u64]),
    "ref_va_is_gva": (i32, [u64]),
    "ref_va_is_known": (i32, [u64]),
    "ref_va_mem_type": (i32, [u64]),
    "ref_va_rank": (i64, [u64]),
    "ref_va_infer_direction": (i32, [u64, u64]),
    "ref_va_reserve": (u64, [u32, u64, i32]),
    "ref_va_unreserve": (None, [u64]),
    "ref_va_range_count": (u64, []),
    "ref_va_reserved_count": (u64, []),
    "ref_mask48": (u64, [u64]),
    "ref_memcpy": (i32, [vp, u64, vp, u64, u32]),
    "ref_batch_copy": (i32, [vpp, vpp, u64p, u32]),
    "ref_extend_try_load": (i32, []),
    "ref_extend_cleanup": (None, []),
    "ref_extend_copy": (i32, [vp, vp, u64, u32, vp]),
    "ref_extend_batch_copy": (i32, [vp, u32, vp, u32, vp]),
}

_oracle = None
_ref = None


def _bind(handle, table):
    for name, (restype, argtypes) in table.items():
        fn = getattr(handle, name)
        fn.restype = restype
        fn.argtypes = argtypes
    return handle


def build_oracle():
    subprocess.run(["make", "-C", ORACLE_DIR, "oracle"], check=True, capture_output=True)


def oracle():
    global _oracle
    if _oracle is None:
        if not os.path.exists(ORACLE_SO):
            build_oracle()
        _oracle = _bind(ctypes.CDLL(ORACLE_SO), _ORACLE_SIG)
    return _oracle


def reference():
    """The library built from the reference's own sources, or None where it was never built."""
    global _ref
    if _ref is None:
        if not os.path.exists(REF_SO):
            return None
        _ref = _bind(ctypes.CDLL(REF_SO), _REF_SIG)
    return _ref


def ptr_array(values):
    arr = (ctypes.c_void_p * len(values))()
    for i, v in enumerate(values):
        arr[i] = int(v)
    return arr


def u64_array(values):
    arr = (ctypes.c_uint64 * len(values))()
    for i, v in enumerate(values):
        arr[i] = int(v)
    return arr


def np_ptr(a):
    return a.ctypes.data
