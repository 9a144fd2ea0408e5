"""The C-ABI libraries load and export every symbol include/*.h declares (no GPU needed)."""

import os
import re
import subprocess

from memfabric_hybrid_amd import native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include")

_DECL = re.compile(r"^\s*(?:const\s+)?[A-Za-z_][A-Za-z0-9_]*[\s\*]+\**\s*((?:hybm|smem|mf|mfrt)_[A-Za-z0-9_]+)\s*\(", re.M)


def _declared(header):
    text = open(os.path.join(INCLUDE, header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(_DECL.findall(text))


def _exported(path):
    out = subprocess.run(["nm", "-D", "--defined-only", path], check=True, capture_output=True, text=True).stdout
    return {line.split()[-1] for line in out.splitlines() if " T " in line}


def test_dataplane_exports_every_declared_symbol():
    stable = _declared("mf_xcopy_api.h") | _declared("mf_hip_dataplane.h")
    unstable = _declared("mf_hip_dataplane_internal.h")
    assert len(stable) > 60 and len(unstable) > 30
    assert stable & unstable == set()
    exported = _exported(native.DATAPLANE_PATH)
    assert (stable | unstable) - exported == set()


def test_stable_header_holds_no_test_views_or_switches():
    """Views of the host logic, replay loops and tuning switches are declared in the internal header only."""
    stable = _declared("mf_hip_dataplane.h")
    for name in stable:
        assert not name.startswith(("mf_va_", "mf_dir_", "mf_gva_", "mf_trans_")), name
        assert "replay" not in name and "tune" not in name and "describe" not in name, name
    assert {"mf_xcopy_batch", "mf_xcopy_device_table", "mf_xcopy_device_table_static", "mf_xcopy_2d_batch",
            "mf_moe_dispatch", "mf_moe_combine", "mfrt_init"} <= stable


def test_binding_table_matches_headers():
    declared = _declared("mf_xcopy_api.h") | _declared("mf_hip_dataplane.h") | _declared("mf_hip_dataplane_internal.h")
    bound, plug = native.declared_symbols()
    assert set(bound) == declared
    assert set(plug) == _declared("mf_hip_copy_extend.h")


def test_plugin_exports_the_two_symbols_and_its_failure_counter():
    """The reference's loader resolves the two copy symbols by name and needs both
    (dl_hybm_copy_extend.cpp:57-68 there); the only other export is the failure counter."""
    exported = _exported(native.PLUGIN_PATH)
    assert exported == {"hybm_copy_extend", "hybm_batch_copy_extend", "mf_copy_extend_failures"}


def test_yardstick_library_exports_its_one_symbol():
    assert _declared("mf_hip_yardstick.h") == {"mf_probe_hbm"}
    assert _exported(native.YARDSTICK_PATH) == {"mf_probe_hbm"}
    native.yardstick()


def test_libraries_load_and_bind():
    lib = native.lib()
    assert lib.hybm_get_error_string(0) == b"success"
    assert lib.hybm_get_error_string(-2) == b"invalid parameter"
    native.plugin()


def test_types_header_compiles_as_c_and_cxx(tmp_path):
    src = tmp_path / "t.c"
    src.write_text('#include "mf_xcopy_api.h"\n#include "mf_hip_dataplane.h"\n#include "mf_hip_dataplane_internal.h"\n#include "mf_hip_copy_extend.h"\n#include "mf_hip_yardstick.h"\nint main(void){return 0;}\n')
    subprocess.run(["gcc", "-std=c11", "-Wall", "-Werror", "-I", INCLUDE, "-c", str(src), "-o", str(tmp_path / "t.o")], check=True)
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Werror", "-x", "c++", "-I", INCLUDE, "-c", str(src), "-o", str(tmp_path / "t2.o")], check=True)


REFERENCE = "/root/reference"


def test_engine_compiles_against_the_reference_operator_header():
    """The copy engine (csrc/host/hip_data_op.cpp) is written against the reference's DataOperator
    contract: with MF_WITH_REFERENCE_HEADERS it includes the reference's own
    src/hybm/csrc/data_operation/hybm_data_operator.h (and hybm_def.h, smem_bm_def.h, ... in place
    of include/mf_xcopy_types.h's definitions) and must compile without an error."""
    import pytest
    header = os.path.join(REFERENCE, "src/hybm/csrc/data_operation/hybm_data_operator.h")
    if not os.path.exists(header):
        pytest.skip("the reference tree is not present on this machine")
    inc = ["src/hybm/include", "src/smem/include/host", "src/hybm/csrc/common", "src/smem/csrc/common",
           "src/hybm/csrc/data_operation", "src/util/csrc", "src/hybm/csrc", "src/util/csrc/ptracer/include"]
    cmd = ["g++", "-std=c++17", "-fsyntax-only", "-H", "-DNO_XPU", "-DMF_WITH_REFERENCE_HEADERS"]
    cmd += ["-I" + os.path.join(REFERENCE, d) for d in inc]
    cmd.append(os.path.join(ROOT, "memfabric_hybrid_amd", "csrc", "host", "hip_data_op.cpp"))
    run = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-3000:]
    used = run.stderr
    assert header in used                                                    # their contract, not our mirror of it
    assert os.path.join(ROOT, "memfabric_hybrid_amd/csrc/host/data_operator.h") not in used
    assert os.path.join(REFERENCE, "src/hybm/include/hybm_def.h") in used
