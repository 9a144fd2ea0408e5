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
    declared = _declared("mf_xcopy_api.h") | _declared("mf_hip_dataplane.h")
    assert len(declared) > 60
    exported = _exported(native.DATAPLANE_PATH)
    assert declared - exported == set()


def test_binding_table_matches_headers():
    declared = _declared("mf_xcopy_api.h") | _declared("mf_hip_dataplane.h")
    bound, plug = native.declared_symbols()
    assert set(bound) == declared
    assert set(plug) == _declared("mf_hip_copy_extend.h")


def test_plugin_exports_exactly_the_two_symbols():
    exported = _exported(native.PLUGIN_PATH)
    assert exported == {"hybm_copy_extend", "hybm_batch_copy_extend"}


def test_libraries_load_and_bind():
    lib = native.lib()
    assert lib.hybm_get_error_string(0) == b"success"
    assert lib.hybm_get_error_string(-2) == b"invalid parameter"
    native.plugin()


def test_types_header_compiles_as_c_and_cxx(tmp_path):
    src = tmp_path / "t.c"
    src.write_text('#include "mf_xcopy_api.h"\n#include "mf_hip_dataplane.h"\n#include "mf_hip_copy_extend.h"\nint main(void){return 0;}\n')
    subprocess.run(["gcc", "-std=c11", "-Wall", "-Werror", "-I", INCLUDE, "-c", str(src), "-o", str(tmp_path / "t.o")], check=True)
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Werror", "-x", "c++", "-I", INCLUDE, "-c", str(src), "-o", str(tmp_path / "t2.o")], check=True)
