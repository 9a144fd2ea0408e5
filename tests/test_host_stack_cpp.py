"""Builds and runs the C++ unit tests of the host stack (tests/cpp) over the CPU stand-in for the
runtime layer: operator priority/fallback semantics and the C API end to end, no GPU needed."""

import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "memfabric_hybrid_amd", "csrc", "host")
SOURCES = ["mf_log.cpp", "xcopy_engine.cpp", "va_manager.cpp", "hip_data_op.cpp", "compose_data_op.cpp",
           "mem_entity.cpp", "hybm_api.cpp", "smem_bm_api.cpp", "dataplane_api.cpp", "copy2d_api.cpp", "moe_api.cpp", "trans_entry.cpp", "smem_trans_api.cpp", "host_copy.cpp", "copy_extend_plugin.cpp"]


def test_host_stack_over_fake_runtime(tmp_path):
    exe = str(tmp_path / "test_host_stack")
    cmd = ["g++", "-O1", "-std=c++17", "-pthread"]
    if os.environ.get("MF_TEST_SANITIZE") == "thread":
        cmd += ["-g", "-fsanitize=thread"]
    elif os.environ.get("MF_TEST_SANITIZE"):
        cmd += ["-g", "-fsanitize=address,undefined"]
    cmd += ["-o", exe, os.path.join(ROOT, "tests", "cpp", "test_host_stack.cpp"),
            os.path.join(ROOT, "tests", "cpp", "fake_rt.cpp")] + [os.path.join(HOST, s) for s in SOURCES]
    build = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert build.returncode == 0, build.stderr[-4000:]
    run = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stdout[-4000:] + run.stderr[-4000:]
    assert "host stack tests passed" in run.stdout
