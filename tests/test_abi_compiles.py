"""The boundary as text that compiles: include/maya_moe.h as plain C11 (no C++-isms, nothing undeclared), and the
reference-side adapter (tests/adapter/maya_moe_adapter.cpp: the reference's operator signatures defined over the C ABI)
against the reference's own headers, the way the reference's HIP build compiles its sources."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference"


def test_header_is_c11(tmp_path):
    src = tmp_path / "use_header.c"
    src.write_text('#include "maya_moe.h"\n'
                   "int use(void) {\n"
                   "    maya_moe_args a = {0};\n"
                   "    maya_exl3_args b = {0};\n"
                   "    maya_mv_job j = {0};\n"
                   "    maya_residency r = {0};\n"
                   "    maya_prefill_plan p = {0};\n"
                   "    (void) b; (void) j; (void) r; (void) p;\n"
                   "    return maya_moe_gate_up(&a, 0) + (int) sizeof(maya_router) + MAYA_TYPE_IQ2_S;\n"
                   "}\n")
    r = subprocess.run(["gcc", "-std=c11", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-I", os.path.join(ROOT, "include"),
                        str(src)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    # and as C++ (the adapter's language)
    cpp = tmp_path / "use_header.cpp"
    cpp.write_text(src.read_text().replace("= {0};", "{};"))
    r = subprocess.run(["g++", "-std=c++17", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-I", os.path.join(ROOT, "include"),
                        str(cpp)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


def test_adapter_compiles_against_the_reference_headers():
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(os.path.join(REF, "include/strata/kernels/glm_fast.hpp")) or not os.path.exists(hipcc):
        pytest.skip("no reference tree (or no hipcc) here")
    # the reference's HIP build force-includes its own cuda_runtime.h shim (cmake/hip_backend.cmake:120-134)
    cmd = [hipcc, "-std=c++20", "-fsyntax-only", "-x", "hip", "--offload-arch=gfx950", "-DSTRATA_USE_HIP=1",
           "-include", os.path.join(REF, "include/strata/hip_compat/cuda_runtime.h"),
           "-I" + os.path.join(REF, "include/strata/hip_compat"), "-I" + os.path.join(REF, "include"), "-I" + os.path.join(REF, "src/ds4"),
           "-I" + os.path.join(ROOT, "include"), "-Wall", "-Werror", "-Wno-unused-command-line-argument",
           os.path.join(ROOT, "tests/adapter/maya_moe_adapter.cpp")]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
