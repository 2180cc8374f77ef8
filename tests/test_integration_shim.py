"""The pybind11 / torch shim that the integration guide shows as the replacement of the reference's
csrc/linear/quant_linear.cpp is a real file (tests/integration/quant_linear_hip.cpp): it must be the text
the guide shows, and it must compile against include/uniql_amd.h and torch's headers."""
import os
import re
import shutil
import subprocess
import sysconfig

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SHIM = os.path.join(ROOT, "tests", "integration", "quant_linear_hip.cpp")


def test_document_shows_the_file():
    doc = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    shown = re.search(r"```cpp\n(// quant_linear_hip\.cpp.*?)```", doc, re.S).group(1)
    assert shown == open(SHIM).read()


def test_shim_compiles_against_the_header():
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    from torch.utils import cpp_extension
    includes = cpp_extension.include_paths(device_type="cuda") if "device_type" in cpp_extension.include_paths.__code__.co_varnames \
        else cpp_extension.include_paths(True)
    includes += [sysconfig.get_paths()["include"], os.path.join(ROOT, "include"), "/opt/rocm/include"]
    cmd = [hipcc, "-std=c++17", "-fsyntax-only", "-x", "c++", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-DTORCH_EXTENSION_NAME=quant_linear_cuda", "-Wno-everything"]
    cmd += [f"-I{p}" for p in includes] + [SHIM]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-3000:]
