"""The C++ operator layer (mllm-advanced_amd/host): the engine-facing classes a maintainer would
drop into mllm/Backends. The GPU test runs the C++ test binary, which drives
registerBackend -> createOp -> load(.mllm) -> dispatch -> D2H and compares with the CPU oracle."""
import ctypes
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "mllm-advanced_amd", "host")
BIN = os.path.join(HOST, "tests", "hip_linear_test")
LIB = os.path.join(ROOT, "mllm-advanced_amd", "libmllm_hip_backend.so")


def test_backend_library_is_built_and_loads():
    assert os.path.exists(LIB), "run __graft_entry__.build()"
    ctypes.CDLL(os.path.join(ROOT, "mllm-advanced_amd", "libw4a32_hip.so"), mode=ctypes.RTLD_GLOBAL)
    ctypes.CDLL(LIB)
    assert os.path.exists(BIN)


def test_container_structs_have_the_on_disk_sizes():
    # head 268 bytes, descriptor 416 bytes: the header static_asserts them; check the text is there
    text = open(os.path.join(HOST, "mllm", "Engine", "ParameterReader.hpp")).read()
    assert "sizeof(ParameterPackHead) == 268" in text and "sizeof(ParameterDescriptor) == 416" in text
    assert "0x519ACE0519ACE000" in text


@pytest.mark.gpu
def test_cpp_operator_tests_pass(tmp_path):
    out = subprocess.run([BIN, str(tmp_path)], capture_output=True, text=True, timeout=300)
    print(out.stdout[-4000:])
    print(out.stderr[-2000:])
    assert out.returncode == 0, out.stdout[-2000:] + out.stderr[-2000:]
    assert "[ PASSED ]" in out.stdout
