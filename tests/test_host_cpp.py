"""The C++ host interface (forja_amd/host/forja_hip.hpp): it must compile on its own against the
C ABI header, and its known-answer program must pass on the device."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "forja_amd", "host")


def test_host_header_compiles_standalone():
    result = subprocess.run(
        ["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-Werror", "-I" + os.path.join(ROOT, "include"),
         "-I" + HOST, "-x", "c++", "-"],
        input='#include "forja_hip.hpp"\nint main() { return 0; }\n', capture_output=True, text=True)
    assert result.returncode == 0, result.stderr


@pytest.mark.gpu
def test_cpp_known_answers_on_device():
    binary = os.path.join(HOST, "conformance")
    assert os.path.exists(binary), "run forja_amd/build.py first"
    result = subprocess.run([binary], capture_output=True, text=True, timeout=120)
    assert result.returncode == 0, result.stdout + result.stderr
    assert "all checks passed" in result.stdout
