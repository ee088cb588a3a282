"""The C-ABI library loads without a GPU and exports every entry point the header declares."""
import ctypes
import os
import re

from forja_amd import hip_backend

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_entry_points():
    text = open(os.path.join(ROOT, "include", "forja_hip.h")).read()
    return sorted(set(re.findall(r"FH_API[^;(]*?\b(fh_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = hip_backend.load_library()
    names = declared_entry_points()
    assert len(names) >= 20
    for name in names:
        assert getattr(lib, name) is not None, name
    assert sorted(hip_backend.EXPORTS) == names


def test_struct_layouts_match_the_header():
    # fh_tensor: u64 + 2*u32 + 8*u32 + 8*u64 + u64
    assert ctypes.sizeof(hip_backend.FhTensor) == 8 + 8 + 32 + 64 + 8
    assert ctypes.sizeof(hip_backend.FhInst) == 20
    assert ctypes.sizeof(hip_backend.FhError) == 32
    expected = 16 * 4 + 2 * 8 + 2 * 4 + 16 * ctypes.sizeof(hip_backend.FhTensor)
    assert ctypes.sizeof(hip_backend.FhDispatch) == expected
    assert hip_backend.load_library().fh_version().startswith(b"forja-hip")


def test_product_package_never_imports_the_oracle():
    """The shipped path must not route through the CPU oracle in any form."""
    package = os.path.join(ROOT, "forja_amd")
    pattern = re.compile(r"(import\s+oracle|from\s+oracle|liboracle|forja_cpu_oracle|orc_\w+\()")
    for directory, _, files in os.walk(package):
        for name in files:
            if name.endswith((".py", ".cpp", ".hip", ".hpp", ".h")):
                text = open(os.path.join(directory, name)).read()
                assert not pattern.search(text), f"{name} references the oracle"
