"""The C-ABI library loads without a GPU and exports every symbol the header declares.
No compute entry point is called here."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "rocal_mi355x.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"RMX_API\s+[\w\s\*]+?\b(rmx_\w+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = _declared()
    assert len(names) >= 35
    for op in ("crop_mirror_normalize", "crop", "flip", "resize", "color_twist", "brightness", "contrast", "hue", "saturation",
               "warp_affine", "rotate"):
        assert "rmx_create_" + op in names and "rmx_update_" + op in names
    for n in ("rmx_ctx_create", "rmx_ctx_destroy", "rmx_ctx_sync", "rmx_op_launch", "rmx_op_destroy", "rmx_last_error",
              "rmx_update_resize_cmn"):
        assert n in names


def test_library_exports_every_declared_symbol():
    from rocal_amd import _lib
    assert os.path.exists(_lib.LIB_PATH), "build the library first: python -m rocal_amd.build"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    missing = [n for n in _declared() if not hasattr(lib, n)]
    assert not missing, "declared in include/rocal_mi355x.h but not exported: %s" % missing
    # the Python binding covers the same surface
    assert sorted(_lib.EXPORTS) == _declared()


def test_error_reporting_needs_no_gpu():
    from rocal_amd import _lib
    lib = _lib.lib()
    assert lib.rmx_version().decode().startswith("rocal-mi355x")
    assert lib.rmx_op_launch(None, None, None) != 0
    assert "NULL" in lib.rmx_last_error().decode()
    assert lib.rmx_op_algorithmic_bytes(None) == 0


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from rocal_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.RmxError, match="not built"):
        _lib.lib()


def test_public_api_header_stands_alone(tmp_path):
    """include/rocal_api_mi355x.h compiles with include/ as the only search path of this repository, and the caller program of the GPU
    tests names nothing outside it."""
    import subprocess
    src = tmp_path / "only_public.cpp"
    src.write_text('#include "rocal_api_mi355x.h"\n#include "rocal_mi355x.h"\nint main() { TimingInfo t{}; (void)t; return rocalGetSeed() == 0u ? 0 : 1; }\n')
    r = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-I", os.path.join(ROOT, "include"), str(src)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    caller = open(os.path.join(ROOT, "tests", "cpp", "api_caller.cpp")).read()
    includes = re.findall(r'#include\s+"([^"]+)"', caller)
    assert includes == ["rocal_api_mi355x.h"]
    # every rocal* entry point the public header declares is exported by the host library
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "rocal_api_mi355x.h")).read(), flags=re.S)
    declared = sorted(set(re.findall(r"ROCAL_API_CALL\s+(rocal\w+)\s*\(", text)))
    assert len(declared) >= 70
    host = os.path.join(ROOT, "rocal_amd", "lib", "librocal_mi355x_host.so")
    assert os.path.exists(host), "build the host layer first: make -C rocal_amd/host"
    syms = subprocess.run(["nm", "-D", "--defined-only", host], capture_output=True, text=True).stdout
    missing = [d for d in declared if (" T " + d + "\n") not in syms]
    assert not missing, missing
