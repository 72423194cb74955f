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
