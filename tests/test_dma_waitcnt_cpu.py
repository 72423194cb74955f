"""Generated code of the streaming bilinear kernel: the wait for a window's loads (s_waitcnt vmcnt(N), N > 0) relies on at
least N store instructions having been issued behind those loads (the held-back stores of the window before). The compiler
is free to merge adjacent stores, so the count is checked in the assembly of every instance of the kernel."""
import os
import re
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = "/opt/rocm/bin/hipcc"


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="needs hipcc")
def test_held_back_stores_cover_the_wait_count():
    from rocal_amd import build as rbuild
    src = os.path.join(ROOT, "rocal_amd", "csrc", "rmx_kernels_resize_dma.hip")
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "dma.s")
        flags = list(rbuild.FLAGS)  # the flags the library is built with
        subprocess.run([HIPCC] + flags + ["-I" + os.path.join(ROOT, "rocal_amd", "csrc"), "-I" + os.path.join(ROOT, "include"), "--cuda-device-only", "-S",
                        src, "-o", out], check=True, capture_output=True, timeout=600)
        text = open(out).read()
    funcs = re.split(r"\n(?=_ZN3rmx21rmx_resize_dma_kernel[^\n]*:\s)", text)
    checked = 0
    for f in funcs:
        m = re.match(r"(_ZN3rmx21rmx_resize_dma_kernel\S*):", f)
        if not m:
            continue
        body = f.split("s_endpgm")[0]
        lines = body.splitlines()
        waits = [int(x) for x in re.findall(r"^\s*s_waitcnt vmcnt\((\d+)\)\s*$", body, re.M)]
        n = max([w for w in waits if w > 0], default=0)
        loads = [i for i, l in enumerate(lines) if "global_load_lds" in l]
        assert loads, m.group(1)
        stores_behind = sum(1 for l in lines[loads[-1]:] if re.match(r"\s*global_store", l))
        assert stores_behind >= n, "%s: waits with vmcnt(%d) but only %d stores follow the loads" % (m.group(1), n, stores_behind)
        checked += 1
    assert checked >= 20  # every instance of the kernel
