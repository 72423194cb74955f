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


def _device_assembly(src_name):
    """The gfx950 assembly of one kernel source, with the flags the library is built with: the file the build keeps next to
    the object when it is newer than the source and every header, else a compilation of its own."""
    from rocal_amd import build as rbuild
    src = os.path.join(ROOT, "rocal_amd", "csrc", src_name)
    kept = rbuild.assembly_path(src_name)
    if os.path.exists(kept) and not os.environ.get("RMX_EXTRA_FLAGS") and os.path.getmtime(kept) > max(os.path.getmtime(src), rbuild._newest_header()):
        return open(kept).read()
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "kernel.s")
        subprocess.run([HIPCC] + list(rbuild.FLAGS) + ["-I" + os.path.join(ROOT, "rocal_amd", "csrc"), "-I" + os.path.join(ROOT, "include"),
                        "--cuda-device-only", "-S", src, "-o", out], check=True, capture_output=True, timeout=900)
        return open(out).read()


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="needs hipcc")
def test_held_back_stores_cover_the_wait_count():
    text = _device_assembly("rmx_kernels_resize_dma.hip")
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
        # The held-back group: the first basic block behind the last load into LDS that stores anything. Only ITS stores
        # are known to lie between the next window's loads and the numbered wait on every path (stores of other blocks
        # further down, e.g. element-wise ones of a partial group, must not be counted).
        tail = "\n".join(lines[loads[-1] + 1:])
        blocks = re.split(r"\n(?=\.LBB\d+_\d+:)", tail)
        held = next((b for b in blocks if re.search(r"^\s*global_store", b, re.M)), "")
        stores_behind = len(re.findall(r"^\s*global_store", held, re.M))
        if n:
            assert stores_behind >= n, "%s: waits with vmcnt(%d) but the held-back group has %d stores" % (m.group(1), n, stores_behind)
            assert "global_load_lds" not in held
        checked += 1
    assert checked >= 20  # every instance of the kernel


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="needs hipcc")
def test_streaming_triangular_kernel_counts_its_stores():
    """The streaming triangular kernel waits for its loads into LDS with s_waitcnt vmcnt(6 x output rows stored since): every
    output row must be exactly six store instructions (written as inline assembly, one per element and lane), no store may
    come from the compiler, nothing may spill to scratch memory (scratch traffic counts as vector memory too), and the only
    waits with a number are the two the source names."""
    # (the kernel's instances are spread over four translation units)
    text = "\n".join(_device_assembly("rmx_kernels_tri_dma_%s.hip" % u) for u in ("2", "4", "8_nchw", "8_nhwc"))
    funcs = re.split(r"\n(?=_ZN3rmx25rmx_resize_tri_dma_kernel[^\n]*:\s)", text)
    checked = 0
    for f in funcs:
        m = re.match(r"(_ZN3rmx25rmx_resize_tri_dma_kernel\S*):", f)
        if not m:
            continue
        body = f.split("s_endpgm")[0]
        stores = re.findall(r"^\s*(global_store_\w+|flat_store_\w+|buffer_store_\w+|scratch_\w+)", body, re.M)
        # tap-count variants of the row loop x accumulator sets it stores from x (two columns x three channels). The kernel's
        # last template argument is the number of sets: 2, 4 or 8; the kernel with eight has six tap-count variants instead of
        # four and every one twice, for samples that use all eight sets and for samples that use the lower four
        slots = int(re.search(r"Li(\d)EEEv8RmxKArgs$", m.group(1)).group(1))
        assert slots in (2, 4, 8)
        # (the kernels with two and four sets: four tap-count variants and two for lanes that own neighbouring columns)
        expected = 6 * (8 + 4) * 6 if slots == 8 else (4 + 2) * slots * 6
        assert len(stores) == expected, "%s: %d store instructions" % (m.group(1), len(stores))
        assert len(set(stores)) == 1 and stores[0].startswith("global_store_"), "%s: %s" % (m.group(1), sorted(set(stores)))
        waits = sorted(set(int(x) for x in re.findall(r"s_waitcnt vmcnt\((\d+)\)", body)))
        assert set(waits) <= {0, 6, 12}, "%s: waits %s" % (m.group(1), waits)
        assert "global_load_lds_dwordx4" in body
        checked += 1
    assert checked == 54  # every instance of the kernel


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="needs hipcc")
def test_warp_kernel_hand_written_lds_reads_are_awaited_before_use():
    """The raw bilinear form of the warp kernel writes the LDS reads of a pixel's taps out by hand and waits for them by a
    count (s_waitcnt lgkmcnt(4): the four reads of the next pixel may still be outstanding). The compiler does not know
    that those registers are filled later, so the generated code of every instance is checked: in a loop that waits this
    way there are exactly the 32 read instructions of 8 pixels and nothing else that counts as an LDS / scalar-memory
    operation; the waits are 7 x lgkmcnt(4) and one lgkmcnt(0); and no instruction between a pixel's reads and the wait
    that covers them touches a register those reads fill."""
    text = _device_assembly("rmx_kernels_warp.hip")

    def regs(tok):
        m = re.match(r"v\[(\d+):(\d+)\]", tok)
        if m:
            return set(range(int(m.group(1)), int(m.group(2)) + 1))
        m = re.match(r"v(\d+)$", tok)
        return {int(m.group(1))} if m else set()

    funcs = re.split(r"\n(?=_ZN3rmx15rmx_warp_kernel[^\n]*:\s)", text)
    loops = 0
    for f in funcs:
        m = re.match(r"(_ZN3rmx15rmx_warp_kernel\S*):", f)
        if not m:
            continue
        body = f.split("s_endpgm")[0]
        blocks = re.split(r"\n(?=\.LBB\d+_\d+:)", body)
        for blk in blocks:
            if not re.search(r"ds_read2_b32 [^\n]* offset0:4[0-9] offset1:4[0-9]", blk):
                continue  # (only the hand-written reads take the row below from an offset inside the instruction)
            ins = [l.strip() for l in blk.splitlines() if l.strip() and not l.strip().startswith((";", "."))]
            lgkm = [i for i in ins if re.match(r"(ds_|s_load|s_buffer_load|s_memtime|s_memrealtime|s_sendmsg|s_dcache)", i)]
            assert len(lgkm) == 32 and all(i.startswith(("ds_read2_b32", "ds_read_b32")) for i in lgkm), (m.group(1), lgkm[:3], len(lgkm))
            waits = [i for i in ins if i.startswith("s_waitcnt")]
            assert [w.split()[-1] for w in waits] == ["lgkmcnt(4)"] * 7 + ["lgkmcnt(0)"], (m.group(1), waits)
            # pixel k's four reads are covered by the k-th wait
            pos_reads = [n for n, i in enumerate(ins) if i.startswith("ds_read")]
            pos_waits = [n for n, i in enumerate(ins) if i.startswith("s_waitcnt")]
            for k in range(8):
                group = pos_reads[4 * k: 4 * k + 4]
                filled = set()
                for n in group:
                    filled |= regs(ins[n].split()[1].rstrip(","))
                for n in range(group[-1] + 1, pos_waits[k]):
                    if ins[n].startswith("ds_read"):
                        continue  # (the next pixel's reads: they fill other registers, checked next)
                    toks = re.findall(r"v\[\d+:\d+\]|v\d+", ins[n])
                    touched = set().union(*[regs(t) for t in toks]) if toks else set()
                    assert not (touched & filled), "%s: '%s' touches a register whose LDS read is not awaited yet" % (m.group(1), ins[n])
                # the next pixel's reads must not fill a register of this pixel before this pixel's wait
                if k + 1 < 8 and pos_reads[4 * k + 4] < pos_waits[k]:
                    nxt = set()
                    for n in pos_reads[4 * k + 4: 4 * k + 8]:
                        nxt |= regs(ins[n].split()[1].rstrip(","))
                    assert not (nxt & filled), m.group(1)
            loops += 1
    assert loops >= 12  # two loops (with and without the ROI test) in each of the six formats
