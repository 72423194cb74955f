"""Compile the HIP sources under rocal_amd/csrc into rocal_amd/lib/librocal_mi355x.so (gfx950)."""
import concurrent.futures as cf
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
# RMX_LIB_NAME / RMX_EXTRA_FLAGS: measurement builds under another name (e.g. the streaming bilinear kernel without its loads,
# stores or arithmetic: RMX_LIB_NAME=librocal_exp4.so RMX_EXTRA_FLAGS=-DRMX_DMA_EXPERIMENT=4), loaded with RMX_LIB=<path>;
# such a build keeps its objects apart from the library's.
_NAME = os.environ.get("RMX_LIB_NAME", "librocal_mi355x.so")
OBJDIR = os.path.join(HERE, "lib", "obj" if _NAME == "librocal_mi355x.so" else "obj_" + os.path.splitext(_NAME)[0])
LIB = os.path.join(LIBDIR, _NAME)
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -ffp-contract=off: the kernels spell every fused multiply-add out (bit-exact parity with the
# CPU checker depends on it). Packed fp32 instructions are switched off for the device pass.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fvisibility=hidden",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function",
         "-Wno-unknown-cuda-version"]


def _newest_header():
    return max(os.path.getmtime(h) for h in glob.glob(os.path.join(CSRC, "*.h")) + [os.path.join(HERE, "..", "include", "rocal_mi355x.h")])


# Sources whose generated code the CPU tests read (explicit wait counts that rely on how many instructions the compiler makes):
# their device assembly is kept next to the object, so that the tests need not compile them a second time.
KEEP_ASSEMBLY = ("rmx_kernels_resize_dma.hip", "rmx_kernels_tri_dma_2.hip", "rmx_kernels_tri_dma_4.hip", "rmx_kernels_tri_dma_8_nchw.hip",
                 "rmx_kernels_tri_dma_8_nhwc.hip", "rmx_kernels_warp.hip")


def assembly_path(src_name):
    return os.path.join(OBJDIR, os.path.splitext(src_name)[0] + "-hip-amdgcn-amd-amdhsa-gfx950.s")


def _compile(src, incremental=False):
    obj = os.path.join(OBJDIR, os.path.basename(src) + ".o")
    if incremental and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(src), _newest_header()):
        return obj, ""
    keep = ["-save-temps=obj"] if os.path.basename(src) in KEEP_ASSEMBLY else []
    cmd = [HIPCC] + FLAGS + keep + os.environ.get("RMX_EXTRA_FLAGS", "").split() + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the packed-fp32 feature name: that warning is expected
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, r.stderr))
    return obj, err


def build(verbose=False, incremental=False):
    """Compiles every source (incremental=True: only those older than their object or than a header)."""
    os.makedirs(OBJDIR, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    # objects of sources that no longer exist must not be linked
    for o in glob.glob(os.path.join(OBJDIR, "*.o")):
        if os.path.join(CSRC, os.path.basename(o)[:-2]) not in srcs:
            os.remove(o)
    with cf.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        results = list(ex.map(lambda s: _compile(s, incremental), srcs))
    objs = [o for o, _ in results]
    if verbose:
        for _, e in results:
            if e.strip():
                print(e, file=sys.stderr)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True, incremental="--incremental" in sys.argv))
