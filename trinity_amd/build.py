"""Build libtrinity_amd.so (gfx950) in-tree with hipcc.

Usage: python -m trinity_amd.build            (also called by __graft_entry__.build)
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libtrinity_amd.so")
KERNEL_SOURCES = ["rmsnorm.hip", "gemm.hip", "skinny.hip", "attn.hip", "attn_few.hip", "scores.hip", "kvfp8.hip"]
# every kernel translation unit is compiled twice: for fp16 elements (namespace tri) and, with these defines, for
# bf16 elements (the same text in namespace tri_bf16); abi.hip dispatches on the element type of a call
BF16_DEFINES = ["-DTRI_BF16", "-Dtri=tri_bf16"]
# diag.hip (the issue probe) has no 16-bit element type of its own: compiled once
UNITS = [("abi.hip", "abi.o", []), ("diag.hip", "diag.o", [])] + [(s, s.replace(".hip", ".o"), []) for s in KERNEL_SOURCES] + \
        [(s, s.replace(".hip", "_bf16.o"), BF16_DEFINES) for s in KERNEL_SOURCES]
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-ignored-attributes",
]


# Kernels whose MFMA results feed ordinary arithmetic at once (softmax, score sums) keep the accumulators in
# architectural VGPRs; left to its default the compiler parks them in AGPRs and pays one v_accvgpr_read per
# element.  The GEMMs keep the default (accumulators in AGPRs free VGPRs for the pipeline).
EXTRA_FLAGS = {
    "scores.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    "attn_few.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
}


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libtrinity_amd.so cannot be built")
    return exe


def build(verbose=True, jobs=7):
    """Compile every translation unit and link the shared library."""
    from concurrent.futures import ThreadPoolExecutor

    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    cc = hipcc()

    def compile_one(unit):
        src, objname, defines = unit
        obj = os.path.join(objdir, objname)
        cmd = [cc] + FLAGS + EXTRA_FLAGS.get(src, []) + defines + ["-c", os.path.join(CSRC, src), "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s\n%s" % (src, r.stdout, r.stderr))
        err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
        if verbose and err.strip():
            sys.stderr.write(err + "\n")
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, UNITS))
    cmd = [cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (r.stdout, r.stderr))
    # a kernel whose host stub went missing only shows up as an unresolved symbol at load time
    import ctypes

    ctypes.CDLL(LIB)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build()
