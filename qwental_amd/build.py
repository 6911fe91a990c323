"""Build recipe of the HIP backend: kernels -> gfx950 code object -> embedded into libqwgpu_hip.so.

    python -m qwental_amd.build

Three steps, all cross-compile without a GPU:
  1. hipcc --genco: csrc/kernels/qw_kernels.hip -> csrc/qw_kernels_gfx950.hsaco (one code object: the same kernels spread over
     several measured 3 % slower on the 48-layer step)
  2. hipcc -c: csrc/qw_noalloc.hip (host + device: the per-device scratch array of the entry point that allocates nothing) -> csrc/qw_noalloc.o
  3. clang -std=c23: csrc/gpu_hip.c (embeds the code object) + csrc/qw_path.c + csrc/qw_gguf.c + csrc/qw_par.c + qw_noalloc.o -> qwental_amd/libqwgpu_hip.so
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HIPCC = os.path.join(ROCM, "bin", "hipcc")
CLANG = os.path.join(ROCM, "llvm", "bin", "clang")
LIB = os.path.join(HERE, "libqwgpu_hip.so")
# Experiments: QW_BUILD_TAG=<tag> makes a second build beside the product's, libqwgpu_hip_<tag>.so with its objects in
# csrc/_<tag>/ (QW_HIP_LIB selects it at run time); QW_BUILD_DEFS adds compiler flags, e.g. -DQW_PARTS=0x37 for a code
# object that holds only some groups of kernels (a short compile).
TAG = os.environ.get("QW_BUILD_TAG", "")
OBJDIR = os.path.join(CSRC, "_" + TAG) if TAG else CSRC
if TAG:
    os.makedirs(OBJDIR, exist_ok=True)
    LIB = os.path.join(HERE, "libqwgpu_hip_%s.so" % TAG)
HSACO = os.path.join(OBJDIR, "qw_kernels_gfx950.hsaco")
# -packed-fp32-ops: packed FP32 instructions are kept out of every kernel of this library
HIPFLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"] + os.environ.get("QW_BUILD_DEFS", "").split()


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode:
        sys.stderr.write(out + "\n")
        raise RuntimeError("build step failed: " + " ".join(cmd))
    return out


def build(verbose=False, kernels=True):
    """kernels=False keeps the code object of the last build (host-side iterations: `python -m qwental_amd.build --host-only`)."""
    if kernels or not os.path.exists(HSACO):
        out = _run([HIPCC] + HIPFLAGS + ["--genco", "-I", os.path.join(CSRC, "kernels"), "-o", HSACO, os.path.join(CSRC, "kernels", "qw_kernels.hip")])
        if verbose and out.strip():
            print(out)
    noalloc_o = os.path.join(OBJDIR, "qw_noalloc.o")
    _run([HIPCC] + HIPFLAGS + ["-fPIC", "-I", CSRC, "-I", os.path.join(ROOT, "include"), "-c", os.path.join(CSRC, "qw_noalloc.hip"), "-o", noalloc_o])
    out = _run([CLANG, "-std=c23", "-O2", "-Wall", "-Wextra", "-fPIC", "-shared", "--embed-dir=" + OBJDIR] + [f for f in os.environ.get("QW_BUILD_DEFS", "").split() if f.startswith("-D")] + ["-I", os.path.join(ROOT, "include"), "-I", CSRC,
                "-I", os.path.join(ROCM, "include"), os.path.join(CSRC, "gpu_hip.c"), os.path.join(CSRC, "qw_path.c"), os.path.join(CSRC, "qw_gguf.c"), os.path.join(CSRC, "qw_par.c"), noalloc_o, "-pthread", "-o", LIB,
                "-L", os.path.join(ROCM, "lib"), "-lamdhip64", "-Wl,-rpath," + os.path.join(ROCM, "lib")])
    if verbose and out.strip():
        print(out)
    if TAG:
        return LIB
    # command-line tool with the reference's dqtest contract
    _run([CLANG, "-std=c23", "-O2", "-Wall", "-I", os.path.join(ROOT, "include"), os.path.join(CSRC, "tools", "dqhip.c"), "-o",
          os.path.join(HERE, "dqhip"), "-L", HERE, "-lqwgpu_hip", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + os.path.join(ROCM, "lib")])
    return LIB


if __name__ == "__main__":
    print(build(verbose=True, kernels="--host-only" not in sys.argv))
