"""qwental_amd — MI355X (gfx950) backend of the quantized decode path behind the reference's GPU interface.

The product is the C library libqwgpu_hip.so (csrc/gpu_hip.c + csrc/qw_path.c + the HIP kernels). This package
holds its build recipe, a ctypes binding used by the tests and the benchmark, and the seeded synthetic generators
of the benchmark configurations. Nothing here computes on the CPU in place of the GPU: without the library or
without a gfx950 device every entry point raises.
"""
from . import synth  # noqa: F401
from .gpu import Gpu, Buf, Path, Tensor, MoeLayer, Gguf, Par, lib_path, load_lib  # noqa: F401
