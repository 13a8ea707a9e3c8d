"""gfx950 blit engine: linear copy, dword fill and batched small copies on one
MI355X, behind the interface of ROCr's core::Blit.

The directory name contains a hyphen, so it is imported by path under the
module name ``rocm_systems_amd`` (see ``__graft_entry__.load_package``).

Contents:
  csrc/      HIP kernels, the C ABI over HIP and the C++ core::Blit adapter
  lib/       built shared libraries (not tracked)
  build.py   compile recipe
  capi.py    ctypes binding of include/mi355_blit.h, used by tests and bench
"""
from . import aql, build, capi  # noqa: F401
