"""MI355X-native SegOp runtime behind Futhark's generated-library C API.

The product is two shared libraries built in-tree by ``futhark_amd.build``:
``libfuthark_amd_kernels.so`` (hand-written gfx950 kernels behind a C ABI) and
``libsegops.so`` (C runtime + the ``futhark_*`` API of the ``segops`` program).
This package only holds the ctypes view of that API used by tests and bench,
and the seeded input generator.
"""
from .capi import Segops, Context, FutharkError, lib_path  # noqa: F401

__all__ = ["Segops", "Context", "FutharkError", "lib_path"]
