"""mograd_amd: MI355X (gfx950) implementation of mograd's backward hot path.

`mograd_amd.runtime` mirrors the reference's kernel-dispatch surface over the C ABI of
libmograd_hip.so (declared in include/mograd_hip.h, built by `python -m mograd_amd.build`).
Importing the package does not load the library; constructing a `Device` does, and raises
if it is missing.
"""
from ._lib import BF16, F16, F32, I32, I64, LibraryMissing, MogradError, load  # noqa: F401
from .runtime import (GRAD_RULES, SCHEDULER_RULES, AnyBuffer, Device, Layout, Node, evaluate, evaluate_many,  # noqa: F401
                      gradient, run)

__version__ = "0.1"
