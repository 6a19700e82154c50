"""MI355X-native (gfx950) implementation of Slang's cooperative-vector operators.

The arithmetic lives in slang_amd/libcoopvec_mi355x.so (hand-written HIP kernels behind the
C-ABI of include/coopvec.h); `slang_amd.coopvec` mirrors the Slang operator names on top of it.
"""
from . import _lib  # noqa: F401

__all__ = ["coopvec", "build"]
