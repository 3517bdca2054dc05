"""coral_amd -- MI355X-native batched graph beam search behind CORAL's search API.

The product is the shared library coral_amd/lib/libcoral_search.so (HIP kernels
for gfx950 + a C ABI, include/coral_search.h) and the C++ class / CLI built on
it.  This package is the thin Python side: a ctypes binding used by the tests
and the benchmark (`coral_amd.capi`), the seeded synthetic data generators of
the benchmark configurations (`coral_amd.synth`) and readers/writers for the
reference's file formats (`coral_amd.formats`).
"""
from . import capi  # noqa: F401

__all__ = ["capi"]
