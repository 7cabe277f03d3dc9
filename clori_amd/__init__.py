"""MI355X (gfx950) attention backend for YVEX: C11 host + hand-written HIP kernels behind
the reference's backend operator contract.  `clori_amd.backend.Backend` wraps the C ABI
declared in include/yvex_rocm.h and include/yvex_rocm_operations.h; the shared library is
clori_amd/libyvex_rocm.so."""

from . import binding  # noqa: F401

__all__ = ["binding"]
