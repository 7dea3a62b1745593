"""hyle_amd -- MI355X (gfx950) compute provider for HYLE's tensor hot path.

`hyle_amd.compute` mirrors the reference's `hyle::compute` prepare/submit interface over
the C ABI of libhyle_hip.so; `hyle_amd.torch_io` is plumbing that lets tests and the
benchmark keep device memory in torch tensors.  Importing `hyle_amd.compute` without the
built library raises: there is no CPU path.
"""
from . import capi  # noqa: F401

__all__ = ["capi", "compute", "torch_io", "build"]
