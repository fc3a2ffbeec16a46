"""amos_amd: the AMOS auto-tensorize hot path on AMD MI355X (gfx950).

`amos_amd.ops` holds tensor-level entry points over the C ABI of
libamos_mi355x.so; `amos_amd.auto_tensorize` mirrors the Python surface of the
reference's `tvm.auto_tensorize` for the GEMM / batched GEMM / conv path.
"""
from . import _lib  # noqa: F401

__all__ = ["_lib"]
