"""deepstrix_amd -- the deepstrix MoE feed-forward path for MI355X (gfx950).

The product is libdsx_moe.so (C ABI in include/dsx_moe.h, HIP sources in csrc/).  The Python
modules here are the host-side mirror of the reference's operator interface used by the
tests and the benchmark: `dispatch` (per-op functions, crates/v4flash-kernels/src/het/dispatch.rs),
`executor` (whole layer, MoeExecutor) and `synth` (synthetic tensors).
"""
from . import capi  # noqa: F401

__all__ = ["capi"]
