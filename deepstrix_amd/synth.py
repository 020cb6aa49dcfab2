"""Synthetic tensors for the benchmark and the tests (libdsx_synth.so, csrc/dsx_synth.hip).

Values are a pure function of (seed, tensor id, element index); the host and the device
generator give identical bytes.  Distributions follow BASELINE configs: weights N(0, 0.02)
quantized to MXFP4 / Q8_0, activations and logits N(0, 1), router bias N(0, 0.01).  The
normal is an Irwin-Hall sum of twelve 16-bit uniforms (integer arithmetic, so exact on
every machine).
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

from .capi import FMT_MXFP4, FMT_Q8_0

PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG, "lib", "libdsx_synth.so")

# tensor ids
T_GATE, T_UP, T_DOWN, T_SH_GATE, T_SH_UP, T_SH_DOWN, T_X, T_LOGITS, T_BIAS, T_ROUTER_W, T_NORM_W = range(11)

_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is missing: run `python -m deepstrix_amd.build`")
        l = C.CDLL(LIB_PATH)
        vp, u64, u32, f32 = C.c_void_p, C.c_uint64, C.c_uint32, C.c_float
        l.dsx_synth_normal_host.argtypes = [vp, u64, u64, u64, u64, f32, f32]
        l.dsx_synth_normal_host.restype = None
        l.dsx_synth_mxfp4_host.argtypes = [vp, u64, u64, u64, u64, u32, f32]
        l.dsx_synth_mxfp4_host.restype = None
        l.dsx_synth_q8_0_host.argtypes = [vp, u64, u64, u64, u64, u32, f32]
        l.dsx_synth_q8_0_host.restype = None
        l.dsx_synth_normal_dev.argtypes = [vp, vp, u64, u64, u64, u64, f32, f32]
        l.dsx_synth_mxfp4_dev.argtypes = [vp, vp, u64, u64, u64, u64, u32, f32]
        l.dsx_synth_q8_0_dev.argtypes = [vp, vp, u64, u64, u64, u64, u32, f32]
        l.dsx_synth_copy_dev.argtypes = [vp, vp, vp, u64]
        l.dsx_synth_read_dev.argtypes = [vp, vp, vp, u64, u32]
        l.dsx_synth_read_tiles_dev.argtypes = [vp, vp, vp, u32, u32, C.c_int]
        _lib = l
    return _lib


def matrix_bytes(fmt: int, rows: int, cols: int) -> int:
    if fmt == FMT_MXFP4:
        if cols <= 0 or cols % 256:
            raise ValueError(f"MXFP4 rows need cols % 256 == 0, got {cols}")
        return rows * (cols // 256) * 136
    if fmt == FMT_Q8_0:
        if cols <= 0 or cols % 32:
            raise ValueError(f"Q8_0 rows need cols % 32 == 0, got {cols}")
        return rows * (cols // 32) * 34
    raise ValueError(f"unknown weight format {fmt}")


def normal_host(seed, tensor_id, n, sigma=1.0, mean=0.0, offset=0) -> np.ndarray:
    out = np.empty(n, np.float32)
    lib().dsx_synth_normal_host(out.ctypes.data, seed, tensor_id, offset, n, sigma, mean)
    return out


def weights_host(fmt, seed, tensor_id, n_rows, cols, sigma=0.02, first_row=0) -> np.ndarray:
    """Rows [first_row, first_row + n_rows) of a [*, cols] weight tensor, engine layout."""
    out = np.empty(matrix_bytes(fmt, n_rows, cols), np.uint8)
    fn = lib().dsx_synth_mxfp4_host if fmt == FMT_MXFP4 else lib().dsx_synth_q8_0_host
    fn(out.ctypes.data, seed, tensor_id, first_row * cols, n_rows, cols, sigma)
    return out


def normal_dev(seed, tensor_id, n, sigma=1.0, mean=0.0, offset=0, device="cuda"):
    import torch
    out = torch.empty(n, dtype=torch.float32, device=device)
    rc = lib().dsx_synth_normal_dev(torch.cuda.current_stream().cuda_stream, out.data_ptr(), seed,
                                    tensor_id, offset, n, sigma, mean)
    if rc:
        raise RuntimeError(f"dsx_synth_normal_dev: hip error {rc}")
    return out


def weights_dev(fmt, seed, tensor_id, n_rows, cols, sigma=0.02, first_row=0, device="cuda", out=None):
    import torch
    nbytes = matrix_bytes(fmt, n_rows, cols)
    if out is None:
        out = torch.empty(nbytes, dtype=torch.uint8, device=device)
    assert out.numel() == nbytes
    fn = lib().dsx_synth_mxfp4_dev if fmt == FMT_MXFP4 else lib().dsx_synth_q8_0_dev
    rc = fn(torch.cuda.current_stream().cuda_stream, out.data_ptr(), seed, tensor_id,
            first_row * cols, n_rows, cols, sigma)
    if rc:
        raise RuntimeError(f"dsx_synth weights: hip error {rc}")
    return out


def copy_dev(dst, src) -> None:
    """dst <- src with the library's plain streaming-copy kernel (byte-counter calibration)."""
    import torch
    assert dst.numel() * dst.element_size() == src.numel() * src.element_size()
    rc = lib().dsx_synth_copy_dev(torch.cuda.current_stream().cuda_stream, dst.data_ptr(),
                                  src.data_ptr(), src.numel() * src.element_size())
    if rc:
        raise RuntimeError(f"dsx_synth_copy_dev: hip error {rc}")


def read_dev(sink, src, workgroups: int = 0) -> None:
    """Streams `src` through the library's plain read kernel (one word per wave into `sink`, 16 bytes
    per workgroup): the read rate a device reaches on a buffer of that size."""
    import torch
    assert sink.numel() * sink.element_size() >= 16 * (workgroups or 4096)
    rc = lib().dsx_synth_read_dev(torch.cuda.current_stream().cuda_stream, sink.data_ptr(), src.data_ptr(),
                                  src.numel() * src.element_size(), workgroups)
    if rc:
        raise RuntimeError(f"dsx_synth_read_dev: hip error {rc}")


def read_tiles_dev(sink, src, n_tiles: int, n_sb: int, operand_order: bool = True) -> None:
    """Streams the first n_tiles 16-row tiles of an MXFP4 matrix (rows of n_sb super-blocks) the way
    the decode kernels stream weights -- or, operand_order=False, the same bytes in memory order
    (one word per wave into `sink`): the read rate that access pattern reaches on a device."""
    import torch
    assert src.numel() * src.element_size() >= n_tiles * 16 * n_sb * 136
    assert sink.numel() * sink.element_size() >= 16 * n_tiles
    rc = lib().dsx_synth_read_tiles_dev(torch.cuda.current_stream().cuda_stream, sink.data_ptr(), src.data_ptr(),
                                        n_tiles, n_sb, 1 if operand_order else 0)
    if rc:
        raise RuntimeError(f"dsx_synth_read_tiles_dev: hip error {rc}")
