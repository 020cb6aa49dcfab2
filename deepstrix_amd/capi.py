"""ctypes binding of libdsx_moe.so (include/dsx_moe.h).

This is the stand-in for the reference's Rust FFI layer (crates/v4flash-hip/src/sys.rs):
plain pointers and sizes in, an int status out, mapped to an exception the way the Rust
wrappers map a status to eyre::Report (crates/v4flash-hip/src/error.rs:10-78).  There is no
fallback: if the library is missing the import fails.
"""
from __future__ import annotations

import ctypes as C
import os

PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG, "lib", "libdsx_moe.so")

FMT_Q8_0 = 8
FMT_MXFP4 = 39
FMT_MXFP4_PLANAR = 1039  # the same matrix with nibble blocks and scales in separate planes (include/dsx_moe.h)
SRC_F32, SRC_BF16, SRC_F8E4M3 = 0, 1, 2  # dsx_q8_0_weights_from_hf source types
ROUTER_SQRT_SOFTPLUS, ROUTER_SIGMOID, ROUTER_SOFTMAX = 0, 1, 2
ERR_INVALID_ARG, ERR_SHAPE, ERR_UNSUPPORTED, ERR_DEVICE = -1, -2, -3, -4
Q8K_BLOCK_BYTES = 292
MXFP4_SUPER_BYTES = 136


class DsxError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"dsx error {code}: {message}")
        self.code = code
        self.message = message


class LayerDesc(C.Structure):
    _fields_ = [
        ("hidden", C.c_uint32), ("inter", C.c_uint32), ("n_expert", C.c_uint32),
        ("n_used", C.c_uint32),
        ("gate_fmt", C.c_int), ("up_fmt", C.c_int), ("down_fmt", C.c_int),
        ("gate", C.c_void_p), ("up", C.c_void_p), ("down", C.c_void_p),
        ("gate_bpe", C.c_uint64), ("up_bpe", C.c_uint64), ("down_bpe", C.c_uint64),
        ("clamp", C.c_float),
        ("router_mode", C.c_uint32), ("n_group", C.c_uint32), ("topk_group", C.c_uint32),
        ("route_scale", C.c_float), ("route_eps", C.c_float),
        ("bias", C.c_void_p),
        ("sh_inter", C.c_uint32),
        ("sh_gate_fmt", C.c_int), ("sh_up_fmt", C.c_int), ("sh_down_fmt", C.c_int),
        ("sh_gate", C.c_void_p), ("sh_up", C.c_void_p), ("sh_down", C.c_void_p),
        ("sh_clamp", C.c_float),
    ]


class HcPostDesc(C.Structure):
    """dsx_hc_post_desc (include/dsx_moe.h)."""
    _fields_ = [("out_hc", C.c_void_p), ("residual_hc", C.c_void_p), ("post", C.c_void_p),
                ("comb", C.c_void_p), ("n_hc", C.c_uint32), ("post_stride", C.c_uint32),
                ("comb_stride", C.c_uint32)]


_vp, _u32, _u64, _f32, _int, _sz = C.c_void_p, C.c_uint32, C.c_uint64, C.c_float, C.c_int, C.c_size_t

# name -> (restype, argtypes); every symbol include/dsx_moe.h declares
SIGNATURES = {
    "dsx_abi_version": (_int, []),
    "dsx_last_error": (C.c_char_p, []),
    "dsx_init": (_int, []),
    "dsx_router_topk": (_int, [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _f32, _f32, _u32, _u32, _u32, _u32]),
    "dsx_router_hash_select": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _f32, _f32, _u32]),
    "dsx_moe_hetsplit_select": (_int, [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32]),
    "dsx_router_logits": (_int, [_vp, _vp, _vp, _vp, _u32, _u32, _u32]),
    "dsx_router_logits_f16": (_int, [_vp, _vp, _vp, _vp, _u32, _u32, _u32]),
    "dsx_q8k_quantize": (_int, [_vp, _vp, _vp, _u32]),
    "dsx_q8_0_quantize": (_int, [_vp, _vp, _vp, _vp, _u32]),
    "dsx_q8_0_quantize_rows": (_int, [_vp, _vp, _vp, _u32, _u32]),
    "dsx_moe_gate_up_batch": (_int, [_vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _u64, _u64, _u32, _f32, _u32, _u32]),
    "dsx_moe_down_batched": (_int, [_vp, _int, _vp, _vp, _vp, _vp, _u64, _u32, _u32, _u32, _u32]),
    "dsx_moe_group_build": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32]),
    "dsx_moe_gate_up_chunked_rows": (_int, [_vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                            _u32, _u64, _u64, _u32, _u32, _f32, _u32, _u32]),
    "dsx_moe_down_by_expert": (_int, [_vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u64,
                                      _u32, _u32, _u32, _u32, _u32]),
    "dsx_moe_reduce_partials": (_int, [_vp, _vp, _vp, _vp, _u32, _u32, _u32]),
    "dsx_dense_ffn_scratch_bytes": (_sz, [_u32, _u32, _u32]),
    "dsx_dense_ffn": (_int, [_vp, _int, _int, _int, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _f32, _int, _vp]),
    "dsx_vec_add_inplace": (_int, [_vp, _vp, _vp, _u64]),
    "dsx_rms_norm": (_int, [_vp, _vp, _vp, _vp, _u32, _f32, _u32]),
    "dsx_swiglu_clamp_weighted": (_int, [_vp, _vp, _vp, _vp, _vp, _f32, _u32, _u32]),
    "dsx_mxfp4_repack_hf_to_v2": (_int, [_vp, _vp, _vp, _vp, _u32, _u32]),
    "dsx_q8_0_weights_from_hf": (_int, [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32, _u32]),
    "dsx_q8_0_repack_rows": (_int, [_vp, _vp, _vp, _u32, _u32]),
    "dsx_mxfp4_rows_to_planar": (_int, [_vp, _vp, _u32, _u32, _u32, _u64]),
    "dsx_mxfp4_planar_to_rows": (_int, [_vp, _vp, _u32, _u32, _u32, _u64]),
    "dsx_dequant_rows": (_int, [_vp, _int, _vp, _vp, _u32, _u32]),
    "dsx_moe_layer_create": (_int, [C.POINTER(LayerDesc), C.POINTER(_vp)]),
    "dsx_moe_layer_destroy": (None, [_vp]),
    "dsx_moe_layer_weights_to_planar": (_int, [_vp, _vp]),
    "dsx_moe_layer_weights_to_rows": (_int, [_vp, _vp]),
    "dsx_moe_layer_set_profile_events": (_int, [_vp, _vp, _vp, _vp]),
    "dsx_moe_layer_set_tuning": (_int, [_vp, _u32, _u32, _u32, _u32]),
    "dsx_moe_layer_get_tuning": (_int, [_vp, C.POINTER(C.c_uint32 * 6)]),
    "dsx_moe_layer_set_decode": (_int, [_vp, _u32, _u32]),
    "dsx_moe_layer_set_trace": (_int, [_vp, _vp, _sz]),
    "dsx_moe_layer_status": (_int, [_vp, _vp, C.POINTER(C.c_uint32)]),
    "dsx_moe_layer_status_ptr": (_int, [_vp, _vp, C.POINTER(_vp)]),
    "dsx_moe_layer_workspace_bytes": (_sz, [_vp, _u32]),
    "dsx_moe_block_forward": (_int, [_vp, _vp, _vp, _vp, _f32, _vp, _u32, _vp, _sz]),
    "dsx_moe_block_forward_f16": (_int, [_vp, _vp, _vp, _vp, _f32, _vp, _u32, _vp, _sz]),
    "dsx_moe_layer_forward_noalloc": (_int, [_vp, _vp, _vp, _vp, _vp, _u32, _vp, _vp, _vp, _vp]),
    "dsx_moe_layer_forward": (_int, [_vp, _vp, _vp, _vp, _vp, _u32, _vp, _sz, _vp, _vp, _vp, _vp]),
    "dsx_moe_layer_forward_hc": (_int, [_vp, _vp, C.POINTER(HcPostDesc), _vp, _vp, _u32, _vp, _sz, _vp, _vp, _vp, _vp]),
    "dsx_hc_post": (_int, [_vp, C.POINTER(HcPostDesc), _vp, _vp, _vp, _u32, _u32]),
}

_lib = None


def lib() -> C.CDLL:
    """Loads the library (raises if it was not built)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m deepstrix_amd.build` "
                "(there is no CPU fallback)")
        l = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        raise DsxError(rc, lib().dsx_last_error().decode("utf-8", "replace"))


_inited = set()


def init() -> None:
    """Verifies the current device is gfx950 (once per device)."""
    import torch
    dev = torch.cuda.current_device()
    if dev not in _inited:
        check(lib().dsx_init())
        _inited.add(dev)
