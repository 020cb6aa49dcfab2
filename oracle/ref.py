"""ctypes front end of the CPU oracle (oracle/dsx_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke()`` and by
the ``cpu_baseline`` leg of bench.py -- never by the shipped package.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass
from typing import Optional

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_DIR, "_build", "libdsx_oracle.so")

FMT_Q8_0 = 8
FMT_MXFP4 = 39
ROUTER_SQRT_SOFTPLUS, ROUTER_SIGMOID, ROUTER_SOFTMAX = 0, 1, 2
Q8K_BLOCK = 292
SUPER = 136


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (seconds)."""
    src = os.path.join(_DIR, "dsx_oracle.c")
    stale = (not os.path.exists(_SO)) or os.path.getmtime(_SO) < max(
        os.path.getmtime(src), os.path.getmtime(os.path.join(_DIR, "dsx_oracle.h")))
    if force or stale:
        subprocess.check_call(["make", "-C", _DIR, "-B" if force else "-s"])
    return _SO


def use_timing_build() -> str:
    """For the timed CPU-baseline leg only: compiles the oracle for the host it runs on
    (-O3 -march=native, same floating-point rules, so the same results) into a temporary
    directory and switches this module to it.  Returns the flags in use; when the compile fails
    the committed portable build stays in place and its flags are returned."""
    global _lib
    import tempfile
    portable = "-O2 -fopenmp -ffp-contract=off -fno-fast-math"
    flags = "-O3 -march=native -fopenmp -ffp-contract=off -fno-fast-math"
    try:
        out = os.path.join(tempfile.mkdtemp(prefix="dsx_oracle_"), "libdsx_oracle_native.so")
        subprocess.check_call(["gcc", *flags.split(), "-fPIC", "-std=c11", "-shared", "-o", out,
                               os.path.join(_DIR, "dsx_oracle.c"), "-lm"],
                              stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
        l = C.CDLL(out)
        _declare(l)
        _lib = l
        return flags
    except (OSError, subprocess.CalledProcessError):
        return portable


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
        _declare(_lib)
    return _lib


class _Cfg(C.Structure):
    _fields_ = [
        ("hidden", C.c_int), ("inter", C.c_int), ("n_expert", C.c_int), ("n_used", C.c_int),
        ("gate_fmt", C.c_int), ("up_fmt", C.c_int), ("down_fmt", C.c_int),
        ("gate", C.c_void_p), ("up", C.c_void_p), ("down", C.c_void_p),
        ("gate_bpe", C.c_uint64), ("up_bpe", C.c_uint64), ("down_bpe", C.c_uint64),
        ("clamp", C.c_float),
        ("sh_inter", C.c_int),
        ("sh_gate_fmt", C.c_int), ("sh_up_fmt", C.c_int), ("sh_down_fmt", C.c_int),
        ("sh_gate", C.c_void_p), ("sh_up", C.c_void_p), ("sh_down", C.c_void_p),
        ("sh_clamp", C.c_float),
    ]


def _declare(l):
    vp, sz, f32, i32 = C.c_void_p, C.c_size_t, C.c_float, C.c_int
    l.dsx_ref_f16_to_f32.restype = f32
    l.dsx_ref_f16_to_f32.argtypes = [C.c_uint16]
    l.dsx_ref_f32_to_f16.restype = C.c_uint16
    l.dsx_ref_f32_to_f16.argtypes = [f32]
    l.dsx_ref_bf16_to_f32.restype = f32
    l.dsx_ref_bf16_to_f32.argtypes = [C.c_uint16]
    l.dsx_ref_f32_to_bf16.restype = C.c_uint16
    l.dsx_ref_f32_to_bf16.argtypes = [f32]
    for n in ("dsx_ref_e8m0_to_f32", "dsx_ref_e8m0_half_to_f32", "dsx_ref_e4m3_to_f32"):
        getattr(l, n).restype = f32
        getattr(l, n).argtypes = [C.c_uint8]
    l.dsx_ref_mxfp4_dequant_ggml.argtypes = [vp, vp, sz]
    l.dsx_ref_mxfp4_dequant_v2.argtypes = [vp, vp, sz, sz]
    l.dsx_ref_mxfp4_repack_hf_to_v2.argtypes = [vp, vp, vp, sz, sz]
    l.dsx_ref_mxfp4_unpack_v2_to_hf.argtypes = [vp, vp, vp, sz, sz]
    l.dsx_ref_mxfp4_quantize_v2.argtypes = [vp, vp, sz, sz]
    l.dsx_ref_q8_0_quantize_block.argtypes = [vp, vp]
    l.dsx_ref_q8_0_quantize_rows.argtypes = [vp, vp, sz, sz]
    l.dsx_ref_q8_0_repack_rows.argtypes = [vp, vp, sz, sz]
    l.dsx_ref_q8_0_from_hf.restype = i32
    l.dsx_ref_q8_0_from_hf.argtypes = [vp, vp, i32, sz, sz, sz, sz, vp]
    l.dsx_ref_q8_0_dequant_rows.argtypes = [vp, vp, sz, sz]
    l.dsx_ref_q8_0_quantize_act.argtypes = [vp, vp, vp, sz]
    l.dsx_ref_dot_q8_0.restype = f32
    l.dsx_ref_dot_q8_0.argtypes = [sz, vp, vp, vp]
    l.dsx_ref_q8k_quantize.argtypes = [vp, vp, sz]
    l.dsx_ref_q8k_dequant.argtypes = [vp, vp, sz]
    l.dsx_ref_dot_mxfp4_q8k.restype = f32
    l.dsx_ref_dot_mxfp4_q8k.argtypes = [sz, vp, vp]
    l.dsx_ref_swiglu.restype = f32
    l.dsx_ref_swiglu.argtypes = [f32, f32, f32, f32]
    l.dsx_ref_rms_norm.argtypes = [vp, vp, vp, sz, f32, sz]
    l.dsx_ref_hc_post.argtypes = [vp, vp, vp, vp, vp, vp, vp, sz, sz, sz, sz, sz]
    l.dsx_ref_hc_post.restype = None
    l.dsx_ref_router_topk.restype = i32
    l.dsx_ref_router_topk.argtypes = [vp, vp, vp, vp, i32, i32, f32, f32, i32, i32, i32, i32]
    l.dsx_ref_router_scores.restype = i32
    l.dsx_ref_router_scores.argtypes = [vp, vp, vp, vp, i32, i32, i32, i32, i32]
    l.dsx_ref_router_logits.argtypes = [vp, vp, vp, i32, i32, i32]
    l.dsx_ref_hetsplit_select.argtypes = [vp, vp, vp, i32, i32, i32, i32, i32]
    l.dsx_ref_router_hash_select.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, f32, f32, i32]
    l.dsx_ref_group_build.restype = i32
    l.dsx_ref_group_build.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32]
    l.dsx_ref_wi_upper_bound.restype = C.c_uint32
    l.dsx_ref_wi_upper_bound.argtypes = [sz, C.c_uint32, C.c_uint32, sz]
    l.dsx_ref_moe_forward.restype = i32
    l.dsx_ref_moe_forward.argtypes = [C.POINTER(_Cfg), vp, vp, vp, i32, vp, vp, vp, vp, i32]
    l.dsx_ref_max_threads.restype = i32


def _p(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


# ---- formats ---------------------------------------------------------------

def mxfp4_dequant_ggml(blocks: np.ndarray) -> np.ndarray:
    blocks = _c(blocks, np.uint8)
    n = blocks.size // 17 * 32
    y = np.empty(n, np.float32)
    lib().dsx_ref_mxfp4_dequant_ggml(_p(blocks), _p(y), n)
    return y


def mxfp4_dequant_v2(rows: np.ndarray, n_rows: int, cols: int) -> np.ndarray:
    rows = _c(rows, np.uint8)
    assert rows.size == n_rows * (cols // 256) * SUPER
    y = np.empty((n_rows, cols), np.float32)
    lib().dsx_ref_mxfp4_dequant_v2(_p(rows), _p(y), n_rows, cols)
    return y


def mxfp4_repack_hf_to_v2(packed: np.ndarray, scale: np.ndarray) -> np.ndarray:
    packed, scale = _c(packed, np.uint8), _c(scale, np.uint8)
    out, nb = scale.shape
    dst = np.empty(out * nb * 17, np.uint8)
    lib().dsx_ref_mxfp4_repack_hf_to_v2(_p(packed), _p(scale), _p(dst), out, nb)
    return dst


def mxfp4_unpack_v2_to_hf(src: np.ndarray, out: int, nb: int):
    src = _c(src, np.uint8)
    packed = np.empty((out, nb * 16), np.uint8)
    scale = np.empty((out, nb), np.uint8)
    lib().dsx_ref_mxfp4_unpack_v2_to_hf(_p(src), _p(packed), _p(scale), out, nb)
    return packed, scale


def mxfp4_quantize_v2(x: np.ndarray) -> np.ndarray:
    x = _c(x, np.float32)
    n_rows, cols = x.shape
    dst = np.empty(n_rows * (cols // 256) * SUPER, np.uint8)
    lib().dsx_ref_mxfp4_quantize_v2(_p(x), _p(dst), n_rows, cols)
    return dst


def q8_0_quantize_block(x32: np.ndarray) -> np.ndarray:
    x32 = _c(x32, np.float32)
    out = np.empty(34, np.uint8)
    lib().dsx_ref_q8_0_quantize_block(_p(x32), _p(out))
    return out


def q8_0_quantize_rows(x: np.ndarray) -> np.ndarray:
    x = _c(x, np.float32)
    n_rows, cols = x.shape
    dst = np.empty(n_rows * (cols // 32) * 34, np.uint8)
    lib().dsx_ref_q8_0_quantize_rows(_p(x), _p(dst), n_rows, cols)
    return dst


def q8_0_repack_rows(ggml: np.ndarray, n_rows: int, blocks: int) -> np.ndarray:
    """ggml blocks [d f16 | 32 i8] -> engine rows [blocks x d | blocks x 32 i8]
    (crates/v4flash-kernels/src/weights.rs:225-240)."""
    ggml = _c(ggml, np.uint8)
    dst = np.empty(n_rows * blocks * 34, np.uint8)
    lib().dsx_ref_q8_0_repack_rows(_p(ggml), _p(dst), n_rows, blocks)
    return dst


SRC_F32, SRC_BF16, SRC_F8E4M3 = 0, 1, 2


def q8_0_from_hf(src: np.ndarray, scale: Optional[np.ndarray], dtype: int) -> np.ndarray:
    """A checkpoint matrix (f32, bf16 bits as uint16, or fp8-e4m3 codes as uint8 with an E8M0
    scale grid) -> ggml Q8_0 blocks (crates/v4flash-core/src/hf_v41.rs:728-805).  Raises where
    the reference returns Err."""
    want = {SRC_F32: np.float32, SRC_BF16: np.uint16, SRC_F8E4M3: np.uint8}[dtype]
    src = _c(src, want)
    out, inn = src.shape
    sr = sc = 0
    if scale is not None:
        scale = _c(scale, np.uint8)
        sr, sc = scale.shape
    dst = np.empty(out * (inn // 32) * 34, np.uint8)
    if lib().dsx_ref_q8_0_from_hf(_p(src), _p(scale), dtype, out, inn, sr, sc, _p(dst)) != 0:
        raise ValueError("q8_0_from_hf: the reference refuses this input")
    return dst


def q8_0_dequant_rows(rows: np.ndarray, n_rows: int, cols: int) -> np.ndarray:
    rows = _c(rows, np.uint8)
    y = np.empty((n_rows, cols), np.float32)
    lib().dsx_ref_q8_0_dequant_rows(_p(rows), _p(y), n_rows, cols)
    return y


def q8_0_quantize_act(x: np.ndarray):
    x = _c(x, np.float32).reshape(-1)
    blocks = x.size // 32
    xq = np.empty(x.size, np.int8)
    xs = np.empty(blocks, np.float32)
    lib().dsx_ref_q8_0_quantize_act(_p(x), _p(xq), _p(xs), blocks)
    return xq, xs


def dot_q8_0(wrow: np.ndarray, xq: np.ndarray, xscale: np.ndarray) -> float:
    wrow, xq, xscale = _c(wrow, np.uint8), _c(xq, np.int8), _c(xscale, np.float32)
    return float(lib().dsx_ref_dot_q8_0(xscale.size, _p(wrow), _p(xq), _p(xscale)))


def q8k_quantize(x: np.ndarray) -> np.ndarray:
    x = _c(x, np.float32).reshape(-1)
    nb = x.size // 256
    out = np.empty(nb * Q8K_BLOCK, np.uint8)
    lib().dsx_ref_q8k_quantize(_p(x), _p(out), nb)
    return out


def q8k_dequant(blocks: np.ndarray) -> np.ndarray:
    blocks = _c(blocks, np.uint8)
    nb = blocks.size // Q8K_BLOCK
    y = np.empty(nb * 256, np.float32)
    lib().dsx_ref_q8k_dequant(_p(blocks), _p(y), nb)
    return y


def dot_mxfp4_q8k(w: np.ndarray, y: np.ndarray) -> float:
    w, y = _c(w, np.uint8), _c(y, np.uint8)
    n_super = w.size // SUPER
    assert y.size == n_super * Q8K_BLOCK
    return float(lib().dsx_ref_dot_mxfp4_q8k(n_super, _p(w), _p(y)))


def swiglu(g: float, u: float, clamp: float, ew: float) -> float:
    return float(lib().dsx_ref_swiglu(g, u, clamp, ew))


def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    x, weight = _c(x, np.float32), _c(weight, np.float32)
    rows, n = x.shape
    out = np.empty_like(x)
    lib().dsx_ref_rms_norm(_p(out), _p(x), _p(weight), n, eps, rows)
    return out


def hc_post(block_out, residual_hc, post, comb, add1=None, add2=None) -> np.ndarray:
    """crates/v4flash-kernels/kernels/hc_post.hip:15-34,40-64,100-141.  block_out [b, n_embd],
    residual_hc [b, n_hc, n_embd], post [b, n_hc], comb [b, n_hc, n_hc] addressed
    [dst + src * n_hc] (so comb[t, src, dst] as a numpy array) -> out_hc [b, n_hc, n_embd]."""
    block_out, residual_hc = _c(block_out, np.float32), _c(residual_hc, np.float32)
    post, comb = _c(post, np.float32), _c(comb, np.float32)
    b, n_hc, n_embd = residual_hc.shape
    assert block_out.shape == (b, n_embd) and post.shape == (b, n_hc) and comb.shape == (b, n_hc, n_hc)
    add1 = None if add1 is None else _c(add1, np.float32)
    add2 = None if add2 is None else _c(add2, np.float32)
    out = np.empty_like(residual_hc)
    lib().dsx_ref_hc_post(_p(out), _p(block_out), _p(add1), _p(add2), _p(residual_hc), _p(post),
                          _p(comb), n_embd, n_hc, b, n_hc, n_hc * n_hc)
    return out


def hc_post_from_split(block_out, residual_hc, split, n_w, add1=None, add2=None) -> np.ndarray:
    """crates/v4flash-kernels/kernels/hc_post.hip:66-98: post and comb read from the packed row
    split[b, n_w + n_hc + n_hc * n_hc] (post at n_w, comb behind it)."""
    block_out, residual_hc, split = _c(block_out, np.float32), _c(residual_hc, np.float32), _c(split, np.float32)
    b, n_hc, n_embd = residual_hc.shape
    stride = n_w + n_hc + n_hc * n_hc
    assert split.shape == (b, stride)
    add1 = None if add1 is None else _c(add1, np.float32)
    add2 = None if add2 is None else _c(add2, np.float32)
    out = np.empty_like(residual_hc)
    flat = split.reshape(-1)
    lib().dsx_ref_hc_post(_p(out), _p(block_out), _p(add1), _p(add2), _p(residual_hc),
                          _p(flat[n_w:]), _p(flat[n_w + n_hc:]), n_embd, n_hc, b, stride, stride)
    return out


# ---- router ------------------------------------------------------------------

def router_topk(logits, bias, n_used, scale, eps, mode, n_group=1, topk_group=1):
    logits = _c(logits, np.float32)
    T, E = logits.shape
    bias = None if bias is None else _c(bias, np.float32)
    sel = np.empty((T, n_used), np.int32)
    w = np.empty((T, n_used), np.float32)
    rc = lib().dsx_ref_router_topk(_p(sel), _p(w), _p(logits), _p(bias), E, n_used, scale, eps,
                                   T, mode, n_group, topk_group)
    if rc != 0:
        raise ValueError(f"dsx_ref_router_topk rc={rc}")
    return sel, w


def router_hash_select(logits, tid2eid, token_ids, scale=1.5, eps=6.103515625e-5):
    """crates/v4flash-kernels/src/routing.rs:21-44: picks from the token's row of tid2eid."""
    logits = _c(logits, np.float32)
    tid2eid = _c(tid2eid, np.int32)
    token_ids = _c(token_ids, np.int32)
    T, E = logits.shape
    vocab, n_used = tid2eid.shape
    assert token_ids.shape == (T,)
    sel = np.empty((T, n_used), np.int32)
    w = np.empty((T, n_used), np.float32)
    lib().dsx_ref_router_hash_select(_p(sel), _p(w), _p(logits), _p(tid2eid), _p(token_ids), E,
                                     n_used, vocab, scale, eps, T)
    return sel, w


def hetsplit_select(selected, remap, mode, cap):
    """Per-slot expert index of one side of the reference's het-split, -1 where the slot is the
    other side's (crates/v4flash-kernels/kernels/mxfp4_pair_matvec.hip:231-284)."""
    selected = _c(selected, np.int32)
    remap = _c(remap, np.int32)
    T, k = selected.shape
    out = np.empty((T, k), np.int32)
    lib().dsx_ref_hetsplit_select(_p(out), _p(selected), _p(remap), mode, cap, k, remap.size, T)
    return out


def router_scores(logits, bias, mode, n_group=1, topk_group=1):
    logits = _c(logits, np.float32)
    T, E = logits.shape
    bias = None if bias is None else _c(bias, np.float32)
    p = np.empty((T, E), np.float32)
    s = np.empty((T, E), np.float32)
    rc = lib().dsx_ref_router_scores(_p(p), _p(s), _p(logits), _p(bias), E, T, mode, n_group,
                                     topk_group)
    if rc != 0:
        raise ValueError(f"dsx_ref_router_scores rc={rc}")
    return p, s


def router_logits(w: np.ndarray, x: np.ndarray) -> np.ndarray:
    w, x = _c(w, np.float32), _c(x, np.float32)
    E, H = w.shape
    T = x.shape[0]
    out = np.empty((T, E), np.float32)
    lib().dsx_ref_router_logits(_p(out), _p(w), _p(x), E, H, T)
    return out


def group_build(selected: np.ndarray, n_expert: int, chunk: int):
    selected = _c(selected, np.int32)
    T, k = selected.shape
    gc = np.empty(n_expert, np.int32)
    off = np.empty(n_expert + 1, np.int32)
    mem = np.zeros(T * k, np.int32)
    wi = np.zeros(n_expert + T * k, np.int32)
    n = lib().dsx_ref_group_build(_p(gc), _p(off), _p(mem), _p(wi), _p(selected), T, k,
                                  n_expert, chunk)
    return gc, off, mem[: off[-1]], wi[:n]


def wi_upper_bound(members: int, groups: int, chunk: int, cap: int) -> int:
    return int(lib().dsx_ref_wi_upper_bound(members, groups, chunk, cap))


# ---- the layer ---------------------------------------------------------------

@dataclass
class MoeWeights:
    """Host copies of one layer's expert tensors in engine layout."""
    hidden: int
    inter: int
    n_expert: int
    n_used: int
    gate: np.ndarray
    up: np.ndarray
    down: np.ndarray
    gate_fmt: int = FMT_MXFP4
    up_fmt: int = FMT_MXFP4
    down_fmt: int = FMT_MXFP4
    clamp: float = 0.0
    sh_inter: int = 0
    sh_gate: Optional[np.ndarray] = None
    sh_up: Optional[np.ndarray] = None
    sh_down: Optional[np.ndarray] = None
    sh_gate_fmt: int = FMT_MXFP4
    sh_up_fmt: int = FMT_MXFP4
    sh_down_fmt: int = FMT_MXFP4
    sh_clamp: float = 0.0


def matrix_bytes(fmt: int, rows: int, cols: int) -> int:
    return rows * (cols // 256) * SUPER if fmt == FMT_MXFP4 else rows * (cols // 32) * 34


def moe_forward(w: MoeWeights, x, selected, weights, n_threads: int = 0, want_parts=False):
    x = _c(x, np.float32)
    T = x.shape[0]
    selected = _c(selected, np.int32).reshape(T, w.n_used)
    weights = _c(weights, np.float32).reshape(T, w.n_used)
    cfg = _Cfg()
    cfg.hidden, cfg.inter, cfg.n_expert, cfg.n_used = w.hidden, w.inter, w.n_expert, w.n_used
    cfg.gate_fmt, cfg.up_fmt, cfg.down_fmt = w.gate_fmt, w.up_fmt, w.down_fmt
    keep = [_c(w.gate, np.uint8), _c(w.up, np.uint8), _c(w.down, np.uint8)]
    cfg.gate, cfg.up, cfg.down = (a.ctypes.data for a in keep)
    cfg.gate_bpe = matrix_bytes(w.gate_fmt, w.inter, w.hidden)
    cfg.up_bpe = matrix_bytes(w.up_fmt, w.inter, w.hidden)
    cfg.down_bpe = matrix_bytes(w.down_fmt, w.hidden, w.inter)
    cfg.clamp = w.clamp
    cfg.sh_inter = w.sh_inter
    if w.sh_inter:
        sh = [_c(w.sh_gate, np.uint8), _c(w.sh_up, np.uint8), _c(w.sh_down, np.uint8)]
        keep += sh
        cfg.sh_gate, cfg.sh_up, cfg.sh_down = (a.ctypes.data for a in sh)
        cfg.sh_gate_fmt, cfg.sh_up_fmt, cfg.sh_down_fmt = w.sh_gate_fmt, w.sh_up_fmt, w.sh_down_fmt
        cfg.sh_clamp = w.sh_clamp
    out = np.empty((T, w.hidden), np.float32)
    mid = np.empty((T, w.n_used, w.inter), np.float32) if want_parts else None
    moe = np.empty((T, w.hidden), np.float32) if want_parts else None
    shared = np.zeros((T, w.hidden), np.float32) if want_parts else None
    rc = lib().dsx_ref_moe_forward(C.byref(cfg), _p(x), _p(selected), _p(weights), T, _p(out),
                                   _p(mid), _p(moe), _p(shared), n_threads)
    if rc != 0:
        raise ValueError(f"dsx_ref_moe_forward rc={rc}")
    if want_parts:
        return out, mid, moe, shared
    return out


def max_threads() -> int:
    return int(lib().dsx_ref_max_threads())
