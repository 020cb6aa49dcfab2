"""Per-operator entry points, named and ordered like the reference's `het::dispatch`
functions and launch wrappers.  Arguments are torch tensors on the GPU (torch only owns the
memory and the stream); every call goes straight through the C ABI.

Reference counterparts (paths relative to the reference tree):
  router_topk .............. crates/v4flash-kernels/src/router_topk.rs:245-364
  q8k_quantize ............. crates/v4flash-kernels/src/q8_k.rs:33-104
  moe_gate_up_batch ........ crates/v4flash-kernels/src/het/dispatch.rs:26-66
  moe_down_batched ......... crates/v4flash-kernels/src/het/dispatch.rs:121-150
  moe_group_build .......... crates/v4flash-kernels/src/moe_group_builder.rs:72-130
  moe_gate_up_chunked_rows . crates/v4flash-kernels/src/het/dispatch.rs:534-570
  moe_down_by_expert ....... crates/v4flash-kernels/src/het/dispatch.rs:580-620
  moe_reduce_partials ...... crates/v4flash-kernels/src/q2_k.rs:454-500
"""
from __future__ import annotations

from typing import Optional

import torch

from . import capi
from .capi import FMT_MXFP4, FMT_MXFP4_PLANAR, FMT_Q8_0, check, lib


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _p(t: Optional[torch.Tensor]) -> Optional[int]:
    if t is None:
        return None
    assert t.is_cuda and t.is_contiguous(), "device-resident contiguous tensors only"
    return t.data_ptr()


def wi_upper_bound(members: int, groups: int, chunk: int) -> int:
    """crates/v4flash-kernels/src/het/dispatch.rs:450-454"""
    g = min(members, groups)
    return min(members, g + -(-members // max(chunk, 1)))


def router_topk(selected, weights, logits, bias, n_expert, n_used, scale, eps, b, mode,
                n_group=1, topk_group=1):
    capi.init()
    check(lib().dsx_router_topk(_stream(), _p(selected), _p(weights), _p(logits), _p(bias),
                                n_expert, n_used, scale, eps, b, mode, n_group, topk_group))


def router_hash_select(selected, weights, logits, tid2eid, token_ids, scale=1.5, eps=6.103515625e-5):
    """crates/v4flash-kernels/src/routing.rs:21-44, on the device (no logits readback)."""
    capi.init()
    b, n_expert = logits.shape
    vocab, n_used = tid2eid.shape
    check(lib().dsx_router_hash_select(_stream(), _p(selected), _p(weights), _p(logits), _p(tid2eid),
                                       _p(token_ids), n_expert, n_used, vocab, scale, eps, b))


def moe_hetsplit_select(selected_side, selected, remap, mode, cap):
    """One side's picks under the reference's het-split rule
    (crates/v4flash-kernels/kernels/mxfp4_pair_matvec.hip:231-284); -1 = not this side's."""
    capi.init()
    b, n_used = selected.shape
    check(lib().dsx_moe_hetsplit_select(_stream(), _p(selected_side), _p(selected), _p(remap), mode,
                                        cap, n_used, remap.numel(), b))


def router_logits(logits, router_w, x, n_expert, hidden, n_tokens):
    """crates/v4flash-kernels/kernels/laguna_ops.hip:57-60 (f32 W . x); f16 router weights as
    crates/v4flash-kernels/src/f16.rs:37-45 keeps them take the f16 entry point."""
    capi.init()
    if router_w.dtype == torch.float16:
        fn = lib().dsx_router_logits_f16
    elif router_w.dtype == torch.float32:
        fn = lib().dsx_router_logits
    else:
        raise TypeError(f"router_w must be float32 or float16, got {router_w.dtype}")
    check(fn(_stream(), _p(logits), _p(router_w), _p(x), n_expert, hidden, n_tokens))


def q8k_quantize(out, x, n_blocks):
    capi.init()
    check(lib().dsx_q8k_quantize(_stream(), _p(out), _p(x), n_blocks))


def q8_0_quantize(xq, xscale, x, blocks):
    capi.init()
    check(lib().dsx_q8_0_quantize(_stream(), _p(xq), _p(xscale), _p(x), blocks))


def q8_0_quantize_rows(out, x, rows, k):
    capi.init()
    check(lib().dsx_q8_0_quantize_rows(_stream(), _p(out), _p(x), rows, k))


def moe_gate_up_batch(dt, mid, gate, up, xq, ew, selected, gbpe, ubpe, n_used, clamp, n_rows,
                      n_blocks):
    capi.init()
    check(lib().dsx_moe_gate_up_batch(_stream(), dt, _p(mid), _p(gate), _p(up), _p(xq), _p(ew),
                                      _p(selected), gbpe, ubpe, n_used, clamp, n_rows, n_blocks))


def moe_down_batched(dt, out, down, xq, selected, dbpe, xq_slot_stride, n_used, n_rows,
                     n_blocks_in):
    capi.init()
    check(lib().dsx_moe_down_batched(_stream(), dt, _p(out), _p(down), _p(xq), _p(selected), dbpe,
                                     xq_slot_stride, n_used, n_rows, n_blocks_in))


def moe_group_build(group_count, group_offset, expert_members, work_items, n_work_items,
                    selected, b, n_used, n_expert, chunk):
    capi.init()
    check(lib().dsx_moe_group_build(_stream(), _p(group_count), _p(group_offset),
                                    _p(expert_members), _p(work_items), _p(n_work_items),
                                    _p(selected), b, n_used, n_expert, chunk))


def moe_gate_up_chunked_rows(dt, mid, gate, up, xq, ew, group_count, group_offset, expert_members,
                             work_items, n_work_items, max_work_items, gbpe, ubpe, n_used, chunk,
                             clamp, n_rows, n_blocks):
    capi.init()
    check(lib().dsx_moe_gate_up_chunked_rows(
        _stream(), dt, _p(mid), _p(gate), _p(up), _p(xq), _p(ew), _p(group_count), _p(group_offset),
        _p(expert_members), _p(work_items), _p(n_work_items), max_work_items, gbpe, ubpe, n_used,
        chunk, clamp, n_rows, n_blocks))


def moe_down_by_expert(dt, partials, down, xq, group_count, group_offset, expert_members,
                       work_items, n_work_items, max_work_items, dbpe, xq_slot_stride, n_used,
                       chunk, n_rows, n_blocks_in):
    capi.init()
    check(lib().dsx_moe_down_by_expert(
        _stream(), dt, _p(partials), _p(down), _p(xq), _p(group_count), _p(group_offset),
        _p(expert_members), _p(work_items), _p(n_work_items), max_work_items, dbpe,
        xq_slot_stride, n_used, chunk, n_rows, n_blocks_in))


def moe_reduce_partials(out, partials, selected, n_used, n_rows, b):
    capi.init()
    check(lib().dsx_moe_reduce_partials(_stream(), _p(out), _p(partials), _p(selected), n_used,
                                        n_rows, b))


def dense_ffn_scratch_bytes(b, hidden, inter) -> int:
    return int(lib().dsx_dense_ffn_scratch_bytes(b, hidden, inter))


def dense_ffn(gate_fmt, up_fmt, down_fmt, out, gate, up, down, x, b, hidden, inter, clamp,
              scratch, accumulate=False):
    capi.init()
    check(lib().dsx_dense_ffn(_stream(), gate_fmt, up_fmt, down_fmt, _p(out), _p(gate), _p(up),
                              _p(down), _p(x), b, hidden, inter, clamp, int(accumulate),
                              _p(scratch)))


def vec_add_inplace(out, rhs, n):
    capi.init()
    check(lib().dsx_vec_add_inplace(_stream(), _p(out), _p(rhs), n))


def hc_post_desc(out_hc, residual_hc, post, comb, n_hc, post_stride=None, comb_stride=None) -> capi.HcPostDesc:
    """dsx_hc_post_desc over device tensors; strides default to separate [b, n_hc] / [b, n_hc, n_hc]
    arrays (pass both as n_w + n_hc + n_hc * n_hc for views into the engine's packed split rows)."""
    d = capi.HcPostDesc()
    d.out_hc, d.residual_hc, d.post, d.comb = _p(out_hc), _p(residual_hc), _p(post), _p(comb)
    d.n_hc = n_hc
    d.post_stride = n_hc if post_stride is None else post_stride
    d.comb_stride = n_hc * n_hc if comb_stride is None else comb_stride
    return d


def hc_post(desc: capi.HcPostDesc, block_out, n_embd, b, add1=None, add2=None):
    """HcPost::launch* (crates/v4flash-kernels/kernels/hc_post.hip:15-141)."""
    import ctypes as C
    capi.init()
    check(lib().dsx_hc_post(_stream(), C.byref(desc), _p(block_out), _p(add1), _p(add2), n_embd, b))


def rms_norm(out, x, weight, n, eps, rows):
    capi.init()
    check(lib().dsx_rms_norm(_stream(), _p(out), _p(x), _p(weight), n, eps, rows))


def swiglu_clamp_weighted(mid, gate, up, expert_w, clamp, ff, n_experts):
    capi.init()
    check(lib().dsx_swiglu_clamp_weighted(_stream(), _p(mid), _p(gate), _p(up), _p(expert_w), clamp,
                                          ff, n_experts))


def mxfp4_repack_hf_to_v2(dst, packed, scale, out, nb):
    capi.init()
    check(lib().dsx_mxfp4_repack_hf_to_v2(_stream(), _p(dst), _p(packed), _p(scale), out, nb))


def q8_0_weights_from_hf(dst, src, scale, src_dtype, out_rows, in_cols, split_rows=True):
    """A checkpoint matrix (f32, bf16 or fp8-e4m3 + E8M0 scale grid) -> Q8_0 weights
    (crates/v4flash-core/src/hf_v41.rs:728-805; split rows as
    crates/v4flash-kernels/src/weights.rs:225-240 lays them out)."""
    capi.init()
    sr, sc = (scale.shape if scale is not None else (0, 0))
    check(lib().dsx_q8_0_weights_from_hf(_stream(), _p(dst), _p(src), _p(scale), src_dtype, out_rows,
                                         in_cols, sr, sc, 1 if split_rows else 0))


def q8_0_repack_rows(dst, src, num_rows, blocks_per_row):
    """crates/v4flash-kernels/src/weights.rs:225-240"""
    capi.init()
    check(lib().dsx_q8_0_repack_rows(_stream(), _p(dst), _p(src), num_rows, blocks_per_row))


def mxfp4_rows_to_planar(w, n_rows, cols, n_matrices=1, stride=None):
    """MXFP4 matrices in the engine's rows -> the planar form, in place (include/dsx_moe.h)."""
    capi.init()
    stride = n_rows * (cols // 256) * 136 if stride is None else stride
    check(lib().dsx_mxfp4_rows_to_planar(_stream(), _p(w), n_rows, cols, n_matrices, stride))


def mxfp4_planar_to_rows(w, n_rows, cols, n_matrices=1, stride=None):
    capi.init()
    stride = n_rows * (cols // 256) * 136 if stride is None else stride
    check(lib().dsx_mxfp4_planar_to_rows(_stream(), _p(w), n_rows, cols, n_matrices, stride))


def dequant_rows(dt, y, rows, n_rows, cols):
    capi.init()
    check(lib().dsx_dequant_rows(_stream(), dt, _p(y), _p(rows), n_rows, cols))


def matrix_bytes(fmt: int, rows: int, cols: int) -> int:
    """bytes_per_expert for one matrix (crates/v4flash-kernels/src/weight_contract.rs:146-158)."""
    if fmt in (FMT_MXFP4, FMT_MXFP4_PLANAR):
        return rows * (cols // 256) * 136
    if fmt == FMT_Q8_0:
        return rows * (cols // 32) * 34
    raise ValueError(f"format {fmt}")
