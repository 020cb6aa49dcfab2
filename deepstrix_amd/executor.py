"""The whole MoE layer behind one object, modelled on the reference's `MoeExecutor`
(crates/v4flash-kernels/src/het/remote_experts.rs:7432-7443): it records device pointers and
dimensions, owns the scratch, and `run` produces f32 [T, hidden].  The sequencing itself
lives in the library (dsx_moe_layer_forward); this class only holds the buffers.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional

import torch

from . import capi
from .capi import FMT_MXFP4, FMT_MXFP4_PLANAR, LayerDesc, check, lib
from .dispatch import matrix_bytes, mxfp4_rows_to_planar


@dataclass
class LayerWeights:
    """Device tensors (uint8) in engine layout; `RoutedExpertWeights` in the reference
    (crates/v4flash-kernels/src/model_weights.rs:41-54)."""
    hidden: int
    inter: int
    n_expert: int
    n_used: int
    gate: torch.Tensor
    up: torch.Tensor
    down: torch.Tensor
    gate_fmt: int = FMT_MXFP4
    up_fmt: int = FMT_MXFP4
    down_fmt: int = FMT_MXFP4
    clamp: float = 0.0
    router_mode: int = capi.ROUTER_SIGMOID
    n_group: int = 1
    topk_group: int = 1
    route_scale: float = 1.0
    route_eps: float = 1e-20
    bias: Optional[torch.Tensor] = None
    sh_inter: int = 0
    sh_gate: Optional[torch.Tensor] = None
    sh_up: Optional[torch.Tensor] = None
    sh_down: Optional[torch.Tensor] = None
    sh_gate_fmt: int = FMT_MXFP4
    sh_up_fmt: int = FMT_MXFP4
    sh_down_fmt: int = FMT_MXFP4
    sh_clamp: float = 0.0
    # pre-norm block (chained layers): RMSNorm weight [hidden], router matrix f32 [n_expert, hidden]
    norm_w: Optional[torch.Tensor] = None
    norm_eps: float = 1e-6
    router_w: Optional[torch.Tensor] = None


    def to_planar(self) -> "LayerWeights":
        """Rewrites every MXFP4 tensor in place into the planar form (FMT_MXFP4_PLANAR: same bytes
        in another order, same results; the grouped GEMMs read it faster) and returns self."""
        def conv(t, fmt, rows, cols, n):
            if fmt != FMT_MXFP4:
                return fmt
            mxfp4_rows_to_planar(t, rows, cols, n)
            return FMT_MXFP4_PLANAR
        self.gate_fmt = conv(self.gate, self.gate_fmt, self.inter, self.hidden, self.n_expert)
        self.up_fmt = conv(self.up, self.up_fmt, self.inter, self.hidden, self.n_expert)
        self.down_fmt = conv(self.down, self.down_fmt, self.hidden, self.inter, self.n_expert)
        if self.sh_inter:
            self.sh_gate_fmt = conv(self.sh_gate, self.sh_gate_fmt, self.sh_inter, self.hidden, 1)
            self.sh_up_fmt = conv(self.sh_up, self.sh_up_fmt, self.sh_inter, self.hidden, 1)
            self.sh_down_fmt = conv(self.sh_down, self.sh_down_fmt, self.hidden, self.sh_inter, 1)
        return self


class MoeLayer:
    # Set by a test-suite whose small shapes stand in for the paths of a large one: layers with
    # fewer experts than this get fixed token thresholds (decode path up to 16 tokens, grouped
    # GEMM from 100; planar: 11 / 17 / narrow tile below 14 picks), so that a token count names the
    # same path on every small shape.  None (the default): the library's own, shape-derived
    # thresholds.
    v3_thresholds_below_experts: Optional[int] = None

    def __init__(self, w: LayerWeights, max_tokens: int):
        capi.init()
        self.w = w
        self.max_tokens = max_tokens
        d = LayerDesc()
        d.hidden, d.inter, d.n_expert, d.n_used = w.hidden, w.inter, w.n_expert, w.n_used
        d.gate_fmt, d.up_fmt, d.down_fmt = w.gate_fmt, w.up_fmt, w.down_fmt
        d.gate, d.up, d.down = w.gate.data_ptr(), w.up.data_ptr(), w.down.data_ptr()
        d.gate_bpe = matrix_bytes(w.gate_fmt, w.inter, w.hidden)
        d.up_bpe = matrix_bytes(w.up_fmt, w.inter, w.hidden)
        d.down_bpe = matrix_bytes(w.down_fmt, w.hidden, w.inter)
        for name, t, bpe in (("gate", w.gate, d.gate_bpe), ("up", w.up, d.up_bpe),
                             ("down", w.down, d.down_bpe)):
            if t.numel() * t.element_size() != bpe * w.n_expert:
                raise ValueError(f"{name}: {t.numel() * t.element_size()} bytes, expected "
                                 f"{bpe * w.n_expert}")
        d.clamp = w.clamp
        d.router_mode, d.n_group, d.topk_group = w.router_mode, w.n_group, w.topk_group
        d.route_scale, d.route_eps = w.route_scale, w.route_eps
        d.bias = w.bias.data_ptr() if w.bias is not None else None
        d.sh_inter = w.sh_inter
        if w.sh_inter:
            d.sh_gate_fmt, d.sh_up_fmt, d.sh_down_fmt = w.sh_gate_fmt, w.sh_up_fmt, w.sh_down_fmt
            d.sh_gate, d.sh_up, d.sh_down = (w.sh_gate.data_ptr(), w.sh_up.data_ptr(),
                                             w.sh_down.data_ptr())
            d.sh_clamp = w.sh_clamp
        self._desc = d
        h = C.c_void_p()
        check(lib().dsx_moe_layer_create(C.byref(d), C.byref(h)))
        self._h = h
        self._pin_v3_thresholds()
        self.workspace_bytes = int(lib().dsx_moe_layer_workspace_bytes(h, max_tokens))
        self.workspace = torch.empty(self.workspace_bytes, dtype=torch.uint8, device=w.gate.device)

    def _pin_v3_thresholds(self):
        w, lim = self.w, MoeLayer.v3_thresholds_below_experts
        if lim is None or w.n_expert >= lim:
            return
        if w.gate_fmt == FMT_MXFP4_PLANAR and w.down_fmt == FMT_MXFP4_PLANAR:   # (a layer with a Q8_0 matrix keeps the rows' thresholds)
            self.set_tuning(gemm_min_tokens=17, decode_max_tokens=11, gemm_narrow_members=14)
        else:
            self.set_tuning(gemm_min_tokens=100, decode_max_tokens=16, gemm_narrow_members=1)

    def __del__(self):
        h = getattr(self, "_h", None)
        if h:
            self._h = None
            try:
                lib().dsx_moe_layer_destroy(h)
            except Exception:  # interpreter shutdown: the module globals are already gone
                pass

    def weights_to_planar(self):
        """Rewrites the layer's MXFP4 tensors (self.w's buffers) in place into the planar form and
        switches the layer over (include/dsx_moe.h: dsx_moe_layer_weights_to_planar)."""
        check(lib().dsx_moe_layer_weights_to_planar(self._h, torch.cuda.current_stream().cuda_stream))
        w = self.w
        for name in ("gate_fmt", "up_fmt", "down_fmt") + (("sh_gate_fmt", "sh_up_fmt", "sh_down_fmt") if w.sh_inter else ()):
            if getattr(w, name) == FMT_MXFP4:
                setattr(w, name, FMT_MXFP4_PLANAR)
        self._pin_v3_thresholds()

    def weights_to_rows(self):
        check(lib().dsx_moe_layer_weights_to_rows(self._h, torch.cuda.current_stream().cuda_stream))
        w = self.w
        for name in ("gate_fmt", "up_fmt", "down_fmt") + (("sh_gate_fmt", "sh_up_fmt", "sh_down_fmt") if w.sh_inter else ()):
            if getattr(w, name) == FMT_MXFP4_PLANAR:
                setattr(w, name, FMT_MXFP4)
        self._pin_v3_thresholds()

    def set_profile_events(self, gate_up_begin=None, gate_up_end=None, down_end=None):
        """hipEvent_t handles (ints) recorded around the gate/up launch and after down."""
        check(lib().dsx_moe_layer_set_profile_events(self._h, gate_up_begin, gate_up_end, down_end))

    def set_tuning(self, by_expert_chunk: int = 0, gemm_min_tokens: int = 0, decode_max_tokens: int = 0,
                   gemm_narrow_members: int = 0):
        """0 keeps the current value (include/dsx_moe.h: dsx_moe_layer_set_tuning)."""
        check(lib().dsx_moe_layer_set_tuning(self._h, by_expert_chunk, gemm_min_tokens,
                                             decode_max_tokens, gemm_narrow_members))

    def tuning(self) -> dict:
        """The thresholds in force (include/dsx_moe.h: dsx_moe_layer_get_tuning)."""
        v = (C.c_uint32 * 6)()
        check(lib().dsx_moe_layer_get_tuning(self._h, C.byref(v)))
        return dict(zip(("by_expert_chunk", "gemm_min_tokens", "gemm_q8_min_tokens", "decode_max_tokens",
                         "gemm_narrow_members", "share_min_tokens"), (int(x) for x in v)))

    def set_decode(self, fused: int = 0, spin_limit: int = 0):
        """fused: 1 = one launch for gate/up + down, pairing tokens that name one expert from 4
        tokens on (default), 3 = never pairing, 4 = pairing from 2 tokens on, 2 = one launch per
        stage; spin_limit: bound of the in-kernel waits (include/dsx_moe.h: dsx_moe_layer_set_decode)."""
        check(lib().dsx_moe_layer_set_decode(self._h, fused, spin_limit))

    def status(self, builtin_scratch: bool = False) -> int:
        """Status word of the last forward on this layer's workspace (0 = ok); synchronizes."""
        torch.cuda.synchronize()
        v = C.c_uint32(0xFFFFFFFF)
        check(lib().dsx_moe_layer_status(self._h, None if builtin_scratch else self.workspace.data_ptr(),
                                         C.byref(v)))
        return int(v.value)

    def block(self, h: torch.Tensor) -> torch.Tensor:
        """In place: h += layer(RMSNorm(h)), router logits = router_w . RMSNorm(h)
        (include/dsx_moe.h: dsx_moe_block_forward)."""
        T = h.shape[0]
        if T > self.max_tokens:
            raise ValueError(f"{T} tokens > max_tokens={self.max_tokens}")
        w = self.w
        if w.norm_w is None or w.router_w is None:
            raise ValueError("block() needs norm_w and router_w")
        if w.router_w.dtype == torch.float16:
            fn = lib().dsx_moe_block_forward_f16
        elif w.router_w.dtype == torch.float32:
            fn = lib().dsx_moe_block_forward
        else:
            raise TypeError(f"router_w must be float32 or float16, got {w.router_w.dtype}")
        check(fn(
            self._h, torch.cuda.current_stream().cuda_stream, h.data_ptr(), w.norm_w.data_ptr(),
            w.norm_eps, w.router_w.data_ptr(), T, self.workspace.data_ptr(), self.workspace_bytes))
        return h

    def run(self, x: torch.Tensor, logits: Optional[torch.Tensor] = None, out=None,
            selected_in=None, weights_in=None, want_routing=False):
        """x f32 [T, hidden], logits f32 [T, n_expert] -> out f32 [T, hidden]."""
        T = x.shape[0]
        if T > self.max_tokens:
            raise ValueError(f"{T} tokens > max_tokens={self.max_tokens}")
        assert x.dtype == torch.float32 and x.is_contiguous()
        if out is None:
            out = torch.empty((T, self.w.hidden), dtype=torch.float32, device=x.device)
        sel_out = w_out = None
        if want_routing:
            sel_out = torch.empty((T, self.w.n_used), dtype=torch.int32, device=x.device)
            w_out = torch.empty((T, self.w.n_used), dtype=torch.float32, device=x.device)
        p = lambda t: None if t is None else t.data_ptr()
        check(lib().dsx_moe_layer_forward(
            self._h, torch.cuda.current_stream().cuda_stream, p(out), p(x), p(logits), T,
            p(self.workspace), self.workspace_bytes, p(sel_out), p(w_out), p(selected_in),
            p(weights_in)))
        if want_routing:
            return out, sel_out, w_out
        return out

    def run_hc(self, x: torch.Tensor, logits: Optional[torch.Tensor], hc, selected_in=None,
               weights_in=None, want_routing=False):
        """`run` whose result goes through the hyper-connection combine `hc` (a capi.HcPostDesc,
        see dispatch.hc_post_desc) instead of to an output buffer (dsx_moe_layer_forward_hc)."""
        T = x.shape[0]
        if T > self.max_tokens:
            raise ValueError(f"{T} tokens > max_tokens={self.max_tokens}")
        assert x.dtype == torch.float32 and x.is_contiguous()
        sel_out = w_out = None
        if want_routing:
            sel_out = torch.empty((T, self.w.n_used), dtype=torch.int32, device=x.device)
            w_out = torch.empty((T, self.w.n_used), dtype=torch.float32, device=x.device)
        p = lambda t: None if t is None else t.data_ptr()
        check(lib().dsx_moe_layer_forward_hc(
            self._h, torch.cuda.current_stream().cuda_stream, C.byref(hc), p(x), p(logits), T,
            p(self.workspace), self.workspace_bytes, p(sel_out), p(w_out), p(selected_in),
            p(weights_in)))
        return (sel_out, w_out) if want_routing else None

    def run_noalloc(self, x: torch.Tensor, logits: Optional[torch.Tensor], out: torch.Tensor,
                    selected_in=None, weights_in=None, selected_out=None, weights_out=None):
        """`run` through dsx_moe_layer_forward_noalloc: the library's built-in scratch array
        instead of this object's workspace, every buffer supplied by the caller.  Refused
        (DsxError, ERR_UNSUPPORTED) when the token count needs more scratch than the array."""
        T = x.shape[0]
        assert x.dtype == torch.float32 and x.is_contiguous() and out.is_contiguous()
        p = lambda t: None if t is None else t.data_ptr()
        check(lib().dsx_moe_layer_forward_noalloc(
            self._h, torch.cuda.current_stream().cuda_stream, p(out), p(x), p(logits), T,
            p(selected_out), p(weights_out), p(selected_in), p(weights_in)))
        return out


class MoeChain:
    """A stack of pre-norm residual MoE blocks run back to back on one stream, optionally
    replayed from a HIP graph (launch-bound at small token counts).  The counterpart of the
    reference's per-layer loop around `issue_igpu_moe`
    (crates/v4flash-kernels/src/het/forward_layer.rs:424-466)."""

    def __init__(self, weights, max_tokens: int):
        self.layers = [MoeLayer(w, max_tokens) for w in weights]
        self.max_tokens = max_tokens
        self._graph = None
        self._static_h = None

    def step(self, h: torch.Tensor) -> torch.Tensor:
        """In place over all layers."""
        for layer in self.layers:
            layer.block(h)
        return h

    def capture(self, n_tokens: int) -> None:
        """Records one step for `n_tokens` tokens into a graph; `replay` then runs it."""
        hidden = self.layers[0].w.hidden
        self._static_h = torch.zeros((n_tokens, hidden), dtype=torch.float32, device="cuda")
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):   # warm-up outside the capture
            self.step(self._static_h)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self._static_h.zero_()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            self.step(self._static_h)
        self._graph = g

    def replay(self, h: torch.Tensor) -> torch.Tensor:
        """One captured step on a copy of h; returns the graph's output buffer (valid until
        the next replay)."""
        self._static_h.copy_(h)
        self._graph.replay()
        return self._static_h
