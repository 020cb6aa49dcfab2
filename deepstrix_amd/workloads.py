"""The synthetic workloads of the benchmark and the tests: layer shapes (the BASELINE configs),
seeded inputs on the host and the same layers generated on the device.  Everything here is a
pure function of a seed (see synth.py); nothing depends on a CPU reference."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import numpy as np

from . import synth
from .capi import FMT_MXFP4, FMT_Q8_0

ROUTER = {"sqrt_softplus": 0, "sigmoid": 1, "softmax": 2}


@dataclass
class Shape:
    hidden: int
    inter: int
    n_expert: int
    n_used: int
    gate_fmt: int = FMT_MXFP4
    down_fmt: int = FMT_MXFP4
    shared: bool = True
    sh_gate_fmt: Optional[int] = None
    sh_down_fmt: Optional[int] = None
    sh_inter: Optional[int] = None   # the shared expert's intermediate size (None: like the routed experts)
    clamp: float = 0.0
    router_mode: int = 1
    n_group: int = 1
    topk_group: int = 1
    route_scale: float = 1.0
    route_eps: float = 1e-20
    bias_sigma: float = 0.0
    seed: int = 0xD5EE0000

    @property
    def shg(self):
        return self.sh_gate_fmt if self.sh_gate_fmt is not None else self.gate_fmt

    @property
    def shd(self):
        return self.sh_down_fmt if self.sh_down_fmt is not None else self.down_fmt

    @property
    def shi(self):
        return self.sh_inter if self.sh_inter is not None else self.inter


# BASELINE configs
CFG1 = Shape(2048, 1408, 64, 6, FMT_Q8_0, FMT_Q8_0, router_mode=2, seed=0xD5EE0001)
CFG2 = Shape(7168, 2048, 256, 8, router_mode=1, n_group=8, topk_group=4, route_scale=2.5,
             bias_sigma=0.01, seed=0xD5EE0002)
CFG5 = Shape(7168, 2048, 256, 8, FMT_MXFP4, FMT_Q8_0, router_mode=1, route_scale=2.5,
             seed=0xD5EE0005)


def host_inputs(s: Shape, T: int, logit_shift: Optional[np.ndarray] = None):
    x = synth.normal_host(s.seed, synth.T_X, T * s.hidden).reshape(T, s.hidden)
    # BASELINE config 2: bf16 activations, converted to f32 exactly
    x = (x.view(np.uint32) & np.uint32(0xFFFF0000)).view(np.float32)
    logits = synth.normal_host(s.seed, synth.T_LOGITS, T * s.n_expert).reshape(T, s.n_expert)
    if logit_shift is not None:
        logits = (logits + logit_shift[None, :]).astype(np.float32)
    bias = synth.normal_host(s.seed, synth.T_BIAS, s.n_expert, s.bias_sigma) if s.bias_sigma else None
    return x, logits, bias


def device_weights(s: Shape, device="cuda", block=False, planar=False):
    """The same layer generated on the GPU (identical bytes); planar: its MXFP4 tensors then
    rewritten into the planar form."""
    import torch
    from deepstrix_amd.executor import LayerWeights
    gate = synth.weights_dev(s.gate_fmt, s.seed, synth.T_GATE, s.n_expert * s.inter, s.hidden)
    up = synth.weights_dev(s.gate_fmt, s.seed, synth.T_UP, s.n_expert * s.inter, s.hidden)
    down = synth.weights_dev(s.down_fmt, s.seed, synth.T_DOWN, s.n_expert * s.hidden, s.inter)
    w = LayerWeights(s.hidden, s.inter, s.n_expert, s.n_used, gate, up, down, s.gate_fmt,
                     s.gate_fmt, s.down_fmt, s.clamp, s.router_mode, s.n_group, s.topk_group,
                     s.route_scale, s.route_eps)
    if s.bias_sigma:
        w.bias = synth.normal_dev(s.seed, synth.T_BIAS, s.n_expert, s.bias_sigma)
    if s.shared:
        w.sh_inter = s.shi
        w.sh_gate = synth.weights_dev(s.shg, s.seed, synth.T_SH_GATE, s.shi, s.hidden)
        w.sh_up = synth.weights_dev(s.shg, s.seed, synth.T_SH_UP, s.shi, s.hidden)
        w.sh_down = synth.weights_dev(s.shd, s.seed, synth.T_SH_DOWN, s.hidden, s.shi)
        w.sh_gate_fmt = w.sh_up_fmt = s.shg
        w.sh_down_fmt = s.shd
        w.sh_clamp = s.clamp
    if block:
        w.norm_w = synth.normal_dev(s.seed, synth.T_NORM_W, s.hidden, 0.02, 1.0)
        w.router_w = synth.normal_dev(s.seed, synth.T_ROUTER_W, s.n_expert * s.hidden, 0.02)
        w.norm_eps = 1e-6
    if planar:
        w.to_planar()
    torch.cuda.synchronize()
    return w


def host_block_params(s: Shape):
    """RMSNorm weight 1 + N(0, 0.02) and router matrix N(0, 0.02) of a pre-norm block
    (BASELINE config 4), the same values device_weights(block=True) generates."""
    norm_w = synth.normal_host(s.seed, synth.T_NORM_W, s.hidden, 0.02, 1.0)
    router_w = synth.normal_host(s.seed, synth.T_ROUTER_W, s.n_expert * s.hidden, 0.02)
    return norm_w, router_w.reshape(s.n_expert, s.hidden)


def zipf_logit_shift(n_expert: int, seed: int, s: float = 1.1) -> np.ndarray:
    """-s * ln(rank) under a seeded permutation of the experts (BASELINE config 3: added to
    N(0,1) logits with a factor chosen so that the top 10 % of experts get ~50 % of the picks)."""
    rng = np.random.default_rng(seed)
    perm = rng.permutation(n_expert)
    shift = np.empty(n_expert, np.float32)
    shift[perm] = (-s * np.log(np.arange(1, n_expert + 1))).astype(np.float32)
    return shift
