"""Freezes the CPU oracle's result for BASELINE config 1 (hidden 2048, 64 + 1 experts, top-6
softmax router fed by the f32 router matvec, inter 1408, Q8_0 weights, T = 4) as a fixture:

    python tests/golden/make_cfg1_fixture.py

Inputs are not stored: they are regenerated from the seeds of tests/helpers.CFG1 by the
counter-based generator (deepstrix_amd/synth.py).  Stored in cfg1_T4.npz (numpy, no pickle):
  logits [4, 64] f32   router W . x
  sel    [4, 6]  i32   picks, weights w [4, 6] f32
  out    [4, 2048] f32 layer output (routed experts in slot order, shared expert added last)
The fixture comes from this repository's oracle, not from the reference (whose path cannot run
here): it guards the oracle against drift and gives the GPU test a committed vector.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from deepstrix_amd import synth  # noqa: E402
from oracle import ref  # noqa: E402
from tests import helpers as H  # noqa: E402


def compute():
    s, T = H.CFG1, 4
    x, _, _ = H.host_inputs(s, T)
    W = synth.normal_host(s.seed, synth.T_ROUTER_W, s.n_expert * s.hidden, 0.02).reshape(s.n_expert, s.hidden)
    logits = ref.router_logits(W, x)
    sel, w = ref.router_topk(logits, None, s.n_used, s.route_scale, s.route_eps, s.router_mode)
    out = ref.moe_forward(H.host_weights(s, experts=np.unique(sel)), x, sel, w)
    return {"logits": logits, "sel": sel, "w": w, "out": out.astype(np.float32)}


if __name__ == "__main__":
    np.savez_compressed(os.path.join(HERE, "cfg1_T4.npz"), **compute())
    print("wrote cfg1_T4.npz")
