"""Seeded random layers against the CPU oracle: shapes, formats, routers, shared-expert variants,
token counts on every path (one-launch decode, by-expert kernels, grouped GEMMs) and both MXFP4
layouts, drawn from a generator instead of being picked by hand.  Every case must be accepted by
dsx_moe_layer_create (the generator only draws shapes the header documents as supported) and meet
the same bar as the hand-picked layer tests."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

from deepstrix_amd.capi import FMT_MXFP4, FMT_Q8_0
from deepstrix_amd.executor import MoeLayer
from tests import helpers as H
from tests.test_gpu_layer import OUT_TOL, run_case

pytestmark = pytest.mark.gpu

TOKEN_COUNTS = [1, 2, 3, 4, 5, 7, 8, 9, 12, 15, 16, 17, 24, 33, 40, 41, 64, 65, 100, 111, 112, 129, 200,
                300, 450]


def draw_case(rng):
    """(Shape, T, planar): MXFP4 matrices have a multiple of 256 columns, Q8_0 ones of 128."""
    gate_fmt, down_fmt = [(FMT_MXFP4, FMT_MXFP4), (FMT_Q8_0, FMT_Q8_0), (FMT_MXFP4, FMT_Q8_0)][rng.integers(3)]
    shared = rng.random() < 0.7
    kw = {}
    if shared and rng.random() < 0.4:
        kw["sh_gate_fmt"], kw["sh_down_fmt"] = [(FMT_Q8_0, FMT_Q8_0), (FMT_MXFP4, FMT_MXFP4),
                                                (FMT_MXFP4, FMT_Q8_0)][rng.integers(3)]
    if shared and rng.random() < 0.3:
        kw["sh_inter"] = 256 * int(rng.integers(1, 4))
    sh_gate = kw.get("sh_gate_fmt", gate_fmt) if shared else gate_fmt
    sh_down = kw.get("sh_down_fmt", down_fmt) if shared else down_fmt
    # hidden is the column count of gate/up (routed and shared), inter that of down
    hidden_unit = 256 if FMT_MXFP4 in (gate_fmt, sh_gate) else 128
    hidden = hidden_unit * int(rng.integers(1, 1536 // hidden_unit + 1))
    inter_unit = 256 if (down_fmt == FMT_MXFP4 or (sh_down == FMT_MXFP4 and "sh_inter" not in kw)) else 128
    inter = inter_unit * int(rng.integers(1, 1024 // inter_unit + 1))
    E = int(rng.choice([4, 6, 8, 16, 24, 32, 64]))
    k = int(rng.integers(1, min(E, 8) + 1))
    mode = int(rng.integers(0, 3))
    ng = 4 if (mode != 2 and E % 4 == 0 and rng.random() < 0.5) else 1
    tg = int(rng.integers(1, ng + 1))
    if ng > 1 and tg * (E // ng) < k:
        tg = ng
    s = H.Shape(hidden, inter, E, k, gate_fmt, down_fmt, shared=shared,
                clamp=float(rng.choice([0.0, 7.0, 10.0])), router_mode=mode, n_group=ng, topk_group=tg,
                route_scale=float(rng.choice([1.0, 2.5])), bias_sigma=float(rng.choice([0.0, 0.01])),
                seed=int(rng.integers(1, 1 << 30)), **kw)
    return s, int(rng.choice(TOKEN_COUNTS)), bool(rng.random() < 0.3)


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_random_layers_match_the_oracle(seed):
    rng = np.random.default_rng(seed)
    for c in range(24):
        s, T, planar = draw_case(rng)
        what = f"seed {seed} case {c}: T={T} planar={planar} {s}"
        print(what, flush=True)
        dw = H.device_weights(s, planar=planar)
        layer = MoeLayer(dw, T)
        out, want, _, _ = run_case(s, T, layer=layer, dw=dw)
        assert H.max_rel(out, want) < OUT_TOL, what
        del layer, dw
