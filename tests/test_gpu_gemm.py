"""GPU parity of the grouped-GEMM path of the layer (many tokens per expert) against the CPU
oracle and against the small-batch by-expert path of the same library."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

from deepstrix_amd.executor import MoeLayer
from oracle import ref
from tests import helpers as H

pytestmark = pytest.mark.gpu

OUT_TOL = 2e-3  # max|a-b| / max|ref|
# The two GPU paths compute the same integer dots but sum the super-blocks in a different
# f32 order; a mid value that lands on the other side of a rounding boundary of the second
# quantization then moves one int8 step (1/127 of its block's largest value).
BASE_TOL = 1e-3


def layer_outputs(s, T, selected=None, weights=None, shift=None):
    """(gemm path, by-expert path, oracle) outputs of one layer on the same inputs."""
    x, logits, bias = H.host_inputs(s, T, shift)
    dw = H.device_weights(s)
    layer = MoeLayer(dw, T)
    dx, dl = torch.from_numpy(x).cuda(), torch.from_numpy(logits).cuda()
    if selected is None:
        layer.set_tuning(gemm_min_tokens=1 << 30)
        base, sel, w = layer.run(dx, dl, want_routing=True)
    else:
        sel, w = torch.from_numpy(selected).cuda(), torch.from_numpy(weights).cuda()
        layer.set_tuning(gemm_min_tokens=1 << 30)
        base = layer.run(dx, None, selected_in=sel, weights_in=w)
    base = base.clone()
    layer.set_tuning(gemm_min_tokens=1)
    got = layer.run(dx, None, selected_in=sel, weights_in=w)
    torch.cuda.synchronize()
    sel_h, w_h = sel.cpu().numpy(), w.cpu().numpy()
    hw = H.host_weights(s, experts=np.unique(sel_h[sel_h >= 0]))
    want = ref.moe_forward(hw, x, sel_h, w_h)
    return got.cpu().numpy(), base.cpu().numpy(), want


@pytest.mark.parametrize("T", [1, 15, 16, 17, 64, 65, 200])
def test_small_layer_gemm_path(T):
    s = H.Shape(1024, 512, 16, 4, router_mode=1, n_group=4, topk_group=2, route_scale=2.5,
                bias_sigma=0.01, clamp=10.0, seed=91)
    got, base, want = layer_outputs(s, T)
    assert H.max_rel(got, want) < OUT_TOL
    assert H.max_rel(got, base) < BASE_TOL


@pytest.mark.parametrize("T", [40, 130])
@pytest.mark.parametrize("narrow", [1, 1 << 20])
def test_both_gemm_tiles_on_the_same_inputs(T, narrow):
    """The 128-column tile (gemm_narrow_members = 1: never narrow) and the 16-column tile
    (always narrow: groups of more than 16 members become several work items) agree with the
    oracle and with the by-expert path."""
    s = H.Shape(1024, 512, 16, 4, router_mode=1, route_scale=2.5, clamp=10.0, seed=95)
    x, logits, bias = H.host_inputs(s, T)
    layer = MoeLayer(H.device_weights(s), T)
    dx, dl = torch.from_numpy(x).cuda(), torch.from_numpy(logits).cuda()
    layer.set_tuning(gemm_min_tokens=1 << 30)
    base, sel, w = layer.run(dx, dl, want_routing=True)
    base = base.clone()
    layer.set_tuning(gemm_min_tokens=1, gemm_narrow_members=narrow)
    got = layer.run(dx, None, selected_in=sel, weights_in=w).cpu().numpy()
    sel_h, w_h = sel.cpu().numpy(), w.cpu().numpy()
    want = ref.moe_forward(H.host_weights(s, experts=np.unique(sel_h)), x, sel_h, w_h)
    assert H.max_rel(got, want) < OUT_TOL
    assert H.max_rel(got, base.cpu().numpy()) < BASE_TOL


def test_gemm_path_without_shared_expert():
    s = H.Shape(512, 256, 8, 2, shared=False, router_mode=0, route_scale=1.5,
                route_eps=6.103515625e-5, seed=92)
    got, base, want = layer_outputs(s, 90)
    assert H.max_rel(got, want) < OUT_TOL
    assert H.max_rel(got, base) < BASE_TOL


def test_gemm_path_all_tokens_on_the_same_experts_and_empty_slots():
    """Worst-case imbalance: every token picks experts {0..3}; a full 128-column tile
    per expert plus a ragged one.  A few slots are empty (-1)."""
    s = H.Shape(1024, 512, 16, 4, clamp=10.0, seed=93)
    T = 150
    sel = np.tile(np.arange(4, dtype=np.int32), (T, 1))
    sel[5, 2] = -1
    sel[77, 0] = -1
    rng = np.random.default_rng(0)
    w = rng.uniform(0.1, 1.0, (T, 4)).astype(np.float32)
    got, base, want = layer_outputs(s, T, sel, w)
    assert H.max_rel(got, want) < OUT_TOL
    assert H.max_rel(got, base) < BASE_TOL


def test_gemm_path_skewed_routing():
    """Zipf-like logit shift: a few experts get most tokens, many get none."""
    s = H.Shape(1024, 512, 32, 4, router_mode=1, route_scale=2.5, seed=94)
    shift = (-1.1 * np.log(np.arange(1, 33))).astype(np.float32) * 3.0
    got, base, want = layer_outputs(s, 300, shift=shift)
    assert H.max_rel(got, want) < OUT_TOL
    assert H.max_rel(got, base) < BASE_TOL


def test_config2_v3_shape_T256_takes_the_gemm_path_by_default():
    s = H.CFG2
    T = 256
    x, logits, bias = H.host_inputs(s, T)
    dw = H.device_weights(s)
    layer = MoeLayer(dw, T)
    out, sel, w = layer.run(torch.from_numpy(x).cuda(), torch.from_numpy(logits).cuda(),
                            want_routing=True)
    torch.cuda.synchronize()
    sel_h, w_h = sel.cpu().numpy(), w.cpu().numpy()
    rsel, _ = H.oracle_route(s, logits, bias)
    _, scores = ref.router_scores(logits, bias, s.router_mode, s.n_group, s.topk_group)
    assert H.routing_mismatch_explained(sel_h, rsel, scores, s.n_used) == []
    # the oracle on a sample of tokens (each token is independent of the others)
    pick = np.arange(0, T, 8)
    hw = H.host_weights(s, experts=np.unique(sel_h[pick]))
    want = ref.moe_forward(hw, x[pick], sel_h[pick], w_h[pick])
    assert H.max_rel(out.cpu().numpy()[pick], want) < OUT_TOL


def test_config3_v3_shape_T4096_zipf_routing():
    """BASELINE config 3 at its full size.  Checked three ways: the routing of all 4096 tokens
    against the oracle; a sample of tokens against the oracle's layer; and the size-independent
    property that a token's output does not depend on its batch -- 64 tokens taken out of the
    4096 and run on their own (by-expert path, T=64) must give the rows they had in the batch."""
    s = H.CFG2
    T = 4096
    shift = 0.416 * H.zipf_logit_shift(s.n_expert, 3)  # top 10 % of the experts get ~50 % of the picks
    x, logits, bias = H.host_inputs(s, T, shift)
    dw = H.device_weights(s)
    layer = MoeLayer(dw, T)
    dx, dl = torch.from_numpy(x).cuda(), torch.from_numpy(logits).cuda()
    out, sel, w = layer.run(dx, dl, want_routing=True)
    torch.cuda.synchronize()
    out_h, sel_h, w_h = out.cpu().numpy(), sel.cpu().numpy(), w.cpu().numpy()
    cnt = np.bincount(sel_h.ravel(), minlength=s.n_expert)
    assert np.sort(cnt)[::-1][:26].sum() > 0.4 * cnt.sum()     # the skew is there
    assert cnt.max() > 8 * 128                                  # several full column tiles

    rsel, _ = H.oracle_route(s, logits, bias)
    _, scores = ref.router_scores(logits, bias, s.router_mode, s.n_group, s.topk_group)
    assert H.routing_mismatch_explained(sel_h, rsel, scores, s.n_used) == []

    pick = np.array([0, 1365, 2730, 4095])
    hw = H.host_weights(s, experts=np.unique(sel_h[pick]))
    want = ref.moe_forward(hw, x[pick], sel_h[pick], w_h[pick])
    assert H.max_rel(out_h[pick], want) < OUT_TOL

    sub = np.arange(17, T, 64)[:64]
    small = MoeLayer(dw, 64)
    got = small.run(torch.from_numpy(x[sub]).cuda(), None,
                    selected_in=torch.from_numpy(sel_h[sub]).cuda(),
                    weights_in=torch.from_numpy(w_h[sub]).cuda())
    torch.cuda.synchronize()
    assert H.max_rel(out_h[sub], got.cpu().numpy()) < BASE_TOL
