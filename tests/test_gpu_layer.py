"""GPU parity of the whole layer (dsx_moe_layer_forward) against the CPU oracle."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

from deepstrix_amd import synth
from deepstrix_amd.executor import MoeLayer
from oracle import ref
from tests import helpers as H

pytestmark = pytest.mark.gpu

OUT_TOL = 2e-3  # max|a-b| / max|ref| (fp32 accumulation), the stated parity bar


def run_case(s: H.Shape, T: int, layer=None, dw=None):
    x, logits, bias = H.host_inputs(s, T)
    rsel, rw = H.oracle_route(s, logits, bias)
    _, scores = ref.router_scores(logits, bias, s.router_mode, s.n_group, s.topk_group)
    if layer is None:
        dw = H.device_weights(s)
        layer = MoeLayer(dw, max(T, 1))
    out, sel, w = layer.run(torch.from_numpy(x).cuda(), torch.from_numpy(logits).cuda(),
                            want_routing=True)
    torch.cuda.synchronize()
    sel, w, out = sel.cpu().numpy(), w.cpu().numpy(), out.cpu().numpy()
    assert H.routing_mismatch_explained(sel, rsel, scores, s.n_used) == []
    # the oracle runs on the GPU's routing so that outputs compare like with like
    hw = H.host_weights(s, experts=np.unique(sel[sel >= 0]))
    want = ref.moe_forward(hw, x, sel, w)
    # beyond the 2e-3 contract the callers assert: every token agrees to 2e-6 of max|ref| or
    # differs by single rounding steps of mid values (helpers.assert_parity_up_to_rounding_steps)
    H.assert_parity_up_to_rounding_steps(out, want, hw, sel, f"T={T}")
    assert layer.status() == 0
    return out, want, sel, rsel


@pytest.mark.parametrize("T", [1, 2, 5, 16])
def test_small_mxfp4_layer(T):
    s = H.Shape(1024, 512, 16, 4, router_mode=1, n_group=4, topk_group=2, route_scale=2.5,
                bias_sigma=0.01, clamp=10.0, seed=77)
    out, want, sel, rsel = run_case(s, T)
    assert np.array_equal(sel, rsel)
    assert H.max_rel(out, want) < OUT_TOL


def test_small_layer_without_shared_expert_and_sqrt_softplus_router():
    s = H.Shape(512, 256, 8, 2, shared=False, router_mode=0, route_scale=1.5,
                route_eps=6.103515625e-5, bias_sigma=0.05, seed=78)
    for T in (1, 3):
        out, want, _, _ = run_case(s, T)
        assert H.max_rel(out, want) < OUT_TOL


def test_pinned_routing_and_row_independence():
    """A token's output does not depend on its co-rows: alone == inside a batch, bitwise
    (the by-expert path computes each (token, slot) partial on its own column)."""
    s = H.Shape(1024, 512, 16, 4, seed=79, route_scale=2.5)
    T = 6
    x, logits, bias = H.host_inputs(s, T)
    dw = H.device_weights(s)
    layer = MoeLayer(dw, T)
    layer.set_tuning(decode_max_tokens=1)   # keep the two-token call on the by-expert path too
    dx = torch.from_numpy(x).cuda()
    out, sel, w = layer.run(dx, torch.from_numpy(logits).cuda(), want_routing=True)
    out2 = layer.run(dx, None, selected_in=sel, weights_in=w)
    assert torch.equal(out, out2)
    pair = layer.run(dx[2:4].contiguous(), None, selected_in=sel[2:4].contiguous(),
                     weights_in=w[2:4].contiguous())
    assert torch.equal(pair, out[2:4])


@pytest.mark.parametrize("T", [2, 3, 4, 7])
def test_per_token_decode_path_equals_by_expert_path(T):
    """Up to decode_max_tokens tokens run the decode kernels once per token (grid.y = token);
    more go through the by-expert path.  Both must agree with the oracle and each other."""
    s = H.Shape(1024, 512, 16, 4, router_mode=1, route_scale=2.5, clamp=10.0, seed=81)
    x, logits, bias = H.host_inputs(s, T)
    dw = H.device_weights(s)
    layer = MoeLayer(dw, T)
    dx, dl = torch.from_numpy(x).cuda(), torch.from_numpy(logits).cuda()
    layer.set_tuning(decode_max_tokens=8)
    a, sel, w = layer.run(dx, dl, want_routing=True)
    a = a.clone()
    layer.set_tuning(decode_max_tokens=1)
    b = layer.run(dx, None, selected_in=sel, weights_in=w)
    torch.cuda.synchronize()
    sel_h, w_h = sel.cpu().numpy(), w.cpu().numpy()
    want = ref.moe_forward(H.host_weights(s, experts=np.unique(sel_h)), x, sel_h, w_h)
    assert H.max_rel(a.cpu().numpy(), want) < OUT_TOL
    assert H.max_rel(b.cpu().numpy(), want) < OUT_TOL
    assert H.max_rel(a.cpu().numpy(), b.cpu().numpy()) < 1e-3
    # an empty slot in the per-token path
    sel2 = sel.clone()
    sel2[T - 1, 1] = -1
    layer.set_tuning(decode_max_tokens=8)
    c = layer.run(dx, None, selected_in=sel2, weights_in=w)
    sel2_h = sel2.cpu().numpy()
    want2 = ref.moe_forward(H.host_weights(s, experts=np.unique(sel2_h[sel2_h >= 0])), x, sel2_h, w_h)
    assert H.max_rel(c.cpu().numpy(), want2) < OUT_TOL


@pytest.mark.parametrize("T", [1, 4, 16, 64])
def test_config2_v3_shape_decode(T, cfg2_layer):
    """BASELINE config 2: hidden 7168, 256 + 1 experts, top-8 sigmoid + bias, 8 groups / top-4,
    scale 2.5, inter 2048, MXFP4, bf16-valued activations."""
    layer, dw = cfg2_layer
    out, want, sel, rsel = run_case(H.CFG2, T, layer, dw)
    assert (sel == rsel).all(axis=1).mean() > 0.95
    assert H.max_rel(out, want) < OUT_TOL


@pytest.fixture(scope="module")
def cfg2_layer():
    dw = H.device_weights(H.CFG2)
    return MoeLayer(dw, 64), dw


@pytest.mark.parametrize("hidden,inter", [(256, 256), (512, 768), (768, 1280), (1280, 1792), (1792, 512),
                                          (2304, 2304), (3072, 1024)])
def test_by_expert_path_over_super_block_counts(hidden, inter):
    """The by-expert kernels run several row tiles per workgroup and keep four super-blocks of
    weights in flight (down) or the k range split over the waves (gate/up): rows of 1 .. 12
    super-blocks cover every way their loops begin and end.  Against the oracle; the first and the
    last token then run alone on the same picks through the per-stage decode kernels, against the
    oracle as well."""
    s = H.Shape(hidden, inter, 8, 3, router_mode=1, route_scale=2.5, clamp=10.0, seed=900 + hidden // 256 + inter)
    T = 11
    x, logits, bias = H.host_inputs(s, T)
    dw = H.device_weights(s)
    layer = MoeLayer(dw, T)
    layer.set_tuning(decode_max_tokens=1, gemm_min_tokens=1 << 20)   # by expert at every token count above 1
    dx, dl = torch.from_numpy(x).cuda(), torch.from_numpy(logits).cuda()
    out, sel, w = layer.run(dx, dl, want_routing=True)
    out = out.clone()
    torch.cuda.synchronize()
    sel_h, w_h = sel.cpu().numpy(), w.cpu().numpy()
    hw = H.host_weights(s, experts=np.unique(sel_h))
    want = ref.moe_forward(hw, x, sel_h, w_h)
    H.assert_parity_up_to_rounding_steps(out.cpu().numpy(), want, hw, sel_h, f"{hidden}x{inter}")
    assert layer.status() == 0
    layer.set_decode(fused=2)   # one launch per stage: k_mxfp4_gate_up / k_mxfp4_down_decode
    for t in (0, T - 1):
        one = layer.run(dx[t:t + 1], None, selected_in=sel[t:t + 1].contiguous(), weights_in=w[t:t + 1].contiguous())
        torch.cuda.synchronize()
        assert H.max_rel(one.cpu().numpy(), want[t:t + 1]) < OUT_TOL


def test_by_expert_chunk_sizes_give_the_same_bits():
    """The members of an expert are served in chunks of `by_expert_chunk` token columns (1 .. 16; the
    kernels are instantiated for 1, 2, 4, 8 and 16 columns, and a chunk wider than a workgroup's
    columns is split over several workgroups): every column is computed on its own, so the chunk
    size must not change a bit of the output."""
    s = H.Shape(1024, 512, 8, 3, router_mode=1, route_scale=2.5, clamp=10.0, seed=931)
    T = 40   # 15 picks per expert: several chunks per group at every size
    x, logits, bias = H.host_inputs(s, T)
    layer = MoeLayer(H.device_weights(s), T)
    layer.set_tuning(decode_max_tokens=1, gemm_min_tokens=1 << 20)
    dx, dl = torch.from_numpy(x).cuda(), torch.from_numpy(logits).cuda()
    ref_out, sel, w = layer.run(dx, dl, want_routing=True)
    ref_out = ref_out.clone()
    sel_h, w_h = sel.cpu().numpy(), w.cpu().numpy()
    hw = H.host_weights(s, experts=np.unique(sel_h))
    H.assert_parity_up_to_rounding_steps(ref_out.cpu().numpy(), ref.moe_forward(hw, x, sel_h, w_h), hw, sel_h, "chunk 4")
    for chunk in (1, 2, 3, 8, 11, 16):
        layer.set_tuning(by_expert_chunk=chunk)
        assert layer.tuning()["by_expert_chunk"] == chunk
        out = layer.run(dx, dl)
        torch.cuda.synchronize()
        assert layer.status() == 0
        assert torch.equal(out, ref_out), f"chunk {chunk}"
