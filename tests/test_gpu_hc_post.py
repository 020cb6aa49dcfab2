"""The hyper-connection combine behind the FFN (crates/v4flash-kernels/kernels/hc_post.hip:15-141,
call site crates/v4flash-kernels/src/het/forward_layer.rs:3126-3133) on the GPU: the operator bit
for bit against the CPU oracle, and the layer entry point that applies it while it stores --
bitwise the operator applied to the plain layer's own output, on every path of the layer."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

from deepstrix_amd import dispatch
from deepstrix_amd.capi import FMT_Q8_0, DsxError
from deepstrix_amd.executor import MoeLayer
from oracle import ref
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _mix(b, n_hc, n_embd, seed):
    rng = np.random.default_rng(seed)
    res = rng.standard_normal((b, n_hc, n_embd)).astype(np.float32)
    post = rng.uniform(0.2, 1.5, (b, n_hc)).astype(np.float32)
    comb = rng.standard_normal((b, n_hc, n_hc)).astype(np.float32)
    return res, post, comb


@pytest.mark.parametrize("b,n_hc,n_embd", [(1, 4, 7168), (2, 4, 7168), (130, 4, 1024), (3, 1, 64), (5, 8, 512), (2, 7, 20)])
def test_operator_is_bit_exact(b, n_hc, n_embd):
    rng = np.random.default_rng(100 + b)
    block = rng.standard_normal((b, n_embd)).astype(np.float32)
    a1 = rng.standard_normal((b, n_embd)).astype(np.float32)
    a2 = rng.standard_normal((b, n_embd)).astype(np.float32)
    res, post, comb = _mix(b, n_hc, n_embd, 200 + b)
    d = lambda a: torch.from_numpy(a).cuda()
    dres, dpost, dcomb, dblock, d1, d2 = d(res), d(post), d(comb), d(block), d(a1), d(a2)
    for adds in ((None, None), (d1, None), (d1, d2)):
        out = torch.full((b, n_hc, n_embd), float("nan"), dtype=torch.float32, device="cuda")
        desc = dispatch.hc_post_desc(out, dres, dpost, dcomb, n_hc)
        dispatch.hc_post(desc, dblock, n_embd, b, *adds)
        want = ref.hc_post(block, res, post, comb, None if adds[0] is None else a1,
                           None if adds[1] is None else a2)
        assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))
    assert torch.equal(dblock, d(block))          # block_out is not written
    # post and comb as views into the packed split rows (hc_post.hip:66-98), in place over the residual
    n_w = 3
    stride = n_w + n_hc + n_hc * n_hc
    split = np.concatenate([rng.standard_normal((b, n_w)).astype(np.float32), post,
                            comb.reshape(b, -1)], axis=1)
    dsplit = d(split).reshape(-1)
    inplace = dres.clone()
    desc = dispatch.hc_post_desc(inplace, inplace, dsplit[n_w:], dsplit[n_w + n_hc:], n_hc, stride, stride)
    dispatch.hc_post(desc, dblock, n_embd, b)
    want = ref.hc_post_from_split(block, res, split, n_w)
    assert np.array_equal(inplace.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_operator_refusals():
    t = torch.zeros(64, device="cuda")
    with pytest.raises(DsxError):
        dispatch.hc_post(dispatch.hc_post_desc(t, t, t, t, 9), t, 4, 1)       # n_hc > 8
    with pytest.raises(DsxError):
        dispatch.hc_post(dispatch.hc_post_desc(t, t, t, t, 2), t, 6, 1)       # n_embd % 4
    with pytest.raises(DsxError):
        dispatch.hc_post(dispatch.hc_post_desc(t, t, t, t, 2), t, 8, 1, None, t)   # add2 without add1


SMALL = H.Shape(1024, 512, 16, 4, router_mode=1, n_group=4, topk_group=2, route_scale=2.5,
                bias_sigma=0.01, clamp=10.0, seed=1301)
SMALL_Q8_SHARED = H.Shape(1024, 512, 16, 4, sh_gate_fmt=FMT_Q8_0, sh_down_fmt=FMT_Q8_0, sh_inter=384,
                          router_mode=1, n_group=4, topk_group=2, route_scale=2.5, bias_sigma=0.01,
                          clamp=10.0, seed=1302)
SMALL_Q8 = H.Shape(512, 256, 8, 2, FMT_Q8_0, FMT_Q8_0, router_mode=2, seed=1303)


def _layer_case(s, layer, T, n_hc=4):
    x, logits, _ = H.host_inputs(s, T)
    res, post, comb = _mix(T, n_hc, s.hidden, 300 + T)
    d = lambda a: torch.from_numpy(a).cuda()
    dx, dl, dres, dpost, dcomb = d(x), d(logits), d(res), d(post), d(comb)
    plain, sel, w = layer.run(dx, dl, want_routing=True)
    out = torch.full((T, n_hc, s.hidden), float("nan"), dtype=torch.float32, device="cuda")
    sel2, w2 = layer.run_hc(dx, dl, dispatch.hc_post_desc(out, dres, dpost, dcomb, n_hc), want_routing=True)
    assert layer.status() == 0
    assert torch.equal(sel, sel2) and torch.equal(w, w2)
    want = ref.hc_post(plain.cpu().numpy(), res, post, comb)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32)), f"T={T}"
    return out, plain, sel.cpu().numpy(), w.cpu().numpy()


@pytest.mark.parametrize("T", [1, 2, 5, 16, 17, 130])
def test_layer_forward_hc_is_the_operator_on_the_layers_own_output(T):
    """One launch decode (1 .. 16 tokens), by-expert (17) and grouped GEMM (130); with fused = 2
    the per-stage decode kernels as well."""
    layer = MoeLayer(H.device_weights(SMALL), T)
    _layer_case(SMALL, layer, T)
    if T <= 16:
        layer.set_decode(fused=2)
        _layer_case(SMALL, layer, T)


@pytest.mark.parametrize("T", [1, 3, 6, 8, 40, 130])
def test_layer_forward_hc_with_a_shared_expert_of_another_format(T):
    """The shared expert inside the launch (up to 6 tokens), on the side stream behind a join (8),
    and beside the by-expert / GEMM paths."""
    layer = MoeLayer(H.device_weights(SMALL_Q8_SHARED), T)
    _layer_case(SMALL_Q8_SHARED, layer, T)
    if T <= 8:
        layer.set_decode(fused=2)
        _layer_case(SMALL_Q8_SHARED, layer, T)


@pytest.mark.parametrize("T", [1, 4, 130])
def test_layer_forward_hc_all_q8_0(T):
    layer = MoeLayer(H.device_weights(SMALL_Q8), T)
    _layer_case(SMALL_Q8, layer, T)


@pytest.mark.parametrize("T", [1, 2, 130])
def test_v3_shape_against_the_oracle(T):
    """n_hc = 4 at the DeepSeek-V3 shape: the whole chain (layer + combine) against the CPU oracle."""
    s = H.CFG2
    dw = H.device_weights(s)
    layer = MoeLayer(dw, T)
    out, plain, sel, w = _layer_case(s, layer, T)     # the oracle on the GPU's routing
    x, logits, bias = H.host_inputs(s, T)
    hw = H.host_weights_from_device(s, dw, experts=np.unique(sel))
    res, post, comb = _mix(T, 4, s.hidden, 300 + T)
    want = ref.hc_post(ref.moe_forward(hw, x, sel, w), res, post, comb)
    H.assert_close(out.cpu().numpy().reshape(T * 4, -1), want.reshape(T * 4, -1), 2e-3, f"V3 T={T}")
