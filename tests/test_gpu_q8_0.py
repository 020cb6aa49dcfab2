"""GPU parity of the Q8_0 expert products and of Q8_0 / mixed-format layers against the CPU
oracle (BASELINE configs 1 and 5)."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

from deepstrix_amd import capi, dispatch, synth
from deepstrix_amd.capi import FMT_MXFP4, FMT_Q8_0
from deepstrix_amd.executor import MoeLayer
from oracle import ref
from tests import helpers as H

pytestmark = pytest.mark.gpu

OUT_TOL = 2e-3


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def q8_case(hidden=256, inter=128, E=6, k=3, seed=31):
    s = H.Shape(hidden, inter, E, k, FMT_Q8_0, FMT_Q8_0, shared=False, clamp=5.0, seed=seed)
    return s, H.host_weights(s)


def act_rows(x, k):
    """[rows] Q8_0 activation rows as the kernels take them, made on the GPU."""
    rows = x.shape[0]
    out = torch.zeros((rows, k + k // 8), dtype=torch.uint8, device="cuda")
    dispatch.q8_0_quantize_rows(out, dev(x), rows, k)
    return out


def test_q8_0_decode_operators_match_oracle():
    s, w = q8_case()
    gb = synth.matrix_bytes(FMT_Q8_0, s.inter, s.hidden)
    db = synth.matrix_bytes(FMT_Q8_0, s.hidden, s.inter)
    x = synth.normal_host(5, synth.T_X, s.hidden)[None]
    sel = np.array([[4, 1, 2]], np.int32)
    ew = np.array([[0.5, 1.25, 0.75]], np.float32)
    out_ref, mid_ref, _, _ = ref.moe_forward(w, x, sel, ew, want_parts=True)
    xq = act_rows(x, s.hidden)
    mid = torch.full((3, s.inter), 9.0, dtype=torch.float32, device="cuda")
    dispatch.moe_gate_up_batch(FMT_Q8_0, mid, dev(w.gate), dev(w.up), xq, dev(ew), dev(sel), gb, gb,
                               3, s.clamp, s.inter, s.hidden // 32)
    assert H.max_rel(mid.cpu().numpy(), mid_ref[0]) < 1e-5
    midq = act_rows(mid_ref[0], s.inter)          # the oracle's mid: isolates the down kernel
    out = torch.zeros(s.hidden, dtype=torch.float32, device="cuda")
    dispatch.moe_down_batched(FMT_Q8_0, out, dev(w.down), midq, dev(sel), db, s.inter + s.inter // 8,
                              3, s.hidden, s.inter // 32)
    assert H.max_rel(out.cpu().numpy(), out_ref[0]) < 1e-5
    # empty slot
    sel2 = np.array([[4, -1, 2]], np.int32)
    out_ref2, mid_ref2, _, _ = ref.moe_forward(w, x, sel2, ew, want_parts=True)
    mid.fill_(7.0)
    dispatch.moe_gate_up_batch(FMT_Q8_0, mid, dev(w.gate), dev(w.up), xq, dev(ew), dev(sel2), gb, gb,
                               3, s.clamp, s.inter, s.hidden // 32)
    m = mid.cpu().numpy()
    assert not m[1].any() and H.max_rel(m, mid_ref2[0]) < 1e-5
    dispatch.moe_down_batched(FMT_Q8_0, out, dev(w.down), act_rows(mid_ref2[0], s.inter), dev(sel2), db,
                              s.inter + s.inter // 8, 3, s.hidden, s.inter // 32)
    assert H.max_rel(out.cpu().numpy(), out_ref2[0]) < 1e-5


def test_q8_0_one_hot_activation_reads_single_weights():
    """x = one int8 step at one position (scale 1): mid before SwiGLU is one dequantized weight."""
    s, w = q8_case(hidden=384, inter=64, E=3, k=1)
    gb = synth.matrix_bytes(FMT_Q8_0, s.inter, s.hidden)
    wg = ref.q8_0_dequant_rows(w.gate, s.n_expert * s.inter, s.hidden).reshape(s.n_expert, s.inter, s.hidden)
    wu = ref.q8_0_dequant_rows(w.up, s.n_expert * s.inter, s.hidden).reshape(s.n_expert, s.inter, s.hidden)
    mid = torch.zeros((1, s.inter), dtype=torch.float32, device="cuda")
    k = s.hidden
    for pos in (0, 1, 31, 32, 33, 127, 128, 383):
        for qv in (1, -128, 127):
            row = np.zeros(k + k // 8, np.uint8)
            row[pos] = np.int8(qv).view(np.uint8)
            row[k:].view(np.float32)[:] = 1.0
            dispatch.moe_gate_up_batch(FMT_Q8_0, mid, dev(w.gate), dev(w.up), dev(row), dev(np.ones(1, np.float32)),
                                       dev(np.array([2], np.int32)), gb, gb, 1, 0.0, s.inter, k // 32)
            g = wg[2][:, pos].astype(np.float64) * qv
            u = wu[2][:, pos].astype(np.float64) * qv
            np.testing.assert_allclose(mid.cpu().numpy()[0], g / (1 + np.exp(-g)) * u, rtol=3e-6, atol=1e-30)


@pytest.mark.parametrize("T,chunk", [(5, 4), (9, 2), (3, 1), (20, 8), (45, 32), (21, 20)])
def test_q8_0_by_expert_chain_matches_oracle(T, chunk):
    s, w = q8_case(hidden=384, inter=128, E=5, k=2, seed=33)
    gb = synth.matrix_bytes(FMT_Q8_0, s.inter, s.hidden)
    db = synth.matrix_bytes(FMT_Q8_0, s.hidden, s.inter)
    x, logits, bias = H.host_inputs(s, T)
    sel, ew = H.oracle_route(s, logits, bias)
    out_ref, mid_ref, _, _ = ref.moe_forward(w, x, sel, ew, want_parts=True)
    E, k = s.n_expert, s.n_used
    gc = torch.zeros(E, dtype=torch.int32, device="cuda")
    off = torch.zeros(E + 1, dtype=torch.int32, device="cuda")
    mem = torch.zeros(T * k, dtype=torch.int32, device="cuda")
    wi = torch.zeros(T * k + E, dtype=torch.int32, device="cuda")
    nwi = torch.zeros(1, dtype=torch.int32, device="cuda")
    dispatch.moe_group_build(gc, off, mem, wi, nwi, dev(sel), T, k, E, chunk)
    max_wi = dispatch.wi_upper_bound(T * k, E, chunk)
    xq = act_rows(x, s.hidden)
    mid = torch.zeros((T * k, s.inter), dtype=torch.float32, device="cuda")
    dispatch.moe_gate_up_chunked_rows(FMT_Q8_0, mid, dev(w.gate), dev(w.up), xq, dev(ew), gc, off, mem, wi,
                                      nwi, max_wi, gb, gb, k, chunk, s.clamp, s.inter, s.hidden // 32)
    assert H.max_rel(mid.cpu().numpy().reshape(T, k, s.inter), mid_ref) < 1e-5
    midq = act_rows(mid_ref.reshape(T * k, s.inter), s.inter)
    part = torch.zeros((T * k, s.hidden), dtype=torch.float32, device="cuda")
    dispatch.moe_down_by_expert(FMT_Q8_0, part, dev(w.down), midq, gc, off, mem, wi, nwi, max_wi, db,
                                s.inter + s.inter // 8, k, chunk, s.hidden, s.inter // 32)
    out = torch.zeros((T, s.hidden), dtype=torch.float32, device="cuda")
    dispatch.moe_reduce_partials(out, part, dev(sel), k, s.hidden, T)
    assert H.max_rel(out.cpu().numpy(), out_ref) < 1e-5


def layer_case(s, T, selected=None, weights=None):
    x, logits, bias = H.host_inputs(s, T)
    dw = H.device_weights(s)
    layer = MoeLayer(dw, T)
    dx = dev(x)
    if selected is None:
        out, sel, w = layer.run(dx, dev(logits), want_routing=True)
        rsel, _ = H.oracle_route(s, logits, bias)
        _, scores = ref.router_scores(logits, bias, s.router_mode, s.n_group, s.topk_group)
        assert H.routing_mismatch_explained(sel.cpu().numpy(), rsel, scores, s.n_used) == []
    else:
        sel, w = dev(selected), dev(weights)
        out = layer.run(dx, None, selected_in=sel, weights_in=w)
    torch.cuda.synchronize()
    sel_h, w_h = sel.cpu().numpy(), w.cpu().numpy()
    hw = H.host_weights(s, experts=np.unique(sel_h[sel_h >= 0]))
    want = ref.moe_forward(hw, x, sel_h, w_h)
    return out.cpu().numpy(), want


@pytest.mark.parametrize("T", [1, 4, 13])
def test_config1_q8_0_layer(T):
    """BASELINE config 1: hidden 2048, 64 + 1 experts, top-6 softmax, inter 1408, Q8_0."""
    out, want = layer_case(H.CFG1, T)
    assert H.max_rel(out, want) < OUT_TOL


@pytest.mark.parametrize("T", [128, 300])
def test_config1_shape_many_tokens_take_the_int8_grouped_gemms(T):
    """An all-Q8_0 layer from 128 tokens on: gate/up (SwiGLU in the epilogue) and down as
    int8-MFMA grouped GEMMs, the shared expert as the extra group."""
    out, want = layer_case(H.CFG1, T)
    assert H.max_rel(out, want) < OUT_TOL


def test_small_q8_0_layer_many_tokens_skewed_groups():
    """Groups of more than 128 members (two column tiles, the second ragged), empty experts."""
    s = H.Shape(512, 256, 8, 2, FMT_Q8_0, FMT_Q8_0, clamp=5.0, seed=38)
    T = 200
    rng = np.random.default_rng(38)
    sel = np.stack([rng.choice(3, 2, replace=False) for _ in range(T)]).astype(np.int32)  # experts 0..2 only
    sel[7, 1] = -1
    w = rng.uniform(0.1, 1.0, (T, 2)).astype(np.float32)
    out, want = layer_case(s, T, sel, w)
    assert H.max_rel(out, want) < OUT_TOL


def test_config1_router_logits_from_fp32_matvec():
    """Config 1 names a router matrix W f32 N(0, 0.02): logits = W . x feed the same layer."""
    s, T = H.CFG1, 4
    x, _, _ = H.host_inputs(s, T)
    W = synth.normal_host(s.seed, synth.T_ROUTER_W, s.n_expert * s.hidden, 0.02).reshape(s.n_expert, s.hidden)
    logits = ref.router_logits(W, x)
    dlog = (dev(x) @ dev(W).T).contiguous()
    np.testing.assert_allclose(dlog.cpu().numpy(), logits, atol=2e-5)
    dw = H.device_weights(s)
    layer = MoeLayer(dw, T)
    out, sel, w = layer.run(dev(x), dlog, want_routing=True)
    rsel, _ = ref.router_topk(logits, None, s.n_used, s.route_scale, s.route_eps, s.router_mode)
    _, scores = ref.router_scores(logits, None, s.router_mode)
    assert H.routing_mismatch_explained(sel.cpu().numpy(), rsel, scores, s.n_used) == []
    sel_h, w_h = sel.cpu().numpy(), w.cpu().numpy()
    want = ref.moe_forward(H.host_weights(s, experts=np.unique(sel_h)), x, sel_h, w_h)
    assert H.max_rel(out.cpu().numpy(), want) < OUT_TOL


def test_config1_against_the_committed_fixture():
    """tests/golden/cfg1_T4.npz: logits, picks, weights and layer output of config 1 at T = 4."""
    import os
    s, T = H.CFG1, 4
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "cfg1_T4.npz"),
                allow_pickle=False)
    x, _, _ = H.host_inputs(s, T)
    W = synth.normal_dev(s.seed, synth.T_ROUTER_W, s.n_expert * s.hidden, 0.02).reshape(s.n_expert, s.hidden)
    dlog = torch.zeros((T, s.n_expert), dtype=torch.float32, device="cuda")
    dispatch.router_logits(dlog, W, dev(x), s.n_expert, s.hidden, T)
    np.testing.assert_allclose(dlog.cpu().numpy(), g["logits"], atol=2e-5)
    layer = MoeLayer(H.device_weights(s), T)
    out, sel, w = layer.run(dev(x), dlog, want_routing=True)
    _, scores = ref.router_scores(g["logits"], None, s.router_mode)
    assert H.routing_mismatch_explained(sel.cpu().numpy(), g["sel"], scores, s.n_used) == []
    if np.array_equal(sel.cpu().numpy(), g["sel"]):
        np.testing.assert_allclose(w.cpu().numpy(), g["w"], rtol=2e-5)
        assert H.max_rel(out.cpu().numpy(), g["out"]) < OUT_TOL


def test_mixed_precision_small_layer():
    s = H.Shape(512, 256, 8, 2, FMT_MXFP4, FMT_Q8_0, clamp=10.0, seed=35, route_scale=2.5)
    for T in (1, 7):
        out, want = layer_case(s, T)
        assert H.max_rel(out, want) < OUT_TOL


@pytest.mark.parametrize("T", [128, 131, 300])
def test_mixed_precision_many_tokens_take_the_grouped_gemms(T):
    """From 128 tokens on: MXFP4 gate/up GEMM with f32 mid rows, Q8_0 rows, int8-MFMA down GEMM
    (groups of more than 128 members at T=300: two column tiles, the second ragged)."""
    s = H.Shape(512, 256, 8, 2, FMT_MXFP4, FMT_Q8_0, clamp=10.0, seed=36, route_scale=2.5)
    out, want = layer_case(s, T)
    assert H.max_rel(out, want) < OUT_TOL
    s = H.Shape(1024, 512, 16, 4, FMT_MXFP4, FMT_Q8_0, shared=False, seed=37)
    out, want = layer_case(s, T)
    assert H.max_rel(out, want) < OUT_TOL


def test_config5_mixed_precision_adversarial_and_uniform_routing():
    """BASELINE config 5 (gate/up MXFP4, down Q8_0, V3 shape) at a reduced token count: every
    token on experts 0..7, then uniform random distinct top-8."""
    s, T = H.CFG5, 24
    rng = np.random.default_rng(5)
    w = rng.uniform(0.05, 0.6, (T, 8)).astype(np.float32)
    adversarial = np.tile(np.arange(8, dtype=np.int32), (T, 1))
    out, want = layer_case(s, T, adversarial, w)
    assert H.max_rel(out, want) < OUT_TOL
    uniform = np.stack([rng.choice(s.n_expert, 8, replace=False) for _ in range(T)]).astype(np.int32)
    out, want = layer_case(s, T, uniform, w)
    assert H.max_rel(out, want) < OUT_TOL


def test_q8_0_shape_contract():
    z = torch.zeros(8192, dtype=torch.uint8, device="cuda")
    f = torch.zeros(4096, dtype=torch.float32, device="cuda")
    i = torch.zeros(16, dtype=torch.int32, device="cuda")
    with pytest.raises(capi.DsxError) as e:   # k = 96: not a multiple of 128
        dispatch.moe_gate_up_batch(FMT_Q8_0, f, z, z, z, f, i, 102, 102, 1, 0.0, 16, 3)
    assert e.value.code == capi.ERR_SHAPE


def test_config5_full_size_T512_adversarial_and_uniform_routing():
    """BASELINE config 5 at its full size (T=512).  Adversarial routing (every token on experts
    0..7: 512 members per group) and uniform routing; a sample of tokens against the oracle and,
    as the size-independent check, 16 tokens taken out of the batch and run on their own."""
    s, T = H.CFG5, 512
    rng = np.random.default_rng(55)
    x, logits, bias = H.host_inputs(s, T)
    w = rng.uniform(0.05, 0.6, (T, 8)).astype(np.float32)
    dw = H.device_weights(s)
    layer = MoeLayer(dw, T)
    small = MoeLayer(dw, 16)
    dx = torch.from_numpy(x).cuda()
    cases = {
        "adversarial": np.tile(np.arange(8, dtype=np.int32), (T, 1)),
        "uniform": np.stack([rng.choice(s.n_expert, 8, replace=False) for _ in range(T)]).astype(np.int32),
    }
    for name, sel in cases.items():
        out = layer.run(dx, None, selected_in=torch.from_numpy(sel).cuda(),
                        weights_in=torch.from_numpy(w).cuda())
        torch.cuda.synchronize()
        out_h = out.cpu().numpy()
        pick = np.array([0, 255, 511])
        hw = H.host_weights(s, experts=np.unique(sel[pick]))
        want = ref.moe_forward(hw, x[pick], sel[pick], w[pick])
        assert H.max_rel(out_h[pick], want) < OUT_TOL, name
        sub = np.arange(3, T, 32)[:16]
        got = small.run(torch.from_numpy(x[sub]).cuda(), None,
                        selected_in=torch.from_numpy(sel[sub]).cuda(),
                        weights_in=torch.from_numpy(w[sub]).cuda())
        torch.cuda.synchronize()
        # the batch takes the grouped GEMM for gate/up, the 16 tokens the by-expert kernel: the
        # same integer dots summed in a different f32 order, so a mid value next to a rounding
        # boundary of the Q8_0 quantization may move one int8 step
        assert H.max_rel(out_h[sub], got.cpu().numpy()) < 1e-3, name
