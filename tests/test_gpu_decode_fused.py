"""The one-launch decode path (gate/up, mid quantization, down and the slot-order sum handed
from workgroup to workgroup inside one grid) against the CPU oracle and against the
one-launch-per-stage path, through the C ABI."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

from deepstrix_amd import capi
from deepstrix_amd.executor import MoeLayer
from oracle import ref
from tests import helpers as H

pytestmark = pytest.mark.gpu

CONTRACT = 2e-3      # max|a-b| / max|ref|, the stated parity bar
REGRESSION = 1e-4    # about ten times what is observed (integer dots are exact; only the
                     # order of f32 sums differs from the oracle)


def _both_modes(s, T, sel_in=None, w_in=None):
    x, logits, _ = H.host_inputs(s, T)
    dw = H.device_weights(s)
    layer = MoeLayer(dw, max(T, 1))
    dx, dl = torch.from_numpy(x).cuda(), torch.from_numpy(logits).cuda()
    outs = {}
    # 1 = one launch (pairs tokens that name one expert from 4 tokens on), 2 = one launch per
    # stage, 3 = one launch, never pairing, 4 = one launch, pairing from 2 tokens on
    for mode in (1, 2, 3, 4):
        layer.set_decode(fused=mode)
        if sel_in is None:
            out, sel, w = layer.run(dx, dl, want_routing=True)
        else:
            out, sel, w = layer.run(dx, None, selected_in=sel_in, weights_in=w_in, want_routing=True)
        assert layer.status() == 0
        outs[mode] = (out.cpu().numpy(), sel.cpu().numpy(), w.cpu().numpy())
    # pairing changes which workgroup computes a (token, slot) column, never a value
    for mode in (1, 4):
        assert np.array_equal(outs[mode][0], outs[3][0]), f"mode {mode} differs from mode 3"
    return x, outs


@pytest.mark.parametrize("T", [1, 2, 5, 12])
@pytest.mark.parametrize("inter", [512, 2048, 2560])   # 2, 8 (straight-line code) and 10 blocks per mid row
def test_one_launch_decode_matches_oracle_and_the_per_stage_path(T, inter):
    s = H.Shape(1024, inter, 16, 4, router_mode=1, n_group=4, topk_group=2, route_scale=2.5,
                bias_sigma=0.01, clamp=10.0, seed=900 + inter)
    x, outs = _both_modes(s, T)
    (a, sel, w), (b, sel2, w2) = outs[1], outs[2]
    assert np.array_equal(sel, sel2) and np.array_equal(w, w2)
    want = ref.moe_forward(H.host_weights(s, experts=np.unique(sel)), x, sel, w)
    assert H.max_rel(a, want) < REGRESSION
    assert H.max_rel(b, want) < REGRESSION
    assert H.max_rel(a, b) < REGRESSION


def test_one_launch_decode_without_shared_expert_and_single_pick():
    for k, shared in ((2, False), (1, True), (1, False)):
        s = H.Shape(512, 256, 8, k, shared=shared, router_mode=0, route_scale=1.5,
                    route_eps=6.103515625e-5, bias_sigma=0.05, seed=910 + k)
        for T in (1, 3):
            x, outs = _both_modes(s, T)
            a, sel, w = outs[1]
            want = ref.moe_forward(H.host_weights(s, experts=np.unique(sel)), x, sel, w)
            assert H.max_rel(a, want) < REGRESSION, (k, shared, T)


def test_empty_and_out_of_range_picks_are_empty_slots():
    """Pinned routing with -1 and with an index past the weights: both are slots that
    contribute nothing (and nothing is read past the expert tensors)."""
    s = H.Shape(1024, 512, 16, 4, route_scale=2.5, clamp=10.0, seed=920)
    T = 3
    rng = np.random.default_rng(5)
    sel = np.stack([rng.choice(s.n_expert, s.n_used, replace=False) for _ in range(T)]).astype(np.int32)
    w = rng.uniform(0.1, 0.9, (T, s.n_used)).astype(np.float32)
    sel[0, 1] = -1
    sel[1, 0] = s.n_expert + 3
    sel[2, :] = -1               # a token whose output is the shared expert alone
    x, outs = _both_modes(s, T, torch.from_numpy(sel).cuda(), torch.from_numpy(w).cuda())
    clean = np.where((sel < 0) | (sel >= s.n_expert), -1, sel)
    want = ref.moe_forward(H.host_weights(s, experts=np.unique(clean[clean >= 0])), x, clean, w)
    for mode in (1, 2, 3, 4):
        out, sel_out, _ = outs[mode]
        assert np.array_equal(sel_out, clean)
        assert H.max_rel(out, want) < REGRESSION, mode


def _picks(kind, T, s, rng):
    """Pinned picks in which tokens name the same experts."""
    k, E = s.n_used, s.n_expert
    base = rng.choice(E, k, replace=False).astype(np.int32)
    if kind == "identical":          # every token: the same experts in the same slots
        sel = np.tile(base, (T, 1))
    elif kind == "permuted":         # the same experts, each token in another slot order
        sel = np.stack([rng.permutation(base) for _ in range(T)])
    elif kind == "odd":              # one expert named by every token (T odd: one is left alone),
        others = np.setdiff1d(np.arange(E), base[:1])       # in a slot that moves from token to token
        sel = np.stack([rng.choice(others, k, replace=False) for _ in range(T)])
        for t in range(T):
            sel[t, t % k] = base[0]
    elif kind == "holes":            # identical picks with empty and out-of-range slots among them
        sel = np.tile(base, (T, 1))
        sel[1, 0] = -1
        sel[T // 2, k - 1] = E + 7
        if T > 2:
            sel[T - 1, :] = -1
    else:
        raise ValueError(kind)
    return np.ascontiguousarray(sel, dtype=np.int32)


@pytest.mark.parametrize("kind", ["identical", "permuted", "odd", "holes"])
@pytest.mark.parametrize("T,k", [(2, 4), (5, 4), (7, 8), (12, 8)])   # 12 x 8 picks: two 64-pick ballots
def test_tokens_that_name_the_same_experts(kind, T, k):
    """Tokens of one step that name the same expert are paired and the expert is streamed once
    per pair.  The result must be bitwise what every token gets on its own (modes 1 and 4
    against mode 3, inside _both_modes) and agree with the oracle and the per-stage path."""
    s = H.Shape(1024, 512, 32, k, route_scale=2.5, clamp=10.0, seed=930 + T)
    rng = np.random.default_rng(1000 + T * 10 + k)
    sel = _picks(kind, T, s, rng)
    if kind == "odd":
        for t in range(T):   # a token names an expert at most once
            assert len(set(sel[t])) == k
    w = rng.uniform(0.1, 0.9, (T, k)).astype(np.float32)
    x, outs = _both_modes(s, T, torch.from_numpy(sel).cuda(), torch.from_numpy(w).cuda())
    clean = np.where((sel < 0) | (sel >= s.n_expert), -1, sel)
    want = ref.moe_forward(H.host_weights(s, experts=np.unique(clean[clean >= 0])), x, clean, w)
    for mode in (1, 2, 3, 4):
        assert H.max_rel(outs[mode][0], want) < REGRESSION, mode
    # a token's output does not depend on which tokens share the step with it
    if kind == "identical" and T > 2:
        layer = MoeLayer(H.device_weights(s), T)
        layer.set_decode(fused=4)
        dx = torch.from_numpy(x).cuda()
        dsel, dw_ = torch.from_numpy(sel).cuda(), torch.from_numpy(w).cuda()
        alone = layer.run(dx[1:2].contiguous(), None, selected_in=dsel[1:2].contiguous(),
                          weights_in=dw_[1:2].contiguous()).cpu().numpy()
        assert np.array_equal(alone[0], outs[4][0][1])


def test_repeated_calls_are_bitwise_equal():
    s = H.CFG2
    x, logits, _ = H.host_inputs(s, 2)
    layer = MoeLayer(H.device_weights(s), 2)
    dx, dl = torch.from_numpy(x).cuda(), torch.from_numpy(logits).cuda()
    first = layer.run(dx, dl).clone()
    for _ in range(20):
        assert torch.equal(layer.run(dx, dl), first)
    assert layer.status() == 0


def test_an_expired_wait_is_reported_and_every_kernel_still_exits():
    """Forced from the host: with a wait bound of one round, down items that start long before
    their slot's gate/up tiles can finish (32 tiles of 16 rows x 32768 columns, while all 545
    work items are resident at once) give up at once.  The launch completes; when a wait did
    expire (whether one does is a matter of timing on the device, so a clean run is accepted too)
    the status word says which, and what could not be read counts as zero -- the output holds no
    NaN.  With the normal bound the same call is exact again."""
    s = H.Shape(32768, 256, 2, 1, route_scale=1.0, seed=930)
    x, logits, _ = H.host_inputs(s, 1)
    dw = H.device_weights(s)
    layer = MoeLayer(dw, 1)
    dx, dl = torch.from_numpy(x).cuda(), torch.from_numpy(logits).cuda()
    good, sel, w = layer.run(dx, dl, want_routing=True)
    assert layer.status() == 0
    want = ref.moe_forward(H.host_weights(s), x, sel.cpu().numpy(), w.cpu().numpy())
    assert H.max_rel(good.cpu().numpy(), want) < REGRESSION
    layer.set_decode(spin_limit=1)
    cut = layer.run(dx, dl).clone()
    status = layer.status()
    assert status in (0, 1, 3)           # ok / DSX_STATUS_MID_WAIT_EXPIRED / _PARTIAL_WAIT_EXPIRED
    assert torch.isfinite(cut).all()
    if status == 0:
        assert torch.equal(cut, good)
    # a bound no counter could reach is cut down to the library's maximum: the call still ends
    layer.set_decode(spin_limit=0xFFFFFFFF)
    again = layer.run(dx, dl)
    assert layer.status() == 0
    assert torch.equal(again, good)
    layer.set_decode(spin_limit=1 << 16)
    again = layer.run(dx, dl)
    assert layer.status() == 0
    assert torch.equal(again, good)


def test_the_status_word_has_a_device_address():
    """dsx_moe_layer_status_ptr: the word a captured graph's owner can test without a copy."""
    import ctypes as C
    from deepstrix_amd.capi import check, lib
    s = H.Shape(1024, 512, 16, 4, seed=931)
    layer = MoeLayer(H.device_weights(s), 1)
    p = C.c_void_p()
    check(lib().dsx_moe_layer_status_ptr(layer._h, layer.workspace.data_ptr(), C.byref(p)))
    assert p.value == layer.workspace.data_ptr()
    x, logits, _ = H.host_inputs(s, 1)
    layer.run(torch.from_numpy(x).cuda(), torch.from_numpy(logits).cuda())
    torch.cuda.synchronize()
    assert int(layer.workspace[:4].view(torch.int32)[0]) == layer.status() == 0
