"""BASELINE configs 3 and 5 at their full sizes, several hundred tokens each against the CPU
oracle (host weights are the device tensors copied back).  The tokens are chosen, not sampled:
first / 128th / 129th / last member of the largest expert group (the edges of its 128-column
GEMM tiles, the last one ragged), the last member of other groups, tokens with an empty slot,
tokens whose picks are all empty (shared expert alone), plus an even spread of the rest."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

from deepstrix_amd.executor import MoeLayer
from oracle import ref
from tests import helpers as H

pytestmark = pytest.mark.gpu

CONTRACT = 2e-3
# A token's output agrees with the oracle to about 2e-7 of max|ref| (exact integer dots, f32 sums
# in another order) unless a mid value lands on the other side of an int8 rounding boundary;
# helpers.assert_parity_up_to_rounding_steps accepts exactly that and nothing else.
TIGHT = 2e-6


def _edge_tokens(sel: np.ndarray, n_expert: int, want: int) -> np.ndarray:
    """Tokens at the column-tile edges of the expert groups (members ascend by token)."""
    T = sel.shape[0]
    cnt = np.bincount(sel[sel >= 0].ravel(), minlength=n_expert)
    order = np.argsort(cnt)[::-1]
    toks = []
    for rank, e in enumerate(order[:12]):
        members = np.nonzero((sel == e).any(axis=1))[0]          # ascending token ids
        if members.size == 0:
            continue
        pos = [0, members.size - 1]
        if rank == 0:                                            # the largest group: every tile edge
            pos += [p for p in range(127, members.size, 128)] + [p for p in range(128, members.size, 128)]
        toks += [int(members[p]) for p in pos]
    toks += np.linspace(0, T - 1, want).astype(int).tolist()
    return np.unique(np.array(toks, np.int64))


def _compare(out_h, x, sel_h, w_h, hw, toks, what):
    want = ref.moe_forward(hw, x[toks], sel_h[toks], w_h[toks])
    H.assert_close(out_h[toks], want, CONTRACT, what)
    st = H.assert_parity_up_to_rounding_steps(out_h[toks], want, hw, sel_h[toks], what, TIGHT, CONTRACT)
    print(what, st, H.compare_stats(out_h[toks], want), flush=True)
    return st


@pytest.mark.parametrize("planar", [False, True], ids=["engine_rows", "planar"])
def test_config3_T4096_zipf_prefill_against_the_oracle_on_chosen_tokens(planar):
    """planar: the same layer after its MXFP4 tensors were rewritten into the planar form -- the
    128-column GEMM instantiation for planar weights with the work items dealt to the XCDs (many
    column tiles per expert), against the oracle and bitwise against the engine's rows."""
    s, T = H.CFG2, 4096
    shift = 0.416 * H.zipf_logit_shift(s.n_expert, 3)
    x, logits, bias = H.host_inputs(s, T, shift)
    dw = H.device_weights(s)
    hw = H.host_weights_from_device(s, dw)
    layer = MoeLayer(dw, T)
    dx, dl = torch.from_numpy(x).cuda(), torch.from_numpy(logits).cuda()
    what = "config 3 (planar weights)" if planar else "config 3"
    if planar:
        on_rows, sel_rows, w_rows = layer.run(dx, dl, want_routing=True)
        layer.weights_to_planar()
        torch.cuda.synchronize()
    out, sel, w = layer.run(dx, dl, want_routing=True)
    torch.cuda.synchronize()
    if planar:
        assert torch.equal(sel, sel_rows) and torch.equal(w, w_rows)
        assert torch.equal(out, on_rows), "planar weights: output differs from the engine's rows"
    out_h, sel_h, w_h = out.cpu().numpy(), sel.cpu().numpy(), w.cpu().numpy()
    cnt = np.bincount(sel_h.ravel(), minlength=s.n_expert)
    assert cnt.max() > 16 * 128 and cnt.max() % 128 != 0          # many tiles, the last one ragged
    # more work items than 1.5 x the experts: the kernel deals them to the XCDs
    assert int(np.ceil(cnt / 128).sum()) + T // 128 > s.n_expert + s.n_expert // 2
    toks = _edge_tokens(sel_h, s.n_expert, 256)
    assert toks.size >= 256
    _compare(out_h, x, sel_h, w_h, hw, toks, what)
    # bit-stability: the same call again gives the same bits
    again = layer.run(dx, dl)
    assert torch.equal(again, out)

    # pinned routing with holes: an empty slot in every third token, and tokens with no pick at
    # all (their output is the shared expert alone)
    sel2 = sel_h.copy()
    sel2[::3, 5] = -1
    sel2[7::97, :] = -1
    out2 = layer.run(dx, None, selected_in=torch.from_numpy(sel2).cuda(), weights_in=w)
    out2_h = out2.cpu().numpy()
    toks2 = np.unique(np.concatenate([np.arange(0, T, 3)[:96], np.arange(7, T, 97), toks[:64]]))
    _compare(out2_h, x, sel2, w_h, hw, toks2, what + " with empty slots")


def test_config5_T512_mixed_precision_against_the_oracle_on_chosen_tokens():
    s, T = H.CFG5, 512
    rng = np.random.default_rng(55)
    x, _, _ = H.host_inputs(s, T)
    w = rng.uniform(0.05, 0.6, (T, 8)).astype(np.float32)
    dw = H.device_weights(s)
    hw = H.host_weights_from_device(s, dw)
    layer = MoeLayer(dw, T)
    dx, dwt = torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()
    adversarial = np.tile(np.arange(8, dtype=np.int32), (T, 1))
    uniform = np.stack([rng.choice(s.n_expert, 8, replace=False) for _ in range(T)]).astype(np.int32)
    holes = uniform.copy()
    holes[::4, 2] = -1
    holes[5::61, :] = -1
    for name, sel in (("adversarial", adversarial), ("uniform", uniform), ("uniform with empty slots", holes)):
        out = layer.run(dx, None, selected_in=torch.from_numpy(sel).cuda(), weights_in=dwt)
        torch.cuda.synchronize()
        toks = _edge_tokens(sel, s.n_expert, 256)
        assert toks.size >= 256
        _compare(out.cpu().numpy(), x, sel, w, hw, toks, f"config 5 {name}")
