"""Pins the oracle's routers and token->expert inversion (CPU only).

None of these tests retypes the oracle's code path: each compares against an independent
statement of the rule (float64 ranking with numpy sorts, exhaustive enumeration on tiny
expert counts, numpy softmax) or against an invariant the definition fixes.

Rules and their sources in the reference tree:
  sqrt(softplus) scores, top-k, p / max(sum, eps) * scale ... crates/v4flash-kernels/tests/
      router_topk_alts.rs:100-110, router_learned.rs:44-66
  sigmoid(logit) + bias ranking, weights from unbiased p ..... crates/v4flash-kernels/tests/
      laguna_spike.rs:601-618
  softmax top-k and group-limited top-k are not in the reference: textbook / DeepSeek-V3
      definitions, enumerated here.
"""
import itertools

import numpy as np
import pytest

from oracle import ref

SQRT_SOFTPLUS, SIGMOID, SOFTMAX = 0, 1, 2


def probs64(logits, mode):
    z = logits.astype(np.float64)
    if mode == SQRT_SOFTPLUS:
        return np.sqrt(np.logaddexp(0.0, z))
    if mode == SIGMOID:
        return 1.0 / (1.0 + np.exp(-z))
    e = np.exp(z - z.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def topk_stable(scores, k):
    """Indices of the k largest, larger first, lower index first among equals."""
    return np.argsort(-scores, kind="stable")[:k]


def gap_ok(scores, k, tol=1e-6):
    s = np.sort(scores)[::-1]
    d = np.diff(s[: k + 1])
    return np.all(np.abs(d) > tol)


@pytest.mark.parametrize("mode", [SQRT_SOFTPLUS, SIGMOID, SOFTMAX])
@pytest.mark.parametrize("E,k", [(64, 6), (256, 8), (384, 8)])
def test_plain_topk_matches_f64_ranking(mode, E, k):
    rng = np.random.default_rng(1000 + 10 * mode + E)
    T = 64
    logits = rng.normal(0, 1.5, (T, E)).astype(np.float32)
    bias = rng.normal(0, 0.01, E).astype(np.float32) if mode == SIGMOID else None
    scale, eps = 2.5, 1e-20
    sel, w = ref.router_topk(logits, bias, k, scale, eps, mode)
    p = probs64(logits, mode)
    s = p + (bias.astype(np.float64) if bias is not None else 0.0)
    checked = 0
    for t in range(T):
        if not gap_ok(s[t], k):
            continue
        checked += 1
        want = topk_stable(s[t], k)
        assert sel[t].tolist() == want.tolist()
        pw = p[t, want]
        np.testing.assert_allclose(w[t], pw / pw.sum() * scale, rtol=2e-6)
    assert checked > T // 2


def test_weights_use_unbiased_probabilities_and_sum_to_scale():
    rng = np.random.default_rng(7)
    E, k = 32, 4
    logits = rng.normal(0, 1, (8, E)).astype(np.float32)
    bias = np.zeros(E, np.float32)
    bias[5] = 10.0  # forces expert 5 into every pick without changing its weight
    sel, w = ref.router_topk(logits, bias, k, 1.0, 1e-20, SIGMOID)
    p = probs64(logits, SIGMOID)
    for t in range(8):
        assert sel[t, 0] == 5
        np.testing.assert_allclose(w[t].sum(), 1.0, rtol=1e-6)
        np.testing.assert_allclose(w[t, 0] / w[t, 1], p[t, 5] / p[t, sel[t, 1]], rtol=1e-5)


def test_ties_go_to_the_lowest_index():
    logits = np.zeros((1, 16), np.float32)
    logits[0, [3, 9, 12]] = 1.0
    for mode in (SQRT_SOFTPLUS, SIGMOID, SOFTMAX):
        sel, w = ref.router_topk(logits, None, 5, 1.0, 1e-20, mode)
        assert sel[0].tolist() == [3, 9, 12, 0, 1]
        assert w[0, 0] == w[0, 1] == w[0, 2] and w[0, 3] == w[0, 4]


def test_weight_sum_floor():
    # sqrt(softplus(-30)) ~ 3e-7 per expert: the sum is below eps, so eps divides
    logits = np.full((1, 8), -30.0, np.float32)
    eps = 6.1035e-5
    sel, w = ref.router_topk(logits, None, 2, 1.5, eps, SQRT_SOFTPLUS)
    p = probs64(logits, SQRT_SOFTPLUS)[0, 0]
    np.testing.assert_allclose(w[0], p / eps * 1.5, rtol=1e-5)


def test_hash_router_select_closed_form_floor_and_empty_slots():
    # crates/v4flash-kernels/src/routing.rs:21-44: picks are the token's row of tid2eid,
    # weights sqrt(softplus(logit)) / max(sum, 6.103515625e-5) * 1.5
    rng = np.random.default_rng(11)
    E, k, vocab, T = 256, 6, 50, 9
    tid2eid = np.stack([rng.choice(E, k, replace=False) for _ in range(vocab)]).astype(np.int32)
    toks = rng.integers(0, vocab, T).astype(np.int32)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[4] = -30.0                                  # sum of p below the floor
    sel, w = ref.router_hash_select(logits, tid2eid, toks)
    assert np.array_equal(sel, tid2eid[toks])
    p = np.take_along_axis(probs64(logits, SQRT_SOFTPLUS), sel.astype(np.int64), axis=1)
    want = p / np.maximum(p.sum(axis=1, keepdims=True), 6.103515625e-5) * 1.5
    np.testing.assert_allclose(w, want, rtol=2e-6)
    np.testing.assert_allclose(np.delete(w, 4, axis=0).sum(axis=1), 1.5, rtol=1e-6)
    assert w[4].sum() < 0.1
    # with the learned router's own picks as the table, the weights are the learned router's
    lsel, lw = ref.router_topk(logits, None, k, 1.5, 6.103515625e-5, SQRT_SOFTPLUS)
    hsel, hw = ref.router_hash_select(logits, lsel, np.arange(T, dtype=np.int32))
    assert np.array_equal(hsel, lsel) and np.array_equal(hw.view(np.uint32), lw.view(np.uint32))
    # ids out of range leave empty slots
    bad = tid2eid.copy()
    bad[toks[0], 2] = E
    bad[toks[0], 3] = -7
    sel2, w2 = ref.router_hash_select(logits[:3], bad, np.concatenate([toks[:1], [vocab, -1]]).astype(np.int32))
    assert sel2[0, 2] == -1 and sel2[0, 3] == -1 and w2[0, 2] == 0 and w2[0, 3] == 0
    np.testing.assert_allclose(w2[0].sum(), 1.5, rtol=1e-6)
    assert (sel2[1:] == -1).all() and (w2[1:] == 0).all()


def test_hetsplit_select_partitions_the_picks():
    # crates/v4flash-kernels/kernels/mxfp4_pair_matvec.hip:231-284: the two sides of the split
    # own disjoint slots that together cover every pick; the mode-1 side owns the first `cap`
    # resident picks of a token in slot order
    rng = np.random.default_rng(31)
    E, k, T = 40, 6, 200
    remap = np.empty(E, np.int32)
    hot = rng.random(E) < 0.5
    remap[hot] = np.arange(hot.sum())                      # dense slots of the resident experts
    remap[~hot] = -(np.arange((~hot).sum()) + 1)           # packed slots of the cold ones
    sel = np.stack([rng.choice(E, k, replace=False) for _ in range(T)]).astype(np.int32)
    sel[3, 2] = -1                                         # an empty slot belongs to nobody
    for cap in (0, 1, 3, 6, 99):
        a = ref.hetsplit_select(sel, remap, 0, cap)
        b = ref.hetsplit_select(sel, remap, 1, cap)
        owned_a, owned_b = a >= 0, b >= 0
        assert not (owned_a & owned_b).any()
        assert np.array_equal(owned_a | owned_b, sel >= 0)
        for t in range(T):
            resident_slots = [s_ for s_ in range(k) if sel[t, s_] >= 0 and hot[sel[t, s_]]]
            want_b = resident_slots[:cap]
            assert [s_ for s_ in range(k) if owned_b[t, s_]] == want_b
            for s_ in range(k):
                e = sel[t, s_]
                if owned_b[t, s_]:
                    assert b[t, s_] == remap[e]            # dense slot on the resident side
                if owned_a[t, s_]:
                    assert a[t, s_] == (e if hot[e] else -remap[e] - 1)
    assert (ref.hetsplit_select(sel, remap, 1, 0) == -1).all()


def test_softmax_matches_numpy():
    rng = np.random.default_rng(11)
    logits = rng.normal(0, 2, (16, 64)).astype(np.float32)
    p, s = ref.router_scores(logits, None, SOFTMAX)
    np.testing.assert_allclose(p, probs64(logits, SOFTMAX), rtol=3e-6, atol=1e-9)
    np.testing.assert_allclose(p.sum(-1), 1.0, rtol=1e-5)
    assert np.array_equal(p, s)


# ---- group-limited top-k ------------------------------------------------------------

def group_limited_bruteforce(p, bias, k, n_group, topk_group):
    """DeepSeek-V3 rule by exhaustive search (float64).

    Among all ways to keep `topk_group` groups, the kept set maximises the sum of group
    scores (group score = sum of the group's two largest biased scores); the picks are the
    k-subset of experts in kept groups with the largest total biased score.
    """
    E = p.shape[0]
    s = p + bias
    per = E // n_group
    gs = [np.sort(s[g * per:(g + 1) * per])[::-1][:2].sum() for g in range(n_group)]
    best_groups = max(itertools.combinations(range(n_group), topk_group),
                      key=lambda c: sum(gs[g] for g in c))
    allowed = [e for g in best_groups for e in range(g * per, (g + 1) * per)]
    best = max(itertools.combinations(allowed, k), key=lambda c: sum(s[e] for e in c))
    return set(best_groups), set(best)


@pytest.mark.parametrize("seed", range(12))
def test_group_limited_matches_exhaustive_search(seed):
    rng = np.random.default_rng(500 + seed)
    E, n_group, topk_group, k = 16, 4, 2, 3
    logits = rng.normal(0, 1, (1, E)).astype(np.float32)
    bias = rng.normal(0, 0.3, E).astype(np.float32)
    sel, w = ref.router_topk(logits, bias, k, 2.5, 1e-20, SIGMOID, n_group, topk_group)
    p = probs64(logits, SIGMOID)[0]
    groups, picks = group_limited_bruteforce(p, bias.astype(np.float64), k, n_group, topk_group)
    assert set(sel[0].tolist()) == picks
    assert {e // (E // n_group) for e in sel[0]} <= groups
    # order: descending biased score; weights: unbiased p renormalised x 2.5
    s = p + bias
    assert np.all(np.diff(s[sel[0]]) <= 0)
    np.testing.assert_allclose(w[0], p[sel[0]] / p[sel[0]].sum() * 2.5, rtol=2e-6)


def test_group_limited_invariants_at_v3_shape():
    rng = np.random.default_rng(3)
    T, E, G, KG, k = 128, 256, 8, 4, 8
    logits = rng.normal(0, 1, (T, E)).astype(np.float32)
    bias = rng.normal(0, 0.01, E).astype(np.float32)
    sel, w = ref.router_topk(logits, bias, k, 2.5, 1e-20, SIGMOID, G, KG)
    p, s = ref.router_scores(logits, bias, SIGMOID, G, KG)
    per = E // G
    for t in range(T):
        assert len(set(sel[t].tolist())) == k
        assert len({e // per for e in sel[t]}) <= KG
        kept = np.isfinite(s[t]).reshape(G, per)
        assert np.all(kept.all(1) | (~kept).all(1)) and kept.all(1).sum() == KG
    np.testing.assert_allclose(w.sum(-1), 2.5, rtol=1e-5)
    # one group, or every group kept: plain top-k
    a = ref.router_topk(logits, bias, k, 2.5, 1e-20, SIGMOID, 1, 1)
    b = ref.router_topk(logits, bias, k, 2.5, 1e-20, SIGMOID, G, G)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


def test_group_limited_differs_from_plain_when_a_strong_expert_sits_in_a_weak_group():
    E, G = 16, 4
    logits = np.full((1, E), -3.0, np.float32)
    logits[0, 0:2] = 2.0     # group 0: two strong
    logits[0, 4:6] = 1.5     # group 1: two fairly strong
    logits[0, 8] = 3.0       # group 2: one very strong, alone -> group score lower
    plain, _ = ref.router_topk(logits, None, 3, 1.0, 1e-20, SIGMOID, 1, 1)
    lim, _ = ref.router_topk(logits, None, 3, 1.0, 1e-20, SIGMOID, G, 2)
    assert 8 in plain[0] and 8 not in lim[0]
    assert set(lim[0].tolist()) <= {0, 1, 4, 5}


def test_router_rejects_bad_arguments():
    logits = np.zeros((1, 8), np.float32)
    with pytest.raises(ValueError):
        ref.router_topk(logits, None, 9, 1.0, 1e-20, SIGMOID)
    with pytest.raises(ValueError):
        ref.router_topk(logits, None, 2, 1.0, 1e-20, SIGMOID, 3, 1)  # 8 % 3 != 0


def test_router_logits_is_a_matvec():
    rng = np.random.default_rng(5)
    W = rng.normal(0, 0.02, (64, 2048)).astype(np.float32)
    x = rng.normal(0, 1, (4, 2048)).astype(np.float32)
    got = ref.router_logits(W, x)
    want = x.astype(np.float64) @ W.astype(np.float64).T
    np.testing.assert_allclose(got, want, rtol=0, atol=2e-5)


# ---- token -> expert inversion --------------------------------------------------------

@pytest.mark.parametrize("T,k,E,chunk", [(1, 8, 256, 4), (7, 6, 64, 4), (64, 8, 256, 8),
                                         (300, 8, 32, 32), (5, 4, 16, 1)])
def test_group_build_is_the_inverse_of_selected(T, k, E, chunk):
    rng = np.random.default_rng(T * 31 + E)
    sel = np.stack([rng.choice(E, k, replace=False) for _ in range(T)]).astype(np.int32)
    if T > 2:
        sel[1, 0] = -1  # an empty slot is skipped
    gc, off, mem, wi = ref.group_build(sel, E, chunk)
    flat = sel.reshape(-1)
    assert np.array_equal(gc, np.bincount(flat[flat >= 0], minlength=E))
    assert np.array_equal(off, np.concatenate([[0], np.cumsum(gc)]))
    seen = set()
    for e in range(E):
        m = mem[off[e]:off[e + 1]]
        assert np.all(np.diff(m) > 0)  # ascending (token, slot)
        for v in m:
            t, s = int(v) >> 16, int(v) & 0xFFFF
            assert sel[t, s] == e
            seen.add((t, s))
    assert len(seen) == int((flat >= 0).sum())
    # work items tile every group in chunks, in (expert, start) order
    want = [(e << 16) | st for e in range(E) for st in range(0, gc[e], chunk)]
    assert wi.tolist() == want
    assert len(want) <= ref.wi_upper_bound(len(seen), E, chunk, 1 << 30)
