"""Pins the oracle's whole-layer composition and the synthetic-tensor generators (CPU only).

The reference pins the layer only against external activation dumps that are not available,
so the composition is pinned here by
  * an independent float64 forward over DEQUANTIZED weights (numpy matmuls; no quantized
    dot product, no shared code with the oracle's inner loops): catches a dropped term, a
    transposed operand, a wrong slot/expert index or a misplaced expert weight;
  * identities the reference's own tests rely on: splitting the picks into two disjoint
    sets and adding the results (crates/v4flash-kernels/tests/mxfp4_pair_oracle.rs:198-241),
    per-token == batched (crates/v4flash-kernels/tests/mtp_moe_grouped.rs:6-15), token
    permutation, empty slots.
"""
import numpy as np
import pytest

from deepstrix_amd import synth
from deepstrix_amd.capi import FMT_MXFP4, FMT_Q8_0
from oracle import ref
from tests.helpers import Shape, host_inputs, host_weights, max_rel, oracle_route

SHAPES = {
    "mxfp4": Shape(512, 256, 8, 3, clamp=7.0, seed=11),
    "q8_0": Shape(256, 96, 8, 3, FMT_Q8_0, FMT_Q8_0, clamp=0.0, seed=12),
    "mixed": Shape(512, 256, 8, 2, FMT_MXFP4, FMT_Q8_0, clamp=7.0, seed=13),
    "no_shared": Shape(256, 256, 6, 2, shared=False, seed=14),
}


def dequant(fmt, buf, rows, cols):
    if fmt == FMT_MXFP4:
        return ref.mxfp4_dequant_v2(buf, rows, cols).astype(np.float64)
    return ref.q8_0_dequant_rows(buf, rows, cols).astype(np.float64)


def act_roundtrip(fmt, v):
    """The activation quantizer the matrix format implies, as a value round trip."""
    v = np.ascontiguousarray(v, np.float32)
    if fmt == FMT_MXFP4:
        return ref.q8k_dequant(ref.q8k_quantize(v)).astype(np.float64)
    q, d = ref.q8_0_quantize_act(v)
    return (q.reshape(-1, 32).astype(np.float64) * d[:, None].astype(np.float64)).reshape(-1)


def ffn64(gfmt, dfmt, g, u, d, x, ew, clamp):
    xq = act_roundtrip(gfmt, x)
    gv, uv = g @ xq, u @ xq
    if clamp > 1e-6:
        gv = np.minimum(gv, clamp)
        uv = np.clip(uv, -clamp, clamp)
    mid = gv / (1.0 + np.exp(-gv)) * uv * ew
    return d @ act_roundtrip(dfmt, mid.astype(np.float32))


def layer64(s: Shape, w: ref.MoeWeights, x, sel, wts):
    gb = synth.matrix_bytes(s.gate_fmt, s.inter, s.hidden)
    db = synth.matrix_bytes(s.down_fmt, s.hidden, s.inter)
    out = np.zeros((x.shape[0], s.hidden))
    cache = {}

    def expert(e):
        if e not in cache:
            cache[e] = (dequant(s.gate_fmt, w.gate[e * gb:(e + 1) * gb], s.inter, s.hidden),
                        dequant(s.gate_fmt, w.up[e * gb:(e + 1) * gb], s.inter, s.hidden),
                        dequant(s.down_fmt, w.down[e * db:(e + 1) * db], s.hidden, s.inter))
        return cache[e]

    for t in range(x.shape[0]):
        for j in range(s.n_used):
            e = int(sel[t, j])
            if e < 0:
                continue
            g, u, d = expert(e)
            out[t] += ffn64(s.gate_fmt, s.down_fmt, g, u, d, x[t], float(wts[t, j]), s.clamp)
        if s.shared:
            out[t] += ffn64(s.shg, s.shd, dequant(s.shg, w.sh_gate, s.inter, s.hidden),
                            dequant(s.shg, w.sh_up, s.inter, s.hidden),
                            dequant(s.shd, w.sh_down, s.hidden, s.inter), x[t], 1.0, s.clamp)
    return out


@pytest.fixture(scope="module", params=list(SHAPES))
def case(request):
    s = SHAPES[request.param]
    w = host_weights(s)
    T = 5
    x, logits, bias = host_inputs(s, T)
    x = x * 3.0  # push some gate/up products past the clamp
    sel, wts = oracle_route(s, logits, bias)
    return s, w, x.astype(np.float32), sel, wts


def test_layer_matches_independent_f64_forward(case):
    s, w, x, sel, wts = case
    got = ref.moe_forward(w, x, sel, wts)
    want = layer64(s, w, x, sel, wts)
    # both sides see the same quantized activations; what differs is f32 vs f64 summation
    assert max_rel(got, want) < 2e-5


def test_parts_add_up(case):
    s, w, x, sel, wts = case
    out, mid, moe, shared = ref.moe_forward(w, x, sel, wts, want_parts=True)
    assert mid.shape == (x.shape[0], s.n_used, s.inter)
    np.testing.assert_array_equal(out, moe + shared)
    if not s.shared:
        assert not shared.any()


def test_per_token_equals_batched_bitwise(case):
    s, w, x, sel, wts = case
    whole = ref.moe_forward(w, x, sel, wts)
    for t in range(x.shape[0]):
        one = ref.moe_forward(w, x[t:t + 1], sel[t:t + 1], wts[t:t + 1])
        np.testing.assert_array_equal(one[0], whole[t])


def test_token_permutation(case):
    s, w, x, sel, wts = case
    perm = np.array([3, 0, 4, 2, 1])
    a = ref.moe_forward(w, x, sel, wts)
    b = ref.moe_forward(w, x[perm], sel[perm], wts[perm])
    np.testing.assert_array_equal(a[perm], b)


def test_pick_set_split_adds_up(case):
    s, w, x, sel, wts = case
    _, _, moe, _ = ref.moe_forward(w, x, sel, wts, want_parts=True)
    sel_a, sel_b = sel.copy(), sel.copy()
    sel_a[:, 1:] = -1
    sel_b[:, :1] = -1
    _, _, moe_a, _ = ref.moe_forward(w, x, sel_a, wts, want_parts=True)
    _, _, moe_b, _ = ref.moe_forward(w, x, sel_b, wts, want_parts=True)
    assert max_rel(moe_a + moe_b, moe) < 1e-6


def test_threads_do_not_change_results(case):
    s, w, x, sel, wts = case
    a = ref.moe_forward(w, x, sel, wts, n_threads=1)
    b = ref.moe_forward(w, x, sel, wts, n_threads=ref.max_threads())
    np.testing.assert_array_equal(a, b)


def test_expert_weight_is_applied_before_the_second_quantization():
    # crates/v4flash-kernels/src/het/forward_layer.rs:456-466: mid carries the routing
    # weight into the Q8_K quantizer, so scaling the weight by 2^n scales the output exactly
    s = SHAPES["no_shared"]
    w = host_weights(s)
    x, logits, bias = host_inputs(s, 2)
    sel, wts = oracle_route(s, logits, bias)
    a = ref.moe_forward(w, x, sel, wts)
    b = ref.moe_forward(w, x, sel, wts * 4.0)
    np.testing.assert_array_equal(a * 4.0, b)


# ---- synthetic tensors ------------------------------------------------------------------

def test_config1_fixture_is_what_the_oracle_computes():
    """tests/golden/cfg1_T4.npz freezes the oracle's config-1 result (inputs from seeds)."""
    import importlib.util
    import os
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    spec = importlib.util.spec_from_file_location("make_cfg1_fixture", os.path.join(here, "make_cfg1_fixture.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    now = mod.compute()
    with np.load(os.path.join(here, "cfg1_T4.npz"), allow_pickle=False) as g:
        assert np.array_equal(g["sel"], now["sel"])
        # expf / logf of another libm may differ in the last bit; everything else is exact
        np.testing.assert_allclose(now["logits"], g["logits"], rtol=1e-6, atol=1e-7)
        np.testing.assert_allclose(now["w"], g["w"], rtol=1e-6)
        np.testing.assert_allclose(now["out"], g["out"], rtol=1e-5, atol=1e-7)


def test_synth_normal_moments_and_determinism():
    a = synth.normal_host(1, synth.T_X, 1 << 16)
    b = synth.normal_host(1, synth.T_X, 1 << 16)
    c = synth.normal_host(1, synth.T_X, 1 << 15, offset=1 << 15)
    np.testing.assert_array_equal(a, b)
    np.testing.assert_array_equal(a[1 << 15:], c)  # a pure function of the element index
    assert abs(a.mean()) < 0.02 and abs(a.std() - 1.0) < 0.02
    assert abs(((a - a.mean()) ** 4).mean() / a.var() ** 2 - 3.0) < 0.2
    assert not np.array_equal(a, synth.normal_host(2, synth.T_X, 1 << 16))


@pytest.mark.parametrize("fmt,cols", [(FMT_MXFP4, 512), (FMT_Q8_0, 96)])
def test_synth_weights_are_the_oracle_quantizer_applied_to_the_normals(fmt, cols):
    rows, seed, sigma = 24, 77, 0.02
    got = synth.weights_host(fmt, seed, synth.T_UP, rows, cols, sigma, first_row=5)
    x = synth.normal_host(seed, synth.T_UP, rows * cols, sigma, offset=5 * cols).reshape(rows, cols)
    want = ref.mxfp4_quantize_v2(x) if fmt == FMT_MXFP4 else ref.q8_0_quantize_rows(x)
    np.testing.assert_array_equal(got, want.reshape(-1))


def test_matrix_bytes_rejects_ragged_rows():
    with pytest.raises(ValueError):
        synth.matrix_bytes(FMT_MXFP4, 16, 64)
    with pytest.raises(ValueError):
        synth.matrix_bytes(FMT_Q8_0, 16, 48)
    assert synth.matrix_bytes(FMT_MXFP4, 2048, 7168) == 7_798_784
    assert synth.matrix_bytes(FMT_Q8_0, 7168, 2048) == 15_597_568
