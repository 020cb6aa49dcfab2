"""GPU parity of the individual operators, through the C ABI, against the CPU oracle."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

from deepstrix_amd import capi, dispatch, synth
from deepstrix_amd.capi import FMT_MXFP4, FMT_Q8_0
from oracle import ref
from tests import helpers as H

pytestmark = pytest.mark.gpu

OUT_TOL = 2e-3  # max|a-b| / max|ref|, the tolerance the parity bar states for fp32 outputs


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_synth_device_equals_host():
    for fmt in (FMT_MXFP4, FMT_Q8_0):
        h = synth.weights_host(fmt, 7, synth.T_UP, 24, 1024, first_row=5)
        d = synth.weights_dev(fmt, 7, synth.T_UP, 24, 1024, first_row=5).cpu().numpy()
        assert np.array_equal(h, d)
    h = synth.normal_host(9, synth.T_X, 5000, 0.5, 0.25, offset=17)
    d = synth.normal_dev(9, synth.T_X, 5000, 0.5, 0.25, offset=17).cpu().numpy()
    assert np.array_equal(h.view(np.uint32), d.view(np.uint32))


def test_q8k_quantize_bit_exact():
    rng = np.random.default_rng(0)
    x = rng.standard_normal(256 * 37).astype(np.float32)
    x[256:512] = 0.0
    x[512:768] = -np.abs(x[512:768])
    x[768] = 3.0
    x[769] = -3.0
    x[770:1024] *= 0.1
    x[1024:1280] *= 1e-3
    x[1280:1536] *= 1e4
    out = torch.zeros(37 * 292, dtype=torch.uint8, device="cuda")
    dispatch.q8k_quantize(out, dev(x), 37)
    assert np.array_equal(out.cpu().numpy(), ref.q8k_quantize(x))


def test_q8_0_quantize_bit_exact():
    rng = np.random.default_rng(1)
    x = rng.standard_normal(32 * 45).astype(np.float32)
    x[32:64] = 0
    xq = torch.zeros(x.size, dtype=torch.int8, device="cuda")
    xs = torch.zeros(45, dtype=torch.float32, device="cuda")
    dispatch.q8_0_quantize(xq, xs, dev(x), 45)
    rq, rs = ref.q8_0_quantize_act(x)
    assert np.array_equal(xq.cpu().numpy(), rq)
    assert np.array_equal(xs.cpu().numpy().view(np.uint32), rs.view(np.uint32))
    rows = torch.zeros(3 * (480 + 60), dtype=torch.uint8, device="cuda")
    dispatch.q8_0_quantize_rows(rows, dev(x), 3, 480)
    got = rows.cpu().numpy().reshape(3, 540)
    for r in range(3):
        assert np.array_equal(got[r, :480].view(np.int8), rq[r * 480:(r + 1) * 480])
        assert np.array_equal(got[r, 480:].view(np.float32).view(np.uint32),
                              rs[r * 15:(r + 1) * 15].view(np.uint32))


@pytest.mark.parametrize("mode,E,k,ng,tg,scale,eps,bias_sigma", [
    (0, 384, 6, 1, 1, 1.5, 6.103515625e-5, 0.05),   # V4.1: sqrt-softplus + bias
    (1, 256, 8, 8, 4, 2.5, 1e-20, 0.01),            # config 2: sigmoid, group-limited
    (1, 256, 10, 1, 1, 2.5, 1e-20, 0.02),           # Laguna: sigmoid top-10
    (2, 64, 6, 1, 1, 1.0, 1e-20, 0.0),              # config 1: softmax
    (1, 16, 4, 4, 2, 1.0, 1e-20, 0.0),
    (0, 500, 8, 1, 1, 1.0, 1e-20, 0.0),             # not a multiple of 64
])
def test_router_matches_oracle(mode, E, k, ng, tg, scale, eps, bias_sigma):
    T = 257
    rng = np.random.default_rng(mode * 100 + E)
    logits = rng.standard_normal((T, E)).astype(np.float32) * 2.0
    logits[0] = 0.0                    # all tied: lowest indices win
    logits[1, :] = -30.0               # softplus / sigmoid tails
    logits[2, :] = 30.0
    bias = (rng.standard_normal(E) * bias_sigma).astype(np.float32) if bias_sigma else None
    sel = torch.full((T, k), -7, dtype=torch.int32, device="cuda")
    w = torch.zeros((T, k), dtype=torch.float32, device="cuda")
    dispatch.router_topk(sel, w, dev(logits), None if bias is None else dev(bias), E, k, scale, eps,
                         T, mode, ng, tg)
    sel, w = sel.cpu().numpy(), w.cpu().numpy()
    rsel, rw = ref.router_topk(logits, bias, k, scale, eps, mode, ng, tg)
    _, scores = ref.router_scores(logits, bias, mode, ng, tg)
    # picks: exact wherever the k-th / (k+1)-th score gap exceeds 1e-4
    assert H.routing_mismatch_explained(sel, rsel, scores, k) == []
    same = np.array([np.array_equal(sel[t], rsel[t]) for t in range(T)])
    assert same.mean() > 0.97
    if bias is None and ng <= 1:
        assert np.array_equal(sel[0], np.arange(k))     # all tied: lowest indices win
    np.testing.assert_allclose(w[same], rw[same], rtol=2e-5, atol=1e-7)
    if ng > 1:
        gs = E // ng
        assert all(len(set((sel[t] // gs).tolist())) <= tg for t in range(T))


def small_case(hidden=512, inter=256, E=8, k=3, seed=11):
    s = H.Shape(hidden, inter, E, k, shared=True, seed=seed, clamp=10.0)
    return s, H.host_weights(s)


def test_gate_up_decode_reads_weights_exactly():
    """A one-hot activation (q = 1 at one position, d = 1) makes mid-before-SwiGLU equal a
    single dequantized weight; with up fixed by a second probe this pins the kernel's
    nibble order, block scales and activation split bit-exactly."""
    s, w = small_case()
    gb = synth.matrix_bytes(FMT_MXFP4, s.inter, s.hidden)
    gate, up = dev(w.gate), dev(w.up)
    sel = dev(np.array([5, 2, 7], np.int32))
    ew = dev(np.ones(3, np.float32))
    wg = ref.mxfp4_dequant_v2(w.gate, s.n_expert * s.inter, s.hidden).reshape(s.n_expert, s.inter, s.hidden)
    wu = ref.mxfp4_dequant_v2(w.up, s.n_expert * s.inter, s.hidden).reshape(s.n_expert, s.inter, s.hidden)
    mid = torch.zeros((3, s.inter), dtype=torch.float32, device="cuda")
    for pos in (0, 1, 15, 16, 17, 31, 32, 255, 256, 300, 511):
        for qv in (1, -128, 127, 16, -1):
            xq = np.zeros(2 * 292, np.uint8)
            for b in range(2):
                xq[b * 292: b * 292 + 4] = np.array([1.0], np.float32).view(np.uint8)
            xq[(pos // 256) * 292 + 4 + pos % 256] = np.int8(qv).view(np.uint8)
            dispatch.moe_gate_up_batch(FMT_MXFP4, mid, gate, up, dev(xq), ew, sel, gb, gb, 3, 0.0,
                                       s.inter, 2)
            got = mid.cpu().numpy().astype(np.float64)
            for j, e in enumerate((5, 2, 7)):
                g = wg[e][:, pos].astype(np.float64) * qv
                u = wu[e][:, pos].astype(np.float64) * qv
                want = g / (1 + np.exp(-g)) * u
                np.testing.assert_allclose(got[j], want, rtol=3e-6, atol=1e-30)


def test_gate_up_and_down_decode_match_oracle():
    s, w = small_case(hidden=1024, inter=256, E=8, k=3)
    gb = synth.matrix_bytes(FMT_MXFP4, s.inter, s.hidden)
    db = synth.matrix_bytes(FMT_MXFP4, s.hidden, s.inter)
    x = synth.normal_host(3, synth.T_X, s.hidden)
    sel = np.array([[6, 0, 3]], np.int32)
    ew = np.array([[0.5, 1.25, 0.75]], np.float32)
    w_no_shared = ref.MoeWeights(**{**w.__dict__, "sh_inter": 0})
    out_ref, mid_ref, _, _ = ref.moe_forward(w_no_shared, x[None], sel, ew, want_parts=True)
    xq = torch.zeros(4 * 292, dtype=torch.uint8, device="cuda")
    dispatch.q8k_quantize(xq, dev(x), 4)
    mid = torch.zeros((3, s.inter), dtype=torch.float32, device="cuda")
    dispatch.moe_gate_up_batch(FMT_MXFP4, mid, dev(w.gate), dev(w.up), xq, dev(ew), dev(sel), gb, gb,
                               3, s.clamp, s.inter, 4)
    assert H.max_rel(mid.cpu().numpy(), mid_ref[0]) < 1e-5
    midq = torch.zeros(3 * 292, dtype=torch.uint8, device="cuda")
    dispatch.q8k_quantize(midq, dev(mid_ref[0]), 3)     # oracle's mid: isolates the down kernel
    out = torch.zeros(s.hidden, dtype=torch.float32, device="cuda")
    dispatch.moe_down_batched(FMT_MXFP4, out, dev(w.down), midq, dev(sel), db, 292, 3, s.hidden, 1)
    assert H.max_rel(out.cpu().numpy(), out_ref[0]) < 1e-5
    # an empty slot contributes nothing and leaves a defined (zero) mid row
    sel2 = np.array([[6, -1, 3]], np.int32)
    out_ref2, mid_ref2, _, _ = ref.moe_forward(w_no_shared, x[None], sel2, ew, want_parts=True)
    mid.fill_(7.0)
    dispatch.moe_gate_up_batch(FMT_MXFP4, mid, dev(w.gate), dev(w.up), xq, dev(ew), dev(sel2), gb, gb,
                               3, s.clamp, s.inter, 4)
    m = mid.cpu().numpy()
    assert not m[1].any() and H.max_rel(m, mid_ref2[0]) < 1e-5
    dispatch.q8k_quantize(midq, dev(mid_ref2[0]), 3)
    dispatch.moe_down_batched(FMT_MXFP4, out, dev(w.down), midq, dev(sel2), db, 292, 3, s.hidden, 1)
    assert H.max_rel(out.cpu().numpy(), out_ref2[0]) < 1e-5


@pytest.mark.parametrize("T,E,k,chunk", [(1, 8, 3, 4), (7, 8, 3, 4), (64, 256, 8, 4), (300, 16, 4, 16),
                                          (33, 8, 8, 1), (700, 16, 4, 64), (4096, 256, 8, 64),
                                          (1000, 5, 3, 7)])
def test_group_build_matches_oracle(T, E, k, chunk):
    rng = np.random.default_rng(T)
    sel = np.stack([rng.choice(E, k, replace=False) for _ in range(T)]).astype(np.int32)
    if T > 2:
        sel[1, 0] = -1          # empty slot is skipped
    gc, off, mem, wi = ref.group_build(sel, E, chunk)
    d_gc = torch.full((E,), -1, dtype=torch.int32, device="cuda")
    d_off = torch.full((E + 1,), -1, dtype=torch.int32, device="cuda")
    d_mem = torch.full((T * k,), -1, dtype=torch.int32, device="cuda")
    d_wi = torch.full((T * k + E,), -1, dtype=torch.int32, device="cuda")
    d_n = torch.full((1,), -1, dtype=torch.int32, device="cuda")
    dispatch.moe_group_build(d_gc, d_off, d_mem, d_wi, d_n, dev(sel), T, k, E, chunk)
    assert np.array_equal(d_gc.cpu().numpy(), gc)
    assert np.array_equal(d_off.cpu().numpy(), off)
    assert np.array_equal(d_mem.cpu().numpy()[: mem.size], mem)
    # the same picks from a buffer that is only 4-byte aligned (no 16-byte loads then)
    shifted = dev(np.concatenate([np.zeros(1, np.int32), sel.ravel()]))[1:]
    d_mem2 = torch.full((T * k,), -1, dtype=torch.int32, device="cuda")
    dispatch.moe_group_build(d_gc, d_off, d_mem2, d_wi, d_n, shifted, T, k, E, chunk)
    assert np.array_equal(d_mem2.cpu().numpy()[: mem.size], mem)
    n = int(d_n.item())
    assert n == wi.size and n <= dispatch.wi_upper_bound(T * k, E, chunk)
    assert np.array_equal(d_wi.cpu().numpy()[:n], wi)
    # every pick appears exactly once
    assert int(gc.sum()) == int((sel >= 0).sum())


# chunk 32 is the reference executor's CHUNK_SIZE (crates/v4flash-kernels/src/het/remote_experts.rs:77):
# a work item wider than one workgroup's columns is served by several workgroups
@pytest.mark.parametrize("T,chunk", [(5, 4), (9, 2), (3, 1), (12, 8), (45, 32), (70, 64), (21, 20)])
def test_by_expert_chain_matches_oracle(T, chunk):
    s, w = small_case(hidden=768, inter=256, E=8, k=3, seed=21)
    gb = synth.matrix_bytes(FMT_MXFP4, s.inter, s.hidden)
    db = synth.matrix_bytes(FMT_MXFP4, s.hidden, s.inter)
    rng = np.random.default_rng(T)
    x = synth.normal_host(5, synth.T_X, T * s.hidden).reshape(T, s.hidden)
    sel = np.stack([rng.choice(s.n_expert, s.n_used, replace=False) for _ in range(T)]).astype(np.int32)
    sel[:, 0] = 4                       # one expert with T members: several work items
    ew = rng.random((T, s.n_used)).astype(np.float32) + 0.25
    w_ns = ref.MoeWeights(**{**w.__dict__, "sh_inter": 0})
    out_ref, mid_ref, _, _ = ref.moe_forward(w_ns, x, sel, ew, want_parts=True)
    k, E = s.n_used, s.n_expert
    nb, nbi = s.hidden // 256, s.inter // 256
    xq = torch.zeros(T * nb * 292, dtype=torch.uint8, device="cuda")
    dispatch.q8k_quantize(xq, dev(x), T * nb)
    gc = torch.zeros(E, dtype=torch.int32, device="cuda")
    off = torch.zeros(E + 1, dtype=torch.int32, device="cuda")
    mem = torch.zeros(T * k, dtype=torch.int32, device="cuda")
    wi = torch.zeros(T * k + E, dtype=torch.int32, device="cuda")
    n = torch.zeros(1, dtype=torch.int32, device="cuda")
    dsel = dev(sel)
    dispatch.moe_group_build(gc, off, mem, wi, n, dsel, T, k, E, chunk)
    max_wi = dispatch.wi_upper_bound(T * k, E, chunk)
    mid = torch.full((T, k, s.inter), np.nan, dtype=torch.float32, device="cuda")
    dispatch.moe_gate_up_chunked_rows(FMT_MXFP4, mid, dev(w.gate), dev(w.up), xq, dev(ew), gc, off, mem,
                                      wi, n, max_wi, gb, gb, k, chunk, s.clamp, s.inter, nb)
    got_mid = mid.cpu().numpy()
    assert np.isfinite(got_mid).all()           # every pick written exactly once
    assert H.max_rel(got_mid, mid_ref) < 1e-5
    midq = torch.zeros(T * k * nbi * 292, dtype=torch.uint8, device="cuda")
    dispatch.q8k_quantize(midq, dev(mid_ref), T * k * nbi)
    partials = torch.full((T * k, s.hidden), np.nan, dtype=torch.float32, device="cuda")
    dispatch.moe_down_by_expert(FMT_MXFP4, partials, dev(w.down), midq, gc, off, mem, wi, n, max_wi, db,
                                nbi * 292, k, chunk, s.hidden, nbi)
    assert np.isfinite(partials.cpu().numpy()).all()
    out = torch.zeros((T, s.hidden), dtype=torch.float32, device="cuda")
    dispatch.moe_reduce_partials(out, partials, dsel, k, s.hidden, T)
    assert H.max_rel(out.cpu().numpy(), out_ref) < 1e-5


def test_hash_router_select_matches_oracle_and_feeds_the_layer():
    # crates/v4flash-kernels/src/routing.rs:21-44, on the device
    rng = np.random.default_rng(12)
    E, k, vocab, T = 256, 6, 129, 300
    tid2eid = np.stack([rng.choice(E, k, replace=False) for _ in range(vocab)]).astype(np.int32)
    tid2eid[5, 1] = E          # out of range: empty slot
    toks = rng.integers(0, vocab, T).astype(np.int32)
    toks[:3] = [5, vocab, -2]
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[7] = -30.0
    sel = torch.full((T, k), 99, dtype=torch.int32, device="cuda")
    w = torch.full((T, k), np.nan, dtype=torch.float32, device="cuda")
    dispatch.router_hash_select(sel, w, dev(logits), dev(tid2eid), dev(toks))
    rsel, rw = ref.router_hash_select(logits, tid2eid, toks)
    assert np.array_equal(sel.cpu().numpy(), rsel)
    np.testing.assert_allclose(w.cpu().numpy(), rw, rtol=2e-6, atol=1e-9)
    # pinned routing: the layer computes with these picks and weights
    s, wts = small_case(hidden=768, inter=256, E=8, k=3, seed=23)
    from deepstrix_amd.executor import MoeLayer
    T2 = 5
    table = np.stack([rng.choice(s.n_expert, s.n_used, replace=False) for _ in range(16)]).astype(np.int32)
    tk = rng.integers(0, 16, T2).astype(np.int32)
    x, lg, _ = H.host_inputs(s, T2)
    dsel = torch.zeros((T2, s.n_used), dtype=torch.int32, device="cuda")
    dw = torch.zeros((T2, s.n_used), dtype=torch.float32, device="cuda")
    dispatch.router_hash_select(dsel, dw, dev(lg), dev(table), dev(tk))
    layer = MoeLayer(H.device_weights(s), T2)
    out = layer.run(dev(x), None, selected_in=dsel, weights_in=dw)
    hsel, hw = ref.router_hash_select(lg, table, tk)
    want = ref.moe_forward(wts, x, hsel, hw)
    assert H.max_rel(out.cpu().numpy(), want) < OUT_TOL


@pytest.mark.parametrize("T", [1, 3, 40])
def test_hetsplit_sides_add_up_to_the_unsplit_layer(T):
    """The reference's het-split identity (crates/v4flash-kernels/tests/mxfp4_pair_oracle.rs:198-241):
    out(side 0) + out(side 1) = out.  Both sides read the same weight buffer here (resident
    experts keep their index as dense slot, cold ones are packed at their own index)."""
    rng = np.random.default_rng(40 + T)
    s = H.Shape(768, 256, 8, 3, shared=False, seed=25, clamp=10.0)
    wts = H.host_weights(s)
    from deepstrix_amd.executor import MoeLayer
    layer = MoeLayer(H.device_weights(s), T)
    x, lg, bias = H.host_inputs(s, T)
    sel, w = H.oracle_route(s, lg, bias)
    hot = rng.random(s.n_expert) < 0.5
    remap = np.where(hot, np.arange(s.n_expert), -(np.arange(s.n_expert) + 1)).astype(np.int32)
    dsel, dw, dx = dev(sel), dev(w), dev(x)
    full = layer.run(dx, None, selected_in=dsel, weights_in=dw).cpu().numpy()
    assert H.max_rel(full, ref.moe_forward(wts, x, sel, w)) < OUT_TOL
    for cap in (1, 2):
        parts = []
        for mode in (0, 1):
            side = torch.full((T, s.n_used), 77, dtype=torch.int32, device="cuda")
            dispatch.moe_hetsplit_select(side, dsel, dev(remap), mode, cap)
            want_side = ref.hetsplit_select(sel, remap, mode, cap)
            assert np.array_equal(side.cpu().numpy(), want_side)
            got = layer.run(dx, None, selected_in=side, weights_in=dw).cpu().numpy()
            assert H.max_rel(got, ref.moe_forward(wts, x, want_side, w)) < OUT_TOL
            parts.append(got)
        assert H.max_rel(parts[0] + parts[1], full) < 1e-5


def test_small_kernels_match_oracle():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((5, 7168)).astype(np.float32)
    wn = (1 + 0.02 * rng.standard_normal(7168)).astype(np.float32)
    out = torch.zeros((5, 7168), dtype=torch.float32, device="cuda")
    dispatch.rms_norm(out, dev(x), dev(wn), 7168, 1e-6, 5)
    np.testing.assert_allclose(out.cpu().numpy(), ref.rms_norm(x, wn, 1e-6), rtol=2e-6, atol=1e-7)
    a, b = rng.standard_normal(1000).astype(np.float32), rng.standard_normal(1000).astype(np.float32)
    da = dev(a)
    dispatch.vec_add_inplace(da, dev(b), 1000)
    assert np.array_equal(da.cpu().numpy(), a + b)
    g = (rng.standard_normal((3, 100)) * 8).astype(np.float32)
    u = (rng.standard_normal((3, 100)) * 8).astype(np.float32)
    ew = rng.random(3).astype(np.float32)
    mid = torch.zeros((3, 100), dtype=torch.float32, device="cuda")
    dispatch.swiglu_clamp_weighted(mid, dev(g), dev(u), dev(ew), 10.0, 100, 3)
    want = np.array([[ref.swiglu(g[e, r], u[e, r], 10.0, ew[e]) for r in range(100)] for e in range(3)])
    np.testing.assert_allclose(mid.cpu().numpy(), want, rtol=2e-6, atol=1e-7)


def test_repack_and_dequant_bit_exact():
    rng = np.random.default_rng(4)
    out_rows, nb = 12, 16
    packed = rng.integers(0, 256, (out_rows, nb * 16), dtype=np.uint8)
    scale = rng.integers(100, 140, (out_rows, nb), dtype=np.uint8)
    dst = torch.zeros(out_rows * nb * 17, dtype=torch.uint8, device="cuda")
    dispatch.mxfp4_repack_hf_to_v2(dst, dev(packed), dev(scale), out_rows, nb)
    v2 = ref.mxfp4_repack_hf_to_v2(packed, scale)
    assert np.array_equal(dst.cpu().numpy(), v2)
    y = torch.zeros((out_rows, nb * 32), dtype=torch.float32, device="cuda")
    dispatch.dequant_rows(FMT_MXFP4, y, dst, out_rows, nb * 32)
    assert np.array_equal(y.cpu().numpy().view(np.uint32),
                          ref.mxfp4_dequant_v2(v2, out_rows, nb * 32).view(np.uint32))
    w8 = synth.weights_host(FMT_Q8_0, 1, synth.T_DOWN, 6, 96)
    y8 = torch.zeros((6, 96), dtype=torch.float32, device="cuda")
    dispatch.dequant_rows(FMT_Q8_0, y8, dev(w8), 6, 96)
    assert np.array_equal(y8.cpu().numpy().view(np.uint32), ref.q8_0_dequant_rows(w8, 6, 96).view(np.uint32))


def test_argument_errors_are_reported_before_launch():
    z = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    f = torch.zeros(4096, dtype=torch.float32, device="cuda")
    i = torch.zeros(16, dtype=torch.int32, device="cuda")
    with pytest.raises(capi.DsxError) as e:
        dispatch.moe_gate_up_batch(FMT_MXFP4, f, z, z, z, f, i, 136, 136, 3, 0.0, 10, 1)
    assert e.value.code == capi.ERR_SHAPE and "multiple of 16" in e.value.message
    with pytest.raises(capi.DsxError) as e:
        dispatch.moe_gate_up_batch(12, f, z, z, z, f, i, 136, 136, 3, 0.0, 16, 1)
    assert e.value.code == capi.ERR_UNSUPPORTED
    with pytest.raises(capi.DsxError) as e:
        dispatch.router_topk(i, f, f, None, 1000, 8, 1.0, 1e-20, 1, 1)
    assert e.value.code == capi.ERR_INVALID_ARG
    with pytest.raises(capi.DsxError) as e:
        dispatch.router_topk(i, f, f, None, 256, 8, 1.0, 1e-20, 1, 1, n_group=7, topk_group=2)
    assert e.value.code == capi.ERR_SHAPE
    # empty problems succeed without touching anything
    dispatch.q8k_quantize(z, f, 0)
    dispatch.router_topk(i, f, f, None, 256, 8, 1.0, 1e-20, 0, 1)
