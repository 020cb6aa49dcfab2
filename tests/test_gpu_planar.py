"""The planar form of MXFP4 matrices (DSX_FMT_MXFP4_PLANAR): the same bytes in another order.

The conversion is checked against the permutation written out in numpy, and every path of the
layer must then give bit-identical results on planar weights and on the engine's rows (same
products, same order of sums); one case per path is also compared with the CPU oracle.  The
reference has no such layout, so there is no reference vector: the pin is the equality with the
row layout, which the other GPU tests compare with the oracle.
"""
import numpy as np
import pytest

from deepstrix_amd.capi import FMT_MXFP4, FMT_MXFP4_PLANAR, FMT_Q8_0, DsxError
from oracle import ref
from tests import helpers as H

pytestmark = pytest.mark.gpu


def planar_of(rows_bytes: np.ndarray, n_rows: int, n_sb: int) -> np.ndarray:
    """One matrix, tile by tile of 16 rows: [row][sb][128 nibble bytes | 8 scales] ->
    [row][sb][128] then [sb][row][8]."""
    m = rows_bytes.reshape(n_rows // 16, 16, n_sb, 136)
    nib = m[:, :, :, :128].reshape(n_rows // 16, -1)
    sc = m[:, :, :, 128:].transpose(0, 2, 1, 3).reshape(n_rows // 16, -1)
    return np.concatenate([nib, sc], axis=1).reshape(-1)


def test_conversion_is_the_permutation_and_round_trips():
    import torch
    from deepstrix_amd import dispatch
    n_rows, cols, n_mat, gap = 48, 768, 5, 272
    n_sb = cols // 256
    mat = n_rows * n_sb * 136
    stride = mat + gap
    rng = np.random.default_rng(7)
    host = rng.integers(0, 256, n_mat * stride, dtype=np.uint8)
    dev = torch.from_numpy(host.copy()).cuda()
    dispatch.mxfp4_rows_to_planar(dev, n_rows, cols, n_mat, stride)
    got = dev.cpu().numpy()
    for i in range(n_mat):
        a = i * stride
        np.testing.assert_array_equal(got[a:a + mat], planar_of(host[a:a + mat], n_rows, n_sb))
        np.testing.assert_array_equal(got[a + mat:a + stride], host[a + mat:a + stride])  # the gap is untouched
    dispatch.mxfp4_planar_to_rows(dev, n_rows, cols, n_mat, stride)
    np.testing.assert_array_equal(dev.cpu().numpy(), host)


def test_conversion_rejects_bad_shapes():
    import torch
    from deepstrix_amd import dispatch
    w = torch.zeros(40 * 136, dtype=torch.uint8, device="cuda")
    with pytest.raises(DsxError):
        dispatch.mxfp4_rows_to_planar(w, 40, 256, 1)         # rows % 16
    with pytest.raises(DsxError):
        dispatch.mxfp4_rows_to_planar(w, 32, 128, 1)         # cols % 256
    with pytest.raises(DsxError):
        dispatch.mxfp4_rows_to_planar(w, 32, 256, 2, 1000)   # stride below one matrix
    with pytest.raises(DsxError):
        dispatch.mxfp4_rows_to_planar(w, 16, 256 * 80, 1)    # a tile that LDS does not hold


SMALL = dict(router_mode=1, n_group=4, topk_group=2, route_scale=2.5, bias_sigma=0.01, clamp=10.0)
SHAPES = {
    # every MXFP4 kernel family: the one-launch decode (8 super-blocks in: the straight-line form),
    # the by-expert kernels, the grouped GEMMs
    "all_mxfp4": H.Shape(1024, 2048, 16, 4, seed=41, **SMALL),
    # ... and the general form of the decode kernel (6 super-blocks in)
    "all_mxfp4_nsb6": H.Shape(1024, 1536, 16, 4, seed=42, **SMALL),
    # Q8_0 down: the MXFP4 gate/up GEMM writes f32 mid rows
    "q8_down": H.Shape(1024, 512, 16, 4, FMT_MXFP4, FMT_Q8_0, seed=43, **SMALL),
    # the reference's own mix: Q8_0 shared expert beside MXFP4 routed ones
    "q8_shared": H.Shape(1024, 512, 16, 4, sh_gate_fmt=FMT_Q8_0, sh_down_fmt=FMT_Q8_0, sh_inter=256,
                         seed=44, **SMALL),
    # an MXFP4 shared expert of another width: the dense kernels on planar weights
    "wide_shared": H.Shape(1024, 512, 16, 4, sh_inter=768, seed=45, **SMALL),
    "no_shared": H.Shape(1024, 512, 16, 4, shared=False, seed=46, **SMALL),
}
TOKENS = [1, 2, 3, 4, 7, 11, 12, 16, 17, 40, 99, 100, 130, 300]
PLANAR_TUNING = dict(gemm_min_tokens=17, decode_max_tokens=11, gemm_narrow_members=14)


def _run(layer, s, T):
    import torch
    x, logits, _ = H.host_inputs(s, T)
    out, sel, w = layer.run(torch.from_numpy(x).cuda(), torch.from_numpy(logits).cuda(), want_routing=True)
    torch.cuda.synchronize()
    assert layer.status() == 0
    return out.cpu().numpy(), sel.cpu().numpy(), w.cpu().numpy(), x


@pytest.mark.parametrize("name", sorted(SHAPES))
def test_layer_is_bitwise_the_same_on_planar_weights(name):
    from deepstrix_amd.executor import MoeLayer
    s = SHAPES[name]
    rows = MoeLayer(H.device_weights(s), max(TOKENS))
    dwp = H.device_weights(s, planar=True)
    assert dwp.gate_fmt == FMT_MXFP4_PLANAR
    planar = MoeLayer(dwp, max(TOKENS))
    # a planar layer has its own thresholds (decode up to 11 tokens, then the grouped GEMMs, narrow
    # tile first): the row layout follows them here, so that both run the same kernels at every
    # token count
    if s.down_fmt == FMT_MXFP4:   # (a layer with a Q8_0 matrix keeps the row layout's thresholds)
        rows.set_tuning(**PLANAR_TUNING)
    hw = H.host_weights(s)
    for T in TOKENS:
        a, sel_a, w_a, x = _run(rows, s, T)
        b, sel_b, w_b, _ = _run(planar, s, T)
        np.testing.assert_array_equal(sel_a, sel_b)
        np.testing.assert_array_equal(a.view(np.uint32), b.view(np.uint32), err_msg=f"{name} T={T}")
        if T in (1, 4, 12, 40, 130):
            want = ref.moe_forward(hw, x, sel_b, w_b)
            H.assert_close(b, want, 2e-3, f"{name} planar T={T}")


@pytest.mark.parametrize("fused", [2, 3, 4])
def test_decode_modes_on_planar_weights(fused):
    """Per-stage decode kernels (2) and the one-launch form without (3) and with pairing from two
    tokens on (4)."""
    from deepstrix_amd.executor import MoeLayer
    s = SHAPES["all_mxfp4"]
    rows = MoeLayer(H.device_weights(s), 16)
    planar = MoeLayer(H.device_weights(s, planar=True), 16)
    rows.set_decode(fused)
    planar.set_decode(fused)
    planar.set_tuning(decode_max_tokens=16)   # (a planar layer leaves the decode path at 12 tokens)
    for T in (1, 2, 5, 12, 16):
        a, _, _, _ = _run(rows, s, T)
        b, _, _, _ = _run(planar, s, T)
        np.testing.assert_array_equal(a.view(np.uint32), b.view(np.uint32), err_msg=f"fused={fused} T={T}")


def test_block_and_noalloc_entry_points_on_planar_weights():
    """The residual block (norm, router matvec, layer, residual add) and the entry point without a
    workspace run the same kernels on planar weights: bit for bit the row layout's results."""
    import torch
    from deepstrix_amd.executor import MoeLayer
    s = SHAPES["all_mxfp4"]
    rows = MoeLayer(H.device_weights(s, block=True), 130)
    planar = MoeLayer(H.device_weights(s, block=True, planar=True), 130)
    rows.set_tuning(**PLANAR_TUNING)
    for T in (1, 3, 20, 130):
        h, logits, _ = H.host_inputs(s, T)
        a, b = torch.from_numpy(h.copy()).cuda(), torch.from_numpy(h.copy()).cuda()
        rows.block(a)
        planar.block(b)
        torch.cuda.synchronize()
        assert torch.equal(a, b), f"block T={T}"
    for T in (1, 5):
        x, logits, _ = H.host_inputs(s, T)
        dx, dl = torch.from_numpy(x).cuda(), torch.from_numpy(logits).cuda()
        want = rows.run(dx, dl)
        got = torch.full((T, s.hidden), float("nan"), dtype=torch.float32, device="cuda")
        planar.run_noalloc(dx, dl, got)
        torch.cuda.synchronize()
        assert planar.status(builtin_scratch=True) == 0
        assert torch.equal(want, got), f"noalloc T={T}"


@pytest.mark.parametrize("name", ["all_mxfp4", "q8_shared", "q8_down"])
def test_a_layer_switches_its_own_weights_over_and_back(name):
    """dsx_moe_layer_weights_to_planar on a layer made on the engine's rows: the buffers become
    what the conversion entry point makes of them, the layer computes what a layer created on
    planar weights computes, and the way back restores the bytes."""
    import torch
    from deepstrix_amd.executor import MoeLayer
    s = SHAPES[name]
    dw = H.device_weights(s)
    before = dw.gate.clone()
    layer = MoeLayer(dw, 130)
    want_planar = H.device_weights(s, planar=True)
    ref_layer = MoeLayer(want_planar, 130)
    layer.weights_to_planar()
    torch.cuda.synchronize()
    assert torch.equal(dw.gate, want_planar.gate) and torch.equal(dw.down, want_planar.down)
    assert dw.gate_fmt == want_planar.gate_fmt and dw.down_fmt == want_planar.down_fmt
    for T in (1, 14, 60, 130):
        a, _, _, _ = _run(layer, s, T)
        b, _, _, _ = _run(ref_layer, s, T)
        np.testing.assert_array_equal(a.view(np.uint32), b.view(np.uint32), err_msg=f"{name} T={T}")
    layer.weights_to_planar()   # a second call changes nothing
    torch.cuda.synchronize()
    assert torch.equal(dw.gate, want_planar.gate)
    layer.weights_to_rows()
    torch.cuda.synchronize()
    assert torch.equal(dw.gate, before) and dw.gate_fmt == FMT_MXFP4


def test_a_layer_whose_tensors_share_memory_is_not_converted():
    """gate and up over the same bytes would be rewritten twice: refused before anything moves."""
    import torch
    from deepstrix_amd.executor import MoeLayer
    s = SHAPES["all_mxfp4"]
    dw = H.device_weights(s)
    dw.up = dw.gate
    before = dw.gate.clone()
    layer = MoeLayer(dw, 4)
    with pytest.raises(DsxError):
        layer.weights_to_planar()
    torch.cuda.synchronize()
    assert torch.equal(dw.gate, before)


def test_a_layer_with_both_layouts_is_refused():
    from deepstrix_amd.executor import MoeLayer
    s = SHAPES["all_mxfp4"]
    dw = H.device_weights(s, planar=True)
    dw.down_fmt = FMT_MXFP4   # claims the engine's rows for one tensor
    with pytest.raises(DsxError):
        MoeLayer(dw, 4)


def test_v3_shape_planar_against_rows():
    """BASELINE's shape (7168 x 2048, 256 experts, top-8 + shared expert): decode and the grouped
    GEMMs with ragged groups, bit for bit against the row layout."""
    from deepstrix_amd.executor import MoeLayer
    s = H.CFG2
    rows = MoeLayer(H.device_weights(s), 600)
    planar = MoeLayer(H.device_weights(s, planar=True), 600)
    rows.set_tuning(**PLANAR_TUNING)
    for T in (1, 6, 33, 48, 600):
        a, _, _, _ = _run(rows, s, T)
        b, _, _, _ = _run(planar, s, T)
        np.testing.assert_array_equal(a.view(np.uint32), b.view(np.uint32), err_msg=f"T={T}")
