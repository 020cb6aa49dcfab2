"""dsx_moe_layer_forward_noalloc (the entry point that takes no workspace: its scratch is a
fixed array inside the library) against dsx_moe_layer_forward, through the C ABI."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

from deepstrix_amd import capi
from deepstrix_amd.executor import MoeLayer
from tests import helpers as H

pytestmark = pytest.mark.gpu

NOALLOC_BYTES = 8 << 20  # DSX_NOALLOC_SCRATCH_BYTES


def _pair(layer, s, T, seed_shift):
    """(existing entry point, no-workspace entry point) on the same seeded inputs."""
    s2 = H.Shape(**{**s.__dict__, "seed": s.seed + seed_shift})
    x, logits, _ = H.host_inputs(s2, T)
    dx, dl = torch.from_numpy(x).cuda(), torch.from_numpy(logits).cuda()
    want, wsel, ww = layer.run(dx, dl, want_routing=True)
    torch.cuda.synchronize()
    out = torch.full((T, s.hidden), float("nan"), dtype=torch.float32, device="cuda")
    sel = torch.full((T, s.n_used), -7, dtype=torch.int32, device="cuda")
    w = torch.full((T, s.n_used), float("nan"), dtype=torch.float32, device="cuda")
    layer.run_noalloc(dx, dl, out, selected_out=sel, weights_out=w)
    torch.cuda.synchronize()
    return (want, wsel, ww), (out, sel, w)


@pytest.mark.parametrize("shape", ["v3", "small"])
def test_noalloc_entry_point_matches_the_workspace_one_on_two_calls_in_a_row(shape):
    """Two calls in a row on the shared array, the second with fewer tokens (its regions are
    carved differently, over what the first call left behind): routing bit-exact, outputs
    bitwise equal to dsx_moe_layer_forward's -- same kernels, same order of operations."""
    if shape == "v3":
        s, t_first, t_second = H.CFG2, 12, 1
    else:
        s = H.Shape(1024, 512, 16, 4, router_mode=1, n_group=4, topk_group=2, route_scale=2.5,
                    bias_sigma=0.01, clamp=10.0, seed=4242)
        t_first, t_second = 40, 3          # by-expert path first, decode kernels second
    dw = H.device_weights(s)
    layer = MoeLayer(dw, t_first)
    assert capi.lib().dsx_moe_layer_workspace_bytes(layer._h, t_first) <= NOALLOC_BYTES
    for i, T in enumerate((t_first, t_second)):
        (want, wsel, ww), (out, sel, w) = _pair(layer, s, T, i)
        assert torch.equal(sel, wsel), f"call {i} (T={T}): picks differ"
        assert torch.equal(w, ww), f"call {i} (T={T}): routing weights differ"
        assert torch.isfinite(out).all()
        assert torch.equal(out, want), (
            f"call {i} (T={T}): max |diff| = {(out - want).abs().max().item():.3e}")


def test_noalloc_entry_point_refuses_what_does_not_fit():
    s = H.Shape(1024, 512, 16, 4, seed=4243)
    dw = H.device_weights(s)
    layer = MoeLayer(dw, 4)
    T = 4096
    assert capi.lib().dsx_moe_layer_workspace_bytes(layer._h, T) > NOALLOC_BYTES
    x = torch.zeros((T, s.hidden), dtype=torch.float32, device="cuda")
    lg = torch.zeros((T, s.n_expert), dtype=torch.float32, device="cuda")
    out = torch.zeros((T, s.hidden), dtype=torch.float32, device="cuda")
    with pytest.raises(capi.DsxError) as e:
        layer.run_noalloc(x, lg, out)
    assert e.value.code == capi.ERR_UNSUPPORTED and "scratch" in e.value.message
