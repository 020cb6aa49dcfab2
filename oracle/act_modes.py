"""Activation formats side by side on the CPU: what the MoE output would be if the expert
inputs were FP8 (E4M3, one UE8M0 scale per 32 values -- DeepSeek's own activation format,
/root/reference/docs/v41/ARCH_SPEC.md:131-133, rule restated from
/root/reference/scripts/v41_oracle/kernel.py:85-106) instead of the engine's Q8_K int8 blocks
(/root/reference/crates/v4flash-kernels/kernels/q8_k_quantize.hip:23-90).

TEST INFRASTRUCTURE ONLY (like the rest of oracle/): a float64 forward over dequantized weights,
parameterised by the activation round trip.  It answers one design question -- can a
single-instruction FP4 x FP8 product replace the exact two-plane int8 product and stay inside
the 2e-3 parity bar -- and is run by tests/test_oracle_act_modes.py and by
`python -m oracle.act_modes` (the table quoted in the design notes).
"""
from __future__ import annotations

import numpy as np

from oracle import ref

E4M3_MAX = 448.0


def e4m3_round(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even onto the OCP FP8 E4M3 grid (no infinities, max 448), f32 in and out.
    Values are expected pre-clamped to [-448, 448].  Pure numpy: 3 mantissa bits above 2^-6,
    a fixed step of 2^-9 below (subnormals)."""
    x = np.asarray(x, np.float64)
    a = np.abs(x)
    e = np.floor(np.log2(np.maximum(a, 2.0 ** -9)))
    e = np.maximum(e, -6.0)                       # subnormal range shares the exponent of 2^-6
    step = 2.0 ** (e - 3.0)
    q = np.rint(a / step) * step                  # np.rint rounds half to even
    return (np.sign(x) * np.minimum(q, E4M3_MAX)).astype(np.float32)


def fp8_ue8m0_roundtrip(x: np.ndarray, block: int = 32) -> np.ndarray:
    """x -> dequantized FP8 with a power-of-two scale per `block` values:
    amax floored at 1e-4, s = 2^ceil(log2(amax / 448)), q = e4m3(clamp(x / s, +-448))."""
    x = np.asarray(x, np.float32)
    g = x.reshape(-1, block).astype(np.float64)
    amax = np.maximum(np.abs(g).max(axis=1, keepdims=True), 1e-4)
    s = np.exp2(np.ceil(np.log2(amax / E4M3_MAX)))
    q = e4m3_round(np.clip(g / s, -E4M3_MAX, E4M3_MAX)).astype(np.float64)
    return (q * s).reshape(x.shape)


def int8_pow2_roundtrip(x: np.ndarray, block: int) -> np.ndarray:
    """x -> dequantized int8 with a POWER-OF-TWO scale per `block` values: s = 2^ceil(log2(amax / 127)),
    q = rint(x / s) (|q| <= 127 by construction).  The question behind it: such a scale could ride
    the matrix instruction's E8M0 operand, so that the sums over a row chain through the
    instruction's accumulator instead of being folded per block on the vector ALU."""
    x = np.asarray(x, np.float32)
    g = x.reshape(-1, block).astype(np.float64)
    amax = np.abs(g).max(axis=1, keepdims=True)
    s = np.exp2(np.ceil(np.log2(np.maximum(amax, 1e-30) / 127.0)))
    q = np.clip(np.rint(g / s), -127, 127)
    return (q * s).reshape(x.shape)


def q8k_roundtrip(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    return ref.q8k_dequant(ref.q8k_quantize(x)).astype(np.float64)


ACT_MODES = {
    "q8_k": q8k_roundtrip,                      # the engine's (and this library's) arithmetic
    "fp8_ue8m0_32": fp8_ue8m0_roundtrip,        # one-plane FP8 operand
    "int8_pow2_256": lambda v: int8_pow2_roundtrip(v, 256),   # int8, power-of-two scale per Q8_K block
    "int8_pow2_32": lambda v: int8_pow2_roundtrip(v, 32),     # ... per 32 values (the instruction's scale group)
    "none": lambda v: np.asarray(v, np.float64),  # unquantized activations
}


def _ffn(g, u, d, x, ew, clamp, act):
    xq = act(x)
    gv, uv = g @ xq, u @ xq
    if clamp > 1e-6:
        gv = np.minimum(gv, clamp)
        uv = np.clip(uv, -clamp, clamp)
    mid = gv / (1.0 + np.exp(-gv)) * uv * ew
    return d @ act(mid.astype(np.float32))


def layer_outputs(w: ref.MoeWeights, x: np.ndarray, sel: np.ndarray, wts: np.ndarray, modes):
    """{mode: out[T, hidden] float64} for an all-MXFP4 layer; each expert is dequantized once."""
    gb = ref.matrix_bytes(ref.FMT_MXFP4, w.inter, w.hidden)
    db = ref.matrix_bytes(ref.FMT_MXFP4, w.hidden, w.inter)
    T = x.shape[0]
    out = {m: np.zeros((T, w.hidden)) for m in modes}
    users = {}
    for t in range(T):
        for j in range(w.n_used):
            e = int(sel[t, j])
            if e >= 0:
                users.setdefault(e, []).append((t, float(wts[t, j])))

    def deq(buf, rows, cols):
        return ref.mxfp4_dequant_v2(buf, rows, cols).astype(np.float64)

    for e, lst in sorted(users.items()):
        g = deq(w.gate[e * gb:(e + 1) * gb], w.inter, w.hidden)
        u = deq(w.up[e * gb:(e + 1) * gb], w.inter, w.hidden)
        d = deq(w.down[e * db:(e + 1) * db], w.hidden, w.inter)
        for t, ew in lst:
            for m in modes:
                out[m][t] += _ffn(g, u, d, x[t], ew, w.clamp, ACT_MODES[m])
    if w.sh_inter:
        g, u = deq(w.sh_gate, w.sh_inter, w.hidden), deq(w.sh_up, w.sh_inter, w.hidden)
        d = deq(w.sh_down, w.hidden, w.sh_inter)
        for t in range(T):
            for m in modes:
                out[m][t] += _ffn(g, u, d, x[t], 1.0, w.sh_clamp, ACT_MODES[m])
    return out


def compare(a: np.ndarray, b_ref: np.ndarray) -> dict:
    """The reference harness's statistics (scratch/kernel_ideas/_infra/kbench.h:249-270):
    max_abs, max_rel (elementwise, where |ref| is not tiny), rmse / ref_rms, and the parity
    metric max|a - ref| / max|ref|."""
    a, b_ref = np.asarray(a, np.float64), np.asarray(b_ref, np.float64)
    d = np.abs(a - b_ref)
    big = np.abs(b_ref) > 1e-3 * np.abs(b_ref).max()
    return {"max_abs": float(d.max()),
            "max_rel_elementwise": float((d[big] / np.abs(b_ref[big])).max()),
            "rel_rmse": float(np.sqrt((d ** 2).mean()) / np.sqrt((b_ref ** 2).mean())),
            "max_over_max": float(d.max() / np.abs(b_ref).max())}


def study(shape, T: int):
    """Errors of the one-plane FP8, of int8 with power-of-two scales (per 256 and per 32 values) and
    of unquantized activations against the Q8_K result, on the
    seeded inputs and GPU-independent oracle routing of `shape` (a tests.helpers.Shape)."""
    from tests import helpers as H
    x, logits, bias = H.host_inputs(shape, T)
    sel, wts = H.oracle_route(shape, logits, bias)
    w = H.host_weights(shape, experts=np.unique(sel))
    outs = layer_outputs(w, x, sel, wts, ("q8_k", "fp8_ue8m0_32", "int8_pow2_256", "int8_pow2_32", "none"))
    return {"fp8_ue8m0_32 vs q8_k": compare(outs["fp8_ue8m0_32"], outs["q8_k"]),
            "int8_pow2_256 vs q8_k": compare(outs["int8_pow2_256"], outs["q8_k"]),
            "int8_pow2_32 vs q8_k": compare(outs["int8_pow2_32"], outs["q8_k"]),
            "q8_k vs unquantized": compare(outs["q8_k"], outs["none"]),
            "int8_pow2_256 vs unquantized": compare(outs["int8_pow2_256"], outs["none"]),
            "int8_pow2_32 vs unquantized": compare(outs["int8_pow2_32"], outs["none"]),
            "fp8_ue8m0_32 vs unquantized": compare(outs["fp8_ue8m0_32"], outs["none"])}


if __name__ == "__main__":
    import json
    import sys
    from tests import helpers as H
    T = int(sys.argv[1]) if len(sys.argv) > 1 else 4
    print(f"config 2 (V3 shape, MXFP4, seeded inputs), T = {T}")
    for k, v in study(H.CFG2, T).items():
        print(f"  {k:30s} {json.dumps({a: float(f'{b:.3e}') for a, b in v.items()})}")
