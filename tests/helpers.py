"""Shared helpers of the test-suite: synthetic layers on host and device, parity metrics."""
from __future__ import annotations

import numpy as np

from deepstrix_amd import synth
from deepstrix_amd.capi import FMT_MXFP4, FMT_Q8_0
from deepstrix_amd.workloads import (CFG1, CFG2, CFG5, ROUTER, Shape, device_weights,  # noqa: F401
                                     host_block_params, host_inputs, zipf_logit_shift)
from oracle import ref


def host_expert(s: Shape, which: int, fmt: int, rows: int, cols: int, e: int) -> np.ndarray:
    return synth.weights_host(fmt, s.seed, which, rows, cols, first_row=e * rows)


def host_weights(s: Shape, experts=None) -> ref.MoeWeights:
    """Host copy of the layer.  `experts`: generate only these experts' bytes (the others are
    left zero), to keep large shapes cheap on the CPU."""
    gb = synth.matrix_bytes(s.gate_fmt, s.inter, s.hidden)
    db = synth.matrix_bytes(s.down_fmt, s.hidden, s.inter)
    gate = np.zeros(s.n_expert * gb, np.uint8)
    up = np.zeros(s.n_expert * gb, np.uint8)
    down = np.zeros(s.n_expert * db, np.uint8)
    for e in (range(s.n_expert) if experts is None else sorted(set(int(v) for v in experts))):
        gate[e * gb:(e + 1) * gb] = host_expert(s, synth.T_GATE, s.gate_fmt, s.inter, s.hidden, e)
        up[e * gb:(e + 1) * gb] = host_expert(s, synth.T_UP, s.gate_fmt, s.inter, s.hidden, e)
        down[e * db:(e + 1) * db] = host_expert(s, synth.T_DOWN, s.down_fmt, s.hidden, s.inter, e)
    w = ref.MoeWeights(s.hidden, s.inter, s.n_expert, s.n_used, gate, up, down, s.gate_fmt,
                       s.gate_fmt, s.down_fmt, s.clamp)
    if s.shared:
        w.sh_inter = s.shi
        w.sh_gate = host_expert(s, synth.T_SH_GATE, s.shg, s.shi, s.hidden, 0)
        w.sh_up = host_expert(s, synth.T_SH_UP, s.shg, s.shi, s.hidden, 0)
        w.sh_down = host_expert(s, synth.T_SH_DOWN, s.shd, s.hidden, s.shi, 0)
        w.sh_gate_fmt = w.sh_up_fmt = s.shg
        w.sh_down_fmt = s.shd
        w.sh_clamp = s.clamp
    return w


def oracle_route(s: Shape, logits, bias):
    return ref.router_topk(logits, bias, s.n_used, s.route_scale, s.route_eps, s.router_mode,
                           s.n_group, s.topk_group)


def host_weights_from_device(s: Shape, dw, experts=None) -> ref.MoeWeights:
    """The layer's bytes copied back from the GPU: the cheap way to a host copy of a full-size
    layer (the device generator makes the same bytes as the host one, which the generator tests
    check on smaller tensors).  `experts`: copy only these experts (the others stay zero)."""
    n = lambda t: t.cpu().numpy()
    if experts is None:
        gate, up, down = n(dw.gate), n(dw.up), n(dw.down)
    else:
        gb = synth.matrix_bytes(s.gate_fmt, s.inter, s.hidden)
        db = synth.matrix_bytes(s.down_fmt, s.hidden, s.inter)
        gate, up = np.zeros(s.n_expert * gb, np.uint8), np.zeros(s.n_expert * gb, np.uint8)
        down = np.zeros(s.n_expert * db, np.uint8)
        for e in sorted(set(int(v) for v in experts if v >= 0)):
            gate[e * gb:(e + 1) * gb] = n(dw.gate.view(-1)[e * gb:(e + 1) * gb])
            up[e * gb:(e + 1) * gb] = n(dw.up.view(-1)[e * gb:(e + 1) * gb])
            down[e * db:(e + 1) * db] = n(dw.down.view(-1)[e * db:(e + 1) * db])
    w = ref.MoeWeights(s.hidden, s.inter, s.n_expert, s.n_used, gate, up, down,
                       s.gate_fmt, s.gate_fmt, s.down_fmt, s.clamp)
    if s.shared:
        w.sh_inter = s.shi
        w.sh_gate, w.sh_up, w.sh_down = n(dw.sh_gate), n(dw.sh_up), n(dw.sh_down)
        w.sh_gate_fmt = w.sh_up_fmt = s.shg
        w.sh_down_fmt = s.shd
        w.sh_clamp = s.clamp
    return w


def compare_stats(a: np.ndarray, b_ref: np.ndarray) -> dict:
    """The reference harness's comparison (scratch/kernel_ideas/_infra/kbench.h:249-270):
    count of elements whose bits differ, max_abs, max_rel (elementwise, over elements that are
    not tiny), rmse / ref_rms -- plus the parity metric max|a - ref| / max|ref|."""
    a32, r32 = np.ascontiguousarray(a, np.float32), np.ascontiguousarray(b_ref, np.float32)
    a64, r64 = a32.astype(np.float64), r32.astype(np.float64)
    d = np.abs(a64 - r64)
    ref_max = float(np.abs(r64).max())
    big = np.abs(r64) > 1e-3 * max(ref_max, 1e-30)
    return {"bit_diffs": int((a32.view(np.uint32) != r32.view(np.uint32)).sum()),
            "max_abs": float(d.max()),
            "max_rel": float((d[big] / np.abs(r64[big])).max()) if big.any() else 0.0,
            "rel_rmse": float(np.sqrt((d ** 2).mean()) / max(np.sqrt((r64 ** 2).mean()), 1e-30)),
            "max_over_max": float(d.max()) / max(ref_max, 1e-30)}


def assert_close(a: np.ndarray, b_ref: np.ndarray, rel: float = 2e-3, what: str = "") -> dict:
    """Parity of an output with the oracle's: the contract max|a - ref| / max|ref| < rel, and
    elementwise |a - ref| <= rel * |ref| + floor with floor = rel / 2 * max|ref| (an element near
    a zero crossing is measured against the size of the output, not against itself)."""
    st = compare_stats(a, b_ref)
    r64 = np.asarray(b_ref, np.float64)
    floor = 0.5 * rel * float(np.abs(r64).max())
    bad = np.abs(np.asarray(a, np.float64) - r64) > rel * np.abs(r64) + floor
    assert st["max_over_max"] < rel, f"{what}: {st}"
    assert not bad.any(), f"{what}: {int(bad.sum())} elements off by more than {rel} * |ref| + {floor:.3e}: {st}"
    return st


def assert_parity_up_to_rounding_steps(out, want, hw: ref.MoeWeights, sel, what: str = "",
                                       tight: float = 2e-6, contract: float = 2e-3,
                                       max_steps: int = 4, analyse: int = 12) -> dict:
    """Layer outputs [n, hidden] against the oracle's, token by token.

    The integer dot products are exact on both sides and only the order of f32 sums differs, so
    a token's output agrees to a few 1e-7 of max|ref| -- unless one of its mid values sits on a
    rounding boundary of the int8 activation quantizer and lands on the other side: then the
    whole output row moves by (one quantization step) x (one column of a down matrix), which can
    reach several 1e-4 of max|ref| when the block's largest value is large.  Such a difference is
    arithmetic, not a defect, and it has a signature a defect does not have.  So every token must
      * agree within `tight` x max|ref|, or
      * differ by a vector that at most `max_steps` single columns of its own down matrices
        explain (greedy fit, each coefficient below 0.5), leaving a remainder within `tight`;
    and every token must meet the contract max|a - ref| / max|ref| < `contract`.  The `analyse`
    worst tokens above `tight` are fitted (dequantizing their down matrices on the host)."""
    out64, want64 = np.asarray(out, np.float64), np.asarray(want, np.float64)
    ref_max = float(np.abs(want64).max())
    err = np.abs(out64 - want64).max(axis=1) / ref_max
    assert err.max() < contract, f"{what}: max|a - ref| / max|ref| = {err.max():.3e}"
    loose = np.nonzero(err > tight)[0]
    stats = {"tokens": int(out64.shape[0]), "within_tight": int(out64.shape[0] - loose.size),
             "stepped": int(loose.size), "worst": float(err.max()),
             "median": float(np.median(err))}
    # a rounding step is rare: a few per cent of the tokens at most
    assert loose.size <= max(3, out64.shape[0] // 8), f"{what}: {loose.size} tokens above {tight}: {stats}"
    cache = {}

    def down_matrix(e):   # e = -1: the shared expert
        if e not in cache:
            if e < 0:
                buf, fmt, cols = hw.sh_down, hw.sh_down_fmt, hw.sh_inter
            else:
                db = ref.matrix_bytes(hw.down_fmt, hw.hidden, hw.inter)
                buf, fmt, cols = hw.down[e * db:(e + 1) * db], hw.down_fmt, hw.inter
            W = (ref.mxfp4_dequant_v2(buf, hw.hidden, cols) if fmt == FMT_MXFP4
                 else ref.q8_0_dequant_rows(buf, hw.hidden, cols)).astype(np.float64)
            cache[e] = (W, np.maximum((W * W).sum(axis=0), 1e-30))
            if len(cache) > 24:
                cache.pop(next(iter(cache)))
        return cache[e]

    for i in loose[np.argsort(err[loose])[::-1]][:analyse]:
        resid = out64[i] - want64[i]
        experts = [int(e) for e in sel[i] if e >= 0] + ([-1] if hw.sh_inter else [])
        steps = []
        for _ in range(max_steps):
            if np.abs(resid).max() <= tight * ref_max:
                break
            best = None
            for e in experts:
                W, n2 = down_matrix(e)
                c = W.T @ resid / n2
                gain = c * c * n2
                k = int(np.argmax(gain))
                if best is None or gain[k] > best[0]:
                    best = (float(gain[k]), e, k, float(c[k]))
            _, e, k, c = best
            assert abs(c) < 0.5, f"{what}: token {i}: implausible step {c} in expert {e} column {k}"
            resid = resid - c * down_matrix(e)[0][:, k]
            steps.append((e, k, c))
        left = float(np.abs(resid).max()) / ref_max
        assert left <= tight, (f"{what}: token {i} differs by {err[i]:.3e} of max|ref| and "
                               f"{len(steps)} single mid-value steps {steps} leave {left:.3e}")
    return stats


def max_rel(a: np.ndarray, b_ref: np.ndarray) -> float:
    """max|a - ref| / max|ref| -- the reference's check() metric
    (crates/v4flash-kernels/tests/mxfp4_pair_oracle.rs:86-100)."""
    denom = float(np.abs(b_ref).max())
    return float(np.abs(a.astype(np.float64) - b_ref.astype(np.float64)).max()) / max(denom, 1e-30)


def routing_mismatch_explained(sel_gpu, sel_ref, scores, n_used, tol=1e-4):
    """True when every token whose pick SET differs has a (k-th, (k+1)-th) score gap <= tol."""
    bad = []
    for t in range(sel_ref.shape[0]):
        if set(sel_gpu[t].tolist()) == set(sel_ref[t].tolist()):
            continue
        s = np.sort(scores[t][np.isfinite(scores[t])])[::-1]
        gap = s[n_used - 1] - s[n_used] if s.size > n_used else np.inf
        if gap > tol:
            bad.append((t, float(gap)))
    return bad
