#!/usr/bin/env python3
"""Benchmark of the MoE feed-forward layer on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload: BASELINE config 2 -- DeepSeek-V3-shape layer (hidden 7168, 256 routed experts + 1
shared, top-8 sigmoid gating with bias, 8 groups / top-4, scale 2.5, intermediate 2048, MXFP4
weights, bf16-valued activations) at T = 1.  One step = one layer forward for one token.
Steps rotate over several independent layers (different weights, different token) so that no
weight byte is served from the last-level cache: the cold-weight regime of real decoding.

Prints ONE JSON line (metric, value, roofline, cpu_baseline, ...).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0                     # MI355X HBM3E
MATRIX_BYTES = 7168 * (2048 // 32) * 17   # one MXFP4 7168 x 2048 matrix = 7,798,784 B
EXPERT_BYTES = 3 * MATRIX_BYTES           # 23,396,352 B
TOKEN_BYTES = 9 * EXPERT_BYTES            # 8 routed + 1 shared = 210,567,168 B / token
GATE_UP_BYTES = 9 * 2 * MATRIX_BYTES      # what one gate/up launch streams at T = 1
COPY_BYTES = 256 << 20                    # size of the calibration copy (read 256 MiB, write 256 MiB)

# The dominant kernel of a decode step: one launch that streams gate, up and down of the 8
# picks and the shared expert.
DOMINANT_KERNEL = "k_mxfp4_decode_fused<8,false,false>"
# HBM bytes one launch of it moves come from hardware counters (two `rocprofv3 --pmc` runs of
# this script: FETCH_SIZE, then WRITE_SIZE, each scaled by what it reads for the calibration
# copy below, whose traffic is known).  The figure is read from the committed summary, which
# names the kernel it was taken on; a summary for another kernel gives None (not measured).
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "moe_layer_decode_T1_cfg2_hbm_counters.txt")
# ... and its average duration under `rocprofv3 --kernel-trace` (line `kernel_trace_avg_us <kernel> <us>`)
TRACE_SUMMARY = os.path.join(ROOT, "profiles", "moe_layer_decode_T1_cfg2_kernel_trace.txt")


def kernel_sources_sha16() -> str:
    """First 16 hex digits of the SHA-256 over the library's kernel sources (csrc/, names and
    contents in sorted order): the committed summaries carry the value they were taken at."""
    import hashlib
    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "deepstrix_amd", "csrc")
    for name in sorted(os.listdir(csrc)):
        h.update(name.encode())
        with open(os.path.join(csrc, name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def summary_figure(path: str, key: str, kernel: str):
    """(value, source) from the line `<key> <kernel> <value>` of a committed profile summary --
    (None, reason) when there is no such line, or when the summary says (line `sources_sha16 <hash>`)
    that it was taken on other kernel sources than the ones in this tree."""
    rel = os.path.relpath(path, ROOT)
    value, sha = None, None
    try:
        with open(path) as f:
            for line in f:
                parts = line.lstrip("# ").split()
                if len(parts) >= 3 and parts[0] == key and parts[1] == kernel:
                    value = float(parts[2])
                if len(parts) >= 2 and parts[0] == "sources_sha16":
                    sha = parts[1]
    except OSError:
        pass
    if value is None:
        return None, f"no `{key}` line for {kernel} in {rel}"
    now = kernel_sources_sha16()
    if sha != now:
        return None, f"{rel} was taken on kernel sources {sha}, this tree has {now}: stale, not quoted"
    return value, rel


def measured_traffic(kernel: str):
    """(bytes per launch, source) of the dominant kernel from the committed counter summary."""
    v, src = summary_figure(TRAFFIC_SUMMARY, "traffic_bytes_per_launch", kernel)
    return (None if v is None else int(v)), src


class Hip:
    """The few HIP runtime calls the harness needs (events on the launch stream)."""

    def __init__(self):
        self.l = C.CDLL("libamdhip64.so")
        self.l.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.l.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        self.l.hipEventSynchronize.argtypes = [C.c_void_p]
        self.l.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        self.l.hipEventDestroy.argtypes = [C.c_void_p]

    def event(self):
        e = C.c_void_p()
        rc = self.l.hipEventCreate(C.byref(e))
        if rc:
            raise RuntimeError(f"hipEventCreate: {rc}")
        return e

    def elapsed_ms(self, a, b) -> float:
        ms = C.c_float()
        rc = self.l.hipEventElapsedTime(C.byref(ms), a, b)
        if rc:
            raise RuntimeError(f"hipEventElapsedTime: {rc}")
        return float(ms.value)


FP8_MFMA_PEAK = 5.0e15   # dense FP8 MFMA, the rate class of the FP4 x FP8 instruction issued
MXFP4_MFMA_PEAK = 10.1e15


def prefill_leg(dw, base, H, torch, np, T=4096, reps=5):
    """BASELINE config 3: the same layer at T = 4096 with Zipf(1.1)-skewed router logits, the
    skew factor calibrated (on the GPU router) so that the top 10 % of experts receive about
    half of the assignments."""
    from deepstrix_amd import dispatch
    from deepstrix_amd.executor import MoeLayer
    s = H.Shape(**{**base.__dict__, "seed": base.seed + 3})
    x, logits, _ = H.host_inputs(s, T)
    shift = H.zipf_logit_shift(s.n_expert, 3)
    dx = torch.from_numpy(x).cuda()
    sel = torch.empty((T, s.n_used), dtype=torch.int32, device="cuda")
    w = torch.empty((T, s.n_used), dtype=torch.float32, device="cuda")
    top = max(1, round(0.1 * s.n_expert))

    def share(alpha):
        dl = torch.from_numpy((logits + alpha * shift[None, :]).astype(np.float32)).cuda()
        dispatch.router_topk(sel, w, dl, dw.bias, s.n_expert, s.n_used, s.route_scale, s.route_eps,
                             T, s.router_mode, s.n_group, s.topk_group)
        cnt = np.bincount(sel.cpu().numpy().ravel(), minlength=s.n_expert)
        return float(np.sort(cnt)[::-1][:top].sum()) / float(cnt.sum()), cnt, dl

    lo, hi = 0.0, 2.0
    for _ in range(14):
        mid = 0.5 * (lo + hi)
        if share(mid)[0] < 0.5:
            lo = mid
        else:
            hi = mid
    alpha = 0.5 * (lo + hi)
    frac, cnt, dl = share(alpha)
    layer = MoeLayer(dw, T)
    out = torch.empty((T, s.hidden), dtype=torch.float32, device="cuda")
    for _ in range(2):
        layer.run(dx, dl, out=out)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        layer.run(dx, dl, out=out)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / reps
    flops = 2.0 * T * (s.n_used + 1) * 3 * s.hidden * s.inter
    del layer
    # the bound of this arithmetic: every product is two instructions at the FP6/FP4 rate (the
    # int8 activations as two exact planes of FP6 codes), so the useful rate tops out at half the
    # MXFP4 peak
    roof = {"bound": "mfma", "kernel": "k_mxfp4_gemm<true,128> + k_mxfp4_gemm<false,128> (whole layer, "
            "wall clock)", "achieved": flops / dt / 1e12, "peak": MXFP4_MFMA_PEAK / 1e12,
            "unit": "TFLOP/s", "frac": flops / dt / MXFP4_MFMA_PEAK,
            "frac_of_two_plane_bound": 2.0 * flops / dt / MXFP4_MFMA_PEAK,
            "frac_of_fp8_peak": flops / dt / FP8_MFMA_PEAK, "traffic": None,
            "algorithmic_flop_per_launch": flops}
    return {"roofline": roof, "tokens_per_s": T / dt, "ms_per_layer": dt * 1e3, "zipf_alpha": alpha,
            "top10pct_share": frac, "max_group": int(cnt.max()), "empty_experts": int((cnt == 0).sum()),
            "column_tiles_of_128": int(np.ceil(cnt / 128).sum()) + T // 128,
            "useful_flop": flops, "useful_TFLOPs": flops / dt / 1e12,
            "mfma_issued": "v_mfma_scale_f32_16x16x128_f8f6f4, A = FP4 weights, B = FP6 (E2M3) planes of "
                           "the int8 activations (two instructions per product, each at the FP4 rate)",
            "mfma_frac_useful_vs_fp8_peak": flops / dt / FP8_MFMA_PEAK,
            "mfma_frac_issued_vs_mxfp4_peak": 2.0 * flops / dt / MXFP4_MFMA_PEAK,
            "mfma_frac_useful_vs_mxfp4_peak": flops / dt / MXFP4_MFMA_PEAK}


def q8_0_leg(H, torch, np):
    """BASELINE config 1 (the reference's CPU-runnable case): all-Q8_0 layer, hidden 2048, 64 + 1
    experts, top-6 softmax, inter 1408, T = 4; and the same layer with 512 tokens."""
    from deepstrix_amd.executor import MoeLayer
    s = H.CFG1
    layer = MoeLayer(H.device_weights(s), 512)
    res = {}
    for T in (4, 512):
        x, logits, _ = H.host_inputs(s, T)
        dx, dl = torch.from_numpy(x).cuda(), torch.from_numpy(logits).cuda()
        out = torch.empty((T, s.hidden), dtype=torch.float32, device="cuda")
        for _ in range(3):
            layer.run(dx, dl, out=out)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        reps = 20
        for _ in range(reps):
            layer.run(dx, dl, out=out)
        torch.cuda.synchronize()
        res[f"T{T}_us_per_layer"] = (time.perf_counter() - t0) / reps * 1e6
    del layer
    torch.cuda.empty_cache()
    return res


def mixed_leg(H, torch, np, T=512):
    """BASELINE config 5: MXFP4 gate/up, Q8_0 down, V3 shape, T = 512; every token on experts
    0..7 (worst-case imbalance) and uniform random distinct top-8."""
    from deepstrix_amd.executor import MoeLayer
    s = H.CFG5
    rng = np.random.default_rng(55)
    x, _, _ = H.host_inputs(s, T)
    layers = {"": MoeLayer(H.device_weights(s), T),
              "_planar_weights": MoeLayer(H.device_weights(s, planar=True), T)}   # (the MXFP4 gate/up matrices)
    dx = torch.from_numpy(x).cuda()
    dw = torch.from_numpy(rng.uniform(0.05, 0.6, (T, s.n_used)).astype(np.float32)).cuda()
    out = torch.empty((T, s.hidden), dtype=torch.float32, device="cuda")
    cases = {"adversarial": np.tile(np.arange(s.n_used, dtype=np.int32), (T, 1)),
             "uniform": np.stack([rng.choice(s.n_expert, s.n_used, replace=False)
                                  for _ in range(T)]).astype(np.int32)}
    res = {"tokens": T}
    for name, sel in cases.items():
        ds = torch.from_numpy(sel).cuda()
        for tag, layer in layers.items():
            for _ in range(2):
                layer.run(dx, None, out=out, selected_in=ds, weights_in=dw)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            reps = 8
            for _ in range(reps):
                layer.run(dx, None, out=out, selected_in=ds, weights_in=dw)
            torch.cuda.synchronize()
            res[f"{name}_ms_per_layer{tag}"] = (time.perf_counter() - t0) / reps * 1e3
    del layers, layer
    torch.cuda.empty_cache()
    return res


def chain_leg(H, torch, np, n_layers=8, T=2, steps=256, planar=False):
    """BASELINE config 4: 8 chained V3-shape MXFP4 layers, each h += MoE(RMSNorm(h)), T = 2
    tokens per step, 256 consecutive steps with fresh N(0,1) inputs.  Latency of one step from
    the host's point of view (submit + run + synchronize), eager and replayed from a graph."""
    from deepstrix_amd.executor import MoeChain
    shapes = [H.Shape(**{**H.CFG2.__dict__, "seed": H.CFG2.seed + 0x1000 + 0x100 * i}) for i in range(n_layers)]
    chain = MoeChain([H.device_weights(s, block=True, planar=planar) for s in shapes], T)
    hidden = H.CFG2.hidden
    inputs = torch.randn((steps, T, hidden), dtype=torch.float32, device="cuda",
                         generator=torch.Generator(device="cuda").manual_seed(4))
    h = torch.empty((T, hidden), dtype=torch.float32, device="cuda")

    def timed(fn):
        for i in range(8):
            fn(inputs[i])
        torch.cuda.synchronize()
        lat = np.empty(steps)
        for i in range(steps):
            t0 = time.perf_counter()
            fn(inputs[i])
            torch.cuda.synchronize()
            lat[i] = (time.perf_counter() - t0) * 1e6
        return lat

    def eager(x):
        h.copy_(x)
        chain.step(h)

    lat_e = timed(eager)
    chain.capture(T)
    lat_g = timed(chain.replay)
    q = lambda a: {"p10": float(np.percentile(a, 10)), "p50": float(np.percentile(a, 50)),
                   "p90": float(np.percentile(a, 90))}
    # Algorithmic bytes of a step: per block the distinct routed experts of its T tokens plus the
    # shared expert ONCE (the definition of the decode legs).  The distinct count is measured on
    # the first steps with the block's operators called one by one (same picks as the fused block).
    from deepstrix_amd import dispatch
    distinct, n_probe = [], 16
    xn = torch.empty((T, hidden), dtype=torch.float32, device="cuda")
    lg = torch.empty((T, H.CFG2.n_expert), dtype=torch.float32, device="cuda")
    for i in range(n_probe):
        h.copy_(inputs[i])
        per_step = 0
        for layer in chain.layers:
            w = layer.w
            dispatch.rms_norm(xn, h, w.norm_w, hidden, w.norm_eps, T)
            dispatch.router_logits(lg, w.router_w, xn, w.n_expert, hidden, T)
            out, sel, _ = layer.run(xn, lg, want_routing=True)
            h += out
            per_step += len(np.unique(sel.cpu().numpy()))
        distinct.append(per_step)
    d_mean = float(np.mean(distinct))
    per_step_bytes = (d_mean + n_layers) * EXPERT_BYTES
    streamed_bytes = n_layers * T * 9 * EXPERT_BYTES   # what the launches stream when no two tokens share a pass
    p50 = float(np.percentile(lat_g, 50))
    return {"layers": n_layers, "tokens_per_step": T, "steps": steps,
            "eager_us_per_step": q(lat_e), "graph_us_per_step": q(lat_g),
            "launches_per_step": n_layers * 3,
            "distinct_routed_experts_per_step": d_mean,
            "algorithmic_bytes_per_step": per_step_bytes,
            "graph_GBps_p50": per_step_bytes / (p50 * 1e-6) / 1e9,
            "graph_frac_of_hbm_peak_p50": per_step_bytes / (p50 * 1e-6) / 1e9 / HBM_PEAK_GBS,
            "streamed_bytes_per_step_upper": streamed_bytes}


def decode_leg(layers_of, H, torch, np, base, T, reps=8):
    """One layer forward for T tokens of config 2, rotating over independent layers.  Returns
    us/token, the measured distinct routed experts D(T), the algorithmic bytes (D(T) + 1) x
    23,396,352 and the rate and fraction of the HBM peak they give."""
    xs, ls, _ = H.host_inputs(H.Shape(**{**base.__dict__, "seed": base.seed + T}), T)
    xs, ls = torch.from_numpy(xs).cuda(), torch.from_numpy(ls).cuda()
    o = torch.empty((T, base.hidden), dtype=torch.float32, device="cuda")
    L = len(layers_of)
    _, sel, _ = layers_of[0].run(xs, ls, want_routing=True)
    d_t = int(len(np.unique(sel.cpu().numpy())))
    for r in range(2):
        layers_of[r % L].run(xs, ls, out=o)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    for r in range(reps):
        layers_of[r % L].run(xs, ls, out=o)
    torch.cuda.synchronize()
    us = (time.perf_counter() - t1) * 1e6 / reps
    nbytes = (d_t + 1) * EXPERT_BYTES
    return {"us_per_token": us / T, "us_per_layer": us, "distinct_routed_experts": d_t,
            "algorithmic_bytes": nbytes, "GBps": nbytes / (us * 1e-6) / 1e9,
            "frac_of_hbm_peak": nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS}


def stream_read_leg(hip, layers, torch, np, synth, stream, H, reps=200):
    """What a plain read reaches on this device: 210,567,168 bytes (the size of a decode step's
    weights) streamed by the library's read kernel from the gate tensors of the rotating layers,
    so that the 256 MB memory-side cache serves none of it; HIP events around each launch."""
    sink = torch.zeros(4 * 8192, dtype=torch.int32, device="cuda")
    srcs = [lay.w.gate.view(-1)[:TOKEN_BYTES] for lay in layers]
    rate = lambda t: TOKEN_BYTES / (t * 1e-6) / 1e9
    by_grid = {}
    for wgs in (1024, 2048, 4096, 8192):   # 4 .. 32 workgroups per compute unit
        for r in range(8):
            synth.read_dev(sink, srcs[r % len(srcs)], wgs)
        torch.cuda.synchronize()
        evs = [(hip.event(), hip.event()) for _ in range(reps)]
        for r, (a, b) in enumerate(evs):
            hip.l.hipEventRecord(a, stream)
            synth.read_dev(sink, srcs[r % len(srcs)], wgs)
            hip.l.hipEventRecord(b, stream)
        torch.cuda.synchronize()
        us = np.array([hip.elapsed_ms(a, b) for a, b in evs]) * 1e3
        by_grid[wgs] = {"us_event_bracket": {"p10": float(np.percentile(us, 10)), "p50": float(np.percentile(us, 50)),
                                             "p90": float(np.percentile(us, 90))},
                        "GBps_p50": rate(np.percentile(us, 50)), "GBps_best": rate(us.min())}
    best = max(by_grid, key=lambda g: by_grid[g]["GBps_p50"])
    # the same bytes read the way the decode kernels stream weights: 16-row tiles of rows of 28
    # super-blocks (a gate or up matrix of the layer), operand order and memory order
    n_sb = H.CFG2.hidden // 256
    n_tiles = TOKEN_BYTES // (16 * n_sb * 136)
    tile_bytes = n_tiles * 16 * n_sb * 136
    tiles = {}
    for name, operand in (("operand_order", True), ("memory_order", False)):
        for r in range(8):
            synth.read_tiles_dev(sink, srcs[r % len(srcs)], n_tiles, n_sb, operand)
        torch.cuda.synchronize()
        evs = [(hip.event(), hip.event()) for _ in range(reps)]
        for r, (a, b) in enumerate(evs):
            hip.l.hipEventRecord(a, stream)
            synth.read_tiles_dev(sink, srcs[r % len(srcs)], n_tiles, n_sb, operand)
            hip.l.hipEventRecord(b, stream)
        torch.cuda.synchronize()
        us = np.array([hip.elapsed_ms(a, b) for a, b in evs]) * 1e3
        tiles[name] = {"us_event_bracket": {"p10": float(np.percentile(us, 10)), "p50": float(np.percentile(us, 50)),
                                            "p90": float(np.percentile(us, 90))},
                       "GBps_p50": tile_bytes / (np.percentile(us, 50) * 1e-6) / 1e9,
                       "GBps_best": tile_bytes / (us.min() * 1e-6) / 1e9}
    return {"weight_tile_pattern": {"kernel": "k_read_tiles (libdsx_synth.so): one workgroup per 16-row tile of 136-byte "
                                              "super-blocks, four waves on every fourth super-block, two in flight per wave: "
                                              "the decode kernels' weight loads and nothing else",
                                    "bytes_per_launch": tile_bytes, **tiles},
            "kernel": "k_read16 (libdsx_synth.so): 256 threads per workgroup, four 16-byte loads in flight per thread",
            "bytes_per_launch": TOKEN_BYTES, "buffers_rotated": len(srcs), "by_workgroups": by_grid,
            "best_workgroups": best, "us_event_bracket": by_grid[best]["us_event_bracket"],
            "GBps_p50": by_grid[best]["GBps_p50"], "GBps_best": by_grid[best]["GBps_best"],
            "frac_of_hbm_peak_p50": by_grid[best]["GBps_p50"] / HBM_PEAK_GBS}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--layers", type=int, default=4, help="independent layers the steps rotate over")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-prefill", action="store_true", help="skip the T=4096 prefill leg")
    ap.add_argument("--no-chain", action="store_true", help="skip the 8-layer chained decode leg")
    ap.add_argument("--no-extra", action="store_true",
                    help="skip the informative legs: T=4/16/64 of config 2 and configs 5 and 1")
    ap.add_argument("--no-small-t", action="store_true", help="skip only the T=4/16/64 legs")
    ap.add_argument("--no-ceiling", action="store_true",
                    help="skip the plain streaming-read leg (what a read of a decode step's size reaches)")
    ap.add_argument("--cpu-seconds", type=float, default=15.0)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU only: this build has no multi-GPU path "
              "(run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from deepstrix_amd import capi, synth
    from deepstrix_amd.executor import MoeLayer
    from deepstrix_amd import workloads as H

    torch.cuda.set_device(0)
    capi.init()
    hip = Hip()
    base = H.CFG2
    K, W, L = args.steps, args.warmup, args.layers
    layers, weights = [], []
    for i in range(L):
        s = H.Shape(**{**base.__dict__, "seed": base.seed + 0x100 * i})
        dw = H.device_weights(s)
        weights.append(dw)
        layers.append(MoeLayer(dw, 64))
    # one fresh token per step (bf16-valued activations, N(0,1) logits)
    n_tok = W + K
    x_all, lg_all, _ = H.host_inputs(base, n_tok)
    x_all = torch.from_numpy(x_all).cuda()
    lg_all = torch.from_numpy(lg_all).cuda()
    out = torch.empty((1, base.hidden), dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream

    def step(i):
        layers[i % L].run(x_all[i:i + 1], lg_all[i:i + 1], out=out)

    for i in range(W):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(W, W + K):
        step(i)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms_per_step = wall_ms / K

    # same steps again with events around the dominant kernel (gate/up) and the whole chain
    evs = [(hip.event(), hip.event(), hip.event(), hip.event()) for _ in range(K)]
    for j, i in enumerate(range(W, W + K)):
        a, b, c, d = evs[j]
        lay = layers[i % L]
        lay.set_profile_events(b, c, None)
        hip.l.hipEventRecord(a, stream)
        step(i)
        hip.l.hipEventRecord(d, stream)
    torch.cuda.synchronize()
    for lay in layers:
        lay.set_profile_events(None, None, None)
    gu_ms = np.array([hip.elapsed_ms(b, c) for (_, b, c, _) in evs])
    chain_ms = np.array([hip.elapsed_ms(a, d) for (a, _, _, d) in evs])
    gu_avg_us = float(gu_ms.mean() * 1e3)
    achieved = TOKEN_BYTES / (gu_avg_us * 1e-6) / 1e9
    traffic, traffic_source = measured_traffic(DOMINANT_KERNEL)
    trace_us, trace_source = summary_figure(TRACE_SUMMARY, "kernel_trace_avg_us", DOMINANT_KERNEL)

    # what the bracket itself costs: the same pair of events around a one-workgroup kernel
    # (a 16-byte add, about a microsecond of kernel time in a kernel trace)
    from deepstrix_amd import dispatch
    tiny_a = torch.zeros(4, dtype=torch.float32, device="cuda")
    tiny_b = torch.ones(4, dtype=torch.float32, device="cuda")
    tiny = [(hip.event(), hip.event()) for _ in range(64)]
    for j, (a, b) in enumerate(tiny):
        step(W + j % K)
        hip.l.hipEventRecord(a, stream)
        dispatch.vec_add_inplace(tiny_a, tiny_b, 4)
        hip.l.hipEventRecord(b, stream)
    torch.cuda.synchronize()
    tiny_us = float(np.median([hip.elapsed_ms(a, b) for a, b in tiny]) * 1e3)
    # and around nothing at all
    empty = [(hip.event(), hip.event()) for _ in range(64)]
    for j, (a, b) in enumerate(empty):
        step(W + j % K)
        hip.l.hipEventRecord(a, stream)
        hip.l.hipEventRecord(b, stream)
    torch.cuda.synchronize()
    empty_us = float(np.median([hip.elapsed_ms(a, b) for a, b in empty]) * 1e3)

    # a copy of known size, so that byte counters collected over this run can be scaled
    c_src = torch.empty(COPY_BYTES, dtype=torch.uint8, device="cuda").random_(0, 255)
    c_dst = torch.empty_like(c_src)
    for _ in range(4):
        synth.copy_dev(c_dst, c_src)
    torch.cuda.synchronize()
    del c_src, c_dst

    # other token counts of the same config (informative)
    step_us = chain_ms * 1e3   # one decode step between two events on the launch stream
    extra = {"dominant_kernel_us_p50": float(np.median(gu_ms) * 1e3),
             "step_us_events": {"p10": float(np.percentile(step_us, 10)), "p50": float(np.percentile(step_us, 50)),
                                "p90": float(np.percentile(step_us, 90))},
             "event_bracket_of_one_workgroup_kernel_us": tiny_us,
             "event_bracket_of_nothing_us": empty_us,
             "chain_us_p50_events": float(np.median(chain_ms) * 1e3),
             "layer_GBps_T1": TOKEN_BYTES / (ms_per_step * 1e-3) / 1e9,
             "layer_frac_of_hbm_peak_T1": TOKEN_BYTES / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS}
    small_t = () if (args.no_extra or args.no_small_t) else (4, 16, 64)
    for T in small_t:
        leg = decode_leg(layers, H, torch, np, base, T)
        extra[f"us_per_token_T{T}"] = leg["us_per_token"]
        extra[f"decode_T{T}"] = leg

    if not args.no_ceiling:
        extra["stream_read_ceiling"] = stream_read_leg(hip, layers, torch, np, synth, stream, H)

    if not args.no_prefill:
        # The figures of the leg are those of the engine's weight rows -- the layout a checkpoint
        # loads into and the one the drop-in boundary fixes.  The planar form of the same matrices
        # (opt-in, rewritten in place once after loading; identical results) is quoted beside them.
        pre = prefill_leg(layers[0].w, base, H, torch, np)
        pre["weights_layout"] = "engine rows (136-byte v2 super-blocks)"
        dwp = H.device_weights(H.Shape(**base.__dict__), planar=True)
        on_planar = prefill_leg(dwp, base, H, torch, np)
        pre["planar_weights"] = {
            "weights_layout": "planar (DSX_FMT_MXFP4_PLANAR: nibble blocks and scales in separate planes, "
                              "made in place by dsx_mxfp4_rows_to_planar)",
            "ms_per_layer": on_planar["ms_per_layer"], "tokens_per_s": on_planar["tokens_per_s"],
            "roofline": on_planar["roofline"]}
        extra["prefill_T4096"] = pre
        # the decode step on planar weights, rotating over as many layers as the headline figure
        del dwp
        lps = [MoeLayer(H.device_weights(H.Shape(**{**base.__dict__, "seed": base.seed + 0x100 * i}), planar=True), 1)
               for i in range(L)]
        for i in range(W):
            lps[i % L].run(x_all[i:i + 1], lg_all[i:i + 1], out=out)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for i in range(W, W + K):
            lps[i % L].run(x_all[i:i + 1], lg_all[i:i + 1], out=out)
        torch.cuda.synchronize()
        extra["us_per_token_T1_planar_weights"] = (time.perf_counter() - t1) * 1e6 / K
        # ... and the other token counts of config 2 (the grouped GEMMs from 12 tokens on)
        for T in small_t:
            lpt = [MoeLayer(lp.w, T) for lp in lps]
            leg = decode_leg(lpt, H, torch, np, base, T)
            extra[f"us_per_token_T{T}_planar_weights"] = leg["us_per_token"]
            extra[f"decode_T{T}"]["planar_weights"] = {k: leg[k] for k in ("us_per_token", "us_per_layer", "GBps",
                                                                            "frac_of_hbm_peak")}
            del lpt
        del lps
    if not args.no_chain:
        extra["chain_8_layers_T2"] = chain_leg(H, torch, np)
        torch.cuda.empty_cache()
        on_planar = chain_leg(H, torch, np, planar=True)
        extra["chain_8_layers_T2"]["planar_weights"] = {k: on_planar[k] for k in ("eager_us_per_step", "graph_us_per_step")}
        torch.cuda.empty_cache()
    if not args.no_extra:
        extra["mixed_precision_T512_cfg5"] = mixed_leg(H, torch, np)
        extra["q8_0_cfg1"] = q8_0_leg(H, torch, np)

    result = {
        "metric": "moe_layer_us_per_token_T1",
        "value": ms_per_step * 1e3,
        "unit": "us/token",
        "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": ms_per_step,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "mxfp4 weights x int8 (Q8_K) activations, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": "BASELINE config 2: V3-shape MXFP4 MoE layer decode, T=1 "
                               "(hidden 7168, 256+1 experts, top-8 sigmoid+bias, 8 groups/top-4, "
                               "scale 2.5, inter 2048); cold weights, steps rotate over "
                               f"{L} layers", "tokens_per_step": 1, "layers_rotated": L,
                   "algorithmic_bytes_per_token": TOKEN_BYTES},
        "roofline": {"bound": "hbm", "kernel": DOMINANT_KERNEL + " (gate + up + SwiGLU, mid quantization, "
                     "down and the slot-order sum of 8 routed + 1 shared expert in one launch)",
                     "achieved": achieved, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                     "traffic_source": traffic_source,
                     "algorithmic_bytes_per_launch": TOKEN_BYTES, "avg_launch_us": gu_avg_us,
                     # the same fraction from the two clocks there are: `frac` above is the event
                     # bracket of this run (it includes what the bracket itself costs, see
                     # extra.event_bracket_of_nothing_us); the kernel-trace figure is the committed
                     # rocprofv3 summary's average duration of the kernel (None when stale)
                     "frac_event_bracket": achieved / HBM_PEAK_GBS,
                     "frac_event_bracket_source": "HIP events on the launch stream around each of this run's "
                                                  f"{K} launches, mean",
                     "frac_kernel_trace": (None if trace_us is None
                                           else TOKEN_BYTES / (trace_us * 1e-6) / 1e9 / HBM_PEAK_GBS),
                     "frac_kernel_trace_source": trace_source, "kernel_trace_avg_us": trace_us},
        "extra": extra,
    }

    if not args.no_cpu:
        # CPU baseline: the oracle (a port of the reference arithmetic) on the host cores,
        # same layer-0 weights, decode tokens one at a time, bounded by --cpu-seconds.
        from oracle import ref
        cpu_flags = ref.use_timing_build()
        dw = weights[0]
        hw = ref.MoeWeights(base.hidden, base.inter, base.n_expert, base.n_used,
                            dw.gate.cpu().numpy(), dw.up.cpu().numpy(), dw.down.cpu().numpy(),
                            clamp=base.clamp, sh_inter=base.inter, sh_gate=dw.sh_gate.cpu().numpy(),
                            sh_up=dw.sh_up.cpu().numpy(), sh_down=dw.sh_down.cpu().numpy())
        bias = dw.bias.cpu().numpy()
        xs = x_all[:256].cpu().numpy()
        ls = lg_all[:256].cpu().numpy()
        threads = ref.max_threads()
        done, t1 = 0, time.perf_counter()
        while (time.perf_counter() - t1) < args.cpu_seconds:
            i = done % xs.shape[0]
            sel, w = ref.router_topk(ls[i:i + 1], bias, base.n_used, base.route_scale,
                                     base.route_eps, base.router_mode, base.n_group,
                                     base.topk_group)
            ref.moe_forward(hw, xs[i:i + 1], sel, w)
            done += 1
        cpu_s = time.perf_counter() - t1
        result["cpu_baseline"] = {
            "value": cpu_s * 1e6 / max(done, 1), "unit": "us/token", "cores": threads,
            "kind": "port",
            "sample": f"{done} tokens decoded one at a time through the C oracle "
                      f"(gcc {cpu_flags}, OpenMP, {threads} threads) on layer 0 of the same workload, "
                      f"{cpu_s:.1f} s"}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
