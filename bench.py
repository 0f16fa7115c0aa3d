#!/usr/bin/env python3
"""Benchmark of the accelerated path on one MI355X.

Default workload (the configuration the headline metric is quoted on): GDN chunk forward,
bf16 in / fp32 accumulation and state, B=4, T=8192, H=32, K=V=128, chunk 64, fp32 initial
state, final state on.  One "step" is one pass of the whole chunk forward over that batch
with inputs resident in HBM.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload gdn_chunk|gdn_bwd|decode|conv1d|kda]

Before the W warm-up steps every workload repeats its step untimed for --preheat-ms (default 300 ms, reported as
`preheat_ms`): the device clock ramps over tens of milliseconds of load, which a 20-step run would otherwise measure.
The default workload then times the decode, conv1d and KDA configurations briefly and reports them under
`secondary` (never part of `value`).

`roofline` describes the dominant kernel of the step: algorithmic FLOPs (or bytes) per launch
divided by its average duration, measured with HIP events recorded on the launch stream by the
library's own per-launch timing hooks in a second pass of K steps directly after the timed region.
`cpu_baseline` times the CPU oracle (a port of the reference's PyTorch CPU path) on the host cores
on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
for _p in (str(ROOT), str(ROOT / "flash-linear-attention-npu_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

# HBM bytes per launch of the dominant kernel, measured offline with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (scaled by the factors a plain copy of known size gives: x2.00 and x1.00).  The summaries with the exact
# commands are the files named here; bench.py cannot collect hardware counters itself.
MEASURED_TRAFFIC = {
    "gdn_fused": (881e6 + 311e6, "profiles/gdn_pipe_kernel_B4_T8192_H32_K128_V128.md"),
    "recurrent_gdn": (544e6 + 539e6, "profiles/recurrent_gdn_kernel_decode_256x32x128x128.md"),
    "conv1d_fwd": (147e6 + 134e6, "profiles/conv1d_dense_kernel_B4_T4096_D4096_W4_silu.md"),
    "kda_intra": (689e6 + 944e6, "profiles/kda_kernels_B2_T8192_H32_K128_V128.md"),
}


def measured_traffic(kernel):
    v = MEASURED_TRAFFIC.get(kernel)
    return (int(v[0]), v[1]) if v else (None, None)

# Dense-tile FLOP count per token-head of the chunk forward (C=64, K=V=128):
#   kkt, w, q.k^T = 3*C*K ; u, P.v_new = 2*C*V ; w.h, k^T.v_new, q.h = 3*K*V ; unit-lower inverse C^2/3
def gdn_flops_per_token_head(C=64, K=128, V=128):
    return 2 * (3 * C * K + 2 * C * V + 3 * K * V + C * C // 3)

# share of those FLOPs executed by each kernel of the step
def gdn_kernel_flops_per_token_head(C=64, K=128, V=128):
    prep = 2 * (2 * C * K + C * V + C * C // 3)          # kkt, inverse, w, u
    scan = 2 * (C * K + C * V + 3 * K * V)               # q.k^T, P.v_new, w.h, k^T.v_new, q.h
    return {"prep": prep, "scan": scan, "total": prep + scan}


def preheat(step, torch, ms):
    """Untimed: repeats ``step`` for at least ``ms`` milliseconds of GPU work so that the timed region that follows
    sees the sustained device clock (a few tens of launches do not ramp it, and after seconds of host-only work -- a
    CPU baseline -- the device needs longer than after a short pause).  It goes on until two consecutive batches take
    the same time to within 3 %, for at most six times ``ms``.  Returns the milliseconds spent."""
    if ms <= 0:
        return 0.0
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    n, prev = 8, None
    while True:
        tb = time.perf_counter()
        for _ in range(n):
            step()
        torch.cuda.synchronize()
        now = time.perf_counter()
        cur, spent = (now - tb) / n, (now - t0) * 1e3
        if (now - tb) * 1e3 < 3.0:      # batches long enough for the host clock to compare them
            n *= 2
            continue
        if spent >= ms and prev is not None and abs(cur - prev) <= 0.03 * prev:
            break
        if spent >= 6 * ms:
            break
        prev = cur
    return round((time.perf_counter() - t0) * 1e3, 1)


def profile_report(lib):
    buf = ctypes.create_string_buffer(1 << 16)
    lib.fla_profile_report.argtypes = [ctypes.c_char_p, ctypes.c_uint64]
    lib.fla_profile_report.restype = ctypes.c_int
    lib.fla_profile_report(buf, len(buf))
    out = {}
    for line in buf.value.decode().splitlines():
        name, n, ms = line.split()
        out[name] = (int(n), float(ms))
    return out


def bench_gdn(args, torch, dev):
    import fla_hip
    from fla_hip import pipeline

    lib = fla_hip.load_library()
    B, T, H, K, V, C = 4, 8192, 32, 128, 128, 64
    F = torch.nn.functional
    g = torch.Generator(device=dev).manual_seed(0)
    q = F.normalize(torch.randn(B, H, T, K, device=dev, generator=g), dim=-1).bfloat16()
    k = F.normalize(torch.randn(B, H, T, K, device=dev, generator=g), dim=-1).bfloat16()
    v = torch.randn(B, H, T, V, device=dev, generator=g).bfloat16()
    beta = torch.sigmoid(torch.randn(B, T, H, device=dev, generator=g))
    gate = F.logsigmoid(torch.randn(B, T, H, device=dev, generator=g))
    h0 = torch.randn(B, H, K, V, device=dev, generator=g) * 0.01
    fused = args.route == "fused"

    def step():
        return pipeline.flash_gated_delta_rule(q, k, v, gate, beta, None, h0, True, chunk_size=C, fused=fused,
                                               use_qk_l2norm_in_kernel=args.l2norm)

    heated = preheat(step, torch, args.preheat_ms)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # one event pair around the timed steps, on the stream the library launches on (torch's current stream)
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(args.steps):
        o, final = step()
    ev1.record()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt * 1e3 / args.steps
    tokens_per_s = B * T * args.steps / dt
    bracket_ms = ev0.elapsed_time(ev1) / args.steps

    # per-kernel durations: second pass with the library's event hooks on the launch stream
    lib.fla_profile_enable.argtypes = [ctypes.c_int]
    lib.fla_profile_enable(1)
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    lib.fla_profile_enable(0)
    prof = profile_report(lib)
    kern = {name: ms / n for name, (n, ms) in prof.items()}
    per_launch_pairs = dict(kern)
    if len(kern) == 1:   # a step is one launch: the pair around all timed steps carries no per-launch event cost
        kern = {name: bracket_ms for name in kern}
    dominant = max(kern, key=kern.get) if kern else None
    th = B * T * H
    fl = gdn_kernel_flops_per_token_head(C, K, V)
    flops_of = {  # algorithmic FLOPs of one launch of each kernel
        "gdn_fused": fl["total"] * th, "gdn_prep": fl["prep"] * th, "gdn_scan": fl["scan"] * th,
        "kkt": 2 * C * K * th, "solve_tri": 2 * (C * C // 3) * th, "wu": 2 * (C * K + C * V) * th,
        "fwd_h": 2 * (2 * K * V) * th, "fwd_o": 2 * (C * K + C * V + K * V) * th,
    }
    roofline = None
    if dominant in flops_of:
        ach = flops_of[dominant] / (kern[dominant] * 1e-3) / 1e12
        traffic, src = measured_traffic(dominant)
        roofline = {"bound": "mfma", "kernel": dominant, "achieved": round(ach, 2), "peak": PEAK_BF16_TFLOPS,
                    "unit": "TFLOP/s", "frac": round(ach / PEAK_BF16_TFLOPS, 4), "traffic": traffic,
                    "traffic_source": src,
                    "avg_kernel_ms": round(kern[dominant], 4),
                    "avg_kernel_ms_with_an_event_pair_per_launch": round(per_launch_pairs[dominant], 4),
                    "all_kernels_ms": {n: round(t, 4) for n, t in kern.items()}}
    step_tflops = gdn_flops_per_token_head(C, K, V) * th / (ms_per_step * 1e-3) / 1e12

    # CPU baseline: the oracle's chunked fp32 path on the host cores, bounded sample
    cpu = None
    if not args.no_cpu:
        from oracle import gdn as ogdn   # the CPU oracle is only ever the baseline being timed
        import torch as _t
        cores = os.cpu_count() or 1
        _t.set_num_threads(cores)
        Ts = args.cpu_tokens
        d = ogdn.make_gdn_inputs(1, Ts, H, K, V, dtype=_t.bfloat16, seed=0, init_std=0.01, head_first_gates=True)
        ogdn.chunk_gated_delta_rule_fwd(d["q"][:, :, :128], d["k"][:, :, :128], d["v"][:, :, :128],
                                        d["g"][:, :, :128], d["beta"][:, :, :128], initial_state=d["initial_state"])
        t1 = time.perf_counter()
        reps = 0
        while reps == 0 or time.perf_counter() - t1 < args.cpu_seconds:
            ogdn.chunk_gated_delta_rule_fwd(d["q"], d["k"], d["v"], d["g"], d["beta"],
                                            initial_state=d["initial_state"], output_final_state=True)
            reps += 1
        cdt = time.perf_counter() - t1
        cpu = {"value": round(Ts * reps / cdt, 1), "unit": "tokens/s", "cores": cores, "kind": "port",
               "sample": f"{reps} x (B=1 T={Ts} H={H} K=V={K}) chunked fp32 torch oracle, {cdt:.1f} s"}
    # sanity of the timed result (not a parity test): finite outputs
    assert bool(torch.isfinite(o.float()).all()) and bool(torch.isfinite(final).all())
    return {
        "metric": "gdn_chunk_fwd_tokens_per_s", "value": round(tokens_per_s, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "preheat_ms": heated, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "GDN chunk forward B=4 T=8192 H=32 K=V=128 chunk=64, fp32 initial+final state",
                   "route": args.route, "use_qk_l2norm_in_kernel": bool(args.l2norm)},
        "algorithmic": {"flops_per_step": gdn_flops_per_token_head(C, K, V) * th,
                        "bytes_per_step": 4 * th * 256 + 2 * B * T * H * 4 + 2 * B * H * K * V * 4},
        "step_tflops": round(step_tflops, 2), "step_frac_of_bf16_peak": round(step_tflops / PEAK_BF16_TFLOPS, 4),
        "roofline": roofline, "cpu_baseline": cpu,
    }


def bench_decode(args, torch, dev):
    import fla_hip
    from fla_hip import ops

    lib = fla_hip.load_library()
    N, H, D = 256, 32, 128
    F = torch.nn.functional
    g = torch.Generator(device=dev).manual_seed(0)
    q = F.normalize(torch.randn(N, H, D, device=dev, generator=g), dim=-1).bfloat16()
    k = F.normalize(torch.randn(N, H, D, device=dev, generator=g), dim=-1).bfloat16()
    v = torch.randn(N, H, D, device=dev, generator=g).bfloat16()
    beta = torch.sigmoid(torch.randn(N, H, device=dev, generator=g)).bfloat16()
    gate = F.logsigmoid(torch.randn(N, H, device=dev, generator=g))
    state = torch.randn(N, H, D, D, device=dev, generator=g) * 0.01
    lens = torch.tensor([0] + [1] * N, dtype=torch.int32, device=dev)
    idx = torch.arange(N, dtype=torch.int32, device=dev)

    def step():
        return ops.recurrent_gated_delta_rule(q, k, v, state, beta=beta, scale=D ** -0.5, actual_seq_lengths=lens,
                                              ssm_state_indices=idx, g=gate)

    # A decode step is shorter than the host side of its launch (the wrapper repeats the reference's argument
    # checks), so the timed loop replays the step from a HIP graph, as a serving loop would; the eager loop is
    # timed as well and reported beside it.
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    eager_dt = time.perf_counter() - t0
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    heated = preheat(graph.replay, torch, args.preheat_ms)
    for _ in range(args.warmup):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        graph.replay()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    lib.fla_profile_enable.argtypes = [ctypes.c_int]
    lib.fla_profile_enable(1)
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    lib.fla_profile_enable(0)
    prof = profile_report(lib)
    n, ms = prof["recurrent_gdn"]
    bytes_per_launch = 2 * N * H * D * D * 4 + 4 * N * H * D * 2 + N * H * (2 + 4)
    ach = bytes_per_launch / (ms / n * 1e-3) / 1e9
    cpu = None
    if not args.no_cpu:
        from oracle import decode as odec   # the CPU oracle is only ever the baseline being timed
        cores = os.cpu_count() or 1
        torch.set_num_threads(cores)
        ns = N
        c = lambda t: t[:ns].cpu()
        cq, ck, cv, cs, cb, cg = c(q), c(k), c(v), c(state), c(beta), c(gate)
        t1 = time.perf_counter()
        reps = 0
        while reps == 0 or time.perf_counter() - t1 < args.cpu_seconds:
            odec.recurrent_gated_delta_rule(cq, ck, cv, cs, beta=cb, scale=D ** -0.5,
                                            actual_seq_lengths=torch.tensor([0] + [1] * ns, dtype=torch.int32),
                                            ssm_state_indices=torch.arange(ns, dtype=torch.int32), g=cg)
            reps += 1
        cdt = time.perf_counter() - t1
        cpu = {"value": round(ns * reps / cdt, 1), "unit": "tokens/s", "cores": cores, "kind": "port",
               "sample": f"{reps} x ({ns} sequences x 1 token, H=32 K=V=128) fp32 torch oracle, {cdt:.1f} s"}
    # the same operator as a variable-length prefill (it routes such a call to the chunk forward): 64 sequences, lengths
    # uniform in [128, 4096]
    gl = torch.Generator().manual_seed(0)
    plens = torch.randint(128, 4097, (64,), generator=gl)
    PT = int(plens.sum())
    pq = F.normalize(torch.randn(PT, H, D, device=dev, generator=g), dim=-1).bfloat16()
    pk = F.normalize(torch.randn(PT, H, D, device=dev, generator=g), dim=-1).bfloat16()
    pv = torch.randn(PT, H, D, device=dev, generator=g).bfloat16()
    pbeta = torch.sigmoid(torch.randn(PT, H, device=dev, generator=g)).bfloat16()
    pgate = F.logsigmoid(torch.randn(PT, H, device=dev, generator=g))
    pstate = torch.randn(64, H, D, D, device=dev, generator=g) * 0.01
    pseq = torch.cat([torch.zeros(1, dtype=torch.int32), plens.to(torch.int32)]).to(dev)
    pidx = torch.repeat_interleave(torch.arange(64, dtype=torch.int32), plens).to(dev)
    prefill = lambda: ops.recurrent_gated_delta_rule(pq, pk, pv, pstate, beta=pbeta, scale=D ** -0.5,
                                                     actual_seq_lengths=pseq, ssm_state_indices=pidx, g=pgate)
    prefill()
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    for _ in range(5):
        prefill()
    torch.cuda.synchronize()
    pdt = (time.perf_counter() - t2) / 5
    # the same prefill through the chunked forward, which is what a prefill belongs to: token-major q/k/v are strided
    # views, the V-first pool rows are transposed into the chunk kernel's [N,H,K,V] state and back (inside the timing)
    from fla_hip import pipeline
    pcu = [0] + torch.cumsum(plens, 0).tolist()
    hm = lambda t: t.transpose(0, 1)[None]

    def prefill_chunked():
        h0 = pstate.transpose(-1, -2).contiguous()
        o, fin = pipeline.flash_gated_delta_rule(hm(pq), hm(pk), hm(pv), pgate[None], pbeta[None].float(), D ** -0.5, h0, True,
                                                 cu_seqlens=pcu)
        return o, fin.transpose(-1, -2).contiguous()

    prefill_chunked()
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    for _ in range(5):
        prefill_chunked()
    torch.cuda.synchronize()
    cdt2 = (time.perf_counter() - t2) / 5
    # the KDA twin of the decode step (per-channel gate, same state tile), V-first fp32 pool in place
    kg = F.logsigmoid(torch.randn(N, 1, H, D, device=dev, generator=g)) * 0.3
    kcu = torch.arange(N + 1, dtype=torch.int32, device=dev)
    kq, kk, kv, kb = q.view(N, 1, H, D), k.view(N, 1, H, D), v.view(N, 1, H, D), beta.view(N, 1, H).float()
    kda_step = lambda: ops.recurrent_kda(kq, kk, kv, kg, kb, state, cu_seqlens=kcu, state_v_first=True)
    for _ in range(5):
        kda_step()
    lib.fla_profile_enable(1)
    for _ in range(50):
        kda_step()
    torch.cuda.synchronize()
    lib.fla_profile_enable(0)
    kn, kms = profile_report(lib)["recurrent_kda"]
    kda_bytes = 2 * N * H * D * D * 4 + 4 * N * H * D * 2 + N * H * D * 4 + N * H * 4
    kda_decode = {"kernel": "recurrent_kda", "avg_kernel_ms": round(kms / kn, 4),
                  "achieved_GBps": round(kda_bytes / (kms / kn * 1e-3) / 1e9, 1),
                  "frac_of_hbm_peak": round(kda_bytes / (kms / kn * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)}
    return {
        "metric": "gdn_decode_tokens_per_s", "value": round(N * args.steps / dt, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "preheat_ms": heated,
        "ms_per_step": round(dt * 1e3 / args.steps, 4), "algorithmic": {"bytes_per_step": bytes_per_launch},
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "GDN recurrent decode 256 sequences x 1 token, H=32 K=V=128, fp32 state in place",
                   "launch": "HIP graph replay"},
        "eager_ms_per_step": round(eager_dt * 1e3 / args.steps, 4),
        "roofline": {"bound": "hbm", "kernel": "recurrent_gdn", "achieved": round(ach, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(ach / PEAK_HBM_GBS, 4), "traffic": measured_traffic("recurrent_gdn")[0],
                     "traffic_source": measured_traffic("recurrent_gdn")[1],
                     "avg_kernel_ms": round(ms / n, 4)},
        "varlen_prefill": {"sequences": 64, "tokens": PT, "ms": round(pdt * 1e3, 3),
                           "tokens_per_s": round(PT / pdt, 1),
                           "through_chunk_forward": {"ms": round(cdt2 * 1e3, 3), "tokens_per_s": round(PT / cdt2, 1)}},
        "kda_decode": kda_decode,
        "cpu_baseline": cpu,
    }


def bench_conv1d(args, torch, dev):
    import fla_hip
    from fla_hip import ops

    lib = fla_hip.load_library()
    B, T, D, W = 4, 4096, 4096, 4
    g = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn(B, T, D, device=dev, generator=g).bfloat16()
    w = (torch.randn(W, D, device=dev, generator=g) * 0.1).bfloat16()
    b = (torch.randn(D, device=dev, generator=g) * 0.01).bfloat16()

    def step():
        return ops.causal_conv1d(x, w, b, activation_mode=1)

    heated = preheat(step, torch, args.preheat_ms)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # A step is one launch of a kernel of about 45 us.  Its duration is taken from ONE pair of HIP events around the
    # timed region on the launch stream (the stream torch has current, which the wrapper hands to the library): a pair
    # of events around every single launch adds a few microseconds to each, more than the kernel's margin to its bound.
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(args.steps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    kernel_ms = ev0.elapsed_time(ev1) / args.steps
    lib.fla_profile_enable.argtypes = [ctypes.c_int]
    lib.fla_profile_enable(1)
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    lib.fla_profile_enable(0)
    n, ms = profile_report(lib)["conv1d_fwd"]
    bytes_per_launch = 2 * B * T * D * 2 + (W + 1) * D * 2
    ach = bytes_per_launch / (kernel_ms * 1e-3) / 1e9
    cpu = None
    if not args.no_cpu:
        from oracle import conv1d as oconv   # the CPU oracle is only ever the baseline being timed
        cores = os.cpu_count() or 1
        torch.set_num_threads(cores)
        xs, ws, bs = x.cpu(), w.cpu(), b.cpu()
        t1 = time.perf_counter()
        reps = 0
        while reps == 0 or time.perf_counter() - t1 < args.cpu_seconds:
            oconv.causal_conv1d(xs, ws, bs, activation_mode=1)
            reps += 1
        cdt = time.perf_counter() - t1
        cpu = {"value": round(B * T * reps / cdt, 1), "unit": "tokens/s", "cores": cores, "kind": "port",
               "sample": f"{reps} x (B=4 T=4096 D=4096 W=4) fp32 torch oracle, {cdt:.1f} s"}
    # backward of the same shape (no activation / SiLU) and the decode-time state update, timed by the same hooks
    dy = torch.randn(B, T, D, device=dev, generator=g).bfloat16()
    ypre = torch.randn(B, T, D, device=dev, generator=g).bfloat16()
    ux = torch.randn(256, D, device=dev, generator=g).bfloat16()
    ucs = torch.randn(256, W - 1, D, device=dev, generator=g).bfloat16()
    other = {}
    for name, fn, nbytes in (
        ("bwd", lambda: ops.causal_conv1d_bwd(x, None, w, dy), 3 * B * T * D * 2),
        ("bwd_silu", lambda: ops.causal_conv1d_bwd(x, ypre, w, dy, activation=1), 4 * B * T * D * 2),
        ("update_256x1", lambda: ops.causal_conv1d(ux, w, b, ucs, activation_mode=1, run_mode=1), 256 * D * 2 * (2 + 2 * (W - 1))),
    ):
        for _ in range(3):
            fn()
        lib.fla_profile_enable(1)
        for _ in range(50):
            fn()
        torch.cuda.synchronize()
        lib.fla_profile_enable(0)
        kern = {k_: ms_ / n_ for k_, (n_, ms_) in profile_report(lib).items()}
        total = sum(kern.values())
        other[name] = {"kernels_ms": {k_: round(v_, 4) for k_, v_ in kern.items()}, "total_ms": round(total, 4),
                       "algorithmic_GBps": round(nbytes / (total * 1e-3) / 1e9, 1)}
    return {
        "other_modes": other,
        "metric": "causal_conv1d_tokens_per_s", "value": round(B * T * args.steps / dt, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "preheat_ms": heated,
        "ms_per_step": round(dt * 1e3 / args.steps, 4), "algorithmic": {"bytes_per_step": bytes_per_launch},
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "causal_conv1d fwd + SiLU B=4 T=4096 D=4096 width=4 + bias, zero left pad"},
        "roofline": {"bound": "hbm", "kernel": "conv1d_fwd", "achieved": round(ach, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(ach / PEAK_HBM_GBS, 4), "traffic": measured_traffic("conv1d_fwd")[0],
                     "traffic_source": measured_traffic("conv1d_fwd")[1],
                     "avg_kernel_ms": round(kernel_ms, 4), "avg_kernel_ms_with_an_event_pair_per_launch": round(ms / n, 4)},
        "cpu_baseline": cpu,
    }


def bench_kda(args, torch, dev):
    """KDA chunk forward and backward at B=2 T=8192 H=32 K=V=128, BSND.  The step (``value``) is the forward (gate
    activation + cumsum, intra-chunk kernel, state scan); the training step -- the forward that keeps its
    intermediates followed by the whole backward (dq, dk, dv, dg, dbeta, dh0 with a final-state gradient) -- is timed
    in the same run and reported under ``fwd_bwd``, every kernel with its dense-tile FLOP count."""
    import fla_hip
    from fla_hip import ops, pipeline
    from fla_hip.ops import _hip_ctypes as raw_ops

    lib = fla_hip.load_library()
    B, T, H, K, V, C = 2, 8192, 32, 128, 128, args.kda_chunk
    F = torch.nn.functional
    gen = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s: torch.randn(*s, device=dev, generator=gen)
    q = F.normalize(rn(B, T, H, K), dim=-1).bfloat16()
    k = F.normalize(rn(B, T, H, K), dim=-1).bfloat16()
    v = rn(B, T, H, V).bfloat16()
    g = F.logsigmoid(rn(B, T, H, K))
    beta = torch.sigmoid(rn(B, T, H))
    h0 = rn(B, H, K, V) * 0.01
    d_o = rn(B, T, H, V).bfloat16()
    dht = rn(B, H, K, V) * 0.01
    scale = K ** -0.5

    def step():
        return ops.chunk_kda_fwd(q, k, v, g, beta, scale, C, layout="BSND", initial_state=h0, output_final_state=True)

    def train_step():
        # the forward as the autograd entry (pipeline.chunk_kda) runs it: every intermediate the backward reads, qg and kg
        # as float16 for the reverse scan, no u
        f = raw_ops.chunk_kda_fwd_for_backward(q, k, v, g, beta, scale, C, layout="BSND", initial_state=h0,
                                               output_final_state=True)
        _o, _final, gk, Aqk, Akk, w, _u, qg, kg, v_new, h, _ = f
        return pipeline.chunk_kda_bwd(q, k, v, beta, gk, Aqk, Akk, w, qg, kg, v_new, h, scale, d_o, dht,
                                      initial_state=h0, layout="BSND", chunk_size=C)

    heated = preheat(step, torch, args.preheat_ms)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt * 1e3 / args.steps

    lib.fla_profile_enable.argtypes = [ctypes.c_int]
    lib.fla_profile_enable(1)
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    lib.fla_profile_enable(0)
    kern = {name: ms / n for name, (n, ms) in profile_report(lib).items()}
    th = B * T * H
    flops = {"kda_intra": 2 * (2 * C * K + C * K + C * V + C * C) * th,          # kk, qk, w, u, inverse
             "kda_scan": 2 * (3 * K * V + C * V) * th}                           # w.S, qg.S, kg^T.v_new, Aqk.v_new
    if C == 128:   # dense-tile count of the 64-token kernels that run: diagonal blocks in kda_intra, the rest in kda_cross
        flops["kda_intra"] = 2 * (3 * 64 * K + 64 * V + 64 * 64) * th
    dominant = max(("kda_intra", "kda_scan"), key=lambda n: kern.get(n, 0.0))
    ach = flops[dominant] / (kern[dominant] * 1e-3) / 1e12
    fwd_flops = flops["kda_intra"] + flops["kda_scan"]
    step_tflops = fwd_flops / (ms_per_step * 1e-3) / 1e12
    # The same step against the memory roofline, which is the nearer of the two for this operator: at 8 TB/s the bytes
    # below take 7 times longer than the FLOPs above at the bf16 peak.  Inputs q, k, v, raw gate, beta; results o, gk,
    # Aqk, Akk; and w, u, qg, kg once out of the intra-chunk kernel and once into the state scan, with Aqk read again.
    io_bytes = th * (2 * K * 2 + V * 2 + K * 4 + 4) + th * (V * 2 + K * 4 + 2 * C * 2)
    hop_bytes = 2 * th * (3 * K * 2 + V * 2) + th * C * 2
    step_gbps = (io_bytes + hop_bytes) / (ms_per_step * 1e-3) / 1e9
    kbytes = {"kda_intra": th * (2 * K * 2 + V * 2 + K * 4 + 4) + th * (K * 4 + 2 * C * 2 + 3 * K * 2 + V * 2),
              "kda_scan": th * (3 * K * 2 + V * 2 + C * 2) + th * V * 2}

    fwd_bwd = None
    if C == 64:   # the backward operators work on 64-token chunks
        n_train = max(3, args.steps // 4)
        for _ in range(3):
            grads = train_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n_train):
            grads = train_step()
        torch.cuda.synchronize()
        train_ms = (time.perf_counter() - t0) * 1e3 / n_train
        assert all(bool(torch.isfinite(t.float()).all()) for t in grads)
        lib.fla_profile_enable(1)
        for _ in range(n_train):
            train_step()
        torch.cuda.synchronize()
        lib.fla_profile_enable(0)
        tk = {name: ms / n for name, (n, ms) in profile_report(lib).items()}
        bwd_flops = {   # dense-tile FLOPs per launch
            "kda_bwd_dav": 2 * (2 * C * V) * th,                       # do v_new^T, Aqk^T do
            "bwd_dhu": 2 * (3 * K * V) * th,                           # k dh, q^T do, w^T dv
            "kda_bwd_dqkwg": 2 * (3 * K * V) * th,                     # do h^T, dv h^T, v_new dh^T
            "kda_bwd_wy": 2 * (2 * C * (K + V) + 2 * C * C) * th,      # dA, Akk^T [dw | du], two 64^3 products
            "kda_bwd_intra": 2 * (5 * C * K) * th,                     # four triangular C x C x K products (fp32 pipe)
        }
        all_flops = dict(flops, **bwd_flops)
        total = sum(all_flops[n] for n in tk if n in all_flops)
        fwd_bwd = {"ms_per_step": round(train_ms, 4), "steps": n_train, "tokens_per_s": round(B * T / (train_ms * 1e-3), 1),
                   "step_tflops": round(total / (train_ms * 1e-3) / 1e12, 2),
                   "frac_of_bf16_peak": round(total / (train_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4),
                   "kernels": {n: {"ms": round(t, 4), "gflop": round(all_flops[n] / 1e9, 2) if n in all_flops else None,
                                   "tflops": round(all_flops[n] / (t * 1e-3) / 1e12, 1) if n in all_flops else None}
                               for n, t in tk.items()}}
    cpu = None
    if not args.no_cpu:
        from oracle import kda as okda   # the CPU oracle is only ever the baseline being timed
        import torch as _t
        cores = os.cpu_count() or 1
        _t.set_num_threads(cores)
        Ts = min(args.cpu_tokens, 2048)
        c = lambda x: x[:1, :Ts].transpose(1, 2).contiguous().cpu()
        cq, ck, cv, cg, cb = c(q), c(k), c(v), c(g), beta[:1, :Ts].transpose(1, 2).contiguous().cpu()
        t1 = time.perf_counter()
        reps = 0
        while reps == 0 or time.perf_counter() - t1 < args.cpu_seconds:
            cgk = okda.kda_gate_cumsum(cg, C)
            okda.chunk_kda_fwd(cq, ck, cv, cgk, cb, scale, C, initial_state=h0[:1].cpu(), output_final_state=True)
            reps += 1
        cdt = time.perf_counter() - t1
        cpu = {"value": round(Ts * reps / cdt, 1), "unit": "tokens/s", "cores": cores, "kind": "port",
               "sample": f"{reps} x (B=1 T={Ts} H={H} K=V={K}) chunked fp32 torch oracle forward, {cdt:.1f} s"}
    assert bool(torch.isfinite(out[0].float()).all()) and bool(torch.isfinite(out[1]).all())
    return {
        "metric": "kda_chunk_fwd_tokens_per_s", "value": round(B * T * args.steps / dt, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "preheat_ms": heated, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"KDA chunk forward B=2 T=8192 H=32 K=V=128 chunk={C} BSND, fp32 initial+final state"},
        "algorithmic": {"flops_per_step": fwd_flops, "bytes_per_step_results_and_inputs": io_bytes,
                        "bytes_per_step_between_the_two_kernels": hop_bytes},
        "step_tflops": round(step_tflops, 2), "step_frac_of_bf16_peak": round(step_tflops / PEAK_BF16_TFLOPS, 4),
        "step_GBps": round(step_gbps, 1), "step_frac_of_hbm_peak": round(step_gbps / PEAK_HBM_GBS, 4),
        "roofline": {"bound": "hbm", "kernel": dominant, "achieved": round(kbytes[dominant] / (kern[dominant] * 1e-3) / 1e9, 1),
                     "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(kbytes[dominant] / (kern[dominant] * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                     "traffic": measured_traffic(dominant)[0], "traffic_source": measured_traffic(dominant)[1],
                     "avg_kernel_ms": round(kern[dominant], 4),
                     "against_bf16_peak": {"achieved_tflops": round(ach, 2), "frac": round(ach / PEAK_BF16_TFLOPS, 4)}},
        "other_kernels_ms": {n: round(t, 4) for n, t in kern.items()},
        "fwd_bwd": fwd_bwd,
        "cpu_baseline": cpu,
    }


def bench_gdn_bwd(args, torch, dev):
    """GDN chunk backward at the headline shape: the reference's composition of the backward operators
    (recompute of A, w, u, h; dv_local; reverse scan; dqkwg; WY backward; reverse cumsum), one step = one
    pass producing dq, dk, dv, dbeta, dg and dh0.  `roofline` describes the kernel that takes the most time."""
    import fla_hip
    from fla_hip import pipeline

    lib = fla_hip.load_library()
    B, T, H, K, V, C = 4, 8192, 32, 128, 128, 64
    F = torch.nn.functional
    gen = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s: torch.randn(*s, device=dev, generator=gen)
    q = F.normalize(rn(B, H, T, K), dim=-1).bfloat16()
    k = F.normalize(rn(B, H, T, K), dim=-1).bfloat16()
    v = rn(B, H, T, V).bfloat16()
    beta = torch.sigmoid(rn(B, T, H))
    gate = F.logsigmoid(rn(B, T, H))
    h0 = rn(B, H, K, V) * 0.01
    do = rn(B, T, H, V).bfloat16()
    dht = rn(B, H, K, V) * 0.01
    scale = K ** -0.5
    G = fla_hip.ops.chunk_local_cumsum(gate.transpose(1, 2).contiguous(), C, head_first=True,
                                       output_dtype=torch.float32).transpose(1, 2).contiguous()

    def step():
        return pipeline.flash_chunk_gated_delta_rule_bwd(q, k, v, G, beta, None, scale, h0, do, dht, chunk_size=C)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt * 1e3 / args.steps
    # the same step when the forward kept its inverted chunk matrices (the six-operator forward does, as the
    # reference's forward does; the fused forward keeps none, which is the case timed above)
    A_saved = fla_hip.ops.chunk_scaled_dot_kkt_inverse(k, G.transpose(1, 2), beta.transpose(1, 2), chunk_size=C)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        pipeline.flash_chunk_gated_delta_rule_bwd(q, k, v, G, beta, A_saved, scale, h0, do, dht, chunk_size=C)
    torch.cuda.synchronize()
    ms_saved_A = (time.perf_counter() - t0) * 1e3 / args.steps
    # training as the autograd entry runs it: the fused forward also writes h, v_new and w, the backward recomputes
    # only the inverted chunk matrices
    def fwd_train():
        return pipeline.flash_chunk_gated_delta_rule_fwd(q, k, v, gate, beta, scale, h0, True, None, C,
                                                         save_for_backward=True)

    def train_step():
        gc, _, _, _, saved = fwd_train()
        return pipeline.flash_chunk_gated_delta_rule_bwd(q, k, v, gc, beta, None, scale, h0, do, dht, chunk_size=C,
                                                         saved=saved)

    def timed(fn):
        for _ in range(max(2, args.warmup // 4)):
            fn()
        torch.cuda.synchronize()
        t_ = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t_) * 1e3 / args.steps

    ms_train = timed(train_step)
    ms_fwd_train = timed(fwd_train)

    # the same step as a model runs it: token-major q, k, v (one row per token holds every head, as a projection
    # leaves them) through the autograd entry, without and with the row normalisation of q and k inside the kernels
    def autograd_step(l2norm):
        tq, tk, tv = (t.transpose(1, 2).contiguous().transpose(1, 2).detach().requires_grad_(True) for t in (q, k, v))
        tg, tb = gate.detach().clone().requires_grad_(True), beta.detach().clone().requires_grad_(True)

        def run():
            o, _ = pipeline.flash_gated_delta_rule(tq, tk, tv, tg, tb, output_final_state=True, use_qk_l2norm_in_kernel=l2norm)
            o.backward(do)
            for t in (tq, tk, tv, tg, tb):
                t.grad = None
        return timed(run)

    ms_autograd, ms_autograd_l2 = autograd_step(False), autograd_step(True)
    ms_fwd_plain = timed(lambda: pipeline.flash_chunk_gated_delta_rule_fwd(q, k, v, gate, beta, scale, h0, True, None, C))
    lib.fla_profile_enable.argtypes = [ctypes.c_int]
    lib.fla_profile_enable(1)
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    lib.fla_profile_enable(0)
    kern = {name: ms / n for name, (n, ms) in profile_report(lib).items()}
    th = B * T * H
    flops_of = {  # dense-tile FLOPs per launch
        "bwd_dv_local": 2 * (C * K + C * V) * th,
        "bwd_dqkwg": 2 * (3 * K * V + C * V + 2 * C * K) * th,
        "wy_bwd_da": 2 * (C * K + C * V + 2 * C * C) * th,
        "wy_bwd_full": 2 * (3 * C * K + C * V) * th,
        "bwd_dhu": 2 * (3 * K * V) * th,
        "kkt": 2 * C * K * th, "solve_tri": 2 * (C * C // 3) * th, "wu": 2 * (C * K + C * V) * th,
        "fwd_h": 2 * (2 * K * V) * th,
    }
    if "bwd_dv_local" not in kern:   # 64-token chunks: the reverse scan forms the intra-chunk dv itself
        flops_of["bwd_dhu"] += flops_of.pop("bwd_dv_local")
    if "wy_bwd_da" not in kern:      # and the WY backward forms dA itself
        flops_of["wy_bwd_full"] += flops_of.pop("wy_bwd_da")
    timed = {n: t for n, t in kern.items() if n in flops_of}
    dominant = max(timed, key=timed.get)
    ach = flops_of[dominant] / (kern[dominant] * 1e-3) / 1e12
    step_flops = sum(flops_of[n] for n in timed)
    cpu = None
    if not args.no_cpu:
        from oracle import gdn as ogdn, gdn_bwd as obwd   # the CPU oracle is only ever the baseline being timed
        import torch as _t
        cores = os.cpu_count() or 1
        _t.set_num_threads(cores)
        Ts = min(args.cpu_tokens, 2048)
        d = ogdn.make_gdn_inputs(1, Ts, H, K, V, dtype=_t.bfloat16, seed=0, init_std=0.01, head_first_gates=True)
        cdo = _t.randn(1, H, Ts, V).bfloat16()
        t1 = time.perf_counter()
        reps = 0
        while reps == 0 or time.perf_counter() - t1 < args.cpu_seconds:
            obwd.chunk_gated_delta_rule_bwd(d["q"], d["k"], d["v"], d["g"], d["beta"], scale, cdo,
                                            initial_state=d["initial_state"], chunk=C)
            reps += 1
        cdt = time.perf_counter() - t1
        cpu = {"value": round(Ts * reps / cdt, 1), "unit": "tokens/s", "cores": cores, "kind": "port",
               "sample": f"{reps} x (B=1 T={Ts} H={H} K=V={K}) composed fp32 torch oracle backward, {cdt:.1f} s"}
    assert all(bool(torch.isfinite(t.float()).all()) for t in out)
    return {
        "metric": "gdn_chunk_bwd_tokens_per_s", "value": round(B * T * args.steps / dt, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "GDN chunk backward B=4 T=8192 H=32 K=V=128 chunk=64, initial state and final-state gradient, "
                               "A recomputed from k, g, beta"},
        "ms_per_step_with_saved_A": round(ms_saved_A, 4),
        "training": {"fwd_bwd_ms": round(ms_train, 4), "fwd_saving_h_vnew_w_ms": round(ms_fwd_train, 4),
                     "bwd_with_saved_ms": round(ms_train - ms_fwd_train, 4), "fwd_inference_ms": round(ms_fwd_plain, 4),
                     "fwd_inference_plus_bwd_recompute_ms": round(ms_fwd_plain + ms_per_step, 4),
                     "autograd_token_major_ms": round(ms_autograd, 4),
                     "autograd_token_major_qk_l2norm_ms": round(ms_autograd_l2, 4)},
        "step_tflops": round(step_flops / (ms_per_step * 1e-3) / 1e12, 2),
        "roofline": {"bound": "mfma", "kernel": dominant, "achieved": round(ach, 2), "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(ach / PEAK_BF16_TFLOPS, 4), "traffic": None,
                     "avg_kernel_ms": round(kern[dominant], 4),
                     "all_kernels_ms": {n: round(t, 4) for n, t in kern.items()}},
        "cpu_baseline": cpu,
    }


def bench_copy(args, torch, dev):
    """Calibration only (not a product kernel): a plain device-to-device copy of known size, used to
    scale the FETCH_SIZE / WRITE_SIZE counters and as the practical bandwidth ceiling of the box."""
    n = 512 * 1024 * 1024  # bytes each way
    x = torch.empty(n, dtype=torch.uint8, device=dev).random_(0, 255)
    y = torch.empty_like(x)
    for _ in range(args.warmup):
        y.copy_(x)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        y.copy_(x)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    gbs = 2 * n * args.steps / dt / 1e9
    return {"metric": "device_copy_GBps", "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": round(dt * 1e3 / args.steps, 4), "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
            "config": {"workload": "torch device copy 512 MiB -> 512 MiB (calibration, not a product kernel)"},
            "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None}, "cpu_baseline": None}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=50)   # the device clock needs some tens of milliseconds of load to ramp
    ap.add_argument("--l2norm", action="store_true", help="gdn_chunk: normalise q and k rows inside the kernel")
    ap.add_argument("--kda-chunk", type=int, default=64, choices=[64, 128], help="kda: tokens per chunk")
    ap.add_argument("--workload", default="gdn_chunk", choices=["gdn_chunk", "gdn_bwd", "decode", "conv1d", "kda", "copy"])
    ap.add_argument("--route", default="fused", choices=["fused", "ops"],
                    help="gdn_chunk: one fused library call, or the six per-stage operators")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-secondary", action="store_true", help="gdn_chunk: skip the brief decode / conv1d / kda legs")
    ap.add_argument("--preheat-ms", type=float, default=300.0,
                    help="untimed repetitions of the step before the warm-up, so that the device clock has ramped")
    ap.add_argument("--cpu-tokens", type=int, default=8192, help="tokens per pass of the CPU baseline sample")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="minimum CPU time spent on the baseline")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; every kernel works on one GPU's share and there are no "
              "collectives to time. Use --gpus 1.", file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible.", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    fn = {"gdn_chunk": bench_gdn, "gdn_bwd": bench_gdn_bwd, "decode": bench_decode, "conv1d": bench_conv1d, "kda": bench_kda, "copy": bench_copy}[args.workload]
    result = fn(args, torch, dev)
    if args.workload == "gdn_chunk" and not args.no_secondary:
        # The other configurations the headline metric names, timed briefly after the main region so that the one
        # line a default run prints carries them too: each with its step time, algorithmic work, roofline fraction
        # and its own bounded CPU baseline.  They never enter `value`.
        brief = argparse.Namespace(**vars(args))
        brief.steps, brief.warmup, brief.preheat_ms = 100, 10, min(args.preheat_ms, 100.0)
        brief.cpu_seconds, brief.cpu_tokens = min(args.cpu_seconds, 2.0), 512
        secondary = {}
        for name, sub in (("kda", bench_kda), ("decode", bench_decode), ("conv1d", bench_conv1d)):
            r = sub(brief, torch, dev)
            keep = ("metric", "value", "unit", "steps", "ms_per_step", "dtype", "config", "algorithmic", "step_tflops",
                    "step_GBps", "step_frac_of_hbm_peak", "roofline", "cpu_baseline", "fwd_bwd", "varlen_prefill", "eager_ms_per_step")
            secondary[name] = {k_: r[k_] for k_ in keep if k_ in r}
            secondary[name]["ms"] = r["ms_per_step"]
            secondary[name]["frac"] = r["roofline"]["frac"]
        result["secondary"] = secondary
    print(json.dumps(result))


if __name__ == "__main__":
    main()
