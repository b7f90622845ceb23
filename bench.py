#!/usr/bin/env python3
"""Benchmark of the chunked linear-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]

A step is one chunk_gla forward on the headline workload (B=8, T=4096, H=16,
K=V=128, bf16 q/k/v, fp32 log-gates and state, initial state given, final state
returned), inputs resident in HBM.  Prints ONE JSON line:

* value            tokens/s of the whole forward: tokens of the K timed steps / the wall time between the two
                   synchronisations that bracket them (ms_per_step = that wall time / K; the host time of a
                   call with the launches stubbed out is in extra.chunk_gla_fwd.host_us_per_call)
* roofline         the dominant kernel of that forward against the HBM roofline:
                   algorithmic bytes per launch / its median duration measured
                   here with HIP events on the launch stream; traffic = HBM bytes per launch from
                   the counter readings kept in profiles/hbm_traffic_counters.txt
* cpu_baseline     the oracle's fp32 naive recurrence timed on the host cores on
                   a bounded sample of the same workload
* extra            the other measured rows: the T=1 decode steps (B=256, H=32),
                   chunk_gated_delta_rule forward on a packed batch, forward + backward
                   of both chunk operators (B=4, T=4096)
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "flash-linear-attention_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

MFMA_PEAK_FLOPS = 2.5e15   # dense bf16 MFMA, FLOP/s
HBM_PEAK_GBS = 8000.0
MIB = 1 << 20
RAMP_SECONDS = 1.0         # untimed load ahead of the warm-up steps (clock ramp): at least this long ...
RAMP_MAX_SECONDS = 5.0     # ... and at most this long, until the step time has settled


def _events(n):
    import torch
    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


ROW_RAMP_SECONDS = 0.2     # untimed load ahead of every timed row other than the headline step


def event_stats(fn, steps, warmup=3, ramp=None, between=None):
    """Device time of one call from HIP events recorded on the launch stream around every call:
    median, min, max and mean in microseconds, the number of intervals longer than twice the median
    (a stalled launch: clock ramp, an allocation, something else on the box) and the wall time of the
    whole timed loop, which is bracketed by synchronize on both sides.  The setup of a row (allocations,
    first calls) leaves the device idle for milliseconds and its clocks drop; `ramp` seconds of the call
    itself run untimed first, so that a 20-launch row and a 200-launch row report the same figure.
    `between`, if given, runs on the same stream ahead of every timed call, outside its pair of events
    (a write over a large buffer that pushes the previous call's tensors out of the last-level cache)."""
    import statistics
    import torch
    if ramp is None:
        ramp = ROW_RAMP_SECONDS
    t_ramp = time.perf_counter()
    while time.perf_counter() - t_ramp < ramp:
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    ev = _events(2 * steps)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        if between is not None:
            between()
        ev[2 * i].record()
        fn()
        ev[2 * i + 1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    us = [ev[2 * i].elapsed_time(ev[2 * i + 1]) * 1e3 for i in range(steps)]
    med = statistics.median(us)
    return {"median_us": med, "min_us": min(us), "max_us": max(us), "mean_us": sum(us) / steps, "n": steps,
            "n_over_2x_median": sum(1 for x in us if x > 2 * med), "wall_us_per_call": wall / steps * 1e6}


def spread(st):
    """The part of event_stats() every row reports beside its median."""
    return {"min_us": round(st["min_us"], 1), "max_us": round(st["max_us"], 1), "n": st["n"],
            "n_over_2x_median": st["n_over_2x_median"]}


def event_avg_us(fn, steps, warmup=3, ramp=None, between=None):
    """Median device time of one call (see event_stats)."""
    return event_stats(fn, steps, warmup, ramp, between)["median_us"]


class _StubLib:
    """Stands in for the loaded library: the named entry points return 0 without launching anything."""

    def __init__(self, real, names):
        self._real, self._names = real, set(names)

    def __getattr__(self, name):
        if name in self._names:
            return lambda *a: 0
        return getattr(self._real, name)


def host_time_us(fn, entry_points, n=2000):
    """Host time of one call of `fn` with the kernel launches of `entry_points` stubbed out (argument
    marshalling, allocations and Python included; the device stays idle)."""
    import torch
    from fla_amd import _backend as be
    real = be.lib()
    be._lib = _StubLib(real, entry_points)
    try:
        for _ in range(50):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        dt = time.perf_counter() - t0
    finally:
        be._lib = real
    return dt / n * 1e6


TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic_counters.txt")


def counter_traffic(kernel):
    """HBM bytes per launch of `kernel` from the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs whose
    readings are kept in profiles/hbm_traffic_counters.txt (one tab-separated line per kernel: name,
    FETCH_SIZE, WRITE_SIZE; a `scale` line holds the bytes per counter unit found with the 1 GiB copy
    of the same runs; the kernels of the roofline blocks also appear as `roofline:<kernel>:<workload>`).
    None if the file or the kernel is missing."""
    try:
        lines = [l.rstrip("\n").split("\t") for l in open(TRAFFIC_FILE) if l.strip() and not l.startswith("#")]
    except OSError:
        return None
    scale = next((l for l in lines if l[0] == "scale"), None)
    row = next((l for l in lines if l[0] == kernel), None)
    if scale is None or row is None:
        return None
    return int(round(float(row[1]) * float(scale[1]) + float(row[2]) * float(scale[2])))


def gla_config1(device):
    import torch
    import torch.nn.functional as F
    torch.manual_seed(0)
    B, T, H, K, V = 8, 4096, 16, 128, 128
    q = torch.randn(B, T, H, K, device=device).bfloat16()
    k = torch.randn(B, T, H, K, device=device).bfloat16()
    v = torch.randn(B, T, H, V, device=device).bfloat16()
    g = F.logsigmoid(torch.randn(B, T, H, K, device=device)) / 16
    h0 = torch.randn(B, H, K, V, device=device) * 0.1
    return dict(B=B, T=T, H=H, K=K, V=V, q=q, k=k, v=v, g=g, h0=h0)


def bench_gla(device, steps, warmup):
    import torch
    from fla_amd.ops.common.chunk_h import chunk_fwd_h
    from fla_amd.ops.gla import chunk_gla
    from fla_amd.ops.gla.chunk import chunk_gla_fwd_o_gk
    c = gla_config1(device)
    q, k, v, g, h0 = c["q"], c["k"], c["v"], c["g"], c["h0"]
    B, T, H, K, V = c["B"], c["T"], c["H"], c["K"], c["V"]

    def step():
        return chunk_gla(q, k, v, g, initial_state=h0, output_final_state=True, head_first=False)

    # The clocks of an idle GPU need load to reach their steady state (the first launches after idle run about
    # 25 % slower, and on a box whose first GPU process this is the ramp takes longer than on a warm one): keep
    # the device busy with the step itself for at least RAMP_SECONDS before the warm-up steps, whatever --warmup
    # says, and on until three consecutive batches of 50 steps take the same time within 0.5 % (at most
    # RAMP_MAX_SECONDS).
    if RAMP_SECONDS > 0:
        t_ramp = time.perf_counter()
        hist = []
        while True:
            t_b = time.perf_counter()
            for _ in range(50):
                step()
            torch.cuda.synchronize()
            now = time.perf_counter()
            hist.append(now - t_b)
            last = hist[-3:]
            steady = len(last) == 3 and max(last) - min(last) <= 0.005 * min(last)
            if now - t_ramp >= RAMP_MAX_SECONDS or (steady and now - t_ramp >= RAMP_SECONDS):
                break

    # `warmup` untimed steps, then exactly `steps` steps between two synchronisations: value = tokens of those
    # steps / the wall time between the two synchronisations (host side of every step included; the host
    # needs a fraction of a step per call, so the launches queue up and the device sets the pace).
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    wall_us = (time.perf_counter() - t0) / steps * 1e6
    ms = wall_us * 1e-3
    tokens_per_s = B * T / (wall_us * 1e-6)

    # host side of one step: the same call with the launch replaced by a stub that returns at once
    host_us = host_time_us(step, ("fla_chunk_gla_fwd_fused",))

    # device time of the kernels of the forward, HIP events on the launch stream.  The operator is one launch
    # of gla_fwd_fused_kernel (its workgroups redo chunks flagged by the range guard after their last chunk:
    # none in this workload); the kernel is timed on its own in that form (guard workspaces given).  The two-kernel
    # pipeline it replaces (state scan + per-chunk output) is timed as well for comparison.
    scale = K ** -0.5

    # pointers and workspaces bound once: the host side of a launch is then a few microseconds, the launches
    # queue up behind each other and an event interval holds device time only
    from fla_amd import _backend as be
    from fla_amd.ops.gla.chunk import _guard_workspaces
    o_buf, ht_buf = torch.empty_like(v), q.new_empty(B, H, K, V, dtype=torch.float32)
    wide, hwide = _guard_workspaces(q, B * (T // 64), H, K * V, keep=False)
    fused_args = (be.ptr(q), be.ptr(k), be.ptr(v), be.ptr(g), be.ptr(h0), be.ptr(o_buf), be.ptr(ht_buf), be.ptr(wide),
                  be.ptr(hwide), None, None, None, None, 0, be.dt(q), be.dt(g), B, T, H, K, V, B, float(scale),
                  be.stream_of(q))
    first_launch = be.lib().fla_chunk_gla_fwd_fused_first_launch

    def run_fused():
        be.check(first_launch(*fused_args), "fla_chunk_gla_fwd_fused_first_launch")

    h_hold = {}

    def run_h():
        h_hold["h"], h_hold["ht"] = chunk_fwd_h(k=k, v=v, g=None, gk=g, gv=None, h0=h0, output_final_state=True,
                                                head_first=False, chunk_size=64, gates_are_cumsum=False,
                                                fragment_layout=True)

    run_h()

    def run_o():
        chunk_gla_fwd_o_gk(q, v, g, None, h_hold["h"], scale, head_first=False, chunk_size=64, k=k,
                           gates_are_cumsum=False)

    n_ev = max(steps, 20)
    st_f = event_stats(run_fused, n_ev, warmup=10)
    us_f = st_f["median_us"]
    us_h = event_avg_us(run_h, 20)
    us_o = event_avg_us(run_o, 20)
    NT = T // 64
    qkv = B * T * H * K * 2                      # one bf16 [B,T,H,128] tensor
    gbytes = B * T * H * K * 4                   # fp32 gates
    hbytes = B * NT * H * K * V * 2              # bf16 per-chunk states
    stb = B * H * K * V * 4                      # one fp32 state
    floor_bytes = 4 * qkv + gbytes + 2 * stb     # q,k,v,o + g + h0,ht: the operator's algorithmic bytes
    bytes_h = 2 * qkv + gbytes + hbytes + 2 * stb          # k, v, g in; h, ht out; h0 in
    bytes_o = 3 * qkv + gbytes + hbytes + qkv              # q, k, v, g, h in; o out
    ach = floor_bytes / (us_f * 1e-6) / 1e9
    flops = B * T * H * (4 * K * V + 2 * 64 * K + 2 * 64 * V)   # dense-tile count of the chunked algorithm
    roofline = {"kernel": "gla_fwd_fused_kernel", "bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBS, 4),
                "traffic": counter_traffic("roofline:gla_fwd_fused_kernel:config1"),
                "avg_us": round(us_f, 1), "bytes_per_launch": floor_bytes,
                "frac_of_mfma_peak": round(flops / (us_f * 1e-6) / MFMA_PEAK_FLOPS, 4), **spread(st_f)}
    op = {"algorithmic_bytes": floor_bytes, "achieved_GBs": round(floor_bytes / (ms * 1e-3) / 1e9, 1),
          "frac_of_hbm_peak": round(floor_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
          "algorithmic_flops": flops, "frac_of_mfma_peak": round(flops / (ms * 1e-3) / MFMA_PEAK_FLOPS, 4),
          "wall_us_per_step": round(wall_us, 1), "host_us_per_call": round(host_us, 1),
          # the step is that one kernel: host-bound would show as a wall time per step well above its device time
          "host_bound": bool(host_us > 0.5 * wall_us or wall_us > 1.08 * us_f),
          "two_kernel_pipeline_us": {"gla_fwd_h_kernel": round(us_h, 1), "gla_fwd_o_kernel": round(us_o, 1)},
          "two_kernel_pipeline_GBs": {"gla_fwd_h_kernel": round(bytes_h / (us_h * 1e-6) / 1e9, 1),
                                      "gla_fwd_o_kernel": round(bytes_o / (us_o * 1e-6) / 1e9, 1)}}
    return ms, tokens_per_s, roofline, op, c


def bench_decode(device, steps=1000):
    """Decode workload: B=256, H=32, K=V=128 single-token step, state in place."""
    import torch
    import torch.nn.functional as F
    from fla_amd.ops.gated_delta_rule import fused_recurrent_gated_delta_rule
    from fla_amd.ops.gla import fused_recurrent_gla
    torch.manual_seed(0)
    B, H, K, V = 256, 32, 128, 128
    out = {}
    q = torch.randn(B, 1, H, K, device=device).bfloat16()
    kk = torch.randn(B, 1, H, K, device=device)
    v = torch.randn(B, 1, H, V, device=device).bfloat16()
    gk = F.logsigmoid(torch.randn(B, 1, H, K, device=device))
    g = F.logsigmoid(torch.randn(B, 1, H, device=device))
    beta = torch.rand(B, 1, H, device=device).sigmoid()
    state_bytes = B * H * K * V * 4
    small = B * H * 128 * 2
    # one state buffer for both recurrences, refilled in place: what a serving loop holds for the whole generation
    S = torch.empty(B, H, K, V, device=device)
    for name in ("gla", "gdr"):
        S.normal_().mul_(0.1)
        if name == "gla":
            k = kk.bfloat16()
            fn = lambda: fused_recurrent_gla(q, k, v, gk, initial_state=S, output_final_state=True,
                                             head_first=False, inplace_state=True)
            nbytes = 2 * state_bytes + 4 * small + B * H * K * 4
        else:
            k = F.normalize(kk, dim=-1).bfloat16()
            fn = lambda: fused_recurrent_gated_delta_rule(q, k, v, g, beta, initial_state=S,
                                                          output_final_state=True, head_first=False,
                                                          inplace_state=True)
            nbytes = 2 * state_bytes + 4 * small + 2 * B * H * 4
        # 1000 consecutive steps: the wall time of the loop per step (what a serving loop sees, host
        # included) and the median of the per-step HIP-event intervals (the device side)
        st = event_stats(fn, steps, 20)
        us = st["wall_us_per_call"]
        assert torch.isfinite(S).all()
        out[name] = {"us_per_step": round(us, 1), "tokens_per_s": round(B / (us * 1e-6), 1),
                     "GBs": round(nbytes / (us * 1e-6) / 1e9, 1),
                     "frac_of_hbm_peak": round(nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                     "bytes_per_step": nbytes, "steps": steps,
                     "event_median_us": round(st["median_us"], 1), **spread(st)}
        # the same step captured once in a HIP graph and replayed: no Python between the launches
        S.normal_().mul_(0.1)
        fn()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            fn()
        stg = event_stats(graph.replay, steps, 20)
        usg = stg["wall_us_per_call"]
        assert torch.isfinite(S).all()
        out[name]["hip_graph_replay"] = {"us_per_step": round(usg, 1), "tokens_per_s": round(B / (usg * 1e-6), 1),
                                         "frac_of_hbm_peak": round(nbytes / (usg * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                                         "event_median_us": round(stg["median_us"], 1), **spread(stg)}
    return out


def bench_decode_layer_step(device, steps=300):
    """One token through what a gated DeltaNet layer runs around its state update at the decode shape (B=256, H=32,
    D=128): short-convolution step, l2 norm of q and k, the in-place recurrent step, gated RMS norm of the output -
    six launches with the shift that derives k - run eagerly (wall time per step, host included) and replayed from one captured HIP graph."""
    import torch
    import torch.nn.functional as F
    from fla_amd.modules import FusedRMSNormSwishGate, ShortConvolution, l2_norm
    from fla_amd.ops.gated_delta_rule import fused_recurrent_gated_delta_rule
    torch.manual_seed(0)
    B, H, D, W = 256, 32, 128, 4
    conv = ShortConvolution(H * D, W, activation="silu").to(device).bfloat16()
    norm = FusedRMSNormSwishGate(D).to(device)
    x = torch.randn(B, 1, H * D, device=device).bfloat16()
    gate_in = torch.randn(B, 1, H * D, device=device).bfloat16()
    g = F.logsigmoid(torch.randn(B, 1, H, device=device))
    beta = torch.rand(B, 1, H, device=device)
    state = torch.randn(B, H, D, D, device=device) * 0.1
    cache = torch.zeros(B, H * D, W, device=device, dtype=torch.bfloat16)

    def step():
        y, _ = conv(x, cache=cache)
        q = l2_norm(y.view(B, 1, H, D))
        k = l2_norm(torch.roll(y, 1, dims=-1).view(B, 1, H, D))
        o, _ = fused_recurrent_gated_delta_rule(q, k, y.view(B, 1, H, D), g, beta, initial_state=state,
                                                output_final_state=True, head_first=False, inplace_state=True)
        return norm(o, gate_in.view(B, 1, H, D))

    def step_fused_norms():   # the two l2 norms inside the recurrent step's launch: four launches
        y, _ = conv(x, cache=cache)
        o, _ = fused_recurrent_gated_delta_rule(y.view(B, 1, H, D), torch.roll(y, 1, dims=-1).view(B, 1, H, D),
                                                y.view(B, 1, H, D), g, beta, initial_state=state,
                                                output_final_state=True, head_first=False, inplace_state=True,
                                                use_qk_l2norm_in_kernel=True)
        return norm(o, gate_in.view(B, 1, H, D))

    def eager_and_graph(fn):
        st_e = event_stats(fn, steps, 20)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            fn()
        st_g = event_stats(graph.replay, steps, 20)
        return {"eager_wall_us_per_step": round(st_e["wall_us_per_call"], 1),
                "eager_event_median_us": round(st_e["median_us"], 1),
                "hip_graph_replay_wall_us_per_step": round(st_g["wall_us_per_call"], 1),
                "hip_graph_replay_event_median_us": round(st_g["median_us"], 1)}

    with torch.no_grad():
        out = {"launches_per_step": 6, **eager_and_graph(step)}
        out["l2norm_in_step"] = {"launches_per_step": 4, **eager_and_graph(step_fused_norms)}
    assert torch.isfinite(state).all()
    return out


def bench_gdr(device, steps=50, warmup=20):
    """chunk_gated_delta_rule forward: the packed workload (12 sequences, 32768 tokens) and the
    fixed-length shape B=8, T=4096 of the headline metric.  Each row carries a roofline block for its
    dominant kernel (the serial scan, gdr_fwd_scan_kernel) and the time of the chunk-parallel launch
    that precedes it (gdr_fwd_prep_kernel), both from HIP events round the single launch."""
    import torch
    import torch.nn.functional as F
    from fla_amd.ops.common.chunk_delta_h import chunk_gated_delta_rule_fwd_scan
    from fla_amd.ops.gated_delta_rule import chunk_gated_delta_rule
    from fla_amd.ops.gated_delta_rule.wy_fast import fwd_prepare_scan_operands
    from fla_amd.utils import VarlenPlan
    torch.manual_seed(0)
    T, H, K, V, N = 32768, 16, 128, 128, 12
    lens = torch.randint(256, 6001, (N,)).double()
    lens = (lens / lens.sum() * T).round().long()
    lens[-1] += T - lens.sum()
    offs = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).to(device)
    q = torch.randn(1, T, H, K, device=device).bfloat16()
    k = F.normalize(torch.randn(1, T, H, K, device=device), dim=-1).bfloat16()
    v = torch.randn(1, T, H, V, device=device).bfloat16()
    g = F.logsigmoid(torch.randn(1, T, H, device=device))
    beta = torch.randn(1, T, H, device=device).sigmoid()
    scale = K ** -0.5
    # q, k, v, o in 16 bit + g, beta fp32 (+ the final states): what the operator must move
    floor = 4 * T * H * K * 2 + 2 * T * H * 4
    # state products 6KV, the chunk-local products 3*2*BT*K + 2*2*BT*V, and the 64x64 triangular solve per chunk
    gdr_flops = T * H * (6 * K * V + 6 * 64 * K + 4 * 64 * V + 5500)
    out = {}

    def row(name, fn, prep, scan, n_states, chunks, tokens):
        st = event_stats(fn, steps, warmup)
        us = st["median_us"]
        st_p = event_stats(prep, steps, 5)
        st_s = event_stats(scan, steps, 5)
        state_bytes = n_states * H * K * V * 4
        tri = chunks * H * 10 * 256 * 2                         # the packed triangular tile
        # algorithmic bytes of each launch: every operand read once, every result written once
        bytes_prep = T * H * K * 2 + 2 * T * H * 4 + T * H * 4 + tri              # k, g, beta in; gamma, tile out
        bytes_scan = 4 * T * H * K * 2 + T * H * 4 + tri + state_bytes            # q, k, v, gamma, tile in; o, ht out
        ach = bytes_scan / (st_s["median_us"] * 1e-6) / 1e9
        out[name] = {
            "us": round(us, 1), **spread(st), "tokens_per_s": round(tokens / (us * 1e-6), 1),
            "operator_floor_bytes": floor + state_bytes,
            "frac_of_hbm_peak": round((floor + state_bytes) / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
            "algorithmic_flops": gdr_flops, "frac_of_mfma_peak": round(gdr_flops / (us * 1e-6) / MFMA_PEAK_FLOPS, 4),
            "roofline": {"kernel": "gdr_fwd_scan_kernel", "bound": "hbm", "achieved": round(ach, 1),
                         "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBS, 4),
                         "traffic": counter_traffic("roofline:gdr_fwd_scan_kernel:" + name),
                         "avg_us": round(st_s["median_us"], 1), "bytes_per_launch": bytes_scan, **spread(st_s)},
            "gdr_fwd_prep_kernel": {"avg_us": round(st_p["median_us"], 1), "bytes_per_launch": bytes_prep,
                                    "GBs": round(bytes_prep / (st_p["median_us"] * 1e-6) / 1e9, 1),
                                    "traffic": counter_traffic("roofline:gdr_fwd_prep_kernel:" + name),
                                    **spread(st_p)},
            "launches_bytes_total": bytes_prep + bytes_scan}

    plan = VarlenPlan(offs, 64)
    AT, gc = fwd_prepare_scan_operands(k, beta, g, offsets=plan.offsets, indices=plan.indices)
    row("config2_varlen",
        lambda: chunk_gated_delta_rule(q, k, v, g, beta, output_final_state=True, offsets=offs, head_first=False),
        lambda: fwd_prepare_scan_operands(k, beta, g, offsets=plan.offsets, indices=plan.indices),
        lambda: chunk_gated_delta_rule_fwd_scan(q, k, v, AT, gc, scale, None, True, offsets=plan.offsets,
                                                chunk_offsets=plan.chunk_offsets, seq_order=plan.seq_order),
        N, plan.NT, T)
    out["config2_varlen"]["sequence_lengths"] = lens.tolist()
    B, T2 = 8, 4096
    q, k, v = (x.view(B, T2, H, -1) for x in (q, k, v))
    g, beta = g.view(B, T2, H), beta.view(B, T2, H)
    AT, gc = fwd_prepare_scan_operands(k, beta, g)
    row("B8_T4096",
        lambda: chunk_gated_delta_rule(q, k, v, g, beta, output_final_state=True, head_first=False),
        lambda: fwd_prepare_scan_operands(k, beta, g),
        lambda: chunk_gated_delta_rule_fwd_scan(q, k, v, AT, gc, scale, None, True),
        B, B * T2 // 64, B * T2)
    return out


def bench_backward(device, steps=20):
    """Training workload: forward + backward of both chunk operators, B=4, T=4096, H=16, K=V=128."""
    import torch
    import torch.nn.functional as F
    from fla_amd.ops.gated_delta_rule import chunk_gated_delta_rule
    from fla_amd.ops.gla import chunk_gla
    torch.manual_seed(0)
    B, T, H, K, V = 4, 4096, 16, 128, 128
    mk = lambda *sh: torch.randn(*sh, device=device)
    q, v = mk(B, T, H, K).bfloat16().requires_grad_(), mk(B, T, H, V).bfloat16().requires_grad_()
    h0 = (mk(B, H, K, V) * 0.1).requires_grad_()
    do, dht = mk(B, T, H, V).bfloat16(), mk(B, H, K, V) * 0.1
    out = {}
    k = mk(B, T, H, K).bfloat16().requires_grad_()
    gk = (F.logsigmoid(mk(B, T, H, K)) / 16).requires_grad_()

    leaves = []

    def clear():
        # gradients are produced, not accumulated: a step is one forward + one backward of the operator
        for x in leaves:
            x.grad = None

    def gla_step():
        clear()
        o, ht = chunk_gla(q, k, v, gk, initial_state=h0, output_final_state=True, head_first=False)
        torch.autograd.backward((o, ht), (do, dht))

    kn = F.normalize(mk(B, T, H, K), dim=-1).bfloat16().requires_grad_()
    g = F.logsigmoid(mk(B, T, H)).requires_grad_()
    beta = mk(B, T, H).sigmoid().requires_grad_()

    def gdr_step():
        clear()
        o, ht = chunk_gated_delta_rule(q, kn, v, g, beta, initial_state=h0, output_final_state=True,
                                       head_first=False)
        torch.autograd.backward((o, ht), (do, dht))

    leaves.extend([q, k, v, gk, h0, kn, g, beta])

    import fla_amd.ops.gated_delta_rule.chunk as gdr_mod
    import fla_amd.ops.gla.chunk as gla_mod

    def saved_bytes(forward):
        """Bytes a forward keeps for its backward: distinct storages among the tensors autograd saves (the operator's
        inputs included; `inputs_bytes` says how much of it they are)."""
        seen = {}

        def pack(t):
            seen[t.untyped_storage().data_ptr()] = t.untyped_storage().nbytes()
            return t

        with torch.autograd.graph.saved_tensors_hooks(pack, lambda t: t):
            outs = forward()
        del outs
        return sum(seen.values())

    gla_fwd = lambda: chunk_gla(q, k, v, gk, initial_state=h0, output_final_state=True, head_first=False)
    gdr_fwd = lambda: chunk_gated_delta_rule(q, kn, v, g, beta, initial_state=h0, output_final_state=True,
                                             head_first=False)
    nbytes = lambda *ts: sum(t.numel() * t.element_size() for t in ts)
    for name, fn, mod, fwd, ins in (("chunk_gla", gla_step, gla_mod, gla_fwd, (q, k, v, gk, h0)),
                                    ("chunk_gated_delta_rule", gdr_step, gdr_mod, gdr_fwd, (q, kn, v, g, beta, h0))):
        st = event_stats(fn, steps, 5)
        us = st["median_us"]
        # forward + backward FLOPs (dense-tile counts): GLA 10KV + 4*BT*(K+V); delta rule 16KV + 2*BT*(9K+5V) + 8*BT^2
        fl = B * T * H * ((10 * K * V + 4 * 64 * (K + V)) if name == "chunk_gla"
                          else (16 * K * V + 2 * 64 * (9 * K + 5 * V) + 8 * 64 * 64))
        out[name] = {"fwd_bwd_us": round(us, 1), **spread(st), "tokens_per_s": round(B * T / (us * 1e-6), 1),
                     "algorithmic_flops": fl, "frac_of_mfma_peak": round(fl / (us * 1e-6) / MFMA_PEAK_FLOPS, 4),
                     "inputs_bytes": nbytes(*ins), "saved_for_backward_bytes": saved_bytes(fwd)}
        # the reference's trade: nothing but the inputs (and the gate-range flags) kept, states recomputed in the backward
        mod.KEEP_STATES_FOR_BACKWARD = False
        try:
            st_r = event_stats(fn, steps, 5)
            out[name]["recompute_states"] = {"fwd_bwd_us": round(st_r["median_us"], 1),
                                             "saved_for_backward_bytes": saved_bytes(fwd)}
        finally:
            mod.KEEP_STATES_FOR_BACKWARD = True
        clear()
    return out


def bench_copy(device, steps=20):
    """The runtime's device-to-device copy of 1 GiB (1 GiB read + 1 GiB written): what a pure stream of
    this size reaches on the box, beside the 8 TB/s the roofline fractions are quoted against."""
    import torch
    src = torch.empty(1 << 30, dtype=torch.uint8, device=device)
    dst = torch.empty_like(src)
    us = event_avg_us(lambda: dst.copy_(src), steps)
    return {"us": round(us, 1), "GBs": round(2 * (1 << 30) / us / 1e3, 1),
            "frac_of_hbm_peak": round(2 * (1 << 30) / us / 1e3 / HBM_PEAK_GBS, 4)}


def bench_cu_feed_rate(device, steps=20):
    """What a CU is fed per nanosecond when it streams rows the way the staging waves of the chunk scans do
    (fla_selftest_stream_tiles: one 256-thread workgroup per CU, 64 rows x 256 bytes per tensor and chunk at a
    4 KiB row pitch, registers refilled as they are consumed, no arithmetic), for the sharing patterns of the
    benchmark shapes: B=16 (every workgroup its own rows), B=8 with two and B=4 with four workgroups per
    (sequence, head) - the value slabs of a head.  A scan's chunk period cannot be shorter than the bytes its
    workgroup moves per chunk divided by this rate."""
    import torch
    from fla_amd import _backend as be
    T, H, nt = 4096, 16, 4
    out = {}
    for B, share in ((16, 1), (8, 2), (4, 4)):
        x = torch.randint(-2**31, 2**31 - 1, (nt, B, T, H, 64), dtype=torch.int32, device=device)
        sink = torch.zeros(B * H * share, dtype=torch.int32, device=device)
        tb = B * T * H * 256
        fn = lambda: be.check(be.lib().fla_selftest_stream_tiles(be.ptr(x), tb, nt, be.ptr(sink), B, T, H, share,
                                                                 be.stream_of(x)), "stream_tiles")
        us = event_stats(fn, steps, 5)["median_us"]
        per_wg = nt * T * 256
        out[f"B{B}_share{share}"] = {
            "us": round(us, 1), "workgroups": B * H * share,
            "bytes_per_ns_per_cu": round(per_wg / us / 1e3, 1),
            "into_cus_TBs": round(per_wg * B * H * share / us / 1e6, 2),
            "from_hbm_TBs": round(nt * tb / us / 1e6, 2)}
        del x
    return out


def bench_layer_steps(device, steps=20):
    """The row-wise steps either side of the operators at the operators' benchmark shape
    (B=8, T=4096, H=16, D=128; the convolution on 2048 channels, kernel 4): device time of each
    kernel (HIP events) and its algorithmic bytes (each tensor read or written once)."""
    import torch
    from fla_amd.modules.convolution import ShortConvolution
    from fla_amd.modules.fused_norm_gate import norm_gate_bwd, norm_gate_fwd
    from fla_amd.modules.l2norm import l2norm_bwd, l2norm_fwd
    B, T, H, D = 8, 4096, 16, 128
    gen = torch.Generator(device=device).manual_seed(4)
    x = torch.randn(B * T * H, D, device=device, generator=gen).bfloat16()
    o = torch.randn(B * T * H, D, device=device, generator=gen).bfloat16()
    dy = torch.randn(B * T * H, D, device=device, generator=gen).bfloat16()
    w = torch.ones(D, device=device)
    nb = x.numel() * 2
    out = {}

    # These rows move 134 MB tensors, which a 256 MB last-level cache partly keeps from one launch to the
    # next: `us` is timed with 1 GiB read between the launches (every operand then comes from HBM, as it
    # does behind the operators inside a layer; a read, because the dirty lines of a 1 GiB write would still
    # be draining under the timed launch), `us_back_to_back` without.  Either way part of a launch's own
    # output can still sit in that cache when its end event fires, so a row above the device-copy rate is
    # not an HBM rate.
    flush = torch.zeros(1 << 28, dtype=torch.int32, device=device)

    def rec(name, fn, nbytes):
        warm = event_avg_us(fn, steps)
        us = event_avg_us(fn, steps, ramp=0.0, between=flush.max)
        out[name] = {"us": round(us, 1), "us_back_to_back": round(warm, 1), "algorithmic_bytes": nbytes,
                     "GBs": round(nbytes / us / 1e3, 1),
                     "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}

    rec("l2norm_fwd", lambda: l2norm_fwd(x), 2 * nb)
    rec("l2norm_bwd", lambda: l2norm_bwd(x, dy), 3 * nb)
    rec("rmsnorm_swish_gate_fwd", lambda: norm_gate_fwd(x, o, w, None, 1e-5, True), 3 * nb)
    y, mean, rstd, _ = norm_gate_fwd(x, o, w, None, 1e-5, True)
    rec("rmsnorm_swish_gate_bwd", lambda: norm_gate_bwd(dy, x, o, w, None, 1e-5, mean, rstd, True), 5 * nb)
    Dc = 2048
    xc = torch.randn(B, T, Dc, device=device, generator=gen).bfloat16()
    dyc = torch.randn(B, T, Dc, device=device, generator=gen).bfloat16()
    conv = ShortConvolution(Dc, 4, activation="silu").to(device)
    nbc = xc.numel() * 2
    with torch.no_grad():
        rec("short_conv_fwd", lambda: conv(xc), 2 * nbc)
    xg = xc.clone().requires_grad_()

    def conv_fb():
        yc, _ = conv(xg)
        yc.backward(dyc)
        xg.grad = None
        conv.weight.grad = None

    rec("short_conv_fwd_bwd", conv_fb, 5 * nbc)
    return out


def bench_gla_stages(device, steps=20):
    """The chunk-parallel GLA stages on the reference's internal operands (scores A [B,T,H,64] fp32,
    row-major fp32 states [B,NT,H,K,V]) at B=4, T=4096, H=16, K=V=128: device time per launch and
    algorithmic bytes (every operand read once, the result written once)."""
    import torch
    from fla_amd.ops.gla.chunk import chunk_gla_bwd_dA, chunk_gla_bwd_dv, chunk_gla_fwd_o_gk
    B, T, H, K, V = 4, 4096, 16, 128, 128
    NT = T // 64
    gen = torch.Generator(device=device).manual_seed(5)
    q, k = (torch.randn(B, T, H, K, device=device, generator=gen).bfloat16() for _ in range(2))
    v, do = (torch.randn(B, T, H, V, device=device, generator=gen).bfloat16() for _ in range(2))
    G = -torch.rand(B, T, H, K, device=device, generator=gen)
    A = torch.randn(B, T, H, 64, device=device, generator=gen)
    h = torch.randn(B, NT, H, K, V, device=device, generator=gen)
    tok = B * T * H
    b_qk, b_v, b_g, b_a, b_h = tok * K * 2, tok * V * 2, tok * K * 4, tok * 64 * 4, h.numel() * 4
    out = {}

    # timed like the layer steps: 1 GiB read between the launches, so that no operand is still in the
    # 256 MB last-level cache (`us`); `us_back_to_back` is the same launch without that read
    flush = torch.zeros(1 << 28, dtype=torch.int32, device=device)

    def rec(name, fn, nbytes):
        warm = event_avg_us(fn, steps)
        us = event_avg_us(fn, steps, ramp=0.0, between=flush.max)
        out[name] = {"us": round(us, 1), "us_back_to_back": round(warm, 1), "algorithmic_bytes": nbytes,
                     "GBs": round(nbytes / us / 1e3, 1),
                     "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}

    rec("chunk_gla_fwd_o_gk", lambda: chunk_gla_fwd_o_gk(q, v, G, A, h, K ** -0.5, head_first=False),
        b_qk + b_g + b_a + b_h + 2 * b_v)
    rec("chunk_gla_bwd_dA", lambda: chunk_gla_bwd_dA(v, do, K ** -0.5, head_first=False), 2 * b_v + b_a)
    rec("chunk_gla_bwd_dv", lambda: chunk_gla_bwd_dv(k, G, A, do, h, head_first=False),
        b_qk + b_g + b_a + b_h + 2 * b_v)
    from fla_amd.ops.common.chunk_h import chunk_bwd_dh
    h0 = torch.zeros(B, H, K, V, device=device)
    rec("chunk_bwd_dh", lambda: chunk_bwd_dh(q, k, v, None, G, None, do, h0, h0, K ** -0.5, head_first=False,
                                             states_in_fp32=True), b_qk + b_g + b_v + b_h)
    return out


def bench_simple_gla(device, steps=20):
    """chunk_simple_gla forward (one log-gate per token and head) at config 1's shape: the operator's own launch
    against the same operator through the per-key-gate kernel on a materialised gate tensor, and its two kernels
    (the delta-rule scan without the delta rule, the GLA kernel's per-head-gate form) side by side."""
    import torch
    import torch.nn.functional as F
    from fla_amd.ops.gla import chunk_gla
    from fla_amd.ops.simple_gla import chunk_simple_gla
    B, T, H, D = 8, 4096, 16, 128
    gen = torch.Generator(device=device).manual_seed(6)
    q, k, v = (torch.randn(B, T, H, D, device=device, generator=gen).bfloat16() for _ in range(3))
    g = F.logsigmoid(torch.randn(B, T, H, device=device, generator=gen))
    h0 = torch.randn(B, H, D, D, device=device, generator=gen) * 0.1
    nbytes = 4 * q.numel() * 2 + g.numel() * 4 + 2 * h0.numel() * 4
    import fla_amd.ops.simple_gla.chunk as sg_mod
    routes = {}
    with torch.no_grad():
        us = event_avg_us(lambda: chunk_simple_gla(q, k, v, g, initial_state=h0, output_final_state=True,
                                                   head_first=False), steps)
        us_b = event_avg_us(lambda: chunk_gla(q, k, v, g[..., None].expand(B, T, H, D), initial_state=h0,
                                              output_final_state=True, head_first=False), steps)
        # the two kernels that can serve a forward without gradients (the plain scan is the default), at B=8 and B=4
        default = sg_mod.SCAN_FORWARD
        try:
            for name, flag in (("plain_scan_kernel", True), ("gla_kernel_per_head_gates", False)):
                sg_mod.SCAN_FORWARD = flag
                for Bx in (8, 4):
                    fn = lambda: chunk_simple_gla(q[:Bx], k[:Bx], v[:Bx], g[:Bx], initial_state=h0[:Bx],
                                                  output_final_state=True, head_first=False)
                    routes[f"{name}_B{Bx}_us"] = round(event_avg_us(fn, steps), 1)
        finally:
            sg_mod.SCAN_FORWARD = default
    # forward + backward at config 4's batch (B=4): per-head-gate forward that keeps the states, per-head-gate backward
    Bb = 4
    leaves = [x[:Bb].clone().requires_grad_() for x in (q, k, v, g)]
    h0b = h0[:Bb].clone().requires_grad_()
    do = torch.randn(Bb, T, H, D, device=device, generator=gen).bfloat16()
    dht = torch.randn(Bb, H, D, D, device=device, generator=gen) * 0.1

    def fb(fn, gate):
        o, ht = fn(leaves[0], leaves[1], leaves[2], gate(leaves[3]), initial_state=h0b, output_final_state=True,
                   head_first=False)
        torch.autograd.backward((o, ht), (do, dht))
        for x in leaves + [h0b]:
            x.grad = None

    us_fb = event_avg_us(lambda: fb(chunk_simple_gla, lambda x: x), steps)
    us_fb_b = event_avg_us(lambda: fb(chunk_gla, lambda x: x[..., None].expand(Bb, T, H, D)), steps)
    return {"us": round(us, 1), "tokens_per_s": round(B * T / us * 1e6, 1), "algorithmic_bytes": nbytes,
            "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
            "through_per_key_gate_kernel_us": round(us_b, 1), **routes,
            "fwd_bwd_B4_us": round(us_fb, 1), "fwd_bwd_B4_through_per_key_gate_kernels_us": round(us_fb_b, 1)}


def bench_layer_fusion(device, steps=20):
    """What folding the steps in front of the operators into their forward launches saves inside a layer, at the
    headline shape (B=8, T=4096, H=16, D=128, nothing differentiated): the gate pre-activation of a GLA layer
    (logsigmoid(x)/16 on the bf16 output of the gate projection, fla/layers/gla.py:214) and the l2 norm of q and k of
    a gated DeltaNet layer (fla/layers/gated_deltanet.py:234-235), as separate launches in front of the operator
    against the opt-in forms in which the operator's own launches do that work."""
    import torch
    import torch.nn.functional as F
    from fla_amd.modules import gla_gate_fwd, l2norm_fwd
    from fla_amd.ops.gated_delta_rule import chunk_gated_delta_rule
    from fla_amd.ops.gla import chunk_gla
    B, T, H, D = 8, 4096, 16, 128
    gen = torch.Generator(device=device).manual_seed(7)
    q, k, v = (torch.randn(B, T, H, D, device=device, generator=gen).bfloat16() for _ in range(3))
    x = torch.randn(B, T, H, D, device=device, generator=gen).bfloat16()
    h0 = torch.randn(B, H, D, D, device=device, generator=gen) * 0.1
    g = F.logsigmoid(torch.randn(B, T, H, device=device, generator=gen))
    beta = torch.randn(B, T, H, device=device, generator=gen).sigmoid()
    nb = q.numel() * 2
    out = {}

    def gla_two_step():
        return chunk_gla(q, k, v, gla_gate_fwd(x, 16.0), initial_state=h0, output_final_state=True, head_first=False)

    def gla_fused():
        return chunk_gla(q, k, v, x, initial_state=h0, output_final_state=True, head_first=False,
                         gate_logit_normalizer=16.0)

    def gdr_two_step():
        return chunk_gated_delta_rule(l2norm_fwd(q), l2norm_fwd(k), v, g, beta, initial_state=h0,
                                      output_final_state=True, head_first=False)

    def gdr_fused():
        return chunk_gated_delta_rule(q, k, v, g, beta, initial_state=h0, output_final_state=True, head_first=False,
                                      use_qk_l2norm_in_kernel=True)

    with torch.no_grad():
        a, b = event_avg_us(gla_two_step, steps), event_avg_us(gla_fused, steps)
        gate = event_avg_us(lambda: gla_gate_fwd(x, 16.0), steps)
        out["gla_gate_logsigmoid"] = {
            "separate_launches_us": round(a, 1), "gate_launch_alone_us": round(gate, 1), "in_kernel_us": round(b, 1),
            "saved_us": round(a - b, 1),
            # logits in (bf16) + fp32 gates out, then the operator on fp32 gates / the operator on the bf16 logits
            "bytes_separate": 7 * nb + 2 * nb + 2 * h0.numel() * 4, "bytes_in_kernel": 5 * nb + 2 * h0.numel() * 4}
        a, b = event_avg_us(gdr_two_step, steps), event_avg_us(gdr_fused, steps)
        out["gdr_qk_l2norm"] = {
            "separate_launches_us": round(a, 1), "in_kernel_us": round(b, 1), "saved_us": round(a - b, 1),
            # two norms (read + write each), then the operator / the operator alone
            "bytes_separate": 8 * nb + 2 * h0.numel() * 4, "bytes_in_kernel": 4 * nb + 2 * h0.numel() * 4}
    return out


def bench_fp32_inputs(device, steps=5):
    """chunk_gla on fp32 q, k, v (the reference's own tests run the operator in fp32) at B=8, T=4096, H=16, K=V=128:
    the default route (scaled to fp16, chunk kernels, fp32 gates and states; the scaling and casts are part of the
    call) and the exact one (FLA_AMD_FP32_EXACT=1: fp32 token-by-token kernels, 1e-4, serial in time)."""
    import torch
    import torch.nn.functional as F
    from fla_amd.ops.gla import chunk_gla
    B, T, H, D = 8, 4096, 16, 128
    gen = torch.Generator(device=device).manual_seed(8)
    q, k, v = (torch.randn(B, T, H, D, device=device, generator=gen) for _ in range(3))
    g = F.logsigmoid(torch.randn(B, T, H, D, device=device, generator=gen)) / 16
    h0 = torch.randn(B, H, D, D, device=device, generator=gen) * 0.1
    import fla_amd.ops.gla.chunk as mod
    fn = lambda: chunk_gla(q, k, v, g, initial_state=h0, output_final_state=True, head_first=False)
    with torch.no_grad():
        us16 = event_avg_us(fn, 20)
        mod.FP32_INPUTS_EXACT = True
        try:
            us = event_avg_us(fn, steps, warmup=2, ramp=0.0)
        finally:
            mod.FP32_INPUTS_EXACT = False
    return {"us": round(us16, 1), "tokens_per_s": round(B * T / us16 * 1e6, 1),
            "exact_fp32_route_us": round(us, 1)}


def bench_gdr_onepass(device, steps=30):
    """The one-launch form of chunk_gated_delta_rule forward (opt-in, FLA_AMD_GDR_ONEPASS=1) beside the default two
    launches at B=8, T=4096, H=16, K=V=128: fewer bytes and one launch, but the extra work sits on the scan's matrix
    waves."""
    import torch
    import torch.nn.functional as F
    import fla_amd.ops.gated_delta_rule.chunk as mod
    B, T, H, D = 8, 4096, 16, 128
    gen = torch.Generator(device=device).manual_seed(9)
    q = torch.randn(B, T, H, D, device=device, generator=gen).bfloat16()
    k = F.normalize(torch.randn(B, T, H, D, device=device, generator=gen), dim=-1).bfloat16()
    v = torch.randn(B, T, H, D, device=device, generator=gen).bfloat16()
    g = F.logsigmoid(torch.randn(B, T, H, device=device, generator=gen))
    beta = torch.randn(B, T, H, device=device, generator=gen).sigmoid()
    fn = lambda: mod.chunk_gated_delta_rule(q, k, v, g, beta, output_final_state=True, head_first=False)
    out = {}
    for flag, name in ((False, "two_launches_us"), (True, "one_launch_us")):
        mod.ONEPASS_FORWARD = flag
        try:
            out[name] = round(event_avg_us(fn, steps), 1)
        finally:
            mod.ONEPASS_FORWARD = False
    return out


def cpu_baseline(c, budget_s=15.0):
    """The oracle's fp32 naive recurrence on the host cores, over as many whole
    sequences of the same workload as fit in about `budget_s` seconds."""
    import torch
    from oracle.recurrent import naive_recurrent_gla
    B = c["B"]
    tokens, spent, used, reps = 0, 0.0, 0, 0
    host = [tuple(c[n][b:b + 1].float().cpu() for n in ("q", "k", "v", "g", "h0")) for b in range(B)]
    while spent < 10.0:
        for b in range(B):
            q, k, v, g, h0 = host[b]
            t0 = time.perf_counter()
            naive_recurrent_gla(q, k, v, g, initial_state=h0, output_final_state=True)
            dt = time.perf_counter() - t0
            tokens += q.shape[1]
            spent += dt
            used = max(used, b + 1)
            if spent + dt > budget_s:
                break
        reps += 1
        if spent + dt > budget_s:
            break
    return {"value": round(tokens / spent, 1), "unit": "tokens/s", "cores": torch.get_num_threads(),
            "kind": "port", "seconds": round(spent, 2),
            "sample": f"oracle naive_recurrent_gla (torch CPU fp32) on batch elements 0..{used - 1} of {B} "
                      f"(T={c['T']}, H={c['H']}, K=V=128 each), {reps} pass(es) over them"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true")
    ap.add_argument("--no-ramp", action="store_true",
                    help="skip the untimed clock-ramp load (for counter-collection runs, whose timings are not used)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 1 GiB device copy (a kernel of known traffic, used to scale the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build measures one GPU only (every (sequence, head) pair is independent; "
              "nothing here uses a second GPU). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    device = torch.device("cuda:0")
    if a.no_ramp:
        global RAMP_SECONDS, ROW_RAMP_SECONDS
        RAMP_SECONDS = ROW_RAMP_SECONDS = 0.0
    ms, tps, roofline, op, cfg = bench_gla(device, a.steps, a.warmup)
    extra = {"chunk_gla_fwd": op}
    if not a.no_extra:
        extra["decode_step"] = bench_decode(device)
        extra["decode_layer_step"] = bench_decode_layer_step(device)
        extra["chunk_gated_delta_rule_fwd"] = bench_gdr(device)
        extra["fwd_bwd_config4"] = bench_backward(device)
        extra["layer_steps"] = bench_layer_steps(device)
        extra["layer_fusion"] = bench_layer_fusion(device)
        extra["chunk_gla_fp32_inputs"] = bench_fp32_inputs(device)
        extra["chunk_gated_delta_rule_fwd_one_launch"] = bench_gdr_onepass(device)
        extra["chunk_simple_gla_fwd"] = bench_simple_gla(device)
        extra["gla_stages_reference_operands"] = bench_gla_stages(device)
        extra["device_copy_1GiB"] = bench_copy(device)
        extra["cu_feed_rate"] = bench_cu_feed_rate(device)
    out = {
        "metric": "chunk fwd tokens/s (GLA, GatedDeltaNet, T=4K, D=128) + % of MFMA/HBM roofline",
        "value": round(tps, 1), "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "chunk_gla forward: B=8 T=4096 H=16 K=V=128, bf16 q/k/v, "
                               "fp32 log-gates logsigmoid(N(0,1))/16, fp32 initial state, final state returned"},
        "roofline": roofline,
        "cpu_baseline": None if a.no_cpu_baseline else cpu_baseline(cfg),
        "extra": extra,
    }
    print(json.dumps(out))
    if a.copy_calibration:
        x = torch.empty(1 << 28, device=device, dtype=torch.float32)
        y = torch.empty_like(x)
        y.copy_(x)
        torch.cuda.synchronize()


if __name__ == "__main__":
    main()
