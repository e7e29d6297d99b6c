#!/usr/bin/env python3
"""Benchmark of the Based sequence-mixer hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--only decode|prefill|swa|conv|stack|projections|copy|machine]

Headline workload (`value`): the recurrent decode step of Taylor linear attention at
B=128, H=16, dv=64 — fp32 kv_state (128,16,1,64,273) + k_state, initialised from a seeded
512-token prefill, bf16 q/k/v ~ N(0,1), K consecutive single-token steps.  One "step" is
one kernel launch over the whole batch; value = B / time-per-step (tokens/s, one layer).
Inputs and state are resident in HBM before the timed region.  The HBM-bound workloads are
timed cold (rotating over several independent state / input sets, working set well beyond the
256 MB last-level cache) and warm (one set); `value` and `roofline` use the slower of the two.

The same JSON line also carries, as secondary objects, the linear-attention prefill at
L=4096 (tokens/s and fraction of bf16 MFMA peak) and the sliding-window attention prefill +
decode of the B=8, H=16, L=4096 configuration.

`roofline.achieved` = algorithmic bytes (or FLOPs) per launch / average launch duration,
timed with HIP events on the stream the kernels are launched on.  The K decode steps are
recorded once in a graph, as the decoding loop issues them, and one replay of it is the timed
region (the kernel's own duration: what the kernel trace shows); the same K launches issued one
by one from the host carry the gap between two launches as well and are reported beside it
(`decode_cold.launched_one_by_one_ms`).
`cpu_baseline` = the CPU oracle (a PyTorch restatement of the reference arithmetic) timed on
this host's cores on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published
D_EXP = 273

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, each scaled by what
# the same counter reads for a plain copy of known size (the summaries and the commands that
# produced them are the text files under profiles/); None until such a run exists for the kernel.
MEASURED_TRAFFIC_BYTES = {
    "lin_step_kernel": 293110357,   # B=128, H=16, dv=64, rotating state sets
    "lin_step_kernel_B64_dv128": 290402458,   # long-context decode
    "lin_prefill_mfma_kernel": {96: 2275537424},  # B=96, L=4096, dv=64, states written: fetch 1,361,103,382 + write 914,434,042 (the fetch varies by 10 % between runs); keyed by batch
    "swa_prefill_kernel": 268706329,   # B=8, H=16, L=4096, four heads per workgroup, runs in both directions: fetch 201,524,085 + write 67,182,244
    "decode_linear_kernel_lm_head": 104920711,   # M=4, 50280 x 1024 + closing norm: fetch 104,309,135 + write 611,576
}


PROBE_SRC = os.path.join(ROOT, "bench_probes.hip")
PROBE_LIB = os.path.join(ROOT, "libbench_probes.so")


def build_probes() -> str:
    """Compiles bench_probes.hip (streaming kernels with no arithmetic, used by `--only machine` and
    `--only copy`) into libbench_probes.so beside this file; cross-compiles, no GPU needed.  The
    probes are measurement tools of this benchmark, not part of the product library."""
    import shutil
    import subprocess

    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    cmd = [hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", PROBE_SRC, "-o", PROBE_LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {PROBE_SRC}:\n{r.stdout}\n{r.stderr}")
    return PROBE_LIB


_probes = None


def probes():
    """The loaded probe library (built beforehand by build_probes(); a GPU run never compiles)."""
    global _probes
    if _probes is None:
        import ctypes as C

        if not os.path.exists(PROBE_LIB):
            raise RuntimeError(f"{PROBE_LIB} not found: build it with `python -c 'import bench; bench.build_probes()'`")
        lib = C.CDLL(PROBE_LIB)
        lib.bench_probe_stream_qkv.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_void_p]
        lib.bench_probe_rmw.argtypes = [C.c_void_p, C.c_int64, C.c_void_p]
        lib.bench_probe_copy.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]
        lib.bench_probe_stream_prefill.argtypes = [C.c_void_p] * 4 + [C.c_int64] * 3 + [C.c_void_p]
        lib.bench_probe_mfma.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.POINTER(C.c_double), C.c_void_p]
        lib.bench_probe_timestamp.argtypes = [C.c_void_p, C.c_void_p]
        lib.bench_probe_timestamp.restype = C.c_int
        lib.bench_probe_clock_khz.argtypes = []
        lib.bench_probe_clock_khz.restype = C.c_int64
        for fn in (lib.bench_probe_stream_qkv, lib.bench_probe_rmw, lib.bench_probe_copy, lib.bench_probe_stream_prefill,
                   lib.bench_probe_mfma):
            fn.restype = C.c_int
        _probes = lib
    return _probes


def _probe_ok(rc):
    if rc != 0:
        raise RuntimeError(f"bench probe refused its arguments or failed to launch (code {rc})")


def _events_ms(torch, fn, steps, warmup, warmup_ms=0.0, pilot=4):
    """Average milliseconds per call of fn(), HIP events on the current stream.  warmup_ms > 0
    keeps launching (untimed) until that much wall time has passed: the board's power management
    needs ~20 ms of sustained MFMA load to settle (boost clock -> overshoot -> steady state), and
    the timed region should see the steady state."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t_w = time.perf_counter()
    while (time.perf_counter() - t_w) * 1e3 < warmup_ms:
        for _ in range(8):
            fn()
        torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    # a few more untimed calls right in front of the timed ones, with no synchronisation in between:
    # the stream is busy when the first event is recorded, so the timed region starts when they end,
    # with its own launches already queued, and holds `steps` launches back to back (after a
    # synchronisation the first launch would count the host's launch latency, 5 - 20 us, as its own)
    for _ in range(pilot):
        fn()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / (steps + pilot)
    return e0.elapsed_time(e1) / steps, wall


LONG_REGION = 256  # steps of the decode leg's second timed region when fewer are asked for


def bench_decode(torch, ops, steps, warmup, B=128, H=16, dv=64, prefill_len=512, n_sets=4, replays=12, long_region_too=False,
                 use_graph=True):
    """Recurrent decode step.  Timed twice: COLD over `n_sets` independent (kv_state, k_state) sets
    visited in turn (n_sets x 145 MB at B=128, dv=64: more than the 256 MB last-level cache, and what
    the linear-attention layers of a stack do per token: every layer has its own state), and WARM
    on one set updated in place every step (145 MB: may be served from the last-level cache).
    The roofline figure is the lower of the two."""
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(0)
    # state from a seeded prefill (same kernels; q only shapes the outputs, not the state)
    kp = torch.randn(B, H, prefill_len, 16, generator=g).bfloat16().to(dev)
    vp = torch.randn(B, H, prefill_len, dv, generator=g).bfloat16().to(dev)
    _, kv_state, k_state = ops.linear_attn_prefill(kp, kp, vp, return_state=True)
    del kp, vp
    states = [(kv_state, k_state)] + [(kv_state.clone(), k_state.clone()) for _ in range(n_sets - 1)]
    n_in = 8  # distinct pre-generated inputs cycled through the steps
    qs = [torch.randn(B, H, 1, 16, generator=g).bfloat16().to(dev) for _ in range(n_in)]
    ks = [torch.randn(B, H, 1, 16, generator=g).bfloat16().to(dev) for _ in range(n_in)]
    vs = [torch.randn(B, H, 1, dv, generator=g).bfloat16().to(dev) for _ in range(n_in)]
    y = torch.empty(B, H, 1, dv, dtype=torch.bfloat16, device=dev)
    from based_amd import _lib

    lib = _lib.lib()
    args = [(qs[i].data_ptr(), ks[i].data_ptr(), vs[i].data_ptr()) for i in range(n_in)]
    st_ptrs = [(a.data_ptr(), b.data_ptr()) for a, b in states]
    it = [0]

    def make_step(sets):
        def step():
            a = args[it[0] % n_in]
            st = st_ptrs[it[0] % sets]
            it[0] += 1
            rc = lib.based_linear_attn_step(a[0], a[1], a[2], st[0], st[1], y.data_ptr(),
                                            B, H, dv, H * 16, 16, H * 16, 16, H * dv, dv, H * dv, dv,
                                            1e-12, 0, torch.cuda.current_stream().cuda_stream)
            if rc:
                _lib.check(rc)
        return step

    timing_note = [None]  # set when the timestamps inside a graph are not what was used

    def in_graph(sets, steps=steps):
        """`replays` samples of exactly `steps` launches each, recorded in ONE graph as the decoding
        loop records its launches (generation.py: capture_graph): per sample the untimed warm-up
        steps, a timestamp launch, the `steps` timed launches, a timestamp launch (bench_probes.hip:
        one lane stores the device's constant-rate clock).  The graph is replayed once untimed and
        once for the figures: the GPU is never idle between the samples, and the difference of a
        sample's two timestamps is the time of its `steps` launches and nothing else (both stamps
        trail the launch before them by the same launch latency).  HIP events cannot be recorded
        inside a graph on this platform, and events around a graph of just the timed steps also
        count the boundary between two graph launches (about 14 us: 0.7 us per step of 20).
        Cross-check in the result: HIP events around the whole replay, per launch of the hot kernel
        (the 2 x `replays` timestamp launches add about 0.1 %)."""
        step = make_step(sets)
        lib_p, khz = None, 0
        if use_graph:
            try:
                lib_p = probes()
                khz = lib_p.bench_probe_clock_khz()
            except (RuntimeError, OSError, AttributeError) as e:
                print(f"bench.py: timestamp probe unavailable ({e}); timing with HIP events", file=sys.stderr)
        if khz <= 0:
            # counter runs (--no-graph: a profiler that collects counters has crashed on replays of
            # graphs this long), or no timestamp probe: the same launches one by one, HIP events
            # around each sample
            timing_note[0] = "launches issued one by one, HIP events around each sample"
            ev = sorted(_events_ms(torch, step, steps, warmup)[0] for _ in range(replays))
            return {"median": ev[len(ev) // 2], "min": ev[0], "max": ev[-1], "events_whole_replay": ev[len(ev) // 2]}
        lead_n = max(warmup, 4)
        stamps = torch.zeros(2 * replays, dtype=torch.int64, device=dev)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(warmup):
                step()
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                sp = torch.cuda.current_stream().cuda_stream
                for r in range(replays):
                    for _ in range(lead_n):
                        step()
                    _probe_ok(lib_p.bench_probe_timestamp(stamps.data_ptr() + 16 * r, sp))
                    for _ in range(steps):
                        step()
                    _probe_ok(lib_p.bench_probe_timestamp(stamps.data_ptr() + 16 * r + 8, sp))
        torch.cuda.current_stream().wait_stream(side)
        graph.replay()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        t = stamps.cpu().tolist()
        samples = sorted((t[2 * r + 1] - t[2 * r]) / khz / steps for r in range(replays))  # ticks / kHz = ms
        return {"median": samples[len(samples) // 2], "min": samples[0], "max": samples[-1],
                "events_whole_replay": e0.elapsed_time(e1) / (replays * (lead_n + steps))}

    eager_cold, wall = _events_ms(torch, make_step(n_sets), steps, warmup)
    eager_warm, _ = _events_ms(torch, make_step(1), steps, warmup)
    sp_cold, sp_warm = in_graph(n_sets), in_graph(1)
    ms_cold, ms_warm = sp_cold["median"], sp_warm["median"]
    bytes_per_launch = B * H * (2 * D_EXP * dv * 4 + 2 * D_EXP * 4 + (2 * 16 + 2 * dv) * 2)
    ms = max(ms_cold, ms_warm)
    gbs = bytes_per_launch / (ms * 1e-3) / 1e9
    spread = sp_cold if ms_cold >= ms_warm else sp_warm
    frac_of = lambda t: round(bytes_per_launch / (t * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
    # With fewer than LONG_REGION steps the same measurement is repeated on LONG_REGION steps and
    # reported beside the figure of the region asked for (which stays `value` and `frac`): samples
    # of 1 ms spread more than samples of 13 ms.
    long_region = None
    if long_region_too and steps < LONG_REGION:
        lc, lw = in_graph(n_sets, LONG_REGION), in_graph(1, LONG_REGION)
        lsp = lc if lc["median"] >= lw["median"] else lw  # the slower leg, as for the region asked for
        long_region = {"steps": LONG_REGION, "cold_ms": round(lc["median"], 5), "warm_ms": round(lw["median"], 5),
                       "frac": frac_of(lsp["median"]), "slowest": frac_of(lsp["max"]), "fastest": frac_of(lsp["min"])}
    assert torch.isfinite(y.float()).all() and all(torch.isfinite(a).all() for a, _ in states)
    return {
        "long_region": long_region,
        "tok_s": B / (ms * 1e-3),
        "ms": ms,
        "wall_ms": wall,
        "cold": {"ms": round(ms_cold, 5), "ms_min": round(sp_cold["min"], 5), "ms_max": round(sp_cold["max"], 5),
                 "GBps": round(bytes_per_launch / (ms_cold * 1e-3) / 1e9, 1), "state_sets": n_sets,
                 "working_set_MB": round(n_sets * (kv_state.numel() + k_state.numel()) * 4 / 1e6, 1),
                 "launched_one_by_one_ms": round(eager_cold, 5),
                 "events_around_the_whole_replay_ms": round(sp_cold["events_whole_replay"], 5)},
        "warm": {"ms": round(ms_warm, 5), "ms_min": round(sp_warm["min"], 5), "ms_max": round(sp_warm["max"], 5),
                 "GBps": round(bytes_per_launch / (ms_warm * 1e-3) / 1e9, 1), "state_sets": 1,
                 "working_set_MB": round((kv_state.numel() + k_state.numel()) * 4 / 1e6, 1),
                 "launched_one_by_one_ms": round(eager_warm, 5),
                 "events_around_the_whole_replay_ms": round(sp_warm["events_whole_replay"], 5)},
        "roofline": {"kernel": "lin_step_kernel", "bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "frac_spread": {"replays": replays, "median": frac_of(spread["median"]),
                                     "slowest": frac_of(spread["max"]), "fastest": frac_of(spread["min"])},
                     "traffic": MEASURED_TRAFFIC_BYTES["lin_step_kernel"] if (B, H, dv) == (128, 16, 64) else (
                         MEASURED_TRAFFIC_BYTES["lin_step_kernel_B64_dv128"] if (B, H, dv) == (64, 16, 128) else None),
                     "algorithmic_bytes_per_launch": bytes_per_launch,
                     "timed": "median over %d samples of exactly the timed steps, the slower of cold (rotating state "
                              "sets) and warm (one set); all samples recorded in one graph (warm-up steps, timestamp "
                              "launch, the timed steps, timestamp launch) and replayed back to back; a sample = the "
                              "difference of its two device timestamps; spread in frac_spread; HIP events around the "
                              "whole replay and the launches issued one by one: see decode_cold / decode_warm" % replays
                              if timing_note[0] is None else
                              "median over %d samples of exactly the timed steps, the slower of cold and warm; %s"
                              % (replays, timing_note[0])},
        "workload": f"linear-attn recurrent decode, B={B} H={H} d=16 dv={dv}, fp32 state from a {prefill_len}-token prefill, "
                    f"bf16 q/k/v, {n_sets} independent state sets visited in turn",
    }


def bench_decode_deferred(torch, ops, period=8, B=128, H=16, dv=64, n_sets=4, cycles=6):
    """The decode step with the write-back of the state deferred (`ops.linear_attn_step_deferred`,
    not the reference's semantics for kv_state between steps, same outputs): `cycles` x `period`
    steps on each of `n_sets` state sets visited in turn (cold, as bench_decode), so that the
    average contains the reading steps and the applying steps in their proportion.  Bytes: the
    variant's own count, i.e. the state read on every step and written on every `period`-th."""
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(0)
    states = [(torch.randn(B, H, 1, dv, D_EXP, generator=g).to(dev), (torch.rand(B, H, 1, 1, D_EXP, generator=g) + 1).to(dev))
              for _ in range(n_sets)]
    rings = [ops.deferred_step_buffers(B, H, dv, dev) for _ in range(n_sets)]
    q = torch.randn(B, H, 1, 16, generator=g).bfloat16().to(dev)
    k = torch.randn(B, H, 1, 16, generator=g).bfloat16().to(dev)
    v = torch.randn(B, H, 1, dv, generator=g).bfloat16().to(dev)
    y = torch.empty(B, H, 1, dv, dtype=torch.bfloat16, device=dev)
    n_steps = cycles * period

    def run():
        for _ in range(n_steps):
            for (kv_state, k_state), ring in zip(states, rings):
                ops.linear_attn_step_deferred(q, k, v, kv_state, k_state, ring, period, out=y)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            run()
    torch.cuda.current_stream().wait_stream(side)
    ms, _ = _events_ms(torch, graph.replay, 10, 2)
    ms /= n_steps * n_sets
    assert torch.isfinite(y.float()).all() and all(bool((r[2] == 0).all()) for r in rings)
    state_bytes = B * H * D_EXP * dv * 4
    small = B * H * (2 * D_EXP * 4 + (2 * 16 + 2 * dv) * 2)
    ring_bytes = B * H * (16 + dv) * 4 * (8 + 1)  # every step reads the whole ring (8 slots); most append one token
    own_bytes = state_bytes * (1 + 1 / period) + small + ring_bytes
    in_place_bytes = 2 * state_bytes + small
    return {"period": period, "us_per_step": round(ms * 1e3, 2), "tok_s": round(B / (ms * 1e-3), 1),
            "bytes_per_step": int(own_bytes), "GBps": round(own_bytes / (ms * 1e-3) / 1e9, 1),
            "frac_of_hbm_peak": round(own_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "in_place_bytes_per_step": in_place_bytes,
            "note": "opt-in (LinearAttention(deferred_state_steps=8)); average over reading and applying steps, "
                    f"{n_sets} state sets in turn; the headline figure is the in-place step"}


def bench_prefill(torch, ops, steps, warmup, B=8, H=16, L=4096, dv=64):
    """Linear-attention prefill.  Launches that move less than the last-level cache holds are timed
    over several independent input sets visited in turn (cold) and on one set (warm); the figure
    reported is the slower of the two.  Larger launches are cold by size."""
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(1)
    byts = B * L * H * (2 * 16 + 2 * dv) * 2
    n_sets = 1 if byts > 400e6 else min(8, -(-800_000_000 // byts))
    # (B, L, H*d) projection layout viewed (B, H, L, d), as the module hands it over
    sets = []
    for _ in range(n_sets):
        sets.append(tuple(torch.randn(B, L, H, d, generator=g).bfloat16().to(dev).transpose(1, 2) for d in (16, 16, dv)))
    it = [0]

    def make(n):
        def f():
            q, k, v = sets[it[0] % n]
            it[0] += 1
            ops.linear_attn_prefill(q, k, v, return_state=True)
        return f

    ms_cold, _ = _events_ms(torch, make(n_sets), steps, warmup, warmup_ms=30.0)
    ms_warm = ms_cold if n_sets == 1 else _events_ms(torch, make(1), steps, warmup, warmup_ms=10.0)[0]
    ms = max(ms_cold, ms_warm)
    flops = B * L * H * (4 * D_EXP * dv + 4 * D_EXP)
    tf = flops / (ms * 1e-3) / 1e12
    return {
        "tok_s": B * L / (ms * 1e-3), "ms": ms, "B": B, "L": L, "dv": dv,
        "cold_ms": round(ms_cold, 5), "warm_ms": round(ms_warm, 5), "input_sets": n_sets,
        "roofline": {"kernel": "lin_prefill_mfma_kernel", "bound": "mfma", "achieved": round(tf, 2),
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES["lin_prefill_mfma_kernel"].get(B) if (L, dv) == (4096, 64) else None,
                     "algorithmic_flops_per_launch": flops, "algorithmic_bytes_per_launch": byts,
                     "hbm_gbs": round(byts / (ms * 1e-3) / 1e9, 1),
                     "hbm_frac": round(byts / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
    }


def bench_swa(torch, ops, steps, warmup, B=8, H=16, L=4096, decode_steps=256, n_sets=4):
    """Sliding-window prefill + decode.  The prefill is timed COLD over `n_sets` different packed
    qkv tensors and outputs visited in turn (n_sets x 268 MB of traffic: beyond the 256 MB
    last-level cache) and WARM on one; the roofline figure is the lower of the two."""
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(2)
    # every prefill leg below is timed after 20 ms of its own launches, like the linear-attention
    # prefill: the first millisecond after an idle period runs at another clock and memory state
    # than a serving loop sees (head dim 112 at one point: 157 us in that transient, 139 us after it)
    SWA_WARMUP_MS = 20.0
    qkvs = [torch.randn(B, L, 3, H, 64, generator=g).bfloat16().to(dev) for _ in range(n_sets)]
    outs = [torch.empty(B, L, H, 64, dtype=torch.bfloat16, device=dev) for _ in range(n_sets)]
    qkv = qkvs[0]
    it = [0]

    def make_pf(sets):
        def pf():
            x, o = qkvs[it[0] % sets], outs[it[0] % sets]
            it[0] += 1
            ops.swa_prefill(x[:, :, 0], x[:, :, 1], x[:, :, 2], w_left=64, out=o)
        return pf

    ms_cold, _ = _events_ms(torch, make_pf(n_sets), steps, warmup, warmup_ms=SWA_WARMUP_MS)
    ms_warm, _ = _events_ms(torch, make_pf(1), steps, warmup, warmup_ms=SWA_WARMUP_MS)
    ms = max(ms_cold, ms_warm)
    byts = B * L * H * 4 * 64 * 2
    gbs = byts / (ms * 1e-3) / 1e9
    # the released checkpoints' window layer: 128 keys to the left, rotary over the whole head, KV cache filled
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, 64, 2, dtype=torch.float32) / 64))
    ang = torch.outer(torch.arange(L).float(), inv_freq)
    rope = (ang.cos().contiguous().to(dev), ang.sin().contiguous().to(dev))
    caches = [torch.empty(B, L, 2, H, 64, dtype=torch.bfloat16, device=dev) for _ in range(n_sets)]

    def make_rel(sets, full):
        def pf():
            i = it[0] % sets
            it[0] += 1
            x = qkvs[i]
            if full:
                ops.swa_prefill(x[:, :, 0], x[:, :, 1], x[:, :, 2], w_left=128, rope=rope, kv_cache=caches[i], out=outs[i])
            else:
                ops.swa_prefill(x[:, :, 0], x[:, :, 1], x[:, :, 2], w_left=128, out=outs[i])
        return pf

    ms_w128_cold, _ = _events_ms(torch, make_rel(n_sets, False), steps, warmup, warmup_ms=SWA_WARMUP_MS)
    ms_w128_warm, _ = _events_ms(torch, make_rel(1, False), steps, warmup, warmup_ms=SWA_WARMUP_MS)
    ms_rel_cold, _ = _events_ms(torch, make_rel(n_sets, True), steps, warmup, warmup_ms=SWA_WARMUP_MS)
    del caches
    # the released 1B / 1.3B window layer: head dim 112 (n_embd 1792 over 16 heads), 128 keys to the left,
    # rotary over the whole head, KV cache filled; the general MFMA kernel
    D1 = 112
    x1 = [torch.randn(B, L, 3, H, D1, generator=g).bfloat16().to(dev) for _ in range(n_sets)]
    o1b = [torch.empty(B, L, H, D1, dtype=torch.bfloat16, device=dev) for _ in range(n_sets)]
    c1b = [torch.empty(B, L, 2, H, D1, dtype=torch.bfloat16, device=dev) for _ in range(n_sets)]
    inv1 = 1.0 / (10000.0 ** (torch.arange(0, D1, 2, dtype=torch.float32) / D1))
    ang1 = torch.outer(torch.arange(L).float(), inv1)
    rope1 = (ang1.cos().contiguous().to(dev), ang1.sin().contiguous().to(dev))

    def make_1b(full):
        def pf():
            i = it[0] % n_sets
            it[0] += 1
            x = x1[i]
            if full:
                ops.swa_prefill(x[:, :, 0], x[:, :, 1], x[:, :, 2], w_left=128, rope=rope1, kv_cache=c1b[i], out=o1b[i])
            else:
                ops.swa_prefill(x[:, :, 0], x[:, :, 1], x[:, :, 2], w_left=128, out=o1b[i])
        return pf

    ms_1b_plain, _ = _events_ms(torch, make_1b(False), steps, warmup, warmup_ms=SWA_WARMUP_MS)
    ms_1b_full, _ = _events_ms(torch, make_1b(True), steps, warmup, warmup_ms=SWA_WARMUP_MS)
    byts_1b = B * L * H * 4 * D1 * 2
    del x1, o1b, c1b
    cache = torch.zeros(B, L + decode_steps, 2, H, 64, dtype=torch.bfloat16, device=dev)
    cache[:, :L] = qkv[:, :, 1:]
    qn = torch.randn(B, 1, 3, H, 64, generator=g).bfloat16().to(dev)
    o1 = torch.empty(B, 1, H, 64, dtype=torch.bfloat16, device=dev)
    pos = [L]
    q1, k1, v1 = qn[:, :, 0], qn[:, :, 1], qn[:, :, 2]

    def dstep():
        ops.swa_step(q1, k1, v1, cache, pos[0], w_left=64, out=o1)
        pos[0] = L + (pos[0] + 1 - L) % decode_steps

    dms, _ = _events_ms(torch, dstep, decode_steps, 8)
    return {
        "prefill_tok_s": B * L / (ms * 1e-3), "prefill_ms": ms, "decode_tok_s": B / (dms * 1e-3), "decode_us": dms * 1e3,
        "B": B, "L": L, "window": 64,
        "cold": {"ms": round(ms_cold, 5), "GBps": round(byts / (ms_cold * 1e-3) / 1e9, 1), "input_sets": n_sets},
        "warm": {"ms": round(ms_warm, 5), "GBps": round(byts / (ms_warm * 1e-3) / 1e9, 1), "input_sets": 1},
        "window_128": {"cold_ms": round(ms_w128_cold, 5), "warm_ms": round(ms_w128_warm, 5),
                       "cold_GBps": round(byts / (ms_w128_cold * 1e-3) / 1e9, 1),
                       "with_rotary_and_cache_fill_cold_ms": round(ms_rel_cold, 5),
                       "note": "same inputs, 128 keys to the left (the released checkpoints' window_size 256)"},
        "head_dim_112": {"kernel": "swa_prefill_wide_kernel", "B": B, "L": L, "H": H, "window_left": 128,
                         "cold_ms": round(ms_1b_plain, 5), "cold_GBps": round(byts_1b / (ms_1b_plain * 1e-3) / 1e9, 1),
                         "frac_of_hbm_peak": round(byts_1b / (ms_1b_plain * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                         "with_rotary_and_cache_fill_cold_ms": round(ms_1b_full, 5),
                         "with_rotary_and_cache_fill_GBps": round(byts_1b * 1.5 / (ms_1b_full * 1e-3) / 1e9, 1),
                         "note": "the released 1B / 1.3B window layer (based-1b.yaml: n_embd 1792, 16 heads); bytes = q, k, v "
                                 "read + o written (+ k, v written to the cache: x 1.5)"},
        "roofline": {"kernel": "swa_prefill_kernel", "bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES["swa_prefill_kernel"], "algorithmic_bytes_per_launch": byts,
                     "timed": "the slower of cold (rotating inputs) and warm (one input)"},
    }


def bench_mfma_rate(torch, steps=20):
    """TFLOP/s of a loop of nothing but dense bf16 MFMA 16x16x32 (bench_probes.hip), after 30 ms of
    that load: what the matrix pipes sustain at the clock the board settles at."""
    import ctypes as C

    lib = probes()
    dev = torch.device("cuda:0")
    wgs = 256 * 4
    buf = torch.empty(wgs * 256, dtype=torch.float32, device=dev)
    flops = C.c_double(0.0)
    stream = torch.cuda.current_stream().cuda_stream
    ms, _ = _events_ms(torch, lambda: _probe_ok(lib.bench_probe_mfma(buf.data_ptr(), wgs, 2000, C.byref(flops), stream)),
                       steps, 2, warmup_ms=30.0)
    return flops.value / (ms * 1e-3) / 1e12


def bench_machine(torch, steps=20, warmup=4, n_sets=4):
    """What this machine's memory delivers for the access patterns of the HBM-bound kernels, measured
    with the probe kernels of bench_probes.hip (no arithmetic) over rotating buffers beyond the
    last-level cache: the ceiling next to which the 8 TB/s figure should be read."""
    lib = probes()
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    out = {}
    # state-update pattern: 145 MB read and rewritten in place per launch, like the B=128 decode step
    n = 128 * 16 * (273 * 64 + 273) * 4 // 16 * 16
    bufs = [torch.zeros(n, dtype=torch.uint8, device=dev) for _ in range(n_sets)]
    it = [0]

    def rmw():
        b = bufs[it[0] % n_sets]
        it[0] += 1
        _probe_ok(lib.bench_probe_rmw(b.data_ptr(), n, stream))

    ms, _ = _events_ms(torch, rmw, steps, warmup)
    out["rmw_cold_GBps"] = round(2 * n / (ms * 1e-3) / 1e9, 1)
    srcs = [torch.ones(n, dtype=torch.uint8, device=dev) for _ in range(n_sets)]

    def cp():
        i = it[0] % n_sets
        it[0] += 1
        _probe_ok(lib.bench_probe_copy(bufs[i].data_ptr(), srcs[i].data_ptr(), n, stream))

    ms, _ = _events_ms(torch, cp, steps, warmup)
    out["copy_cold_GBps"] = round(2 * n / (ms * 1e-3) / 1e9, 1)
    del bufs, srcs
    # packed-qkv pattern of the window attention (B=8, H=16, L=4096), 1 / 2 / 4 heads per workgroup
    B, H, L = 8, 16, 4096
    xs = [torch.ones(B, L, 3, H, 64, dtype=torch.bfloat16, device=dev) for _ in range(n_sets)]
    os_ = [torch.empty(B, L, H, 64, dtype=torch.bfloat16, device=dev) for _ in range(n_sets)]
    for g in (1, 2, 4):
        def st():
            i = it[0] % n_sets
            it[0] += 1
            _probe_ok(lib.bench_probe_stream_qkv(xs[i].data_ptr(), os_[i].data_ptr(), B, H, L, g, stream))

        ms, _ = _events_ms(torch, st, steps, warmup)
        out[f"stream_qkv_cold_GBps_{g}_heads"] = round(B * L * H * 512 / (ms * 1e-3) / 1e9, 1)
    del xs, os_
    # memory side of the linear-attention prefill (B=96, H=16, L=4096, dv=64: 2.01 GB per launch, cold by size)
    B, H, L = 96, 16, 4096
    q = torch.ones(B, L, H * 16, dtype=torch.bfloat16, device=dev)
    k = torch.ones(B, L, H * 16, dtype=torch.bfloat16, device=dev)
    v = torch.ones(B, L, H * 64, dtype=torch.bfloat16, device=dev)
    y = torch.empty(B, L, H * 64, dtype=torch.bfloat16, device=dev)
    ms, _ = _events_ms(torch, lambda: _probe_ok(lib.bench_probe_stream_prefill(q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                                                                   y.data_ptr(), B, H, L, stream)), steps, warmup)
    out["stream_prefill_B96_ms"] = round(ms, 4)
    out["stream_prefill_B96_GBps"] = round(B * L * H * 320 / (ms * 1e-3) / 1e9, 1)
    del q, k, v, y
    out["mfma_bf16_sustained_TFLOPs"] = round(bench_mfma_rate(torch), 1)
    out["note"] = ("probe kernels of bench_probes.hip over %d rotating buffer sets; GB/s of bytes read + written; "
                   "mfma: a loop of dense bf16 MFMA only, after 30 ms of that load" % n_sets)
    return out


def bench_conv(torch, ops, steps, warmup, B=4, L=2048, D=2048, K=3, decode_B=128):
    """Gated short convolution at the shape of the 27-layer configuration (d_inner = 2048)."""
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(2)
    n_sets = 8   # 8 x 67 MB of inputs (+ outputs): cold; one set: warm
    us = [torch.randn(B, L, 2 * D, generator=g).bfloat16().to(dev) for _ in range(n_sets)]
    w = (torch.randn(D, 1, K, generator=g) * 0.5).bfloat16().to(dev)
    it = [0]

    def make(sets):
        def f():
            it[0] += 1
            ops.gated_conv_prefill(us[it[0] % sets], w)
        return f

    ms_cold, _ = _events_ms(torch, make(n_sets), steps, warmup)
    ms_warm, _ = _events_ms(torch, make(1), steps, warmup)
    ms = max(ms_cold, ms_warm)
    del us
    byts = B * L * D * 3 * 2
    state = torch.zeros(decode_B, D, K, dtype=torch.bfloat16, device=dev)
    u1 = torch.randn(decode_B, 1, 2 * D, generator=g).bfloat16().to(dev)
    dms, _ = _events_ms(torch, lambda: ops.gated_conv_step(u1, state, w), 64, 8)
    return {
        "prefill_tok_s": B * L / (ms * 1e-3), "prefill_ms": ms, "B": B, "L": L, "D": D, "K": K,
        "decode_tok_s": decode_B / (dms * 1e-3), "decode_us": dms * 1e3, "decode_B": decode_B,
        "cold": {"ms": round(ms_cold, 5), "GBps": round(byts / (ms_cold * 1e-3) / 1e9, 1), "input_sets": n_sets},
        "warm": {"ms": round(ms_warm, 5), "GBps": round(byts / (ms_warm * 1e-3) / 1e9, 1), "input_sets": 1},
        "roofline": {"kernel": "gated_conv_prefill_kernel", "bound": "hbm", "achieved": round(byts / (ms * 1e-3) / 1e9, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(byts / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "traffic": None, "algorithmic_bytes_per_launch": byts,
                     "timed": "the slower of cold (rotating inputs) and warm (one input)"},
    }


def bench_stack(torch, B=4, prefill_len=2048, new_tokens=128, released=False):
    """configs[3]: the 27-layer 360M-shaped stack (random weights, bf16): prefill of 2048 tokens,
    then greedy decoding, eagerly and through the recorded decode graph.  released=True: the
    released checkpoint's configuration instead (window_size 256, rotary, graph decoding only)."""
    from based_amd.stack import GPTLMHeadModel, based_360m_config, based_360m_released_config

    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    cfg = based_360m_released_config() if released else based_360m_config()
    model = GPTLMHeadModel(cfg, device=dev, dtype=torch.bfloat16).eval()
    ids = torch.randint(0, 50277, (B, prefill_len), dtype=torch.long, device=dev)
    out = {"B": B, "prefill_len": prefill_len, "new_tokens": new_tokens}
    with torch.inference_mode():
        model(ids[:, :64])  # warm-up (library handles, workspaces)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        model(ids, num_last_tokens=1)
        torch.cuda.synchronize()
        out["prefill_ms"] = (time.perf_counter() - t0) * 1e3
        out["prefill_tok_s"] = B * prefill_len / (out["prefill_ms"] * 1e-3)
    for name, cg in ((("graph", True),) if released else (("eager", False), ("graph", True))):
        model.generate(input_ids=ids, max_length=prefill_len + new_tokens, cg=cg)  # warm-up / graph capture
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        model.generate(input_ids=ids, max_length=prefill_len + new_tokens, cg=cg)
        torch.cuda.synchronize()
        total = (time.perf_counter() - t0) * 1e3
        ms_tok = (total - out["prefill_ms"]) / new_tokens
        out[f"decode_{name}_ms_per_token"] = ms_tok
        out[f"decode_{name}_tok_s"] = B / (ms_tok * 1e-3)
    out["decode_graph_note"] = "greedy sampling recorded in the graph (based_greedy_step): one replay per token"
    return out


def bench_projections(torch, M=4):
    """The projections of one decoding step of the 27-layer configuration (`based_decode_linear`, M rows =
    the decoding batch), each timed as a recorded graph of launches over enough independent
    weight matrices to exceed the last-level cache, next to `torch.nn.functional.linear` on the
    same matrices.  The LM head (103 MB of weights per launch) carries an HBM roofline."""
    import torch.nn.functional as F

    from based_amd import ops

    with torch.inference_mode():  # as the decoding loop runs (and as graphs recorded after it must)
        return _bench_projections(torch, F, ops, M)


def _bench_projections(torch, F, ops, M):
    dev = torch.device("cuda:0")
    D, F1, V = 1024, 2048, 50280

    def timed_graph(fn, n_sets):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for i in range(n_sets):
                fn(i)
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for i in range(n_sets):
                    fn(i)
        torch.cuda.current_stream().wait_stream(side)
        ms, _ = _events_ms(torch, graph.replay, 10, 2)
        return ms * 1e3 / n_sets

    def weights(n, k, n_sets):
        return [torch.randn(n, k, device=dev).mul_(0.05).to(torch.bfloat16) for _ in range(n_sets)]

    x = torch.randn(M, D, device=dev).to(torch.bfloat16)
    xg = torch.randn(M, F1, device=dev).to(torch.bfloat16)
    res = torch.randn(M, D, device=dev)
    res_out = torch.empty_like(res)
    nw = torch.ones(D, device=dev, dtype=torch.bfloat16)
    norm = dict(prologue=ops.PROLOGUE_ADD_RMS_NORM, residual_in=res, residual_out=res_out, norm_weight=nw, eps=1e-5)
    out = {"M": M, "note": "us per launch inside a recorded graph, weights rotating over > 256 MB; torch = F.linear alone "
                           "(without the norm / gate / convolution step the fused launch contains)"}
    cases = [
        ("out_proj 1024x1024", D, D, lambda w, y: ops.decode_linear(x, w, out=y), x),
        ("fc2 / conv out_proj 1024x2048", D, F1, lambda w, y: ops.decode_linear(xg, w, out=y), xg),
        ("norm + qkv 1536x1024", 1536, D, lambda w, y: ops.decode_linear(x, w, out=y, **norm), x),
        ("norm + fc1 4096x1024 + gate", 2 * F1, D,
         lambda w, y: ops.decode_linear(x, w, out=y[:, :F1], epilogue=ops.EPILOGUE_SWIGLU, **norm), x),
    ]
    for name, n, k, fn, xin in cases:
        n_sets = min(64, max(4, int(400e6 / (n * k * 2))))
        ws = weights(n, k, n_sets)
        y = torch.empty(M, n, dtype=torch.bfloat16, device=dev)
        mine = timed_graph(lambda i: fn(ws[i], y), n_sets)
        ref = timed_graph(lambda i: F.linear(xin, ws[i]), n_sets)
        out[name] = {"us": round(mine, 2), "torch_linear_us": round(ref, 2), "weight_MB": round(n * k * 2 / 1e6, 1),
                     "weight_sets": n_sets}
        del ws
    # in_proj of BaseConv with the convolution step in its tail
    n_sets = 48
    ws = weights(2 * F1, D, n_sets)
    state = torch.zeros(M, F1, 3, device=dev, dtype=torch.bfloat16)
    cw = torch.randn(F1, 1, 3, device=dev).to(torch.bfloat16)
    cb = torch.zeros(F1, device=dev, dtype=torch.bfloat16)
    y = torch.empty(M, F1, dtype=torch.bfloat16, device=dev)
    mine = timed_graph(lambda i: ops.decode_linear(x, ws[i], out=y, epilogue=ops.EPILOGUE_GATED_CONV_STEP, conv_state=state,
                                                   conv_weight=cw, conv_bias=cb, **norm), n_sets)
    ref = timed_graph(lambda i: F.linear(x, ws[i]), n_sets)
    out["norm + in_proj 4096x1024 + conv step"] = {"us": round(mine, 2), "torch_linear_us": round(ref, 2),
                                                    "weight_MB": round(2 * F1 * D * 2 / 1e6, 1), "weight_sets": n_sets}
    del ws
    # LM head: closing norm + 50280 x 1024 projection, 103 MB of weights per launch
    n_sets = 4
    ws = weights(V, D, n_sets)
    y = torch.empty(M, V, dtype=torch.bfloat16, device=dev)
    mine = timed_graph(lambda i: ops.decode_linear(x, ws[i], out=y, prologue=ops.PROLOGUE_ADD_RMS_NORM, residual_in=res,
                                                   norm_weight=nw, eps=1e-5), n_sets)
    ref = timed_graph(lambda i: F.linear(x, ws[i]), n_sets)
    nbytes = V * D * 2 + M * D * 6 + M * V * 2
    gbs = nbytes / (mine * 1e-6) / 1e9
    out["norm + lm_head 50280x1024"] = {
        "us": round(mine, 2), "torch_linear_us": round(ref, 2), "weight_MB": round(V * D * 2 / 1e6, 1), "weight_sets": n_sets,
        "roofline": {"kernel": "decode_linear_kernel", "bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES["decode_linear_kernel_lm_head"] if M == 4 else None,
                     "algorithmic_bytes_per_launch": nbytes}}
    return out


def cpu_baseline_decode(torch, B=128, H=16, dv=64, sample_steps=8):
    """The oracle's recurrent step on the host: `sample_steps` of the 256 steps at full batch."""
    from oracle import based_oracle as O

    g = torch.Generator().manual_seed(0)
    kv = torch.randn(B, H, 1, dv, D_EXP, generator=g)
    ks = torch.randn(B, H, 1, 1, D_EXP, generator=g).abs() + 1
    q = torch.randn(B, H, 1, 16, generator=g).bfloat16()
    k = torch.randn(B, H, 1, 16, generator=g).bfloat16()
    v = torch.randn(B, H, 1, dv, generator=g).bfloat16()
    O.linear_attn_step(kv, ks, q.float(), k.float(), v.float())  # warm-up
    t0 = time.perf_counter()
    for _ in range(sample_steps):
        O.linear_attn_step(kv, ks, q.float(), k.float(), v.float())
    dt = (time.perf_counter() - t0) / sample_steps
    return {"value": round(B / dt, 1), "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{sample_steps} of 256 decode steps at B={B}, H={H}, dv={dv} (oracle linear_attn_step, fp32, torch CPU)",
            "host_cpu_count": os.cpu_count(), "ms_per_step": round(dt * 1e3, 2)}


def cpu_baseline_prefill(torch, H=16, L=1024, dv=64, reps=3):
    """configs[0] on the host: the quadratic causal form (the reference's default
    parallel_forward), B=1, fp32, plus the compiled reference C++ causal product when present."""
    from oracle import based_oracle as O
    from oracle import ref_loader

    g = torch.Generator().manual_seed(0)
    q = torch.randn(1, H, L, 16, generator=g) * 0.25
    k = torch.randn(1, H, L, 16, generator=g) * 0.25
    v = torch.randn(1, H, L, dv, generator=g)
    O.linear_attn_quadratic(q, k, v)
    t0 = time.perf_counter()
    for _ in range(reps):
        O.linear_attn_quadratic(q, k, v)
    dt = (time.perf_counter() - t0) / reps
    out = {"value": round(L / dt, 1), "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
           "sample": f"configs[0]: B=1 H={H} L={L} dv={dv} fp32, oracle linear_attn_quadratic, {reps} passes",
           "ms": round(dt * 1e3, 2)}
    if ref_loader.available():
        fq, fk = O.taylor_exp(q), O.taylor_exp(k)
        ref_loader.causal_dot_product(fq, fk, v)
        t0 = time.perf_counter()
        ref_loader.causal_dot_product(fq, fk, v)
        dt = time.perf_counter() - t0
        out["reference_cpp"] = {"value": round(L / dt, 1), "unit": "tokens/s", "kind": "reference", "ms": round(dt * 1e3, 2),
                                "sample": "same inputs, compiled causal_dot_product on precomputed 273-dim feature maps "
                                          "(numerator only), 1 pass"}
    return out


def cpu_baseline_swa(torch, H=16, L=4096, reps=2):
    """One batch entry of configs[2] on the host (masked-softmax statement of the window attention)."""
    from oracle import based_oracle as O

    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(1, L, H, 64, generator=g) for _ in range(3))
    O.sliding_window_attn(q, k, v, w_left=64)
    t0 = time.perf_counter()
    for _ in range(reps):
        O.sliding_window_attn(q, k, v, w_left=64)
    dt = (time.perf_counter() - t0) / reps
    return {"value": round(L / dt, 1), "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"B=1 of configs[2]'s 8: H={H} L={L} window 64 fp32, oracle sliding_window_attn, {reps} passes",
            "ms": round(dt * 1e3, 2)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-graph", action="store_true",
                    help="decode legs: launches issued one by one, HIP events (for counter runs under a profiler)")
    ap.add_argument("--only", choices=["decode", "prefill", "swa", "conv", "stack", "projections", "copy", "machine"], default=None,
                    help="one workload only; 'copy' is a plain 256 MiB device copy (the copy probe of bench_probes.hip) used to "
                         "calibrate the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run; 'machine' the memory "
                         "probes alone")
    ap.add_argument("--prefill-batches", default="1,8,32,96",
                    help="comma-separated batch sizes of the L=4096 prefill lines")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path is measured on ONE GPU (every (batch, head) pair is independent; "
              "nothing here uses a second device). Re-run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from based_amd import ops

    if args.only == "copy":
        n = 256 * 1024 * 1024
        src = torch.empty(n, dtype=torch.uint8, device="cuda:0").fill_(1)
        dst = torch.empty_like(src)
        stream = torch.cuda.current_stream().cuda_stream
        ms, _ = _events_ms(torch, lambda: _probe_ok(probes().bench_probe_copy(dst.data_ptr(), src.data_ptr(), n, stream)),
                           args.steps, args.warmup)
        assert bool((dst == 1).all())
        print(json.dumps({"workload": "plain device copy (probe_rw_kernel)", "bytes_read": n, "bytes_written": n,
                          "ms": round(ms, 5), "GBps": round(2 * n / (ms * 1e-3) / 1e9, 1)}))
        return
    if args.only == "machine":
        print(json.dumps({"machine": bench_machine(torch)}))
        return

    out = {
        "metric": "prefill tok/s @L=4096 + decode tok/s @B=128, Based-360m mixers, 1 GPU",
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
    }
    if args.only in (None, "decode"):
        d = bench_decode(torch, ops, args.steps, args.warmup, long_region_too=not args.no_graph, use_graph=not args.no_graph)
        if d["long_region"] is not None:
            d["roofline"]["long_region"] = d["long_region"]
        out.update({"value": round(d["tok_s"], 1), "ms_per_step": round(d["ms"], 5),
                    "config": {"workload": "configs[1]: " + d["workload"], "layers": 1},
                    "roofline": d["roofline"], "wall_ms_per_step": round(d["wall_ms"], 5),
                    "decode_cold": d["cold"], "decode_warm": d["warm"]})
        with torch.inference_mode():
            out["decode_deferred"] = bench_decode_deferred(torch, ops)
    if args.only in (None, "prefill"):
        pre = [bench_prefill(torch, ops, 30, 3, B=b) for b in sorted({int(x) for x in args.prefill_batches.split(',')})]
        if args.only is None or args.prefill_batches == "1,8,32,96":
            pre.append(bench_prefill(torch, ops, 30, 3, B=32, dv=112))   # the released 1B / 1.3B head dim
        out["prefill"] = [{k: (round(v, 3) if isinstance(v, float) else v) for k, v in p.items()} for p in pre]
        # the same fractions against what a loop of nothing but MFMA sustains on this board (the
        # published peak assumes the maximum clock, which the board does not hold under that load)
        sustained = bench_mfma_rate(torch)
        for p in out["prefill"]:
            p["roofline"]["mfma_sustained_TFLOPs"] = round(sustained, 1)
            p["roofline"]["frac_of_sustained_mfma"] = round(p["roofline"]["achieved"] / sustained, 4)
    if args.only in (None, "prefill"):
        # configs[4]: one 32K-token sequence at head dim 128, and its decode batch of 64
        c5 = bench_prefill(torch, ops, 30, 3, B=1, L=32768, dv=128)
        d5 = bench_decode(torch, ops, 64, 8, B=64, dv=128, prefill_len=256, use_graph=not args.no_graph)
        out["long_context"] = {"prefill": {k: (round(v, 3) if isinstance(v, float) else v) for k, v in c5.items()},
                               "decode": {"tok_s": round(d5["tok_s"], 1), "ms": round(d5["ms"], 5), "B": 64, "dv": 128,
                                          "cold": d5["cold"], "warm": d5["warm"], "roofline": d5["roofline"]}}
    if args.only in (None, "swa"):
        s = bench_swa(torch, ops, 20, 3)
        out["swa"] = {k: (round(v, 3) if isinstance(v, float) else v) for k, v in s.items()}
    if args.only in (None, "conv"):
        c = bench_conv(torch, ops, 20, 3)
        out["conv"] = {k: (round(v, 3) if isinstance(v, float) else v) for k, v in c.items()}
    if args.only == "conv":
        out.update({"value": round(out["conv"]["prefill_tok_s"], 1), "ms_per_step": out["conv"]["prefill_ms"], "dtype": "bf16",
                    "config": {"workload": "gated short convolution prefill B=4 L=2048 D=2048 K=3"},
                    "roofline": out["conv"]["roofline"]})
    if args.only in (None, "stack"):
        st = bench_stack(torch)
        out["stack"] = {k: (round(v, 3) if isinstance(v, float) else v) for k, v in st.items()}
        rel = bench_stack(torch, released=True)
        out["stack"]["released_config"] = {k: (round(v, 3) if isinstance(v, float) else v) for k, v in rel.items()
                                           if k in ("prefill_ms", "prefill_tok_s", "decode_graph_ms_per_token", "decode_graph_tok_s")}
        out["stack"]["released_config"]["note"] = "window_size 256, rotary_emb_fraction 1, fla_parallel (based-360m.yaml)"
    if args.only in (None, "stack", "projections"):
        out["projections"] = bench_projections(torch)
    if args.only == "projections":
        lm = out["projections"]["norm + lm_head 50280x1024"]
        out.update({"value": round(4 / (lm["us"] * 1e-6), 1), "ms_per_step": round(lm["us"] * 1e-3, 5), "dtype": "bf16",
                    "config": {"workload": "closing norm + LM head projection of a decoding step, M=4, 50280 x 1024 bf16"},
                    "roofline": lm["roofline"]})
    if args.only == "stack":
        out.update({"value": round(out["stack"]["decode_graph_tok_s"], 1),
                    "ms_per_step": out["stack"]["decode_graph_ms_per_token"], "dtype": "bf16",
                    "config": {"workload": "configs[3]: 27-layer stack, B=4, prefill 2048 + 128 greedy tokens (decode graph)"}})
    if args.only == "prefill":
        p = [x for x in out["prefill"] if x["dv"] == 64][-1]
        out.update({"value": round(p["tok_s"], 1), "ms_per_step": p["ms"], "dtype": "bf16",
                    "config": {"workload": f"linear-attn prefill B={p['B']} L={p['L']} dv={p['dv']}"}, "roofline": p["roofline"]})
    if args.only == "swa":
        out.update({"value": round(out["swa"]["prefill_tok_s"], 1), "ms_per_step": out["swa"]["prefill_ms"], "dtype": "bf16",
                    "config": {"workload": "configs[2]: sliding-window prefill B=8 H=16 L=4096 w=64"},
                    "roofline": out["swa"]["roofline"]})
    if args.only is None:
        out["machine"] = bench_machine(torch)
    if not args.no_cpu and args.only in (None, "decode"):
        out["cpu_baseline"] = cpu_baseline_decode(torch)
    if not args.no_cpu and args.only is None:
        out["cpu_baseline_prefill"] = cpu_baseline_prefill(torch)
        out["cpu_baseline_swa"] = cpu_baseline_swa(torch)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
