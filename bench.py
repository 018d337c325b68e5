#!/usr/bin/env python3
"""Benchmark of the KV-cache attention path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload llama3b_decode_8k|...]

Default workload = benchmark configuration 2: Llama-3.2-3B-shaped decode attention, 28 layers, batch 1, 24 query heads,
8 KV heads, head_dim 128, f16 KV cache at 8192 context (seeded N(0,1)), RoPE theta 5e5 ("normal" pairing), one token
appended per layer then flash-decode SDPA. A "step" is one decode step = 28 x (fused RoPE + append, flash decode).
Inputs are resident in HBM before the timed region. The K steps are recorded into HIP graphs of 16 steps each
(position lives in device memory), replayed back to back, and timed with a synchronize on both sides.

Prints ONE JSON line: steps/s, the roofline of the dominant kernel (per-launch HIP-event timing from a separate
eager pass over the same workload), and a CPU baseline (the oracle, timed on a bounded sample).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "test-burn_amd"))
sys.path.insert(0, os.path.join(ROOT, "tests"))

import foundry_attn as fa  # noqa: E402

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, AMD's published figure
GRAPH_STEPS = 16

_COLLECT = None  # a list while the default run gathers the other configurations' lines instead of printing them


def emit(result):
    """A workload's JSON line: printed, or kept for the default run's "configs" object."""
    if _COLLECT is not None:
        _COLLECT.append(result)
    else:
        print(json.dumps(result))



def make_llama3b_decode(f, rng, start_ctx, room):
    """Allocates and fills the 28-layer Llama-3.2-3B-shaped decode state; returns a dict of device buffers."""
    L, H, Hkv, D = 28, 24, 8, 128
    cap = start_ctx + room
    cap = (cap + 127) // 128 * 128  # the reference aligns capacity to 128 (src/model/context.rs:213-219)
    st = dict(L=L, H=H, Hkv=Hkv, D=D, cap=cap, start=start_ctx, theta=5e5, rope_mode=fa.ROPE_NORMAL)
    cos, sin = fa.rope_tables(st["theta"], D, cap)
    st["cos_h"], st["sin_h"] = cos, sin
    st["dcos"], st["dsin"] = f.array(cos), f.array(sin)
    st["kc"], st["vc"] = [], []
    for i in range(L):
        k = np.zeros((Hkv, cap, D), np.float16)
        v = np.zeros((Hkv, cap, D), np.float16)
        k[:, :start_ctx] = rng.standard_normal((Hkv, start_ctx, D), dtype=np.float32).astype(np.float16)
        v[:, :start_ctx] = rng.standard_normal((Hkv, start_ctx, D), dtype=np.float32).astype(np.float16)
        st["kc"].append(f.array(k))
        st["vc"].append(f.array(v))
        if i < 2:  # host copies of two layers feed the CPU baseline and the end-of-run check
            st.setdefault("host_kv", []).append((k, v))
    # fresh q/k/v per (slot, layer); slot = step % GRAPH_STEPS
    st["q_h"] = rng.standard_normal((GRAPH_STEPS, L, H * D), dtype=np.float32).astype(np.float16)
    st["k_h"] = rng.standard_normal((GRAPH_STEPS, L, Hkv * D), dtype=np.float32).astype(np.float16)
    st["v_h"] = rng.standard_normal((GRAPH_STEPS, L, Hkv * D), dtype=np.float32).astype(np.float16)
    st["dq"], st["dk"], st["dv"] = f.array(st["q_h"]), f.array(st["k_h"]), f.array(st["v_h"])
    st["dqr"] = f.zeros((L, H * D))
    st["dout"] = f.zeros((L, H * D))
    st["dpos"] = f.array(np.array([start_ctx], np.uint32))
    st["params"] = fa.KvPrepFusedParams.make(H, Hkv, D, 1, 0, cap, st["rope_mode"])
    return st


def enqueue_step(f, st, slot, fused=True):
    """One decode step: per layer, RoPE + KV append + flash decode (one fused launch, or the two separate ops);
    then advance the position."""
    L, H, Hkv, D, cap = st["L"], st["H"], st["Hkv"], st["D"], st["cap"]
    dm, kvd = H * D, Hkv * D
    for i in range(L):
        qo = (slot * L + i) * dm * 2
        ko = (slot * L + i) * kvd * 2
        if fused:
            f.decode_step_fused(st["dq"].arg((1, dm), offset=qo), st["dk"].arg((1, kvd), offset=ko),
                                st["dv"].arg((1, kvd), offset=ko), None, st["kc"][i].arg(), st["vc"][i].arg(),
                                st["dcos"].arg(), st["dsin"].arg(), st["dout"].arg((1, dm), offset=i * dm * 2),
                                st["params"], d_position=st["dpos"], kv_len_bound=cap)
            continue
        f.kv_prep_fused(st["dq"].arg((1, dm), offset=qo), st["dk"].arg((1, kvd), offset=ko),
                        st["dv"].arg((1, kvd), offset=ko), st["dqr"].arg((1, dm), offset=i * dm * 2), st["kc"][i].arg(),
                        st["vc"][i].arg(), st["dcos"].arg(), st["dsin"].arg(), st["params"], d_position=st["dpos"])
        f.flash_decode_dyn(st["dqr"].arg((1, dm), offset=i * dm * 2), st["kc"][i].arg(), st["vc"][i].arg(),
                           st["dout"].arg((1, dm), offset=i * dm * 2), H, D, st["dpos"], 1, cap)
    f.u32_add(st["dpos"], 1, 1)


def layer_bytes(st, n):
    """Algorithmic HBM bytes of one layer of one decode step at kv_len n (after the append): K and V read once per
    KV head (2*Hkv*n*D*2), the appended K/V rows written (2*Hkv*D*2), q read and out written (2*H*D*2), the new
    token's raw k/v read (2*Hkv*D*2) and one cos + one sin row (2*(D/2)*2)."""
    H, Hkv, D = st["H"], st["Hkv"], st["D"]
    return 2 * Hkv * n * D * 2 + 2 * Hkv * D * 2 + 2 * H * D * 2 + 2 * Hkv * D * 2 + 2 * (D // 2) * 2


def step_bytes(st, n):
    return st["L"] * layer_bytes(st, n)


def run_steps(f, st, graph16, graph1, steps, room, history=None):
    """Replays `steps` decode steps; the position wraps to the start every `room` steps (cache capacity).
    Appends (position, input slot) of every step to `history`."""
    done = 0
    while done < steps:
        seg = min(room, steps - done)
        if done > 0:
            st["dpos"].upload(np.array([st["start"]], np.uint32))
        for _ in range(seg // GRAPH_STEPS):
            graph16.launch()
        for _ in range(seg % GRAPH_STEPS):
            graph1.launch()
        if history is not None:
            slots = list(range(GRAPH_STEPS)) * (seg // GRAPH_STEPS) + [0] * (seg % GRAPH_STEPS)
            history.extend((st["start"] + i, sl) for i, sl in enumerate(slots))
        done += seg


def cpu_baseline(st, sample_seconds, room):
    """The oracle (scalar C restatement of the reference arithmetic, OpenMP over heads) on the same workload: decode
    steps of the timed window over 2 of the 28 layers, scaled to 28 layers; once on one thread and once on every host
    core the process may use (about a third and two thirds of sample_seconds of wall time)."""
    import orc

    host_cpus = os.cpu_count() or 1
    try:
        usable = len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        usable = host_cpus
    all_threads = max(1, min(usable, orc.lib().orc_max_threads()))
    L, H, Hkv, D, cap, start = st["L"], st["H"], st["Hkv"], st["D"], st["cap"], st["start"]
    layers = len(st["host_kv"])

    def sample(threads, seconds):
        kv = [(k.copy(), v.copy()) for k, v in st["host_kv"]]
        done = 0
        t0 = time.perf_counter()
        while True:
            s = done % room
            for i in range(layers):
                k, v = kv[i]
                qr = orc.kv_prep_fused(st["q_h"][s % GRAPH_STEPS, i:i + 1], st["k_h"][s % GRAPH_STEPS, i:i + 1],
                                       st["v_h"][s % GRAPH_STEPS, i:i + 1], k, v, st["cos_h"], st["sin_h"],
                                       orc.make_params(H, Hkv, D, 1, start + s, cap, rope_mode=1))
                orc.sdpa_decode(qr[:, 0].copy(), k, v, H, Hkv, D, cap, start + s + 1, n_threads=threads)
            done += 1
            dt = time.perf_counter() - t0
            if dt >= seconds:
                break
        per_step = dt / done * (L / layers)
        return {"value": 1.0 / per_step, "unit": "steps/s", "cores": threads, "host_cpus": host_cpus, "kind": "port",
                "sample": "%d decode steps x %d of %d layers from kv_len %d, scaled to %d layers (%.1f s wall on %d thread%s)"
                          % (done, layers, L, start + 1, L, dt, threads, "" if threads == 1 else "s")}

    one = sample(1, sample_seconds / 3.0)
    many = sample(all_threads, sample_seconds * 2.0 / 3.0)
    many["one_thread"] = one
    return many


def check_against_oracle(f, st, history):
    """After the run: layer 0's cache and last output must match the oracle replaying the same appends."""
    import orc

    H, Hkv, D, cap = st["H"], st["Hkv"], st["D"], st["cap"]
    k, v = (a.copy() for a in st["host_kv"][0])
    out = None
    for idx, (pos, slot) in enumerate(history):
        qr = orc.kv_prep_fused(st["q_h"][slot, 0:1], st["k_h"][slot, 0:1], st["v_h"][slot, 0:1], k, v, st["cos_h"],
                               st["sin_h"], orc.make_params(H, Hkv, D, 1, pos, cap, rope_mode=1))
        if idx == len(history) - 1:
            out = orc.sdpa_decode(qr[:, 0].copy(), k, v, H, Hkv, D, cap, pos + 1, n_threads=8)
    got_k = st["kc"][0].download()
    got_out = st["dout"].download()[0]
    cache_ok = bool(np.array_equal(got_k.view(np.uint16), k.view(np.uint16)))
    err = float(np.max(np.abs(got_out.astype(np.float32) - out.astype(np.float32))))
    return cache_ok, err


# HBM bytes per launch of the fused decode kernel come from the FETCH_SIZE / WRITE_SIZE counter runs summarised in
# profiles/decode_llama3b_8k_hbm_counters.txt (a counter run cannot be made from inside this script). The summary names
# the hash of the kernel sources it was measured on: when those have changed since, the figure is reported as null.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "decode_llama3b_8k_hbm_counters.txt")
KERNEL_SOURCES = ["fa_decode_impl.h", "fa_decode.hip", "fa_internal.h"]


def kernel_source_hash():
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "test-burn_amd", "csrc", name), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def measured_traffic():
    """(bytes per launch or None, note) from the `traffic_bytes_per_launch=` / `kernel_source_sha256_16=` lines of the
    committed counter summary."""
    import re
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return None, "no counter summary"
    m_b = re.search(r"^traffic_bytes_per_launch=([0-9.eE+]+)", text, re.M)
    m_h = re.search(r"^kernel_source_sha256_16=([0-9a-f]{16})", text, re.M)
    if not m_b or not m_h:
        return None, "counter summary carries no machine-readable figure"
    if m_h.group(1) != kernel_source_hash():
        return None, "counter summary is for kernel sources %s, these are %s" % (m_h.group(1), kernel_source_hash())
    return float(m_b.group(1)), "profiles/decode_llama3b_8k_hbm_counters.txt"


def calibration_copy(f, reps=3):
    """A plain copy of known size through the library's gather kernel (pool rows -> contiguous rows): the HBM
    counters of a profiler run read against it give the factor between counter units and bytes."""
    Hkv, D, bs, tokens = 8, 128, 16, 65536
    nblk = tokens // bs
    k_pool, v_pool = f.zeros((nblk, Hkv, bs, D)), f.zeros((nblk, Hkv, bs, D))
    bt, lens = f.array(np.arange(nblk, dtype=np.int32).reshape(1, nblk)), f.array(np.array([tokens], np.uint32))
    desc = fa.paged_kv(k_pool, v_pool, bt, lens, nblk, Hkv, bs, D, 1, nblk)
    k_out, v_out = f.empty((Hkv, tokens, D)), f.empty((Hkv, tokens, D))
    for _ in range(reps):
        f.paged_gather(desc, 0, tokens, k_out, v_out, tokens)
    f.synchronize()
    nbytes = 2 * Hkv * tokens * D * 2  # read once, written once
    for b in (k_pool, v_pool, bt, lens, k_out, v_out):
        b.free()
    return {"kernel": "paged_gather_kernel", "launches": reps, "bytes_read": nbytes, "bytes_written": nbytes}


MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense f16 / bf16 matrix peak


def bench_prefill(f, args, tokens=2048):
    """Llama-3.2-3B-shaped prefill of one layer: `tokens` tokens (2048 = benchmark configuration 4), RoPE + append into an
    empty paged cache, then causal flash prefill from the paged cache. One step = both launches."""
    H, Hkv, D, M, bs = 24, 8, 128, tokens, 16
    rng = np.random.default_rng(0xF0DD + 4)
    nblk = M // bs
    perm = rng.permutation(nblk).astype(np.int32).reshape(1, nblk)
    k_pool, v_pool = f.zeros((nblk, Hkv, bs, D)), f.zeros((nblk, Hkv, bs, D))
    bt, lens = f.array(perm), f.array(np.array([0], np.uint32))
    desc = fa.paged_kv(k_pool, v_pool, bt, lens, nblk, Hkv, bs, D, 1, nblk)
    q, k, v = (rng.standard_normal((M, n * D), dtype=np.float32).astype(np.float16) for n in (H, Hkv, Hkv))
    cos, sin = fa.rope_tables(5e5, D, M)
    dq, dk, dv, dcos, dsin = (f.array(x) for x in (q, k, v, cos, sin))
    dqr, dout = f.zeros((H, M, D)), f.zeros((M, H * D))
    p = fa.KvPrepFusedParams.make(H, Hkv, D, M, 0, 0, fa.ROPE_NORMAL)

    def step():
        f.kv_prep_fused_paged(dq.arg(), dk.arg(), dv.arg(), dqr.arg(), desc, 0, dcos.arg(), dsin.arg(), p)
        f.flash_prefill_paged(dqr.arg(), desc, 0, dout.arg(), True, 0, H, M, M)

    step()
    f.synchronize()
    # a step's device time: (append, attention) pairs recorded into a HIP graph and replayed between two events on the stream
    per_step, n_timed = graph_replay_seconds(f, lambda i: step(), 8 if M <= 2048 else 2, args.warmup, min(args.steps, 80 if M <= 2048 else 8))

    # parity: cache bit-exact against the oracle's append; the last 64 query rows against the oracle's prefill
    import orc  # the CPU oracle is only the checker here
    kc, vc = np.zeros((Hkv, M, D), np.float16), np.zeros((Hkv, M, D), np.float16)
    qr = orc.kv_prep_fused(q, k, v, kc, vc, cos, sin, orc.make_params(H, Hkv, D, M, 0, M, rope_mode=1))
    cache_ok = (np.array_equal(orc.paged_gather(k_pool.download(), perm[0], Hkv, bs, D, M).view(np.uint16), kc.view(np.uint16))
                and np.array_equal(orc.paged_gather(v_pool.download(), perm[0], Hkv, bs, D, M).view(np.uint16), vc.view(np.uint16))
                and np.array_equal(dqr.download().view(np.uint16), qr.view(np.uint16)))
    tail = 64
    want = orc.sdpa_prefill(np.ascontiguousarray(qr[:, M - tail:]), kc, vc, H, Hkv, D, tail, M, M - tail, M, causal=True,
                            out_layout="head_major", n_threads=max(1, min(16, os.cpu_count() or 1, orc.lib().orc_max_threads())))
    got = dout.download().reshape(M, H, D).transpose(1, 0, 2)[:, M - tail:]
    err = float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64))))

    prof_steps = 20
    f.profile_reset()
    f.profile_enable(True)
    for _ in range(prof_steps):
        step()
    pf_kernel = "flash_prefill_dma_kernel"  # the paged cache selects the LDS-direct two-phase kernel
    n_pf, ms_pf = f.profile_query(pf_kernel)
    if n_pf == 0:
        pf_kernel = "flash_prefill_mfma_kernel"
        n_pf, ms_pf = f.profile_query(pf_kernel)
    n_kp, ms_kp = f.profile_query("kv_prep_fused")
    f.profile_enable(False)
    f.profile_reset()
    # the attention launch alone, back to back: a graph of 10, replayed, timed by two events on the stream
    f.start_capture()
    for _ in range(10):
        f.flash_prefill_paged(dqr.arg(), desc, 0, dout.arg(), True, 0, H, M, M)
    g = f.end_capture()
    for _ in range(2):
        g.launch()
    f.synchronize()
    reps = 10 if M <= 2048 else 4
    f.timer_start()
    for _ in range(reps):
        g.launch()
    b2b_us = f.timer_stop() * 1e3 / (10 * reps)
    g.destroy()
    flops = 4.0 * D * H * M * (M + 1) / 2  # QK^T and PV over the causal pairs
    avg_pf_s = ms_pf / 1e3 / max(1, n_pf)
    achieved = flops / avg_pf_s / 1e12
    append_bytes = 2.0 * M * (H + 2 * Hkv) * D * 2  # read q, k, v; write q_rot and the cache rows
    result = {
        "metric": "prefill-attn steps/s + achieved f16 MFMA TFLOP/s (%% peak), Llama-3.2-3B shape, %d tokens" % M,
        "value": 1.0 / per_step, "unit": "steps/s", "n_gpus": 1, "steps": n_timed, "warmup": args.warmup,
        "ms_per_step": per_step * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "timing": "ms_per_step = device time per step: HIP graph replays between two events on the kernels' stream",
        "config": {"workload": "llama3.2-3b prefill attention, one layer: RoPE + append of %d tokens into an empty paged "
                               "f16 cache (16-token blocks, permuted block table), then causal flash prefill, H24/Hkv8/D128, "
                               "graph replays" % M},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / MFMA_F16_PEAK_TFLOPS, "traffic": None, "kernel": pf_kernel,
                     "avg_launch_us": avg_pf_s * 1e6, "launches": n_pf, "flops_per_launch": flops,
                     "timing": "HIP events around each eager dispatch, each after the append of the whole prompt",
                     "back_to_back_graph_avg_launch_us": b2b_us, "back_to_back_graph_frac": flops / b2b_us / 1e6 / MFMA_F16_PEAK_TFLOPS},
        "append": {"kernel": "kv_prep_fused_vec_kernel", "avg_launch_us": ms_kp * 1e3 / max(1, n_kp),
                   "achieved_gbps": append_bytes / (ms_kp / 1e3 / max(1, n_kp)) / 1e9, "bytes_per_launch": append_bytes,
                   "frac_of_hbm_peak": append_bytes / (ms_kp / 1e3 / max(1, n_kp)) / 1e9 / HBM_PEAK_GBPS},
        "parity": {"cache_bit_exact": bool(cache_ok), "prefill_max_abs_err_last64": err},
    }
    emit(result)
    if not cache_ok or err > 2e-3:
        sys.exit("parity check failed: cache_bit_exact=%s prefill_max_abs_err=%g" % (cache_ok, err))


def graph_replay_seconds(f, step, per_graph, warmup, steps):
    """Device seconds per step of `step(i)` recorded `per_graph` times into one HIP graph and replayed: two events on the
    kernels' stream around the replays (per-dispatch profiling off), divided by the steps in them. Returns (seconds per
    step, steps timed)."""
    f.start_capture()
    for i in range(per_graph):
        step(i)
    graph = f.end_capture()
    for _ in range(max(1, warmup // per_graph)):
        graph.launch()
    f.synchronize()
    reps = max(1, steps // per_graph)
    f.timer_start()
    for _ in range(reps):
        graph.launch()
    per_step = f.timer_stop() / 1e3 / (reps * per_graph)
    graph.destroy()
    return per_step, reps * per_graph


def eager_kernel_us(f, step, n_steps, kernels):
    """{kernel: (launches, average us)} from an eager pass with HIP events attached to every dispatch (the events add a few
    tenths of a microsecond to what they measure)."""
    f.profile_reset()
    f.profile_enable(True)
    for i in range(n_steps):
        step(i)
    out = {}
    for k in kernels:
        n, ms = f.profile_query(k)
        if n:
            out[k] = (n, ms * 1e3 / n)
    f.profile_enable(False)
    f.profile_reset()
    return out


def _finish_secondary(f, args, name, workload, kernel, bytes_per_launch, dt, parity, extra=None, unit="layer-steps/s",
                      graph=None):
    """graph = (device seconds per step from graph replays, steps timed): then `value` and `ms_per_step` are device time per
    step, and - when the step is that one kernel - so is the roofline's launch duration; the eager per-dispatch event
    figure stays as a sub-field. Without it (legacy lines) the host's wall time over eager launches is reported."""
    n, ms = f.profile_query(kernel)
    eager_s = ms / 1e3 / max(1, n)
    steps = args.steps
    if graph is not None:
        per_step, steps = graph
        dt = per_step * steps
    one_kernel_step = graph is not None and (extra or {}).get("kernels_per_step", 1) == 1
    avg_s = graph[0] if one_kernel_step else eager_s
    achieved = bytes_per_launch / avg_s / 1e9
    result = {
        "metric": name, "value": steps / dt, "unit": unit, "n_gpus": 1, "steps": steps,
        "warmup": args.warmup, "ms_per_step": dt / steps * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic", "config": {"workload": workload},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": None, "kernel": kernel, "avg_launch_us": avg_s * 1e6,
                     "launches": steps if one_kernel_step else n, "bytes_per_launch": bytes_per_launch,
                     "timing": ("HIP events on the stream around the graph replays / launches in them" if one_kernel_step
                                else "HIP events around each eager dispatch"),
                     "eager_dispatch_avg_launch_us": eager_s * 1e6, "eager_dispatch_launches": n},
        "parity": parity,
    }
    if graph is not None:
        result["timing"] = "ms_per_step = device time per step: HIP graph replays between two events on the kernels' stream"
        result["whole_step_hbm_frac_of_peak"] = bytes_per_launch / graph[0] / 1e9 / HBM_PEAK_GBPS
    if extra:
        result.update({k: v for k, v in extra.items() if k != "kernels_per_step"})
    emit(result)


def bench_small_decode(f, args):
    """Qwen2.5-0.5B-shaped single-layer decode step at 1024 context (contiguous cache): launch-latency bound."""
    import orc
    H, Hkv, D, pos, cap, NL = 14, 2, 64, 1024, 1152, 16
    rng = np.random.default_rng(0xF0DD + 1)
    cos, sin = fa.rope_tables(1e6, D, cap)
    dcos, dsin = f.array(cos), f.array(sin)
    host, caches = [], []
    for i in range(NL):  # distinct caches so that no launch finds the previous one's data in cache
        kc, vc = np.zeros((Hkv, cap, D), np.float16), np.zeros((Hkv, cap, D), np.float16)
        kc[:, :pos] = rng.standard_normal((Hkv, pos, D), dtype=np.float32).astype(np.float16)
        vc[:, :pos] = rng.standard_normal((Hkv, pos, D), dtype=np.float32).astype(np.float16)
        caches.append((f.array(kc), f.array(vc)))
        if i == 0:
            host = [kc, vc]
    q, k, v = (rng.standard_normal((1, n * D), dtype=np.float32).astype(np.float16) for n in (H, Hkv, Hkv))
    dq, dk, dv, dqr, dout = f.array(q), f.array(k), f.array(v), f.zeros((H, 1, D)), f.zeros((1, H * D))
    p = fa.KvPrepFusedParams.make(H, Hkv, D, 1, pos, cap, fa.ROPE_NEOX)

    def step(i):
        kc, vc = caches[i % NL]
        f.decode_step_fused(dq.arg(), dk.arg(), dv.arg(), dqr.arg(), kc.arg(), vc.arg(), dcos.arg(), dsin.arg(),
                            dout.arg(), p)

    step(0)
    f.synchronize()
    want_qr = orc.kv_prep_fused(q, k, v, host[0], host[1], cos, sin, orc.make_params(H, Hkv, D, 1, pos, cap, rope_mode=0))
    want = orc.sdpa_decode(want_qr[:, 0].copy(), host[0], host[1], H, Hkv, D, cap, pos + 1)
    err = float(np.max(np.abs(dout.download().reshape(-1).astype(np.float64) - want.reshape(-1).astype(np.float64))))
    ok = bool(np.array_equal(caches[0][0].download().view(np.uint16), host[0].view(np.uint16)))
    graph = graph_replay_seconds(f, step, 4 * NL, args.warmup, args.steps)
    f.profile_reset()
    f.profile_enable(True)
    for i in range(2 * NL):
        step(i)
    nbytes = 2.0 * Hkv * (pos + 1) * D * 2 + 2 * Hkv * D * 2 + 2 * H * D * 2 + 2 * D
    _finish_secondary(f, args, "decode-attn layer-steps/s + achieved HBM GB/s, Qwen2.5-0.5B shape @1K ctx",
                      "qwen2.5-0.5b single-layer decode step: RoPE + KV append + flash decode, batch 1, H14/Hkv2/D64, "
                      "kv_len 1025, graph replays over 16 layers' caches", "fused_rope_append_decode_kernel", nbytes, 0.0,
                      {"cache_bit_exact": ok, "decode_max_abs_err": err}, graph=graph)
    f.profile_enable(False)


def bench_kv_growth(f, args):
    """KV-cache growth of a Llama-3.2-3B session at 8448 tokens: the first 8448 rows of every head of all 56 cache
    tensors [8, 8448, 128] move into tensors of twice the capacity (one batched prefix copy)."""
    import orc
    L, Hkv, D, pos = 28, 8, 128, 8448
    new_cap = fa.grown_capacity(pos, pos + 1, 131072)
    rng = np.random.default_rng(0xF0DD + 6)
    base = rng.standard_normal((Hkv, pos, D), dtype=np.float32).astype(np.float16)
    old, new = [], []
    for i in range(2 * L):
        host = base if i == 0 else np.roll(base, i, axis=1)
        old.append(f.array(host))
        new.append(f.zeros((Hkv, new_cap, D)))
    srcs, dsts = [b.arg() for b in old], [b.arg() for b in new]

    def step(i):
        f.kv_prefix_copy_batch(srcs, dsts, pos)

    step(0)
    f.synchronize()
    want = np.zeros((Hkv, new_cap, D), np.float16)
    orc.kv_prefix_copy(np.roll(base, 5, axis=1), want, pos)
    ok = bool(np.array_equal(new[5].download().view(np.uint16), want.view(np.uint16)))
    for i in range(args.warmup):
        step(i)
    f.synchronize()
    f.profile_reset()
    f.profile_enable(True)
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    f.synchronize()
    dt = time.perf_counter() - t0
    nbytes = 2.0 * 2 * L * Hkv * pos * D * 2  # read + written
    _finish_secondary(f, args, "KV-cache growth copies/s + achieved HBM GB/s, Llama-3.2-3B caches @8448 tokens",
                      "llama3.2-3b KV-cache growth %d -> %d rows: per-head prefix copy of 56 tensors [8, 8448, 128] f16, "
                      "one launch (profiling events on)" % (pos, new_cap), "kv_prefix_copy_vec_kernel", nbytes, dt,
                      {"copy_bit_exact": ok}, unit="growths/s")
    f.profile_enable(False)


def bench_fused_qkv(f, args, q8=False, q4=False):
    """The step before the path at Llama-3.2-3B decode shape: RMSNorm + Q/K/V projections of one token, F16 (or Q8_0)
    weights in the reference's canonical blocked layout, one layer per step over 8 distinct layers' weights."""
    import orc
    K, N, NK, NL = 3072, 3072, 1024, 8
    rng = np.random.default_rng(0xF0DD + 7)
    x = rng.uniform(-1, 1, (1, K)).astype(np.float16)
    g = rng.uniform(0.5, 1.5, K).astype(np.float16)
    layers, host0 = [], None
    for i in range(NL):  # distinct weights so that no launch finds the previous one's in cache
        ws = [rng.uniform(-0.1, 0.1, (n, K)).astype(np.float16) for n in (N, NK, NK)]
        if q4:
            ws = [orc.quantize_q4_0(w) for w in ws]
            packed = [orc.pack_q4_0(fa.canonical_layout(w)) for w, _ in ws]
            layers.append(([f.array(p) for p in packed], [f.array(sc) for _, sc in ws]))
            ws = [(orc.unpack_q4_0(p), sc) for p, (_, sc) in zip(packed, ws)]
        elif q8:
            ws = [orc.quantize_q8_0(w) for w in ws]
            layers.append(([f.array(fa.canonical_layout(w)) for w, _ in ws], [f.array(sc) for _, sc in ws]))
        else:
            layers.append(([f.array(fa.canonical_layout(w)) for w in ws], None))
        if i == 0:
            host0 = ws
    dx, dg = f.array(x), f.array(g)
    oq, ok, ov = f.zeros((1, N)), f.zeros((1, NK)), f.zeros((1, NK))

    def step(i):
        w, sc = layers[i % NL]
        wa = [t.arg(dims=(n, K), dtype=fa.DTYPE_Q4_0) for t, n in zip(w, (N, NK, NK))] if q4 else [t.arg() for t in w]
        f.fused_qkv(dx.arg(), wa[0], wa[1], wa[2], oq.arg(), ok.arg(), ov.arg(), K, N, NK, 1, gamma=dg.arg(),
                    scales=[t.arg() for t in sc] if sc else None)

    step(0)
    f.synchronize()
    if q4:
        want = orc.fused_qkv_q8(x, [w for w, _ in host0], [sc for _, sc in host0], gamma=g, layout=1)
    elif q8:
        want = orc.fused_qkv_q8(x, [w for w, _ in host0], [sc for _, sc in host0], gamma=g)
    else:
        want = orc.fused_qkv(x, *host0, gamma=g)
    err = max(float(np.max(np.abs(o.download().astype(np.float64) - w.astype(np.float64)))) for o, w in zip((oq, ok, ov), want))
    for i in range(args.warmup):
        step(i)
    f.synchronize()
    f.profile_reset()
    f.profile_enable(True)
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    f.synchronize()
    dt = time.perf_counter() - t0
    wbytes = (0.5 + 2.0 / 32) if q4 else (1.0 + 2.0 / 32) if q8 else 2.0  # per weight: nibble / int8 + an f16 scale per 32, or f16
    nbytes = wbytes * (N + 2 * NK) * K + 2 * K * 2 + 2 * (N + 2 * NK)  # weights, input + gamma, outputs
    _finish_secondary(f, args, "FusedQkv layer-steps/s + achieved HBM GB/s, Llama-3.2-3B decode shape",
                      "llama3.2-3b FusedQkv at decode: RMSNorm + Q/K/V projections of one token, k_dim 3072, n_dim 3072, "
                      "n_kv 1024, %s canonical weights, eager launches (profiling events on)" % ("Q4_0" if q4 else "Q8_0" if q8 else "F16"),
                      "fused_qkv_kernel", nbytes, dt, {"qkv_max_abs_err": err})
    f.profile_enable(False)


def bench_fused_qkv_chunk(f, args, m, q8=False):
    """FusedQkv on a prefill chunk of m tokens at Llama-3.2-3B shape (F16 or Q8_0 canonical weights, with RMSNorm): the tiled GEMM
    (norm kernel in front; split-K and a finish kernel when the chunk is short). m = 32 is the reference's default chunk
    - still a weight stream, priced against HBM; m = 2048 is the C4 prompt in one piece, priced against the matrix cores."""
    import orc
    K, N, NK, NL = 3072, 3072, 1024, 8
    rng = np.random.default_rng(0xF0DD + 11)
    x = rng.uniform(-1, 1, (m, K)).astype(np.float16)
    g = rng.uniform(0.5, 1.5, K).astype(np.float16)
    layers, host0 = [], None
    for i in range(NL):
        ws = [rng.uniform(-0.1, 0.1, (n, K)).astype(np.float16) for n in (N, NK, NK)]
        if q8:
            ws = [orc.quantize_q8_0(w) for w in ws]
            layers.append(([f.array(fa.canonical_layout(w)) for w, _ in ws], [f.array(sc) for _, sc in ws]))
        else:
            layers.append(([f.array(fa.canonical_layout(w)) for w in ws], None))
        if i == 0:
            host0 = ws
    dx, dg = f.array(x), f.array(g)
    oq, ok, ov = f.zeros((m, N)), f.zeros((m, NK)), f.zeros((m, NK))

    def step(i):
        w, sc = layers[i % NL]
        f.fused_qkv(dx.arg(), w[0].arg(), w[1].arg(), w[2].arg(), oq.arg(), ok.arg(), ov.arg(), K, N, NK, m, gamma=dg.arg(),
                    scales=[t.arg() for t in sc] if sc else None)

    step(0)
    f.synchronize()
    rows = min(m, 64)  # the oracle on the first rows (seconds of CPU time at most)
    if q8:  # the GEMM's arithmetic for block-quantised weights: f16(q * scale), then the F16 product
        want = orc.fused_qkv(x[:rows], *[orc.dequantize_blocks(w, sc) for w, sc in host0], gamma=g)
    else:
        want = orc.fused_qkv(x[:rows], *host0, gamma=g)
    err = max(float(np.max(np.abs(o.download()[:rows].astype(np.float64) - w.astype(np.float64)))) for o, w in zip((oq, ok, ov), want))
    for i in range(args.warmup):
        step(i)
    f.synchronize()
    f.profile_reset()
    f.profile_enable(True)
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    f.synchronize()
    dt = time.perf_counter() - t0
    kernels = {k: f.profile_query(k) for k in ("fused_qkv_rows32_kernel", "rmsnorm_rows_kernel", "fused_qkv_gemm_kernel", "gemm_finish_kernel")}
    f.profile_enable(False)
    us = {k: (ms * 1e3 / n if n else 0.0) for k, (n, ms) in kernels.items()}
    total_s = sum(us.values()) * 1e-6
    flops = 2.0 * m * (N + 2 * NK) * K
    wbytes = (1.0 + 2.0 / 32) if q8 else 2.0  # per weight: int8 + an f16 scale per 32, or f16
    nbytes = wbytes * (N + 2 * NK) * K + 2.0 * m * K + 2.0 * K + 2.0 * m * (N + 2 * NK)
    if m <= 128:
        roof = {"bound": "hbm", "achieved": nbytes / total_s / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": nbytes / total_s / 1e9 / HBM_PEAK_GBPS, "bytes_per_step": nbytes}
    else:
        roof = {"bound": "mfma", "achieved": flops / total_s / 1e12, "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": flops / total_s / 1e12 / MFMA_F16_PEAK_TFLOPS, "flops_per_step": flops}
    roof.update({"traffic": None, "kernel": " + ".join(k for k, (n, _) in kernels.items() if n) + " (the launches of one step, summed)",
                 "avg_launch_us": us, "launches": max(n for n, _ in kernels.values())})
    emit(({
        "metric": "FusedQkv chunk-steps/s, Llama-3.2-3B prefill chunk of %d tokens" % m, "value": args.steps / dt,
        "unit": "chunk-steps/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "llama3.2-3b FusedQkv on a chunk of %d tokens: RMSNorm + Q/K/V projections, k_dim 3072, n_dim "
                               "3072, n_kv 1024, %s canonical weights, eager launches (profiling events on)"
                               % (m, "Q8_0" if q8 else "F16")},
        "roofline": roof, "parity": {"qkv_max_abs_err_first_rows": err, "rows_checked": rows}}))


def bench_o_proj(f, args, q8=False):
    """The step after the path at Llama-3.2-3B decode shape: attn_out [1, 3072] x W_o^T + hidden (MatMul with residual,
    alpha = beta = 1), F16 weights in the canonical blocked layout, one layer per step over 12 layers' weights."""
    import orc
    K, N, NL = 3072, 3072, 12
    rng = np.random.default_rng(0xF0DD + 8)
    x = rng.uniform(-1, 1, (1, K)).astype(np.float16)
    c = rng.uniform(-1, 1, (1, N)).astype(np.float16)
    layers, host0 = [], None
    for i in range(NL):  # distinct weights so that no launch finds the previous one's in cache
        w = rng.uniform(-0.1, 0.1, (N, K)).astype(np.float16)
        if q8:
            w8, sc = orc.quantize_q8_0(w)
            layers.append((f.array(fa.canonical_layout(w8)), f.array(sc)))
            w = (w8, sc)
        else:
            layers.append((f.array(fa.canonical_layout(w)), None))
        if i == 0:
            host0 = w
    dx, dc, out = f.array(x), f.array(c), f.zeros((1, N))

    def step(i):
        w, sc = layers[i % NL]
        f.matmul(dx.arg(), w.arg(), out.arg(), 1, N, K, c=dc.arg(), transpose_b=False, alpha=1.0, beta=1.0,
                 b_scales=sc.arg() if sc else None)

    step(0)
    f.synchronize()
    want = orc.matmul_gemv_q8(x, host0[0], host0[1], None, c, 0, 32, 1.0, 1.0) if q8 else orc.matmul_gemv(x, host0, None, c, 0, 32, 1.0, 1.0)
    err = float(np.max(np.abs(out.download().astype(np.float64) - want.astype(np.float64))))
    for i in range(args.warmup):
        step(i)
    f.synchronize()
    f.profile_reset()
    f.profile_enable(True)
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    f.synchronize()
    dt = time.perf_counter() - t0
    nbytes = ((1.0 + 2.0 / 32) if q8 else 2.0) * N * K + 2 * K + 2 * 2 * N  # weights, input, residual + output
    _finish_secondary(f, args, "o_proj MatMul layer-steps/s + achieved HBM GB/s, Llama-3.2-3B decode shape",
                      "llama3.2-3b o_proj at decode: attn_out [1, 3072] x W_o^T + hidden, n 3072, k 3072, %s canonical "
                      "weights, eager launches (profiling events on)" % ("Q8_0" if q8 else "F16"), "matmul_gemv_kernel", nbytes,
                      dt, {"max_abs_err": err})
    f.profile_enable(False)


def bench_long_decode(f, args, ctx=131072):
    """Llama-3.2-3B-shaped single-layer decode step at 131072 tokens of context (contiguous cache, 537 MB of K and V
    per layer): the decode kernel where one launch is large. Two layers' caches in rotation (more than the last-level
    cache holds); at ctx = 65536 / 32768 (llama3b_decode_64k / _32k) four / eight."""
    import orc
    H, Hkv, D, pos, NL = 24, 8, 128, ctx - 1, 2 * (131072 // ctx)
    cap = pos + 1 + 128
    rng = np.random.default_rng(0xF0DD + 9)
    cos, sin = fa.rope_tables(5e5, D, cap)
    dcos, dsin = f.array(cos), f.array(sin)
    block = rng.standard_normal((Hkv, 8192, D), dtype=np.float32).astype(np.float16)
    caches, host0 = [], None
    for i in range(NL):
        kc = np.tile(np.roll(block, i, axis=1), (1, (cap + 8191) // 8192, 1))[:, :cap].copy()
        vc = np.tile(np.roll(block, i + 7, axis=1), (1, (cap + 8191) // 8192, 1))[:, :cap].copy()
        caches.append((f.array(kc), f.array(vc)))
        if i == 0:
            host0 = [kc, vc]
    q, k, v = (rng.standard_normal((1, n * D), dtype=np.float32).astype(np.float16) for n in (H, Hkv, Hkv))
    dq, dk, dv, dout = f.array(q), f.array(k), f.array(v), f.zeros((1, H * D))
    p = fa.KvPrepFusedParams.make(H, Hkv, D, 1, pos, cap, fa.ROPE_NORMAL)

    def step(i):
        kc, vc = caches[i % NL]
        f.decode_step_fused(dq.arg(), dk.arg(), dv.arg(), None, kc.arg(), vc.arg(), dcos.arg(), dsin.arg(), dout.arg(), p)

    step(0)
    f.synchronize()
    want_qr = orc.kv_prep_fused(q, k, v, host0[0], host0[1], cos, sin, orc.make_params(H, Hkv, D, 1, pos, cap, rope_mode=1))
    want = orc.sdpa_decode(want_qr[:, 0].copy(), host0[0], host0[1], H, Hkv, D, cap, pos + 1, n_threads=16)
    err = float(np.max(np.abs(dout.download().reshape(-1).astype(np.float64) - want.reshape(-1).astype(np.float64))))
    for i in range(args.warmup):
        step(i)
    f.synchronize()
    f.profile_reset()
    f.profile_enable(True)
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    f.synchronize()
    dt = time.perf_counter() - t0
    nbytes = 2.0 * Hkv * (pos + 1) * D * 2 + 2 * Hkv * D * 2 + 2 * H * D * 2 + 2 * Hkv * D * 2 + 2 * D
    _finish_secondary(f, args, "decode-attn layer-steps/s + achieved HBM GB/s, Llama-3.2-3B shape @%dK ctx" % (ctx // 1024),
                      "llama3.2-3b single-layer decode step at long context: RoPE + KV append + flash decode, batch 1, "
                      "H24/Hkv8/D128, kv_len %d, eager launches (profiling events on)" % ctx, "fused_rope_append_decode_kernel",
                      nbytes, dt, {"decode_max_abs_err": err})
    f.profile_enable(False)


def bench_short_decode(f, args, pos=2047):
    """Llama-3.2-3B-shaped single-layer decode step at a short context (pos + 1 keys): where a launch is mostly its fixed
    cost. Eight layers' caches in rotation, a graph of 32 launches replayed, two events on the stream.
    FOUNDRY_ATTN_DECODE_WAVES=8 forces the 8-wave workgroups that longer contexts use."""
    import orc
    H, Hkv, D, NL = 24, 8, 128, 8
    cap = pos + 1 + 64
    rng = np.random.default_rng(0xF0DD + 15)
    cos, sin = fa.rope_tables(5e5, D, cap)
    dcos, dsin = f.array(cos), f.array(sin)
    host = [(rng.standard_normal((Hkv, cap, D), dtype=np.float32).astype(np.float16),
             rng.standard_normal((Hkv, cap, D), dtype=np.float32).astype(np.float16)) for _ in range(NL)]
    caches = [(f.array(kc), f.array(vc)) for kc, vc in host]
    q, k, v = (rng.standard_normal((1, n * D), dtype=np.float32).astype(np.float16) for n in (H, Hkv, Hkv))
    dq, dk, dv, dout = f.array(q), f.array(k), f.array(v), f.zeros((1, H * D))
    p = fa.KvPrepFusedParams.make(H, Hkv, D, 1, pos, cap, fa.ROPE_NORMAL)

    def step(i):
        kc, vc = caches[i % NL]
        f.decode_step_fused(dq.arg(), dk.arg(), dv.arg(), None, kc.arg(), vc.arg(), dcos.arg(), dsin.arg(), dout.arg(), p)

    step(0)
    f.synchronize()
    want_qr = orc.kv_prep_fused(q, k, v, host[0][0], host[0][1], cos, sin, orc.make_params(H, Hkv, D, 1, pos, cap, rope_mode=1))
    want = orc.sdpa_decode(want_qr[:, 0].copy(), host[0][0], host[0][1], H, Hkv, D, cap, pos + 1, n_threads=8)
    err = float(np.max(np.abs(dout.download().reshape(-1).astype(np.float64) - want.reshape(-1).astype(np.float64))))
    per_graph = 4 * NL
    f.start_capture()
    for i in range(per_graph):
        step(i)
    graph = f.end_capture()
    for _ in range(max(1, args.warmup // per_graph)):
        graph.launch()
    f.synchronize()
    reps = max(1, args.steps // per_graph)
    f.timer_start()
    for _ in range(reps):
        graph.launch()
    per_step = f.timer_stop() / 1e3 / (reps * per_graph)
    graph.destroy()
    nbytes = 2.0 * Hkv * (pos + 1) * D * 2 + 2 * Hkv * D * 2 + 2 * H * D * 2 + 2 * Hkv * D * 2 + 2 * D
    emit({
        "metric": "decode-attn layer-steps/s + achieved HBM GB/s, Llama-3.2-3B shape @%d keys" % (pos + 1),
        "value": 1.0 / per_step, "unit": "layer-steps/s", "n_gpus": 1, "steps": reps * per_graph, "warmup": args.warmup,
        "ms_per_step": per_step * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "llama3.2-3b single-layer decode step at a short context: RoPE + KV append + flash decode, batch 1, "
                               "H24/Hkv8/D128, kv_len %d, graph replays" % (pos + 1)},
        "roofline": {"bound": "hbm", "achieved": nbytes / per_step / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": nbytes / per_step / 1e9 / HBM_PEAK_GBPS, "traffic": None, "kernel": "fused_rope_append_decode_kernel",
                     "avg_launch_us": per_step * 1e6, "bytes_per_launch": nbytes,
                     "timing": "HIP events on the stream around the graph replays / launches in them"},
        "parity": {"decode_max_abs_err": err}})


def bench_attn_block(f, args):
    """The attention block of a Llama-3.2-3B decode step, all 28 layers, as the reference's graph runs it
    (models/llama.json:509-585): FusedQkv (RMSNorm + projections) -> RoPE + KV append + flash decode -> o_proj MatMul
    with residual; F16 weights in the canonical layout, 8192 keys of context, one HIP graph of the 28 layers per step.
    The MLP between the blocks is not part of this path; each layer's block reads the previous one's residual."""
    L, H, Hkv, D, pos = 28, 24, 8, 128, 8192
    dm, kvd, cap = H * D, Hkv * D, 8448
    rng = np.random.default_rng(0xF0DD + 10)
    cos, sin = fa.rope_tables(5e5, D, cap)
    dcos, dsin = f.array(cos), f.array(sin)
    base_kv = rng.standard_normal((Hkv, cap, D), dtype=np.float32).astype(np.float16)
    wq = fa.canonical_layout(rng.uniform(-0.05, 0.05, (dm, dm)).astype(np.float16))
    wk = fa.canonical_layout(rng.uniform(-0.05, 0.05, (kvd, dm)).astype(np.float16))
    layers = []
    for i in range(L):  # distinct device buffers per layer (contents rolled copies: only the addresses matter for timing)
        layers.append(dict(kc=f.array(np.roll(base_kv, i, axis=1)), vc=f.array(np.roll(base_kv, i + 3, axis=1)),
                           wq=f.array(np.roll(wq, i)), wk=f.array(np.roll(wk, i)), wv=f.array(np.roll(wk, i + 5)),
                           wo=f.array(np.roll(wq, i + 9)), g=f.array(rng.uniform(0.5, 1.5, dm).astype(np.float16))))
    hid = [f.array(rng.uniform(-1, 1, (1, dm)).astype(np.float16)), f.zeros((1, dm))]
    dq, dk, dv, dattn = f.zeros((1, dm)), f.zeros((1, kvd)), f.zeros((1, kvd)), f.zeros((1, dm))
    dpos = f.array(np.array([pos], np.uint32))
    p = fa.KvPrepFusedParams.make(H, Hkv, D, 1, 0, cap, fa.ROPE_NORMAL)

    def enqueue():
        for i, ly in enumerate(layers):
            src, dst = hid[i % 2], hid[(i + 1) % 2]
            f.fused_qkv(src.arg(), ly["wq"].arg(), ly["wk"].arg(), ly["wv"].arg(), dq.arg(), dk.arg(), dv.arg(), dm, dm, kvd, 1,
                        gamma=ly["g"].arg())
            f.decode_step_fused(dq.arg(), dk.arg(), dv.arg(), None, ly["kc"].arg(), ly["vc"].arg(), dcos.arg(), dsin.arg(),
                                dattn.arg(), p, d_position=dpos, kv_len_bound=cap)
            f.matmul(dattn.arg(), ly["wo"].arg(), dst.arg(), 1, dm, dm, c=src.arg(), transpose_b=False, alpha=1.0, beta=1.0)

    f.start_capture()
    enqueue()
    graph = f.end_capture()
    for _ in range(args.warmup):
        graph.launch()
    f.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        graph.launch()
    f.synchronize()
    dt = time.perf_counter() - t0
    finite = bool(np.all(np.isfinite(hid[0].download())))
    nbytes = L * (2.0 * (dm + 2 * kvd) * dm + 2.0 * dm * dm + 2.0 * 2 * Hkv * (pos + 1) * D)
    per_step = dt / args.steps
    emit(({
        "metric": "attention-block steps/s + achieved HBM GB/s, Llama-3.2-3B decode @8K ctx", "value": 1.0 / per_step,
        "unit": "steps/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": per_step * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "llama3.2-3b attention block x 28 layers per step: FusedQkv, fused RoPE + append + decode "
                               "(+ merge), o_proj with residual; one HIP graph per step"},
        "roofline": {"bound": "hbm", "achieved": nbytes / per_step / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": nbytes / per_step / 1e9 / HBM_PEAK_GBPS, "traffic": None, "kernel": "whole step (4 kernels per layer)",
                     "bytes_per_step": nbytes, "us_per_layer": per_step * 1e6 / L},
        "parity": {"outputs_finite": finite, "note": "stage-by-stage parity of this chain: tests/test_gpu_block.py"}}))


def bench_chunk_block(f, args, m=32, prefix=8160):
    """The attention block of the reference's default prefill mode: a chunk of m = 32 rows (src/model/executor.rs:232-250)
    after `prefix` cached tokens goes through all 28 layers of a Llama-3.2-3B-shaped model - FusedQkv + KvPrepFused (one
    op: RMSNorm, projections, RoPE, append of the chunk's rows), causal FlashAttention of the chunk against the prefix and
    itself, o_proj MatMul with residual - as ONE HIP graph per step; F16 canonical weights, distinct buffers per layer.
    The MLP between the blocks is not part of this path. HBM-bound: a layer reads its weights and the prefix once."""
    L, H, Hkv, D = 28, 24, 8, 128
    dm, kvd = H * D, Hkv * D
    N, cap = prefix + m, prefix + 512
    rng = np.random.default_rng(0xF0DD + 16)
    cos, sin = fa.rope_tables(5e5, D, cap)
    dcos, dsin = f.array(cos), f.array(sin)
    base_kv = rng.standard_normal((Hkv, cap, D), dtype=np.float32).astype(np.float16)
    wq = fa.canonical_layout(rng.uniform(-0.05, 0.05, (dm, dm)).astype(np.float16))
    wk = fa.canonical_layout(rng.uniform(-0.05, 0.05, (kvd, dm)).astype(np.float16))
    layers = []
    for i in range(L):  # distinct device buffers per layer (contents rolled copies: only the addresses matter for timing)
        layers.append(dict(kc=f.array(np.roll(base_kv, i, axis=1)), vc=f.array(np.roll(base_kv, i + 3, axis=1)),
                           wq=f.array(np.roll(wq, i)), wk=f.array(np.roll(wk, i)), wv=f.array(np.roll(wk, i + 5)),
                           wo=f.array(np.roll(wq, i + 9)), g=f.array(rng.uniform(0.5, 1.5, dm).astype(np.float16))))
    hid = [f.array(rng.uniform(-1, 1, (m, dm)).astype(np.float16)), f.zeros((m, dm))]
    dqr, dattn = f.zeros((H, m, D)), f.zeros((m, dm))
    p = fa.KvPrepFusedParams.make(H, Hkv, D, m, prefix, cap, fa.ROPE_NORMAL)

    def enqueue():
        for i, ly in enumerate(layers):
            src, dst = hid[i % 2], hid[(i + 1) % 2]
            f.fused_qkv_kv_prep(src.arg(), ly["wq"].arg(), ly["wk"].arg(), ly["wv"].arg(), dm, dqr.arg(), dcos.arg(), dsin.arg(), p,
                                k_cache=ly["kc"].arg(), v_cache=ly["vc"].arg(), gamma=ly["g"].arg())
            f.flash_attention(dqr.arg(), ly["kc"].arg(), ly["vc"].arg(), dattn.arg(), True, prefix, H, D, N, m)
            f.matmul(dattn.arg(), ly["wo"].arg(), dst.arg(), m, dm, dm, c=src.arg(), transpose_b=False, alpha=1.0, beta=1.0)

    enqueue()  # (workspaces reach their size before the capture)
    f.synchronize()
    f.start_capture()
    enqueue()
    graph = f.end_capture()
    for _ in range(max(args.warmup, 1)):
        graph.launch()
    f.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        graph.launch()
    f.synchronize()
    dt = time.perf_counter() - t0
    graph.destroy()
    finite = bool(np.all(np.isfinite(hid[0].download())))
    nbytes = L * (2.0 * (dm + 2 * kvd) * dm + 2.0 * dm * dm + 2.0 * 2 * Hkv * N * D + 4.0 * 2 * m * dm)
    per_step = dt / args.steps
    emit(({
        "metric": "prefill-chunk attention-block steps/s + achieved HBM GB/s, Llama-3.2-3B, %d rows after %d tokens" % (m, prefix),
        "value": 1.0 / per_step, "unit": "steps/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": per_step * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "llama3.2-3b attention block x 28 layers per step on a prefill chunk of %d rows after %d tokens: "
                               "FusedQkv + KvPrepFused (one op), causal FlashAttention, o_proj with residual; one HIP graph per step"
                               % (m, prefix)},
        "roofline": {"bound": "hbm", "achieved": nbytes / per_step / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": nbytes / per_step / 1e9 / HBM_PEAK_GBPS, "traffic": None, "kernel": "whole step (the launches of 28 layers)",
                     "bytes_per_step": nbytes, "us_per_layer": per_step * 1e6 / L},
        "parity": {"outputs_finite": finite, "note": "stage-by-stage parity of these ops: tests/test_gpu_qkv_kv_prep.py, tests/test_gpu_prefill.py, tests/test_gpu_qkv.py"}}))


def bench_prefill_chunk(f, args, m=32, prefix=8160):
    """One prefill chunk of m rows (32 = the reference's default chunk, src/model/executor.rs:232-250) attending a contiguous
    Llama-3.2-3B-shaped cache that already holds `prefix` tokens: the short-chunk kernel (partitions merged inside the
    launch) or, under another prefill variant, the split-K prefill kernel + its merge kernel; timed as graph replays over
    as many layers' caches in rotation as take about 1 GB (28 at 8K tokens), so that no replay finds its rows in a cache.
    HBM-bound: every launch reads the whole prefix once."""
    H, Hkv, D = 24, 8, 128
    N, cap = prefix + m, prefix + 512
    L = max(4, min(28, int(np.ceil(0.94e9 / (2.0 * Hkv * N * D * 2)))))
    rng = np.random.default_rng(0xF0DD + 14)
    k0 = rng.standard_normal((Hkv, cap, D), dtype=np.float32).astype(np.float16)
    v0 = rng.standard_normal((Hkv, cap, D), dtype=np.float32).astype(np.float16)
    caches = [(f.array(k0), f.array(v0)) for _ in range(L)]  # (the same rows in every layer's buffers)
    q = rng.standard_normal((H, m, D), dtype=np.float32).astype(np.float16)
    dq, dout = f.array(q), f.zeros((m, H * D))

    def step(i):
        kc, vc = caches[i % L]
        f.flash_attention(dq.arg(), kc.arg(), vc.arg(), dout.arg(), True, prefix, H, D, N, m)

    step(0)
    f.synchronize()
    import orc  # the CPU oracle is only the checker here
    want = orc.sdpa_prefill(q, caches[0][0].download(), caches[0][1].download(), H, Hkv, D, m, N, prefix, cap, causal=True,
                            out_layout="head_major", n_threads=max(1, min(16, os.cpu_count() or 1, orc.lib().orc_max_threads())))
    got = dout.download().reshape(m, H, D).transpose(1, 0, 2)
    err = float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64))))
    per_graph = 2 * L
    f.start_capture()
    for i in range(per_graph):
        step(i)
    graph = f.end_capture()
    for _ in range(max(1, args.warmup // per_graph)):
        graph.launch()
    f.synchronize()
    reps = max(1, args.steps // per_graph)
    f.timer_start()
    for _ in range(reps):
        graph.launch()
    per_step = f.timer_stop() / 1e3 / (reps * per_graph)
    graph.destroy()
    f.profile_reset()
    f.profile_enable(True)
    for i in range(per_graph):
        step(i)
    us = {}
    for kname in ("flash_chunk_kernel", "flash_prefill_dma_kernel", "flash_prefill_mfma_kernel", "flash_prefill_merge_kernel"):
        n, ms = f.profile_query(kname)
        if n:
            us[kname] = ms * 1e3 / n
    f.profile_enable(False)
    nbytes = 2.0 * Hkv * N * D * 2 + 2.0 * H * m * D * 2  # K and V once per KV head, q in, out
    emit({
        "metric": "prefill-chunk steps/s + achieved HBM GB/s, Llama-3.2-3B shape, %d rows after %d tokens" % (m, prefix),
        "value": 1.0 / per_step, "unit": "steps/s", "n_gpus": 1, "steps": reps * per_graph, "warmup": args.warmup,
        "ms_per_step": per_step * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "llama3.2-3b prefill chunk of %d rows after a %d-token prefix, one layer per step: causal attention "
                               "split over the keys, merge %s, contiguous cache, %d layers' caches in rotation, graph replays"
                               % (m, prefix, "inside the launch" if "flash_chunk_kernel" in us else "as a second launch", L)},
        "roofline": {"bound": "hbm", "achieved": nbytes / per_step / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": nbytes / per_step / 1e9 / HBM_PEAK_GBPS, "traffic": None,
                     "kernel": "flash_chunk_kernel" if "flash_chunk_kernel" in us else "prefill kernel + merge kernel (one step)",
                     "avg_launch_us": us, "bytes_per_step": nbytes,
                     "timing": "HIP events on the stream around the graph replays / steps in them"},
        "parity": {"max_abs_err_vs_oracle": err}})


def bench_phase_timeline(f, args, which="decode_8k"):
    """Where a launch's time goes, from clock stamps the kernels take themselves: only a development build of the
    library has them (python test-burn_amd/build.py with FOUNDRY_ATTN_BUILD_TAG=_trace and
    FOUNDRY_ATTN_BUILD_FLAGS=-DFA_DECODE_TRACE in the environment builds libfoundry_attn_trace.so beside the product library;
    FOUNDRY_ATTN_LIB selects it). Every wave stamps the 100 MHz wall clock at the kernel's phase boundaries and leaves the
    stamps in the clock buffer; the workload is replayed as a HIP graph and the phases are reported in microseconds after
    the first workgroup's entry, as min / median / 90th percentile / max over the waves that reached them.
    which: decode_8k (the fused decode step of the main configuration), decode_1k (the same step in its 4-wave form:
    Qwen2.5-0.5B shape at 1K context, a launch that is all latency), sage_32k (the int8 step, wave 0 of every workgroup
    = the wave that prepares the query and owns the open block), chunk32_8k (the short-chunk prefill kernel)."""
    rng = np.random.default_rng(0xF0DD + 21)
    if which == "decode_8k":
        st = make_llama3b_decode(f, rng, 8192, 64)
        per_graph, waves, rows = 2 * 28, 8, 256 * 8
        names = ["entry", "start barrier released", "block requests issued", "query operand ready", "first round: S done",
                 "first round: V in LDS", "block loop done", "state in LDS", "fold starts", "records stored", "merge done"]

    elif which == "decode_1k":
        H, Hkv, D, pos, cap, NL = 14, 2, 64, 1024, 1152, 16
        cos, sin = fa.rope_tables(1e6, D, cap)
        dcos, dsin = f.array(cos), f.array(sin)
        caches = []
        for i in range(NL):
            kc, vc = np.zeros((Hkv, cap, D), np.float16), np.zeros((Hkv, cap, D), np.float16)
            kc[:, :pos] = rng.standard_normal((Hkv, pos, D), dtype=np.float32).astype(np.float16)
            vc[:, :pos] = rng.standard_normal((Hkv, pos, D), dtype=np.float32).astype(np.float16)
            caches.append((f.array(kc), f.array(vc)))
        q, k, v = (rng.standard_normal((1, n * D), dtype=np.float32).astype(np.float16) for n in (H, Hkv, Hkv))
        dq, dk, dv, dqr, dout = f.array(q), f.array(k), f.array(v), f.zeros((H, 1, D)), f.zeros((1, H * D))
        p1k = fa.KvPrepFusedParams.make(H, Hkv, D, 1, pos, cap, fa.ROPE_NEOX)
        per_graph, waves, rows = 2 * NL, 4, 512 * 4
        names = ["entry", "start barrier released", "block requests issued", "query operand ready", "first round: S done",
                 "first round: V in LDS", "block loop done", "state in LDS", "fold starts", "records stored", "merge done"]

        def step(i):
            kc, vc = caches[i % NL]
            f.decode_step_fused(dq.arg(), dk.arg(), dv.arg(), dqr.arg(), kc.arg(), vc.arg(), dcos.arg(), dsin.arg(), dout.arg(), p1k)
    elif which == "sage_32k":
        H, Hkv, D, N, NL = 16, 4, 128, 32768, 6
        P = N - 1
        cos, sin = fa.rope_tables(5e6, D, N)
        dcos, dsin = f.array(cos), f.array(sin)
        k = rng.standard_normal((Hkv, N, D), dtype=np.float32).astype(np.float16)
        v = rng.standard_normal((Hkv, N, D), dtype=np.float32).astype(np.float16)
        k[:, P:], v[:, P:] = 0, 0
        layers = []
        for _ in range(NL):
            dk, dv = f.array(k), f.array(v)
            desc, bufs = fa.sage_cache(f, H, Hkv, N, D, dv)
            f.sage_cache_build(dk, P, desc)
            f.synchronize()
            dk.free()
            layers.append((desc, bufs))
        q, kn, vn = (rng.standard_normal((1, n * D), dtype=np.float32).astype(np.float16) for n in (H, Hkv, Hkv))
        dq, dkn, dvn, dout = f.array(q), f.array(kn), f.array(vn), f.zeros((H * D,))
        params = [fa.KvPrepFusedParams.make(H, Hkv, D, 1, P, N, fa.ROPE_NEOX, layer_idx=i, no_rope_layer_step=4) for i in range(NL)]
        per_graph, waves, rows = 2 * NL, 8, 256 * 8
        names = ["entry", "start barrier released", "block requests issued", "query operand ready", "first round: S done",
                 "first round: V in LDS", "block loop done", "state in LDS", "fold starts", "records stored", "merge done",
                 "wave 0: table row and mean in LDS", "wave 0: open block's scale known", "wave 0: open block quantised",
                 "wave 0: open block attended"]

        def step(i):
            f.sage_decode_step(dq.arg(), dkn.arg(), dvn.arg(), layers[i % NL][0], dcos.arg(), dsin.arg(), dout.arg(), params[i % NL])
    else:
        H, Hkv, D, L, m, prefix = 24, 8, 128, 28, 32, 8160
        N, cap = prefix + m, prefix + 512
        k0 = rng.standard_normal((Hkv, cap, D), dtype=np.float32).astype(np.float16)
        v0 = rng.standard_normal((Hkv, cap, D), dtype=np.float32).astype(np.float16)
        caches = [(f.array(k0), f.array(v0)) for _ in range(L)]
        dq, dout = f.array(rng.standard_normal((H, m, D), dtype=np.float32).astype(np.float16)), f.zeros((m, H * D))
        per_graph, waves, rows = L, 8, 256 * 8
        names = ["entry", "query rows requested", None, "round 0 in LDS (seen by this wave)", "last tile attended", "after the barrier",
                 "key halves folded", "state stored", "merge starts", "rows written", "all (m, l) of the first batch seen",
                 "sums of the first pass folded", "producer 0: entry", "producer 0: in its branch", "producer 0: round 0 requested",
                 "producer 0: round 0 landed"]

        def step(i):
            kc, vc = caches[i % L]
            f.flash_attention(dq.arg(), kc.arg(), vc.arg(), dout.arg(), True, prefix, H, D, N, m)
    if which == "decode_8k":
        def run(n):  # (the decode bench's own step: 28 layers per call)
            for s_ in range(n // 28):
                enqueue_step(f, st, s_, True)
    else:
        def run(n):
            for i in range(n):
                step(i)
    run(per_graph)
    f.synchronize()
    buf = fa.DevBuf(f, (rows * 16,), np.uint64)
    buf.upload(np.zeros((rows * 16,), np.uint64))
    f.profile_clock_buffer(buf, rows * 8)
    f.start_capture()
    run(per_graph)
    graph = f.end_capture()
    phases, span = {}, None
    for rep in range(4):
        graph.launch()
        f.synchronize()
    t = buf.download().reshape(rows, 16).astype(np.float64)  # the last launch of the last replay
    f.profile_clock_buffer(None, 0)
    graph.destroy()
    live = t[:, 0] > 0
    if not live.any():
        sys.exit("no stamps in the clock buffer: this library was built without -DFA_DECODE_TRACE (see the workload's description)")
    t0 = t[live, 0].min()
    for i, nm in enumerate(names):
        if nm is None:
            continue
        col = t[:, i][t[:, i] > 0]
        if col.size:
            us = (col - t0) / 100.0
            phases[nm] = {"waves": int(col.size), "min": round(float(us.min()), 2), "p50": round(float(np.median(us)), 2),
                          "p90": round(float(np.percentile(us, 90)), 2), "max": round(float(us.max()), 2)}
    emit({"metric": "phase timeline of one launch, us after the first workgroup's entry (%s)" % which, "value": max(p["max"] for p in phases.values()),
          "unit": "us", "n_gpus": 1, "steps": per_graph, "warmup": per_graph, "ms_per_step": None, "higher_is_better": False,
          "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
          "config": {"workload": "clock stamps inside the kernel, development build of the library; graph replays, the stamps of "
                                 "the last launch of the last replay"},
          "phases": phases})


def bench_prefill_block(f, args, fused=False):
    """The attention block of one Llama-3.2-3B layer on a 2048-token prompt in one chunk (models/llama.json:509-585):
    FusedQkv (norm kernel + GEMM) -> KvPrepFused (RoPE + append of 2048 rows) -> FlashAttention (causal prefill) -> o_proj
    MatMul with residual (GEMM); F16 canonical weights, contiguous cache, eager launches, 4 layers' buffers in rotation.
    fused: the first two as one op (fa_fused_qkv_kv_prep: KvPrepFused is the GEMM's write stage)."""
    L, H, Hkv, D, M = 4, 24, 8, 128, 2048
    dm, kvd, cap = H * D, Hkv * D, 2048
    rng = np.random.default_rng(0xF0DD + 12)
    cos, sin = fa.rope_tables(5e5, D, cap)
    dcos, dsin = f.array(cos), f.array(sin)
    wq = fa.canonical_layout(rng.uniform(-0.05, 0.05, (dm, dm)).astype(np.float16))
    wk = fa.canonical_layout(rng.uniform(-0.05, 0.05, (kvd, dm)).astype(np.float16))
    layers = []
    for i in range(L):
        layers.append(dict(kc=f.zeros((Hkv, cap, D)), vc=f.zeros((Hkv, cap, D)), wq=f.array(np.roll(wq, i)),
                           wk=f.array(np.roll(wk, i)), wv=f.array(np.roll(wk, i + 5)), wo=f.array(np.roll(wq, i + 9)),
                           g=f.array(rng.uniform(0.5, 1.5, dm).astype(np.float16))))
    hid = f.array(rng.uniform(-1, 1, (M, dm)).astype(np.float16))
    dq, dk, dv = f.zeros((M, dm)), f.zeros((M, kvd)), f.zeros((M, kvd))
    dqr, dattn, dout = f.zeros((H, M, D)), f.zeros((M, dm)), f.zeros((M, dm))
    p = fa.KvPrepFusedParams.make(H, Hkv, D, M, 0, cap, fa.ROPE_NORMAL)

    def step(i):
        ly = layers[i % L]
        if fused:
            f.fused_qkv_kv_prep(hid.arg(), ly["wq"].arg(), ly["wk"].arg(), ly["wv"].arg(), dm, dqr.arg(), dcos.arg(), dsin.arg(), p,
                                k_cache=ly["kc"].arg(), v_cache=ly["vc"].arg(), gamma=ly["g"].arg())
        else:
            f.fused_qkv(hid.arg(), ly["wq"].arg(), ly["wk"].arg(), ly["wv"].arg(), dq.arg(), dk.arg(), dv.arg(), dm, dm, kvd, M,
                        gamma=ly["g"].arg())
            f.kv_prep_fused(dq.arg(), dk.arg(), dv.arg(), dqr.arg(), ly["kc"].arg(), ly["vc"].arg(), dcos.arg(), dsin.arg(), p)
        f.flash_attention(dqr.arg(), ly["kc"].arg(), ly["vc"].arg(), dattn.arg(), True, 0, H, D, M, M)
        f.matmul(dattn.arg(), ly["wo"].arg(), dout.arg(), M, dm, dm, c=hid.arg(), transpose_b=False, alpha=1.0, beta=1.0)

    for i in range(max(args.warmup, 1)):
        step(i)
    f.synchronize()
    f.profile_reset()
    f.profile_enable(True)
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    f.synchronize()
    dt = time.perf_counter() - t0
    names = ("rmsnorm_rows_kernel", "fused_qkv_gemm_kernel", "kv_prep_fused", "flash_prefill_dma_kernel",
             "flash_prefill_mfma_kernel", "matmul_gemm_kernel")
    us = {}
    for k in names:
        n, ms = f.profile_query(k)
        if n:
            us[k] = ms * 1e3 / n
    f.profile_enable(False)
    finite = bool(np.all(np.isfinite(dout.download())))
    flops = 2.0 * M * (dm + 2 * kvd) * dm + 4.0 * D * H * M * (M + 1) / 2 + 2.0 * M * dm * dm
    total_s = sum(us.values()) * 1e-6
    emit(({
        "metric": "attention-block layer-steps/s, Llama-3.2-3B prefill of 2048 tokens", "value": args.steps / dt,
        "unit": "layer-steps/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "llama3.2-3b attention block on a 2048-token prompt, one layer per step: "
                               + ("FusedQkv with KvPrepFused as its write stage (one op), " if fused else "FusedQkv, KvPrepFused, ")
                               + "causal FlashAttention, o_proj with residual; eager launches (profiling events on)"},
        "roofline": {"bound": "mfma", "achieved": flops / total_s / 1e12, "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": flops / total_s / 1e12 / MFMA_F16_PEAK_TFLOPS, "traffic": None, "kernel": "sum of the block's kernels",
                     "avg_launch_us": us, "flops_per_step": flops},
        "parity": {"outputs_finite": finite, "note": "stage-by-stage parity of this chain: tests/test_gpu_block.py"}}))


def bench_paged_decode(f, args):
    """Qwen2.5-3B-shaped batched paged decode, one layer per step: 32 ragged sequences, 16-token blocks."""
    import orc
    H, Hkv, D, bs, B, NL = 16, 2, 128, 16, 32, 4
    rng = np.random.default_rng(0xF0DD + 3)
    lens = rng.integers(512, 16385, size=B).astype(np.uint32)
    need = [(int(n) + 1 + bs - 1) // bs for n in lens]
    mb, nblk = max(need), sum(need) + 3
    cos, sin = fa.rope_tables(1e6, D, 16400)
    dcos, dsin = f.array(cos), f.array(sin)
    layers, host0 = [], None
    for i in range(NL):  # distinct pools, each larger than the last-level cache
        perm = rng.permutation(nblk).astype(np.int32)
        bt = np.zeros((B, mb), np.int32)
        o = 0
        for s_, n in enumerate(need):
            bt[s_, :n] = perm[o:o + n]
            o += n
        kp = rng.standard_normal((nblk, Hkv, bs, D), dtype=np.float32).astype(np.float16)
        vp = rng.standard_normal((nblk, Hkv, bs, D), dtype=np.float32).astype(np.float16)
        dkp, dvp, dbt, dl = f.array(kp), f.array(vp), f.array(bt), f.array(lens)
        layers.append((dkp, dvp, dbt, dl, fa.paged_kv(dkp, dvp, dbt, dl, nblk, Hkv, bs, D, B, mb)))
        if i == 0:
            host0 = (kp, vp, bt)
    q, k, v = (rng.standard_normal((B, n * D), dtype=np.float32).astype(np.float16) for n in (H, Hkv, Hkv))
    dq, dk, dv, dqr, dout = f.array(q), f.array(k), f.array(v), f.zeros((B, H, D)), f.zeros((B, H * D))
    p = fa.KvPrepFusedParams.make(H, Hkv, D, B, 0, 0, fa.ROPE_NEOX)

    def step(i):
        f.decode_step_fused_paged(dq.arg(), dk.arg(), dv.arg(), dqr.arg(), layers[i % NL][4], dcos.arg(), dsin.arg(),
                                  dout.arg(), p, 16400)

    step(0)
    f.synchronize()
    got = dout.download().reshape(B, H, D)
    err = 0.0
    for b_ in (0, int(np.argmin(lens)), int(np.argmax(lens))):  # three sequences against the oracle
        n = int(lens[b_])
        kc = orc.paged_gather(host0[0], host0[2][b_], Hkv, bs, D, n, n + 1)
        vc = orc.paged_gather(host0[1], host0[2][b_], Hkv, bs, D, n, n + 1)
        qr = orc.kv_prep_fused(q[b_:b_ + 1], k[b_:b_ + 1], v[b_:b_ + 1], kc, vc, cos, sin,
                               orc.make_params(H, Hkv, D, 1, n, n + 1, rope_mode=0))
        want = orc.sdpa_decode(qr[:, 0].copy(), kc, vc, H, Hkv, D, n + 1, n + 1, n_threads=8).reshape(H, D)
        err = max(err, float(np.max(np.abs(got[b_].astype(np.float64) - want.astype(np.float64)))))
    graph = graph_replay_seconds(f, step, 4 * NL, args.warmup, args.steps)
    f.profile_reset()
    f.profile_enable(True)
    for i in range(4 * NL):
        step(i)
    n_mrg, ms_mrg = f.profile_query("flash_decode_merge_kernel")
    total = float(np.sum(lens.astype(np.float64) + 1))
    nbytes = 2.0 * Hkv * total * D * 2 + B * (2 * Hkv * D * 2 + 2 * H * D * 2 + 2 * D + 4) + 4.0 * sum(need)
    _finish_secondary(f, args, "paged decode-attn layer-steps/s + achieved HBM GB/s, Qwen2.5-3B shape, 32 ragged sequences",
                      "qwen2.5-3b batched paged decode, one layer per step: 32 sequences of %d..%d tokens (sum %d), "
                      "H16/Hkv2/D128, 16-token blocks with a permuted block table, RoPE + append + flash decode in one "
                      "launch%s, graph replays over 4 layers' pools" % (int(lens.min()), int(lens.max()), int(lens.sum()),
                                                                       " + merge launch" if n_mrg else ", merge inside"),
                      "fused_rope_append_decode_kernel", nbytes, 0.0, {"decode_max_abs_err_3_sequences": err},
                      {"kernels_per_step": 2 if n_mrg else 1,
                       "merge_kernel_avg_launch_us": (ms_mrg * 1e3 / n_mrg) if n_mrg else None}, graph=graph)
    f.profile_enable(False)


def bench_sage_decode(f, args):
    """SmolLM3-shaped decode step with int8 Q/K (per-32-token scales, mean-smoothed K) at 32K context, one layer per
    step: RoPE + append of the new token into the int8 cache (open block quantised anew) + int8 decode. Every 4th layer
    skips RoPE (the model's rule); six layers' states in rotation."""
    import orc
    H, Hkv, D, N, NL = 16, 4, 128, 32768, 6
    P = N - 1  # the new token's position
    rng = np.random.default_rng(0xF0DD + 5)

    def outliers(shape):
        x = rng.standard_normal(shape, dtype=np.float32)
        mask = rng.random(shape) < 0.01
        x[mask] = np.sign(x[mask]) * 8.0
        return x.astype(np.float16)

    cos, sin = fa.rope_tables(5e6, D, N)
    dcos, dsin = f.array(cos), f.array(sin)
    layers, host0 = [], None
    for i in range(NL):
        k, v = outliers((Hkv, N, D)), outliers((Hkv, N, D))
        k[:, P:], v[:, P:] = 0, 0
        dk, dv = f.array(k), f.array(v)
        desc, bufs = fa.sage_cache(f, H, Hkv, N, D, dv)
        f.sage_cache_build(dk, P, desc)
        f.synchronize()
        dk.free()
        layers.append((desc, bufs))
        if i == 0:
            host0 = (k, v)
    q, kn, vn = outliers((1, H * D)), outliers((1, Hkv * D)), outliers((1, Hkv * D))
    dq, dkn, dvn, dout = f.array(q), f.array(kn), f.array(vn), f.zeros((H * D,))
    params = [fa.KvPrepFusedParams.make(H, Hkv, D, 1, P, N, fa.ROPE_NEOX, layer_idx=i, no_rope_layer_step=4) for i in range(NL)]

    def step(i):
        f.sage_decode_step(dq.arg(), dkn.arg(), dvn.arg(), layers[i % NL][0], dcos.arg(), dsin.arg(), dout.arg(), params[i % NL])

    step(0)
    f.synchronize()
    got = dout.download().reshape(H, D).astype(np.float64)
    # the checker: the oracle's f16 append, its quantiser with the state's mean, its int8 decode model
    kc, vc = host0[0].copy(), host0[1].copy()
    qr = orc.kv_prep_fused(q, kn, vn, kc, vc, cos, sin, orc.make_params(H, Hkv, D, 1, P, N, rope_mode=0, layer_idx=0, no_rope_layer_step=4))
    mean = layers[0][1]["k_mean"].download()
    want_kq, want_ks = orc.sage_quantize_k(kc, mean, Hkv, N, D, N)
    state_ok = bool(np.array_equal(layers[0][1]["k_q"].download(), want_kq) and
                    np.array_equal(layers[0][1]["k_scale"].download().view(np.uint16), want_ks.view(np.uint16)))
    qq, qs = orc.sage_quantize_q(np.ascontiguousarray(qr[:, 0]), H, D)
    model = orc.sage_decode(qq, qs, want_kq, want_ks, vc, H, Hkv, D, N, N, n_threads=8).reshape(H, D).astype(np.float64)
    err_model = float(np.max(np.abs(got - model)))
    kf, vf, qf = kc.astype(np.float64), vc.astype(np.float64), qr[:, 0].astype(np.float64)
    full = np.zeros((H, D))
    for h in range(H):  # f16 SDPA on the unquantised tensors, in float64
        s_ = kf[h // (H // Hkv)] @ qf[h] / np.sqrt(D)
        w = np.exp(s_ - s_.max())
        full[h] = (w / w.sum()) @ vf[h // (H // Hkv)]
    err_full = float(np.max(np.abs(got - full)))
    # timed as HIP-graph replays (short launches: eager, the host's call overhead would be what is measured)
    per_graph = 4 * NL
    f.start_capture()
    for i in range(per_graph):
        step(i)
    graph = f.end_capture()
    for _ in range(max(1, args.warmup // per_graph)):
        graph.launch()
    f.synchronize()
    reps = max(1, args.steps // per_graph)
    t0 = time.perf_counter()
    for _ in range(reps):
        graph.launch()
    f.synchronize()
    dt = (time.perf_counter() - t0) * args.steps / (reps * per_graph)  # scaled to args.steps steps
    graph.destroy()
    # per-kernel times: an eager pass with events attached to the dispatches
    f.profile_reset()
    f.profile_enable(True)
    for i in range(per_graph):
        step(i)
    n_ap, ms_ap = f.profile_query("sage_append_kernel")
    one_launch = n_ap == 0  # the default: append and attention in one kernel (FOUNDRY_ATTN_SAGE_FUSED=0: two)
    nbytes = float(Hkv * N * D + Hkv * (N // 32) * 2 + Hkv * N * D * 2 + 2 * H * D * 2)
    _finish_secondary(f, args, "int8-QK decode-attn layer-steps/s + achieved HBM GB/s, SmolLM3 shape @32K ctx",
                      "smollm3 decode step with int8 Q/K (K mean-smoothed with a fixed mean, per-32-token f16 scales; f16 V), one "
                      "layer per step: RoPE (every 4th layer none) + append into the int8 cache + int8 decode, batch 1, "
                      "H16/Hkv4/D128, kv_len 32768, 1% of entries at 8 sigma" + (", one launch per step" if one_launch else ", two launches per step"),
                      "sage_fused_append_decode_kernel" if one_launch else "sage_decode_mfma_kernel",
                      nbytes, dt, {"int8_state_bit_exact": state_ok, "max_abs_err_vs_int8_cpu_model": err_model,
                                   "max_abs_err_vs_f16_sdpa_unquantised": err_full},
                      {"dtype": "i8 (QK^T) / f16 (PV)",
                       "append": None if one_launch else {"kernel": "sage_append_kernel", "avg_launch_us": ms_ap * 1e3 / max(1, n_ap)}})
    f.profile_enable(False)


def bench_floors(f, args):
    """What a launch of this size costs with the library's simplest kernels, for reading the decode figures against: an
    (almost) empty launch, and plain copies that move as many bytes as one decode launch reads (Llama-3.2-3B layer at
    8K: 33.6 MB) and as the paged batch's launch reads (240 MB). All through the C ABI, in HIP graphs, buffers rotated
    so that nothing is served from the last-level cache."""
    Hkv, D = 8, 128
    out = {"metric": "launch and copy floors", "unit": "us", "n_gpus": 1, "config": {"workload": "floors"}, "floors": {}}
    word = f.array(np.zeros(4, np.uint32))
    n_launch = 256
    f.start_capture()
    for _ in range(n_launch):
        f.u32_add(word, 1, 1)
    g = f.end_capture()
    for _ in range(3):
        g.launch()
    f.synchronize()
    reps = 10
    t0 = time.perf_counter()
    for _ in range(reps):
        g.launch()
    f.synchronize()
    dt = time.perf_counter() - t0
    g.destroy()
    out["floors"]["launch"] = {"kernel": "u32_add_kernel (one workgroup)", "us_per_launch": dt / (reps * n_launch) * 1e6,
                               "what": "back-to-back dependent launches of a one-workgroup kernel in a HIP graph"}
    for name, rows, n_rot in (("copy_33.6MB", 8192, 28), ("copy_240MB", 58594, 8)):
        srcs = [f.zeros((Hkv, rows, D)) for _ in range(n_rot)]
        dsts = [f.zeros((Hkv, rows, D)) for _ in range(n_rot)]
        f.start_capture()
        for s_, d_ in zip(srcs, dsts):
            f.kv_prefix_copy(s_.arg(), d_.arg(), rows)
        g = f.end_capture()
        for _ in range(3):
            g.launch()
        f.synchronize()
        reps = 20
        t0 = time.perf_counter()
        for _ in range(reps):
            g.launch()
        f.synchronize()
        dt = time.perf_counter() - t0
        g.destroy()
        moved = 2.0 * Hkv * rows * D * 2  # read + written
        us = dt / (reps * n_rot) * 1e6
        out["floors"][name] = {"kernel": "kv_prefix_copy_vec_kernel", "bytes_moved": moved, "us_per_launch": us,
                               "gbps": moved / us / 1e3, "frac_of_hbm_peak": moved / us / 1e3 / HBM_PEAK_GBPS,
                               "what": "fa_kv_prefix_copy of one [8, %d, 128] f16 tensor (half read, half written), %d "
                                       "tensor pairs in rotation, HIP graph" % (rows, n_rot)}
        for b in srcs + dsts:
            b.free()
    # Launches that only READ as many bytes: the column-sum kernel behind fa_sage_k_mean (it streams its input once with
    # 16-byte non-temporal loads and stores a few KB of partial sums; a second, tiny launch finishes the mean), over
    # [16, rows, 128] f16 tensors in rotation. The read-only launch by itself is timed with events attached to its eager
    # dispatches; the pair as graph replays.
    for name, rows, n_rot in (("read_33.6MB", 8200, 28), ("read_240MB", 58594, 8)):
        heads = 16
        srcs = [f.zeros((heads, rows, D)) for _ in range(n_rot)]
        mean = f.zeros((heads, D), np.float32)

        def read_step(i):
            f.sage_k_mean(srcs[i % n_rot], heads, rows, D, rows, mean)

        pair_s, _ = graph_replay_seconds(f, read_step, n_rot, 3 * n_rot, 20 * n_rot)
        ev = eager_kernel_us(f, read_step, 4 * n_rot, ("sage_k_colsum_kernel", "sage_k_mean_finish_kernel"))
        us = ev["sage_k_colsum_kernel"][1]
        nread = float(heads * rows * D * 2)
        out["floors"][name] = {"kernel": "sage_k_colsum_kernel", "bytes_read": nread, "us_per_launch": us,
                               "gbps": nread / us / 1e3, "frac_of_hbm_peak": nread / us / 1e3 / HBM_PEAK_GBPS,
                               "finish_kernel_us": ev["sage_k_mean_finish_kernel"][1], "graph_us_per_call_both_kernels": pair_s * 1e6,
                               "what": "the streaming launch of fa_sage_k_mean over one [16, %d, 128] f16 tensor (read once, "
                                       "%d tensors in rotation): HIP events attached to its eager dispatches; "
                                       "graph_us_per_call_both_kernels = that launch + the finish launch as graph replays" % (rows, n_rot)}
        for b in srcs + [mean]:
            b.free()
    word.free()
    # Shader clock the board sustains: under back-to-back MFMAs on every CU (fa_measure_clock), and inside the prefill
    # kernel itself (fa_profile_clock_buffer: each resident workgroup's shader-clock ticks over its 100 MHz wall ticks)
    # on random and on all-zero inputs. The published matrix peak is the figure at 2.4 GHz.
    clocks = {}
    mhz, busy = f.measure_clock(True, 200000)
    clocks["mfma_probe"] = {"shader_mhz": mhz, "busy_ms": busy, "what": "fa_measure_clock: 8 waves of dependent-free v_mfma_f32_32x32x16_f16 per CU"}
    H = 24
    rng = np.random.default_rng(11)
    for M in (2048, 8192):
        for data in ("random", "zero"):
            mk = (lambda n: f.array(rng.standard_normal((n, M, D), dtype=np.float32).astype(np.float16))) if data == "random" else (lambda n: f.zeros((n, M, D)))
            q, k, v, o = mk(H), mk(Hkv), mk(Hkv), f.zeros((M, H * D))
            n_wg = min(f.n_cus(), -(-M // 128) * H)
            buf = fa.DevBuf(f, (n_wg, 2), np.int64)
            for rep in range(24):  # long enough for the power management to settle; the last launch's readings count
                if rep == 23:
                    f.profile_clock_buffer(buf, n_wg)
                f.flash_attention(q.arg(), k.arg(), v.arg(), o.arg(), True, 0, H, D, M, M)
            f.synchronize()
            f.profile_clock_buffer(None, 0)
            h = buf.download().astype(np.float64)
            clocks["prefill_%d_%s" % (M, data)] = {"shader_mhz": float(np.mean(h[:, 0] / h[:, 1]) * 100.0),
                                                    "cycles_per_workgroup_median": float(np.median(h[:, 0])),
                                                    "what": "flash_prefill_dma_kernel, Llama-3.2-3B shape, %d tokens, %s inputs" % (M, data)}
            for b in (q, k, v, o, buf):
                b.free()
    out["floors"]["clock"] = clocks
    emit(out)


SECONDARY = {"floors": bench_floors, "llama3b_attn_block": bench_attn_block, "llama3b_chunk_block": bench_chunk_block, "llama3b_prefill_block": bench_prefill_block, "llama3b_prefill_chunk32_8k": bench_prefill_chunk, "llama3b_prefill_chunk32_32k": lambda f, args: bench_prefill_chunk(f, args, 32, 32736), "llama3b_prefill_chunk64_8k": lambda f, args: bench_prefill_chunk(f, args, 64, 8128), "timeline_decode_8k": bench_phase_timeline, "timeline_decode_1k": lambda f, args: bench_phase_timeline(f, args, "decode_1k"), "timeline_sage_32k": lambda f, args: bench_phase_timeline(f, args, "sage_32k"), "timeline_chunk32_8k": lambda f, args: bench_phase_timeline(f, args, "chunk32_8k"), "llama3b_prefill_block_fused": lambda f, args: bench_prefill_block(f, args, fused=True), "llama3b_decode_128k": bench_long_decode, "llama3b_decode_64k": lambda f, args: bench_long_decode(f, args, 65536), "llama3b_decode_32k": lambda f, args: bench_long_decode(f, args, 32768), "llama3b_decode_2k": bench_short_decode, "llama3b_decode_512": lambda f, args: bench_short_decode(f, args, 511), "llama3b_prefill_2k": bench_prefill,
             "llama3b_prefill_8k": lambda f, args: bench_prefill(f, args, 8192), "qwen05b_decode_1k": bench_small_decode,
             "qwen3b_paged_decode": bench_paged_decode, "smollm3_sage_decode_32k": bench_sage_decode,
             "llama3b_kv_growth": bench_kv_growth, "llama3b_fused_qkv": bench_fused_qkv,
             "llama3b_o_proj": bench_o_proj,
             "llama3b_fused_qkv_chunk32": lambda f, args: bench_fused_qkv_chunk(f, args, 32),
             "llama3b_fused_qkv_chunk512": lambda f, args: bench_fused_qkv_chunk(f, args, 512),
             "llama3b_fused_qkv_prefill_2k": lambda f, args: bench_fused_qkv_chunk(f, args, 2048),
             "llama3b_fused_qkv_q8_chunk32": lambda f, args: bench_fused_qkv_chunk(f, args, 32, q8=True),
             "llama3b_fused_qkv_q8_prefill_2k": lambda f, args: bench_fused_qkv_chunk(f, args, 2048, q8=True),
             "llama3b_fused_qkv_q8": lambda f, args: bench_fused_qkv(f, args, q8=True),
             "llama3b_fused_qkv_q4": lambda f, args: bench_fused_qkv(f, args, q4=True),
             "llama3b_o_proj_q8": lambda f, args: bench_o_proj(f, args, q8=True)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--workload", default="llama3b_decode_8k")
    ap.add_argument("--cpu-sample-seconds", type=float, default=12.0)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--keys-per-split", type=int, default=0)
    ap.add_argument("--merge", type=int, default=2)
    ap.add_argument("--unfused", action="store_true", help="two launches per layer (KvPrepFused, FlashAttention)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run a copy kernel of known size (reference point for profiler HBM counters)")
    ap.add_argument("--no-configs", action="store_true",
                    help="only the headline workload: skip the other benchmark configurations and the floors")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this path is built and measured on a single MI355X (--gpus 1); it uses no "
                 "collectives (the path shards by KV head or by sequence without any exchange)")
    if args.workload in SECONDARY:  # secondary lines: the other configurations of the path, one layer per step
        f = fa.Foundry(0)
        args.steps, args.warmup = min(args.steps, 200), min(args.warmup, 20)
        SECONDARY[args.workload](f, args)
        f.close()
        return
    if args.workload != "llama3b_decode_8k":
        sys.exit("unknown workload %r (llama3b_decode_8k is the bench line; secondary: %s)"
                 % (args.workload, ", ".join(sorted(SECONDARY))))

    room = 256  # the metric's timed window: 256 consecutive decode steps from 8192 context
    rng = np.random.default_rng(0xF0DD + 2)
    f = fa.Foundry(0)
    name, cus, mem = f.device_info()
    f.set_decode_variant(args.keys_per_split, args.merge)
    st = make_llama3b_decode(f, rng, 8192, room)

    f.start_capture()
    fused = not args.unfused
    for s in range(GRAPH_STEPS):
        enqueue_step(f, st, s, fused)
    graph16 = f.end_capture()
    f.start_capture()
    enqueue_step(f, st, 0, fused)
    graph1 = f.end_capture()

    # warmup (untimed), then reset the position so the timed window starts at 8192 context
    history = []
    if args.warmup > 0:
        run_steps(f, st, graph16, graph1, args.warmup, room, history)
    f.synchronize()
    st["dpos"].upload(np.array([st["start"]], np.uint32))
    f.synchronize()
    # the timed region, bracketed on the host (value) and by two HIP events on the stream the kernels run on (roofline)
    t0 = time.perf_counter()
    f.timer_start()
    run_steps(f, st, graph16, graph1, args.steps, room, history)
    gpu_ms = f.timer_stop()
    f.synchronize()
    dt = time.perf_counter() - t0

    cache_ok, err = check_against_oracle(f, st, history)

    # per-launch timing of the dominant kernel: eager pass with HIP events around every launch on the op stream
    prof_steps = min(32, room)
    st["dpos"].upload(np.array([st["start"]], np.uint32))
    f.profile_reset()
    f.profile_enable(True)
    for s in range(prof_steps):
        enqueue_step(f, st, s % GRAPH_STEPS, fused)
    kernel = "fused_rope_append_decode_kernel" if fused else "flash_decode_mfma_kernel"
    n_dec, ms_dec = f.profile_query(kernel)
    n_mrg, ms_mrg = f.profile_query("flash_decode_merge_kernel")
    f.profile_enable(False)
    f.profile_reset()
    eager_dec_s = ms_dec / 1e3 / max(1, n_dec)  # events around each eager dispatch (they add to what they measure)
    # the dominant kernel's average launch duration over the timed region: device time between the two events divided by
    # its launches there (the one u32_add per step and every launch gap are left in: nothing is subtracted)
    launches_timed = args.steps * st["L"] * (1 if fused else 2)
    avg_dec_s = gpu_ms / 1e3 / launches_timed if fused else eager_dec_s
    ns_timed = [st["start"] + 1 + (i % room) for i in range(args.steps)]
    bytes_per_launch = sum(layer_bytes(st, n) for n in ns_timed) / len(ns_timed)
    achieved = bytes_per_launch / avg_dec_s / 1e9

    traffic, traffic_note = measured_traffic()
    ns = [st["start"] + 1 + (i % room) for i in range(args.steps)]
    bytes_total = sum(step_bytes(st, n) for n in ns)
    result = {
        "metric": "decode-attn steps/s + achieved HBM GB/s (% peak), Llama-3.2-3B shape @8K ctx",
        "value": args.steps / dt,
        "unit": "steps/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": dt / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "llama3.2-3b decode attention: 28 layers x (RoPE + KV append + flash decode), batch 1, "
                               "H24/Hkv8/D128, f16 contiguous KV cache, kv_len 8193..%d, %d-step HIP graphs"
                               % (st["start"] + min(args.steps, room), GRAPH_STEPS),
                   "device": name, "compute_units": cus},
        "whole_step_hbm_gbps": bytes_total / dt / 1e9,
        "whole_step_hbm_frac_of_peak": bytes_total / dt / 1e9 / HBM_PEAK_GBPS,
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": traffic, "traffic_source": traffic_note,
                     "kernel": kernel, "avg_launch_us": avg_dec_s * 1e6, "launches": launches_timed if fused else n_dec,
                     "timing": ("HIP events on the kernels' stream around the timed region / launches of the kernel in it"
                                if fused else "HIP events around each eager dispatch"),
                     "bytes_per_launch": bytes_per_launch,
                     "eager_dispatch_avg_launch_us": eager_dec_s * 1e6, "eager_dispatch_launches": n_dec,
                     "merge_kernel_avg_launch_us": (ms_mrg * 1e3 / n_mrg) if n_mrg else None},
        "parity": {"cache_bit_exact": cache_ok, "decode_max_abs_err": err},
    }
    if args.calibration_copy:
        result["calibration_copy"] = calibration_copy(f)
    graph16.destroy()
    graph1.destroy()
    for b in st["kc"] + st["vc"]:
        b.free()
    if not args.no_configs:
        # the other benchmark configurations (one layer per step, a bounded number of steps each) and the floors, so that
        # one run records them all; each is the same code as its --workload line
        global _COLLECT
        sub = argparse.Namespace(**vars(args))
        sub.steps, sub.warmup = 100, 10
        result["configs"], result["floors"] = {}, None
        for tag, fn in (("C1_qwen05b_decode_1k", bench_small_decode), ("C3_qwen3b_paged_decode", bench_paged_decode),
                        ("C4_llama3b_prefill_2k", bench_prefill), ("C5_smollm3_sage_decode_32k", bench_sage_decode),
                        ("llama3b_prefill_chunk32_8k", bench_prefill_chunk), ("llama3b_attn_block", bench_attn_block),
                        ("llama3b_chunk_block", bench_chunk_block), ("floors", bench_floors)):
            _COLLECT = []
            g = fa.Foundry(0)
            sub.steps, sub.warmup = (20, 3) if fn in (bench_attn_block, bench_chunk_block) else (100, 10)  # (28 layers per step)
            try:
                fn(g, sub)
            finally:
                g.close()
            line, _COLLECT = _COLLECT[0], None
            if tag == "floors":
                result["floors"] = line["floors"]
            else:
                result["configs"][tag] = {k: line[k] for k in ("metric", "value", "unit", "steps", "ms_per_step", "dtype",
                                                                "config", "roofline", "parity", "timing",
                                                                "whole_step_hbm_frac_of_peak", "eager_dispatch_avg_launch_us",
                                                                "merge_kernel_avg_launch_us") if k in line}
                for k in ("append",):  # the append kernel of a configuration, where it is a launch of its own
                    if k in line:
                        result["configs"][tag][k] = line[k]
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(st, args.cpu_sample_seconds, room)
    print(json.dumps(result))
    f.close()
    if not cache_ok or err > 2e-3:
        sys.exit("parity check failed: cache_bit_exact=%s decode_max_abs_err=%g" % (cache_ok, err))


if __name__ == "__main__":
    main()
