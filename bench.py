#!/usr/bin/env python
"""Benchmark of the Palimpsa attention operator on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-decode] [--no-simple-gla]
                    [--no-layer-slice] [--no-configs] [--no-recurrent]

Headline workload (the metric's own configuration): chunked forward+backward at
B=8, T=2048, H=12, dk=dv=64, bf16 rows and gates (--gates fp32: fp32 gates), fp32 states, 64-token tiles,
synthetic seeded inputs, timed through the public entry point
(palimpsa_amd.ops.palimpsa.chunk_palimpsa + autograd), inputs resident in HBM.
One JSON line is printed; it also carries
  roofline      dominant kernel (chunk_bwd_local_kernel) against the bf16 MFMA peak,
                duration from HIP events recorded around every launch of the timed region
  cpu_baseline  the naive fp32 recurrence (oracle port) timed on this host's cores
  extra.decode  config 3 (B=256, H=16, d=128, 1024 single-token steps) against the HBM peak
  extra.simple_gla  the operator pair without the precision state (chunk_simple_gla forward+backward) on the
                headline shape, its tile kernel against the HBM peak
  extra.layer_slice  fused prologue -> chunk_palimpsa -> fused epilogue, forward+backward, on the headline shape
                (the layer between its projections and o_proj), the prologue backward against the HBM peak
  extra.mamba_layer_slice  the same for the reference's other caller (MetaMamba2.forward) on its 170M shape
  extra.c0      config 0 (fp32 recurrent forward, B=2 T=256 H=4 d=32), with the CPU port beside it
  extra.c2      config 2 (packed 32768 tokens, lognormal documents, H=16 d=96, chunked forward+backward)
  extra.c4      config 4 (one sequence of 65536 tokens, H=16 d=128, chunked forward with initial and final state)
  extra.recurrent  the token-serial entry point (fused_recurrent_palimpsa) forward and forward+backward at B=8 T=2048 H=12
                d=64 fp32 (long sequences: the backward runs the chunked kernels) and at B=256 T=64 with that hand-over
                switched off (the token-serial backward kernel, against the HBM peak as the metric asks; it is bound by serial latency)
Every chunked leg carries two bounds: the bf16 matrix peak priced with the fixed formula of the metric and the
fp32 vector peak priced with the vector instructions the kernel issues (counter figures from profiles/counter_table.txt).
The decode leg of the metric is also carried as flat decode_* scalars inside the headline line's roofline object.
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

PEAK_BF16_MFMA_TFLOPS = 2500.0   # MI355X dense bf16 matrix peak
PEAK_HBM_GBS = 8000.0            # MI355X HBM3E peak
PEAK_FP32_VALU_TFLOPS = 157.3    # MI355X fp32 vector peak (an FMA counted as 2 flops on every lane)
CHUNK = 64
COUNTER_TABLE = os.path.join(ROOT, "profiles", "counter_table.txt")


def load_counter_table(path=COUNTER_TABLE):
    """Per-kernel figures that only the profiler can read (rocprofv3 --pmc, one run per counter): HBM bytes per launch
    (FETCH_SIZE + WRITE_SIZE, scaled by a copy of known size) and vector-ALU instructions per state entry
    (SQ_INSTS_VALU minus the matrix instructions, times 64 lanes, per token x value row x key column).  They are kept in a
    small table under profiles/ next to the summaries they come from, one line per (workload, kernel) with the commit the
    kernels were at when they were collected, so that a stale figure shows in the line this script prints."""
    table = {}
    with open(path) as fh:
        for ln in fh:
            ln = ln.strip()
            if not ln or ln.startswith("#"):
                continue
            workload, kernel, traffic, valu, commit = ln.split()[:5]
            table[(workload, kernel)] = {"traffic": None if traffic == "-" else float(traffic),
                                         "valu_ops_per_entry": None if valu == "-" else float(valu),
                                         "measured_at": commit}
    return table


COUNTERS = load_counter_table()


def counter(workload, kernel, field):
    return COUNTERS.get((workload, kernel), {}).get(field)


def add_traffic(roof, workload, kernel):
    """Attach the profiler's HBM bytes per launch, and the commit they were measured at, to a roofline entry."""
    roof["traffic"] = counter(workload, kernel, "traffic")
    roof["traffic_measured_at"] = counter(workload, kernel, "measured_at")
    return roof


def make_inputs(torch, B, T, H, dk, dv, seed, dtype):
    """q,k ~ N(0,1) L2-normalised per head; v ~ N(0,1); b, gt = sigmoid(N(0,1)); g = Ip = 1 (seeded, CPU generator)."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    q = torch.nn.functional.normalize(torch.randn(B, T, H, dk, generator=gen), dim=-1)
    k = torch.nn.functional.normalize(torch.randn(B, T, H, dk, generator=gen), dim=-1)
    v = torch.randn(B, T, H, dv, generator=gen)
    b = torch.sigmoid(torch.randn(B, T, H, dv, generator=gen))
    gt = torch.sigmoid(torch.randn(B, T, H, generator=gen))
    return dict(q=q.to(dtype), k=k.to(dtype), v=v.to(dtype), b=b.to(dtype), gt=gt,
                g=torch.ones(H), Ip=torch.ones(H))


def make_varlen_lengths(total_tokens=32768, mu=6.5, sigma=1.0, lo=16, hi=4096, seed=0):
    """cu_seqlens of config 2: document lengths round(exp(N(mu, sigma))) clipped to [lo, hi], drawn until the sum
    reaches total_tokens; the last one is cut to fit (merged into the one before when shorter than lo)."""
    import math

    import numpy as np
    rng = np.random.RandomState(seed)
    lens, tot = [], 0
    while tot < total_tokens:
        ln = int(np.clip(round(math.exp(rng.normal(mu, sigma))), lo, hi))
        ln = min(ln, total_tokens - tot)
        if ln < lo and lens:
            lens[-1] += ln
        else:
            lens.append(ln)
        tot += ln
    cu = [0]
    for ln in lens:
        cu.append(cu[-1] + ln)
    return cu


def timed_loop(torch, step, steps, warmup):
    """warmup untimed steps, then exactly `steps` steps between two synchronisations (mean, the contract's figure);
    then the same number again with an event pair around every step (median of the per-step device times: what
    A/B comparisons should read) and with the library's per-kernel events on."""
    from palimpsa_amd import _lib as L
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms_mean = (time.perf_counter() - t0) * 1e3 / steps
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for a, b in ev:
        a.record()
        step()
        b.record()
    torch.cuda.synchronize()
    per = sorted(a.elapsed_time(b) for a, b in ev)
    ms_median = per[len(per) // 2]
    L.profile_enable(True)
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    kern = L.profile_read()
    L.profile_enable(False)
    kernels = {k: {"avg_ms": v[0] / v[1], "launches": v[1]} for k, v in kern.items()}
    return ms_mean, ms_median, kernels


def mfma_roofline(workload, kernel, kernels, flops_per_launch, entries, note):
    """Roofline entry of a chunked kernel: the bf16 matrix peak priced with the metric's fixed flop formula, and the
    fp32 vector peak priced with the vector instructions the kernel issues per state entry."""
    avg_ms = kernels.get(kernel, {"avg_ms": float("nan")})["avg_ms"]
    achieved = flops_per_launch / (avg_ms * 1e-3) / 1e12
    out = {"bound": "mfma", "kernel": kernel, "achieved": achieved, "peak": PEAK_BF16_MFMA_TFLOPS, "unit": "TFLOP/s",
           "frac": achieved / PEAK_BF16_MFMA_TFLOPS, "traffic": None, "algorithmic_flops_per_launch": flops_per_launch,
           "avg_launch_ms": avg_ms, "note": note}
    add_traffic(out, workload, kernel)
    ops = counter(workload, kernel, "valu_ops_per_entry")
    if ops is not None:
        valu = ops * entries * 2 / (avg_ms * 1e-3) / 1e12
        out["valu"] = {"ops_per_entry": ops, "achieved": valu, "peak": PEAK_FP32_VALU_TFLOPS, "unit": "TFLOP/s",
                       "frac": valu / PEAK_FP32_VALU_TFLOPS,
                       "note": "vector (non-matrix) lane instructions per state entry x entries x 2 / time: the fp32 "
                               "rate the vector ALUs would show if every instruction were an FMA; the peak assumes "
                               "packed FMA issue, plain fp32 instructions issue at 0.73 of it on this GPU "
                               "(profiles/issue_rates.txt), and matrix instructions stall the vector issue of "
                               "their SIMD for their whole duration"}
    return out


def bench_chunk(torch, dev, steps, warmup, gates="bf16"):
    from palimpsa_amd import _lib as L
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa

    B, T, H, d = 8, 2048, 12, 64
    inp = make_inputs(torch, B, T, H, d, d, 0, torch.bfloat16)
    if gates == "bf16":     # the benchmark configuration stores the per-token gates in bf16 like the rows
        inp["gt"] = inp["gt"].to(torch.bfloat16)
    leaves = {n: inp[n].to(dev).requires_grad_(True) for n in ("q", "k", "v", "b", "gt", "g", "Ip")}
    do = torch.randn(B, T, H, d, generator=torch.Generator().manual_seed(1)).to(dev, torch.bfloat16)

    def step():
        for x in leaves.values():
            x.grad = None
        o = chunk_palimpsa(leaves["q"], leaves["k"], leaves["v"], leaves["b"], leaves["gt"], leaves["g"],
                           leaves["Ip"], chunk_size=CHUNK)
        o.backward(do)

    ms_per_step, ms_median, kernels = timed_loop(torch, step, steps, warmup)
    tokens = B * T
    E = d * d
    token_heads = B * T * H
    # algorithmic flops of the dense contractions of the exact chunked algorithm, causal-exact
    flops_step = (6 * CHUNK + 14) * E * token_heads
    # share of the dominant kernel: recompute L@X (M and J) + reverse L^T@dMloc (M and J)
    flops_local = 4 * (CHUNK + 1) * E * token_heads
    roofline = mfma_roofline(
        "c1", "chunk_bwd_local_kernel", kernels, flops_local, token_heads * E,
        "flops = 4(C+1)*dk*dv per token-head (recompute + reverse triangular contractions, C=64); step_frac uses "
        "(6C+14)*dk*dv over the whole fwd+bwd step.  The kernel is bound by fp32 vector issue in the tile epilogues "
        "(one division per state entry), not by the matrix cores: see roofline.valu and "
        "profiles/bench_c1.sq_counters_pmc.txt")
    if "valu" in roofline:      # flat copies: nested objects do not survive every consumer of this line
        roofline["valu_frac"] = roofline["valu"]["frac"]
        roofline["valu_ops_per_entry"] = roofline["valu"]["ops_per_entry"]
    roofline["step_frac"] = flops_step / (ms_per_step * 1e-3) / 1e12 / PEAK_BF16_MFMA_TFLOPS
    out_roof = mfma_roofline("c1", "chunk_out_kernel", kernels, 2 * (CHUNK + 1) * E * token_heads, token_heads * E,
                             "flops = 2(C+1)*dk*dv per token-head (prefix products of M and J)")
    return dict(value=tokens / (ms_per_step * 1e-3), ms_per_step=ms_per_step, ms_per_step_median=ms_median,
                roofline=roofline, roofline_forward=out_roof, kernels=kernels,
                config={"workload": f"c1: chunked fwd+bwd B=8 T=2048 H=12 dk=dv=64 bf16 rows {gates} gates fp32 states C=64",
                        "B": B, "T": T, "H": H, "dk": d, "dv": d, "chunk": CHUNK})


def bench_decode(torch, dev, steps):
    from palimpsa_amd import _lib as L
    from palimpsa_amd.ops.palimpsa import fused_recurrent_palimpsa

    B, H, d = 256, 16, 128
    ncyc = 16
    inp = make_inputs(torch, B, ncyc, H, d, d, 0, torch.bfloat16)
    rows = [{n: inp[n][:, t:t + 1].contiguous().to(dev) for n in ("q", "k", "v", "b", "gt")} for t in range(ncyc)]
    g, Ip = inp["g"].to(dev), inp["Ip"].to(dev)
    gen = torch.Generator().manual_seed(3)
    mu = (torch.randn(B, H, d, d, generator=gen) * 0.1).to(dev)
    I = torch.nn.functional.softplus(torch.randn(B, H, d, d, generator=gen)).to(dev)

    def step(t, mu, I):
        r = rows[t % ncyc]
        o, mu, I = fused_recurrent_palimpsa(r["q"], r["k"], r["v"], r["b"], r["gt"], g, Ip,
                                            initial_mu_state=mu, initial_I_state=I, output_final_state=True)
        return mu, I

    for t in range(8):
        mu, I = step(t, mu, I)
    torch.cuda.synchronize()
    L.profile_enable(True)
    t0 = time.perf_counter()
    for t in range(steps):
        mu, I = step(t, mu, I)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    kern = L.profile_read()
    L.profile_enable(False)
    E = d * d
    bytes_step = (16 * E + 2 * (2 * d + 2 * d) + 4 + 2 * d) * B * H   # state in+out fp32, bf16 rows, fp32 gate, bf16 o
    ms_k, n_k = kern.get("recurrent_fwd_kernel", (float("nan"), 1))
    avg_ms = ms_k / max(n_k, 1)
    gbs_kernel = bytes_step / (avg_ms * 1e-3) / 1e9

    # the same steps with the mean state kept in bf16 between steps (an optional cache format: 12 bytes per state
    # entry and step instead of 16), through the bound step a server would use
    from palimpsa_amd.ops.palimpsa import DecodeStep, mu_to_cache
    dec = DecodeStep(B, H, d, d, dev, torch.bfloat16, mu_dtype=torch.bfloat16)
    mu16, I16 = mu_to_cache(mu), I.clone()
    bound = [dec] + [DecodeStep(B, H, d, d, dev, torch.bfloat16, mu_dtype=torch.bfloat16) for _ in range(ncyc - 1)]
    for t, ds in enumerate(bound):
        r = rows[t]
        ds.bind(r["q"], r["k"], r["v"], r["b"], r["gt"], g, Ip, mu16, I16)
    for t in range(8):
        bound[t % ncyc].step()
    torch.cuda.synchronize()
    L.profile_enable(True)
    t0 = time.perf_counter()
    for t in range(steps):
        bound[t % ncyc].step()
    torch.cuda.synchronize()
    elapsed16 = time.perf_counter() - t0
    kern16 = L.profile_read()
    L.profile_enable(False)
    bytes16 = (12 * E + 2 * (2 * d + 2 * d) + 4 + 2 * d) * B * H
    ms16, n16 = kern16.get("recurrent_fwd_kernel", (float("nan"), 1))
    avg16 = ms16 / max(n16, 1)
    bf16_mu = {
        "workload": "c3 shape with the mean state kept in bf16 between steps (DecodeStep(mu_dtype=bfloat16)), I fp32",
        "steps": steps, "tokens_per_s": B * steps / elapsed16, "ms_per_step": elapsed16 * 1e3 / steps,
        "roofline": {"bound": "hbm", "kernel": "recurrent_fwd_kernel", "achieved": bytes16 / (avg16 * 1e-3) / 1e9,
                     "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": bytes16 / (avg16 * 1e-3) / 1e9 / PEAK_HBM_GBS,
                     "traffic": None, "algorithmic_bytes_per_launch": bytes16, "avg_launch_ms": avg16},
    }
    return {
        "bf16_mean_state": bf16_mu,
        "workload": "c3: single-token decode B=256 H=16 dk=dv=128 bf16 rows fp32 states",
        "steps": steps, "tokens_per_s": B * steps / elapsed, "ms_per_step": elapsed * 1e3 / steps,
        "hbm_gbs_wall": bytes_step * steps / elapsed / 1e9,
        "roofline": {"bound": "hbm", "kernel": "recurrent_fwd_kernel", "achieved": gbs_kernel, "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": gbs_kernel / PEAK_HBM_GBS,
                     "traffic": counter("c3", "recurrent_fwd_kernel", "traffic"),
                     "traffic_measured_at": counter("c3", "recurrent_fwd_kernel", "measured_at"),
                     "algorithmic_bytes_per_launch": bytes_step, "avg_launch_ms": avg_ms},
    }


def bench_simple_gla(torch, dev, steps, warmup):
    """chunk_simple_gla forward+backward (what the layer runs with its precision state switched off) on the
    headline shape; g = -gt so that the decays are those of the headline workload."""
    from palimpsa_amd import _lib as L
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla

    B, T, H, d = 8, 2048, 12, 64
    inp = make_inputs(torch, B, T, H, d, d, 0, torch.bfloat16)
    leaves = {n: inp[n].to(dev).requires_grad_(True) for n in ("q", "k", "v")}
    leaves["g"] = (-inp["gt"]).to(dev).requires_grad_(True)
    do = torch.randn(B, T, H, d, generator=torch.Generator().manual_seed(1)).to(dev, torch.bfloat16)

    def step():
        for x in leaves.values():
            x.grad = None
        o, _ = chunk_simple_gla(q=leaves["q"], k=leaves["k"], v=leaves["v"], g=leaves["g"])
        o.backward(do)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    # the step is timed without the per-launch events (they cost host time on a step this short) ...
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    # ... and the kernels in a second pass with them
    L.profile_enable(True)
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    kern = L.profile_read()
    L.profile_enable(False)
    # the same step recorded once into a HIP graph and replayed: at 0.15 ms of kernels per step the host side of an
    # eager step (autograd, buffers, eight launches) is as long as the kernels
    static_q = [x.detach().clone().requires_grad_(True) for x in leaves.values()]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            o, _ = chunk_simple_gla(q=static_q[0], k=static_q[1], v=static_q[2], g=static_q[3])
            torch.autograd.grad(o, static_q, do)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o_g, _ = chunk_simple_gla(q=static_q[0], k=static_q[1], v=static_q[2], g=static_q[3])
        grads_g = torch.autograd.grad(o_g, static_q, do)
    for _ in range(warmup):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.replay()
    torch.cuda.synchronize()
    ms_graph = (time.perf_counter() - t0) * 1e3 / steps
    del graph, o_g, grads_g
    # algorithmic bytes of one launch of the forward tile kernel: q, k, v rows in, tile-start state (bf16) in, o out, gates
    tiles = B * (T // CHUNK) * H
    bytes_out = tiles * (CHUNK * (2 * d + d) * 2 + d * d * 2 + CHUNK * d * 2 + CHUNK * 4)
    ms_out, n_out = kern.get("gla_out_kernel", (float("nan"), 1))
    avg_out_ms = ms_out / max(n_out, 1)
    achieved = bytes_out / (avg_out_ms * 1e-3) / 1e9
    kernels = {k: {"avg_ms": v[0] / v[1], "launches": v[1]} for k, v in kern.items()}
    # decode on the shape of config 3 (B=256, H=16, d=128): single-token steps, state [N,H,dk,dv] fed back
    from palimpsa_amd.ops.simple_gla import fused_recurrent_simple_gla
    Bd, Hd, dd, dsteps = 256, 16, 128, 256
    gen = torch.Generator(device="cpu").manual_seed(2)
    rows = [torch.randn(Bd, 1, Hd, dd, generator=gen).to(dev, torch.bfloat16) for _ in range(3)]
    gd = (-torch.rand(Bd, 1, Hd, generator=gen)).to(dev)
    S = (torch.randn(Bd, Hd, dd, dd, generator=gen) * 0.1).to(dev)
    with torch.no_grad():
        for _ in range(3):
            _, S = fused_recurrent_simple_gla(q=rows[0], k=rows[1], v=rows[2], g=gd, initial_state=S, output_final_state=True)
        torch.cuda.synchronize()
        L.profile_enable(True)
        t0 = time.perf_counter()
        for _ in range(dsteps):
            _, S = fused_recurrent_simple_gla(q=rows[0], k=rows[1], v=rows[2], g=gd, initial_state=S, output_final_state=True)
        torch.cuda.synchronize()
        d_elapsed = time.perf_counter() - t0
        dk_ms, dk_n = L.profile_read().get("gla_recurrent_fwd_kernel", (float("nan"), 1))
        L.profile_enable(False)
    bytes_dec = Bd * Hd * (8 * dd * dd + 2 * (2 * dd + dd) + 4 + 2 * dd)     # state in+out fp32, q,k,v bf16, gate, o
    dec_gbs = bytes_dec / (dk_ms / max(dk_n, 1) * 1e-3) / 1e9
    decode = {"workload": "fused_recurrent_simple_gla B=256 H=16 dk=dv=128, single-token steps, state fed back",
              "tokens_per_s": Bd * dsteps / d_elapsed, "ms_per_step": d_elapsed * 1e3 / dsteps,
              "roofline": {"bound": "hbm", "kernel": "gla_recurrent_fwd_kernel", "achieved": dec_gbs, "peak": PEAK_HBM_GBS,
                           "unit": "GB/s", "frac": dec_gbs / PEAK_HBM_GBS,
                           "traffic": counter("gla_decode", "gla_recurrent_fwd_kernel", "traffic"),
                           "traffic_measured_at": counter("gla_decode", "gla_recurrent_fwd_kernel", "measured_at"),
                           "algorithmic_bytes_per_launch": bytes_dec, "avg_launch_ms": dk_ms / max(dk_n, 1)}}
    return {"workload": "chunk_simple_gla fwd+bwd B=8 T=2048 H=12 dk=dv=64 bf16 rows fp32 gates", "decode": decode,
            "tokens_per_s": B * T / (ms * 1e-3), "ms_per_step": ms, "kernel_ms_per_step": sum(v[0] for v in kern.values()) / steps,
            "graph_replay": {"tokens_per_s": B * T / (ms_graph * 1e-3), "ms_per_step": ms_graph,
                             "note": "the eager step above recorded once into a HIP graph (torch.cuda.graph) and replayed"},
            "kernels": kernels,
            "roofline": {"bound": "hbm", "kernel": "gla_out_kernel", "achieved": achieved, "peak": PEAK_HBM_GBS,
                         "unit": "GB/s", "frac": achieved / PEAK_HBM_GBS,
                         "traffic": counter("gla_c1", "gla_out_kernel", "traffic"),
                         "traffic_measured_at": counter("gla_c1", "gla_out_kernel", "measured_at"),
                         "algorithmic_bytes_per_launch": bytes_out, "avg_launch_ms": avg_out_ms}}


def bench_layer_slice(torch, dev, steps, warmup):
    """What the reference layer does between its projections and o_proj (layers/palimpsa.py:263-343): inputs of
    the operator from the projections' outputs, the operator, residual + gated RMS norm; forward and backward."""
    from palimpsa_amd import _lib as L
    from palimpsa_amd.ops.layer_glue import palimpsa_inputs, palimpsa_output_norm
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa

    B, T, H, d = 8, 2048, 12, 64
    gen = torch.Generator(device="cpu").manual_seed(0)
    r = lambda *shape: torch.randn(*shape, generator=gen)
    bf = torch.bfloat16
    leaves = dict(q_raw=r(B, T, H, d).to(bf), k_raw=r(B, T, H, d).to(bf), x=r(B, T, H, d).to(bf),
                  dt_raw=(r(B, T, H) - 1.0).to(bf), dt_bias=r(H), bs_raw=r(B, T, H).to(bf),
                  b_raw=r(B, T, H, d).to(bf), b_scale=torch.ones(H))
    leaves = {n: v.to(dev).requires_grad_(True) for n, v in leaves.items()}
    gate = r(B, T, H, d).to(dev, bf).requires_grad_(True)
    weight = torch.ones(d, device=dev, requires_grad=True)
    D = torch.ones(H, device=dev, requires_grad=True)
    A = torch.ones(H, device=dev, requires_grad=True)
    Ip = torch.ones(H, device=dev)
    dy = r(B, T, H, d).to(dev, bf)
    params = list(leaves.values()) + [gate, weight, D, A]

    def step():
        for x in params:
            x.grad = None
        q, k, v, b, gt = palimpsa_inputs(**leaves)
        o = chunk_palimpsa(q, k, v, b, gt, A, Ip, chunk_size=CHUNK)
        y = palimpsa_output_norm(o, leaves["x"], D, gate, weight, 1e-6)
        y.backward(dy)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    L.profile_enable(True)
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    kern = L.profile_read()
    L.profile_enable(False)
    rows = B * T * H
    # algorithmic bytes of the prologue backward: q_raw, k_raw, dq, dk, x, dv, b_raw, db in; dq_raw, dk_raw, dx, db_raw
    # out (bf16 rows), plus the per-(token, head) scalars dt_raw, bs_raw (bf16) and dgt (fp32) in, ddt_raw, dbs_raw out
    bytes_pb = rows * (12 * d * 2 + 2 * 2 + 4 + 2 * 2)
    ms_pb, n_pb = kern.get("prologue_bwd_kernel", (float("nan"), 1))
    avg_pb = ms_pb / max(n_pb, 1)
    achieved = bytes_pb / (avg_pb * 1e-3) / 1e9
    glue = ("prologue_fwd_kernel", "prologue_bwd_kernel", "epilogue_fwd_kernel", "epilogue_bwd_kernel")
    return {"workload": "prologue -> chunk_palimpsa -> epilogue, fwd+bwd, B=8 T=2048 H=12 dk=dv=64 bf16",
            "tokens_per_s": B * T / (ms * 1e-3), "ms_per_step": ms,
            "glue_kernel_ms_per_step": sum(kern[k][0] for k in glue if k in kern) / steps,
            "kernels": {k: {"avg_ms": v[0] / v[1], "launches": v[1]} for k, v in kern.items()},
            "roofline": {"bound": "hbm", "kernel": "prologue_bwd_kernel", "achieved": achieved, "peak": PEAK_HBM_GBS,
                         "unit": "GB/s", "frac": achieved / PEAK_HBM_GBS,
                         "traffic": counter("layer_slice", "prologue_bwd_kernel", "traffic"),
                         "traffic_measured_at": counter("layer_slice", "prologue_bwd_kernel", "measured_at"),
                         "algorithmic_bytes_per_launch": bytes_pb, "avg_launch_ms": avg_pb}}


def bench_mamba_layer_slice(torch, dev, steps, warmup):
    """What MetaMamba2.forward does between its convolution and out_proj (layers/meta_mamba2.py:283-363) on the shape
    of the reference's meta_mamba2_170M configuration (16 heads, head_dim 96, state_size 48, 16 groups): time step,
    x dt and b dt, the operator with scale 1 on the raw B, C rows, residual and gated norm over the token; fwd+bwd."""
    from palimpsa_amd import _lib as L
    from palimpsa_amd.ops.layer_glue import metamamba2_inputs, metamamba2_output_norm
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa

    B, T, H, G, dk, dv = 8, 2048, 16, 16, 48, 96
    gen = torch.Generator(device="cpu").manual_seed(0)
    r = lambda *shape: torch.randn(*shape, generator=gen)
    bf = torch.bfloat16
    leaves = dict(C=(0.5 * r(B, T, G, dk)).to(bf), Bm=(0.5 * r(B, T, G, dk)).to(bf), x=r(B, T, H, dv).to(bf),
                  dt_raw=(r(B, T, H) - 1.0).to(bf), dt_bias=torch.ones(H), b_raw=r(B, T, H, dv).to(bf), b_scale=torch.ones(H),
                  gate=r(B, T, H * dv).to(bf), weight=torch.ones(H * dv), D=torch.ones(H),
                  A_log=torch.log(torch.arange(1, H + 1).float()))
    leaves = {n: v.to(dev).requires_grad_(True) for n, v in leaves.items()}
    Ip = torch.ones(H, device=dev)
    dy = r(B, T, H, dv).to(dev, bf)

    def step():
        for x in leaves.values():
            x.grad = None
        v, b, dt = metamamba2_inputs(leaves["x"], leaves["dt_raw"], leaves["dt_bias"], leaves["b_raw"], leaves["b_scale"])
        o = chunk_palimpsa(leaves["C"], leaves["Bm"], v, b, dt, leaves["A_log"].exp(), Ip, scale=1.0, chunk_size=CHUNK)
        y = metamamba2_output_norm(o, leaves["x"], leaves["D"], leaves["gate"], leaves["weight"], 1e-5)
        y.backward(dy)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    L.profile_enable(True)
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    kern = L.profile_read()
    L.profile_enable(False)
    rows = B * T * H
    # algorithmic bytes of the epilogue backward: o, x, gate, dy in; d_o, dx, dgate out (bf16 rows)
    bytes_eb = rows * dv * 2 * 7
    ms_eb, n_eb = kern.get("epilogue_bwd_kernel", (float("nan"), 1))
    avg_eb = ms_eb / max(n_eb, 1)
    achieved = bytes_eb / (avg_eb * 1e-3) / 1e9
    glue = ("prologue_fwd_kernel", "prologue_bwd_kernel", "epilogue_fwd_kernel", "epilogue_bwd_kernel")
    return {"workload": "metamamba2 prologue -> chunk_palimpsa (scale 1) -> epilogue over the token, fwd+bwd, "
                        "B=8 T=2048 H=16 dk=48 dv=96 bf16 (meta_mamba2_170M)",
            "tokens_per_s": B * T / (ms * 1e-3), "ms_per_step": ms,
            "glue_kernel_ms_per_step": sum(kern[k][0] for k in glue if k in kern) / steps,
            "kernels": {k: {"avg_ms": v[0] / v[1], "launches": v[1]} for k, v in kern.items()},
            "roofline": {"bound": "hbm", "kernel": "epilogue_bwd_kernel", "achieved": achieved, "peak": PEAK_HBM_GBS,
                         "unit": "GB/s", "frac": achieved / PEAK_HBM_GBS, "traffic": None,
                         "algorithmic_bytes_per_launch": bytes_eb, "avg_launch_ms": avg_eb}}


def bench_c0(torch, dev, steps, warmup, with_cpu):
    """Config 0: fp32 token-serial forward, B=2 T=256 H=4 dk=dv=32, final states returned."""
    from palimpsa_amd.ops.palimpsa import fused_recurrent_palimpsa
    B, T, H, d = 2, 256, 4, 32
    inp = make_inputs(torch, B, T, H, d, d, 0, torch.float32)
    dv_ = {n: x.to(dev) for n, x in inp.items()}

    def step():
        fused_recurrent_palimpsa(dv_["q"], dv_["k"], dv_["v"], dv_["b"], dv_["gt"], dv_["g"], dv_["Ip"],
                                 output_final_state=True)

    ms, med, kernels = timed_loop(torch, step, steps, warmup)
    bytes_alg = B * T * H * (4 * (2 * d + 2 * d) + 4 + 4 * d) + 2 * B * H * d * d * 4
    k_ms = kernels.get("recurrent_fwd_kernel", {"avg_ms": float("nan")})["avg_ms"]
    out = {"workload": "c0: fused-recurrent forward fp32 B=2 T=256 H=4 dk=dv=32, final states",
           "tokens_per_s": B * T / (ms * 1e-3), "ms_per_step": ms, "ms_per_step_median": med, "kernels": kernels,
           "roofline": {"bound": "hbm", "kernel": "recurrent_fwd_kernel", "achieved": bytes_alg / (k_ms * 1e-3) / 1e9,
                        "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": bytes_alg / (k_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                        "traffic": None, "algorithmic_bytes_per_launch": bytes_alg, "avg_launch_ms": k_ms,
                        "note": "256 dependent token steps on 64 waves: the launch is bound by serial latency "
                                "(about 0.2 us per token), not by any throughput roofline"}}
    if with_cpu:
        from oracle import palimpsa_oracle as po
        t0 = time.perf_counter()
        with torch.no_grad():
            po.palimpsa_recurrence(inp["q"], inp["k"], inp["v"], inp["b"], inp["gt"], inp["g"], inp["Ip"])
        el = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": B * T / el, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"the whole configuration, forward, fp32, {el * 1e3:.1f} ms"}
    return out


def bench_c2(torch, dev, steps, warmup):
    """Config 2: one packed row of 32768 tokens, documents ~ lognormal(6.5, 1.0) clipped to [16, 4096], H=16,
    dk=dv=96, bf16, chunked forward+backward, state reset at every document boundary."""
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa
    cu = make_varlen_lengths(seed=0)
    T, H, d = cu[-1], 16, 96
    inp = make_inputs(torch, 1, T, H, d, d, 0, torch.bfloat16)
    leaves = {n: inp[n].to(dev).requires_grad_(True) for n in ("q", "k", "v", "b", "gt", "g", "Ip")}
    do = torch.randn(1, T, H, d, generator=torch.Generator().manual_seed(1)).to(dev, torch.bfloat16)
    cu_t = torch.tensor(cu, device=dev, dtype=torch.int32)

    def step():
        for x in leaves.values():
            x.grad = None
        o = chunk_palimpsa(leaves["q"], leaves["k"], leaves["v"], leaves["b"], leaves["gt"], leaves["g"], leaves["Ip"],
                           chunk_size=CHUNK, cu_seqlens=cu_t)
        o.backward(do)

    ms, med, kernels = timed_loop(torch, step, steps, warmup)
    E, th = d * d, T * H
    roof = mfma_roofline("c2", "chunk_bwd_local_kernel", kernels, 4 * (CHUNK + 1) * E * th, th * E,
                         "flops = 4(C+1)*dk*dv per token-head; step_frac uses (6C+14)*dk*dv; dk = 96 runs the tile kernel "
                         "in three passes of two column blocks (two workgroups per compute unit)")
    roof["step_frac"] = (6 * CHUNK + 14) * E * th / (ms * 1e-3) / 1e12 / PEAK_BF16_MFMA_TFLOPS
    return {"workload": f"c2: packed varlen chunked fwd+bwd, {len(cu) - 1} documents, 32768 tokens, H=16 dk=dv=96 bf16",
            "documents": len(cu) - 1, "tokens_per_s": T / (ms * 1e-3), "ms_per_step": ms, "ms_per_step_median": med,
            "kernels": kernels, "roofline": roof}


def bench_c4(torch, dev, steps, warmup):
    """Config 4: chunked forward of one sequence of 65536 tokens, H=16, dk=dv=128, bf16, with a non-zero fp32
    initial state passed in and the final state returned."""
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa
    T, H, d = 65536, 16, 128
    inp = make_inputs(torch, 1, T, H, d, d, 0, torch.bfloat16)
    dv_ = {n: x.to(dev) for n, x in inp.items()}
    gen = torch.Generator().manual_seed(3)
    mu0 = (torch.randn(1, H, d, d, generator=gen) * 0.1).to(dev)
    I0 = (1.0 + torch.nn.functional.softplus(torch.randn(1, H, d, d, generator=gen))).to(dev)

    def step():
        with torch.no_grad():
            chunk_palimpsa(dv_["q"], dv_["k"], dv_["v"], dv_["b"], dv_["gt"], dv_["g"], dv_["Ip"], chunk_size=CHUNK,
                           initial_mu_state=mu0, initial_I_state=I0, output_final_state=True)

    ms, med, kernels = timed_loop(torch, step, steps, warmup)
    E, th = d * d, T * H
    # the forward runs in windows of tiles: the per-kernel averages are per window, the flops likewise
    n_launch = max(1, kernels.get("chunk_out_kernel", {"launches": steps})["launches"] // steps)
    roof = mfma_roofline("c4", "chunk_out_kernel", kernels, 2 * (CHUNK + 1) * E * th / n_launch, th * E / n_launch,
                         f"flops = 2(C+1)*dk*dv per token-head (prefix products of M and J); the sequence is run in "
                         f"{n_launch} windows of tiles handed through the state, one launch each; step_frac uses "
                         "(2C+6)*dk*dv over the whole forward")
    roof["step_frac"] = (2 * CHUNK + 6) * E * th / (ms * 1e-3) / 1e12 / PEAK_BF16_MFMA_TFLOPS
    return {"workload": "c4: chunked forward B=1 T=65536 H=16 dk=dv=128 bf16, initial and final state",
            "tokens_per_s": T / (ms * 1e-3), "ms_per_step": ms, "ms_per_step_median": med, "kernels": kernels,
            "roofline": roof}


def bench_recurrent(torch, dev, steps, warmup):
    """Token-serial forward and backward (the reference has no such backward) at the headline batch, fp32."""
    from palimpsa_amd.ops.palimpsa import fused_recurrent_palimpsa
    B, T, H, d = 8, 2048, 12, 64
    inp = make_inputs(torch, B, T, H, d, d, 0, torch.float32)
    leaves = {n: inp[n].to(dev).requires_grad_(True) for n in ("q", "k", "v", "b", "gt", "g", "Ip")}
    do = torch.randn(B, T, H, d, generator=torch.Generator().manual_seed(1)).to(dev)
    names = ("q", "k", "v", "b", "gt", "g", "Ip")

    def fwd():
        with torch.no_grad():
            fused_recurrent_palimpsa(*[leaves[n] for n in names])

    def fwd_bwd():
        for x in leaves.values():
            x.grad = None
        fused_recurrent_palimpsa(*[leaves[n] for n in names]).backward(do)

    ms_f, med_f, k_f = timed_loop(torch, fwd, steps, warmup)
    ms_fb, med_fb, k_fb = timed_loop(torch, fwd_bwd, steps, warmup)
    # the same number of tokens as 256 sequences of 64 tokens (the longest the reference layer hands to this entry
    # point), with the hand-over to the chunked kernels switched off: the token-serial backward kernel itself
    Bs, Ts = 256, 64
    inp_s = make_inputs(torch, Bs, Ts, H, d, d, 0, torch.float32)
    leaves_s = {n: inp_s[n].to(dev).requires_grad_(True) for n in names}
    do_s = torch.randn(Bs, Ts, H, d, generator=torch.Generator().manual_seed(1)).to(dev)

    def fwd_bwd_short():
        for x in leaves_s.values():
            x.grad = None
        fused_recurrent_palimpsa(*[leaves_s[n] for n in names]).backward(do_s)

    from palimpsa_amd import _lib as L
    keep = L.recurrent_bwd_chunk_min()
    L.set_recurrent_bwd_chunk_min(None)
    try:
        ms_s, med_s, k_s = timed_loop(torch, fwd_bwd_short, steps, warmup)
    finally:
        L.set_recurrent_bwd_chunk_min(keep)
    rows = B * T * H
    bytes_f = rows * (4 * 4 * d + 4 + 4 * d)                      # q,k,v,b in, gt in, o out (fp32)
    bytes_b = rows * (4 * 5 * d + 4 + 4 * 4 * d + 4)              # q,k,v,b,do + gt in; dq,dk,dv,db + dgt out (fp32)

    def roof(kernel, kernels, nbytes, note):
        k_ms = kernels.get(kernel, {"avg_ms": float("nan")})["avg_ms"]
        gbs = nbytes / (k_ms * 1e-3) / 1e9
        return {"bound": "hbm", "kernel": kernel, "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": gbs / PEAK_HBM_GBS, "traffic": None, "algorithmic_bytes_per_launch": nbytes, "avg_launch_ms": k_ms,
                "note": note}

    return {"workload": "token-serial forward, and forward+backward, B=8 T=2048 H=12 dk=dv=64 fp32 rows",
            "forward": {"tokens_per_s": B * T / (ms_f * 1e-3), "ms_per_step": ms_f, "ms_per_step_median": med_f, "kernels": k_f,
                        "roofline": roof("recurrent_fwd_kernel", k_f, bytes_f,
                                         "rows in, outputs out; 2048 dependent steps per wave with the state in registers: "
                                         "bound by fp32 vector work and serial latency, not by HBM")},
            "forward_backward": {"tokens_per_s": B * T / (ms_fb * 1e-3), "ms_per_step": ms_fb, "ms_per_step_median": med_fb,
                                 "kernels": k_fb,
                                 "note": "sequences of 64 tokens or more: the backward of this entry point runs the "
                                         "chunked backward kernels (fp32 rows: split operands, the fp32 bar) on "
                                         "tile-start states from a states-only forward pass"},
            "forward_backward_short": {
                "workload": f"token-serial forward+backward kernels, B={Bs} T={Ts} H={H} dk=dv={d} fp32 rows (same token count; "
                            "the hand-over of the backward to the chunked kernels switched off)",
                "tokens_per_s": Bs * Ts / (ms_s * 1e-3), "ms_per_step": ms_s, "ms_per_step_median": med_s, "kernels": k_s,
                "roofline": add_traffic(roof("recurrent_bwd_kernel", k_s, bytes_b,
                                             "rows and dO in, gradients out; the kernel also re-reads its state "
                                             "checkpoints and writes per-tile partial sums (workspace traffic, in the "
                                             "counter figure but not in the algorithmic bytes)"),
                                        "rec_short", "recurrent_bwd_kernel")}}


def cpu_baseline(torch):
    """Naive fp32 recurrence (CPU oracle, a port of the reference's palimpsa_ref) with autograd, on a bounded
    sample of the headline workload: batch rows 0-3 of 8, all heads, all 2048 tokens (about 15 s on 16 cores,
    ~5 GB of per-token states kept by autograd); sequences are independent, so the time is scaled x2."""
    from oracle import palimpsa_oracle as po

    B, T, H, d = 8, 2048, 12, 64
    sb = 4
    inp = make_inputs(torch, sb, T, H, d, d, 0, torch.bfloat16)
    names = ["q", "k", "v", "b", "gt", "g", "Ip"]
    leaves = [inp[n].float().requires_grad_(True) for n in names]
    do = torch.randn(sb, T, H, d, generator=torch.Generator().manual_seed(1))
    cores = torch.get_num_threads()
    t0 = time.perf_counter()
    o, _, _, _ = po.palimpsa_recurrence(*leaves, compute_dtype=torch.float32)
    (o * do).sum().backward()
    el = time.perf_counter() - t0
    scale = B / sb
    return {"value": B * T / (el * scale), "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"fwd+autograd-bwd of batch rows 0-{sb - 1} of 8, all 12 heads, all {T} tokens, fp32, {el:.1f} s; "
                      f"time scaled x{scale:.0f} to B=8 (sequences are independent)"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--decode-steps", type=int, default=1024)
    ap.add_argument("--gates", choices=("bf16", "fp32"), default="bf16",
                    help="element type of the per-token gate tensor gt of the headline workload (the reference layer "
                         "passes fp32; the benchmark configuration says bf16)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-decode", action="store_true")
    ap.add_argument("--no-simple-gla", action="store_true")
    ap.add_argument("--no-layer-slice", action="store_true")
    ap.add_argument("--no-configs", action="store_true", help="skip the legs for configurations 0, 2 and 4")
    ap.add_argument("--no-recurrent", action="store_true", help="skip the token-serial forward/backward leg")
    ap.add_argument("--only", choices=("c0", "c2", "c4", "recurrent", "decode"), default=None,
                    help="profiling aid: run this one leg alone and print its object (not the contract's line), so that "
                         "per-kernel profiler averages belong to one workload")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy (for scaling rocprofv3 FETCH_SIZE/WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the operator shards over batch/heads without any "
              "exchange); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP kernels have no CPU fallback", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.copy_calibration:
        # a copy kernel of known size: 1 GiB read + 1 GiB written per launch
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.only is not None:
        short = max(5, min(args.steps, 20))
        leg = {"c0": lambda: bench_c0(torch, dev, args.steps, args.warmup, False),
               "c2": lambda: bench_c2(torch, dev, short, min(args.warmup, 3)),
               "c4": lambda: bench_c4(torch, dev, short, min(args.warmup, 3)),
               "recurrent": lambda: bench_recurrent(torch, dev, max(3, min(args.steps, 10)), 2),
               "decode": lambda: bench_decode(torch, dev, args.decode_steps)}[args.only]()
        print(json.dumps({"only": args.only, "leg": leg}))
        return
    res = bench_chunk(torch, dev, args.steps, args.warmup, args.gates)
    extra = {"kernels": res["kernels"], "ms_per_step_median": res["ms_per_step_median"],
             "roofline_forward": res["roofline_forward"]}
    if not args.no_decode:
        extra["decode"] = dec = bench_decode(torch, dev, args.decode_steps)
        # the second half of the metric (decode tokens/s, fraction of the HBM peak) as flat scalars of the headline
        # line's roofline object
        dr = dec["roofline"]
        res["roofline"].update({
            "decode_workload": dec["workload"], "decode_tokens_per_s": dec["tokens_per_s"],
            "decode_ms_per_step": dec["ms_per_step"], "decode_kernel_avg_ms": dr["avg_launch_ms"],
            "decode_algorithmic_bytes": dr["algorithmic_bytes_per_launch"], "decode_gbs": dr["achieved"],
            "decode_peak_gbs": dr["peak"], "decode_frac": dr["frac"], "decode_traffic": dr["traffic"],
            "decode_traffic_measured_at": dr["traffic_measured_at"]})
    if not args.no_simple_gla:
        extra["simple_gla"] = bench_simple_gla(torch, dev, args.steps, args.warmup)
    if not args.no_layer_slice:
        extra["layer_slice"] = bench_layer_slice(torch, dev, args.steps, args.warmup)
        extra["mamba_layer_slice"] = bench_mamba_layer_slice(torch, dev, max(args.steps // 2, 1), args.warmup)
    if not args.no_configs:
        short = max(5, min(args.steps, 20))     # 8-10 ms per step
        extra["c0"] = bench_c0(torch, dev, args.steps, args.warmup, not args.no_cpu_baseline)
        extra["c2"] = bench_c2(torch, dev, short, min(args.warmup, 3))
        extra["c4"] = bench_c4(torch, dev, short, min(args.warmup, 3))
    if not args.no_recurrent:
        extra["recurrent"] = bench_recurrent(torch, dev, max(3, min(args.steps, 10)), 2)
    line = {
        "metric": "chunk fwd+bwd tokens/s (H=12,d=64,T=2048) %MFMA peak; decode tokens/s %HBM BW",
        "value": res["value"], "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": res["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic", "config": res["config"], "roofline": res["roofline"],
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(torch)
    line["extra"] = extra
    print(json.dumps(line))


if __name__ == "__main__":
    main()
