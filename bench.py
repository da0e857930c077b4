#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-extras]
    python bench.py --model-shapes     (a table instead: see below)

A "step" is one call of the joint-attention forward on the Flux-1024 shape
(B=1, H=24, S=4608 = 512 text + 4096 image tokens, D=128, bf16, non-causal, BHSD-contiguous,
q/k per-head RMSNorm'd), inputs resident in HBM, with the library's default options (fixed work
geometry: results reproducible bit for bit).  Prints ONE JSON line:
  value        TFLOP/s of the step (algorithmic FLOPs 4*B*H*Sq*Sk*D over wall-clock per step)
  ms_per_step  wall-clock per call over exactly K calls, synchronised on both sides, after W
               warm-up calls.  Before the warm-up calls the process brings the chip to its loaded
               state (`conditioning` in the JSON: about 0.2 s of the same call): coming out of idle
               the chip's power management lets a few calls run fast, then overshoots downwards
               for some 100 calls (25 ms) before it settles, and a denoising run, which issues
               thousands of such calls between GEMMs, lives in the settled state.  The same K calls
               of a fresh process WITHOUT that conditioning are reported as `also.c2_flux1024_first25`
  roofline     the same kernel's HIP-event average launch duration against the dense bf16 MFMA peak
  cpu_baseline torch's CPU scaled_dot_product_attention (what the reference's SDPA adapter calls,
               xfuser/core/distributed/attention_backend.py:499-501) on a bounded sample of the
               same workload, timed on this host's cores
  also         the other named shapes: HunyuanVideo-720p head shard (bf16), Wan2.1 720p head
               shard (fp8), the 4-chunk ring with its fp32 merges, the merge kernel's GB/s, the
               fp8 quantiser and the fused norm + rotary prologue (GB/s against the HBM peak)
               and torch's own GPU flash attention (the op behind the reference's default
               SDPA_FLASH backend, attention_backend.py:504-516) on the same tensors and GPU;
               the PixArt-512 fp32 case; the Flux step's first 25 calls and its steady state in a
               fresh process (per-call HIP-event pairs: median and min); the same step with
               streamed sharing (the opt-in launch whose results are reproducible to rounding
               only); host time per call
  Entries of `also` carry the median ("ms" / "us"), the minimum and the mean of per-call
  HIP-event pairs (the reference times its own runs with events around synchronised regions
  and discards the first iteration: xfuser/model_executor/models/runner_models/base_model.py:631-644).
--model-shapes prints, instead of the JSON line, one row per attention shape of the reference's
model families (self, joint and cross attention; head_dim 128, 64, 72, 88): this library against
torch's GPU flash attention on the same tensors, with the largest difference between the outputs.
Everything runs on one GPU; --gpus above 1 is refused (this build has no multi-GPU path).
"""
import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_FP8_TFLOPS = 5000.0    # MI355X dense fp8 MFMA
PEAK_FP32_TFLOPS = 157.3    # MI355X dense fp32 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "attn_fwd_bf16_flux1024_hbm_traffic.md")


def measured_traffic():
    """HBM bytes per Flux-1024 step as the committed counter summary states them (a line
    `traffic_bytes_per_step: N` plus the commit the counters were taken at); None if absent."""
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return None, None
    import re
    m = re.search(r"^traffic_bytes_per_step:\s*([0-9.eE+]+)", text, re.M)
    c = re.search(r"^measured_at_commit:\s*(\S+)", text, re.M)
    return (float(m.group(1)) if m else None), (c.group(1) if c else None)


def make_inputs(B, H, S, D, seed, device, rmsnorm=True, dtype=torch.bfloat16):
    """Synthetic q, k, v ~ N(0,1) (BHSD); q and k get a per-head RMSNorm over head_dim with a gain
    vector ~ U(0.8, 1.2), as a DiT block's norm_q / norm_k produce."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    def n():
        return torch.randn((B, H, S, D), generator=g, dtype=torch.float32)
    q, k, v = n(), n(), n()
    if rmsnorm:
        gq = 0.8 + 0.4 * torch.rand(D, generator=g)
        gk = 0.8 + 0.4 * torch.rand(D, generator=g)
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + 1e-6) * gq
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + 1e-6) * gk
    return q.to(dtype).to(device), k.to(dtype).to(device), v.to(dtype).to(device)


def time_calls(fn, steps, warmup):
    """(wall ms per call, HIP-event ms per call) over exactly `steps` calls."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0) * 1e3 / steps, e0.elapsed_time(e1) / steps


def time_each(fn, steps, warmup):
    """Per-call HIP-event pairs on the current stream -> dict(ms median, ms_min, ms_mean)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for a, b in ev:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    t = sorted(a.elapsed_time(b) for a, b in ev)
    return {"ms": round(t[len(t) // 2], 5), "ms_min": round(t[0], 5), "ms_mean": round(sum(t) / len(t), 5)}


def host_us_per_call(fn, batch=40, repeats=5):
    """Host time of a call that only queues work: `batch` calls back to back without waiting for
    the GPU, smallest per-call average over `repeats` batches (the queue is drained in between)."""
    best = None
    for _ in range(repeats):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(batch):
            fn()
        t = (time.perf_counter() - t0) / batch
        best = t if best is None or t < best else best
    torch.cuda.synchronize()
    return round(best * 1e6, 2)


def with_rate(stat, flops, peak=None):
    stat = dict(stat)
    stat["tflops"] = round(flops / stat["ms"] / 1e9, 1)
    if peak:
        stat["frac_peak"] = round(flops / stat["ms"] / 1e9 / peak, 4)
    return stat


def _fresh_process_series(calls):
    """Per-call HIP-event times (us) of the first `calls` Flux-1024 steps of THIS process, printed as
    one JSON list.  main() runs it in a child process (`python -c "import bench; ..."`), so that the
    steps are the first GPU work of a process that has just started: no conditioning, no warm-up."""
    from xdit_amd import ops
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    q, k, v = make_inputs(1, 24, 4608, 128, 1002, dev)
    out = torch.empty_like(q)
    lse = torch.empty(1, 24, 4608, dtype=torch.float32, device=dev)
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(calls)]
    for a, b in ev:
        a.record()
        ops.attn_fwd(q, k, v, out=out, lse=lse)
        b.record()
    torch.cuda.synchronize()
    print(json.dumps([round(a.elapsed_time(b) * 1e3, 1) for a, b in ev]))


def condition(fn, seconds=0.2):
    """Runs `fn` back to back for about `seconds`: the chip's power management is then in the state
    it keeps under a sustained load of such calls.  Returns the number of calls made."""
    fn()
    torch.cuda.synchronize()
    n = 0
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
        n += 20
    return n


def attn_flops(B, H, Sq, Sk, D):
    return 4.0 * B * H * Sq * Sk * D


def torch_flash(q, k, v):
    """torch's GPU flash attention: the call inside the reference's SDPA_FLASH adapter
    (xfuser/core/distributed/attention_backend.py:504-516), its default backend."""
    from torch.nn.attention import SDPBackend, sdpa_kernel
    with sdpa_kernel([SDPBackend.FLASH_ATTENTION]):
        return torch.nn.functional.scaled_dot_product_attention(q, k, v, dropout_p=0.0, is_causal=False)


# Attention calls of the reference's model families at their usual resolutions, bf16:
# (name, B, H, Sq, Sk, D)
MODEL_SHAPES = [
    ("Flux-1024 joint", 1, 24, 4608, 4608, 128),
    ("Flux-1024 joint, 3 of 24 heads", 1, 3, 4608, 4608, 128),
    ("Flux-2048 joint", 1, 24, 16896, 16896, 128),
    ("HunyuanVideo-720p, 3 of 24 heads", 1, 3, 119056, 119056, 128),
    ("Wan2.1-480p self", 1, 40, 32760, 32760, 128),
    ("Wan2.1-480p cross (512 text keys)", 1, 40, 32760, 512, 128),
    ("SD3-1024 joint", 2, 24, 4250, 4250, 64),
    ("CogVideoX-5B", 2, 48, 17776, 17776, 64),
    ("PixArt-1024 self", 2, 16, 4096, 4096, 72),
    ("PixArt-1024 cross (120 text keys)", 2, 16, 4096, 120, 72),
    ("HunyuanDiT-1024 self", 2, 16, 4096, 4096, 88),
]


def model_shapes(dev):
    from xdit_amd import ops
    print("| shape | B H Sq Sk D | this library us | TFLOP/s | torch flash us | TFLOP/s | speed-up | max abs diff of out |")
    print("|---|---|---|---|---|---|---|---|")
    for name, B, H, Sq, Sk, D in MODEL_SHAPES:
        g = torch.Generator(device="cpu").manual_seed(Sq + D)
        q, k, v = (torch.randn(B, H, n, D, generator=g).bfloat16().to(dev) for n in (Sq, Sk, Sk))
        fl = attn_flops(B, H, Sq, Sk, D)
        steps, warm = (5, 3) if fl > 5e12 else (20, 40)
        _, ms = time_calls(lambda: ops.attn_fwd(q, k, v), steps, warm)
        o, _ = ops.attn_fwd(q, k, v)
        try:
            ro = torch_flash(q, k, v)
            _, rms = time_calls(lambda: torch_flash(q, k, v), steps, min(warm, 10))
            ref = "%.1f | %.0f | %.2fx | %.4f" % (rms * 1e3, fl / rms / 1e9, rms / ms, (ro.float() - o.float()).abs().max().item())
        except Exception as e:  # the comparison is optional: report, do not fail
            ref = "failed: %s | | |" % str(e)[:60]
        print("| %s | %d %d %d %d %d | %.1f | %.0f | %s |" % (name, B, H, Sq, Sk, D, ms * 1e3, fl / ms / 1e9, ref), flush=True)
        del q, k, v, o


def _median_time(fn, budget_s, max_runs):
    times = []
    t_start = time.perf_counter()
    while True:
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
        if time.perf_counter() - t_start > budget_s or len(times) >= max_runs:
            break
    return sorted(times)[len(times) // 2], len(times)


def cpu_baseline(q, k, v, budget_s=8.0):
    """The reference's CPU SDPA path (torch CPU scaled_dot_product_attention, the call inside its
    SDPA adapter) on this host's cores.  Headline figure: the same Flux-1024 tensors, all heads,
    fp32, median of full-shape runs over about `budget_s` seconds.  `others`: the same tensors in
    bf16, PixArt-512 in fp32 at full shape, and for the two video shards the first 2048 query
    rows against the full keys/values (measured) with the linear-in-Sq figure for the whole
    shard next to it, labelled as extrapolated."""
    from oracle import attn_oracle as O   # the checker/baseline module; never used by the GPU leg
    B, H, S, D = q.shape
    qc, kc, vc = (t.float().cpu().contiguous() for t in (q, k, v))
    O.sdpa_cpu(qc[:, :1], kc[:, :1], vc[:, :1])  # warm the thread pool
    t, runs = _median_time(lambda: O.sdpa_cpu(qc, kc, vc), budget_s, 200)
    others = {}
    qb, kb, vb = (x.bfloat16() for x in (qc, kc, vc))
    tb, rb = _median_time(lambda: O.sdpa_cpu(qb, kb, vb), 3.0, 50)
    others["c2_flux1024_bf16"] = {"s": round(tb, 4), "tflops": round(attn_flops(B, H, S, S, D) / tb / 1e12, 4), "runs": rb}
    g = torch.Generator().manual_seed(1001)
    q1, k1, v1 = (torch.randn(1, 16, 1024, 72, generator=g) for _ in range(3))
    t1, r1 = _median_time(lambda: O.sdpa_cpu(q1, k1, v1), 1.5, 200)
    others["c1_pixart512_fp32"] = {"s": round(t1, 5), "tflops": round(attn_flops(1, 16, 1024, 1024, 72) / t1 / 1e12, 4), "runs": r1}
    for name, (Hs, Ss, fp8) in (("c4_hunyuan720p_shard", (3, 118800 + 256, False)),
                                ("c5_wan720p_shard_dequantised_fp32", (5, 75600, True))):
        # the configurations' own tensors: RMSNorm'd q/k for the HunyuanVideo shard; for the Wan shard
        # the fp8 tensors with per-head scales, dequantised to fp32 (what an fp32 reference sees)
        rows = 2048
        cfg = O.make_config("c5_wan720p_shard_fp8" if fp8 else "c4_hunyuan720p_shard")
        if fp8:
            qs, ks, vs = (O.dequant(cfg[n], cfg[n + "_descale"]) for n in ("q", "k", "v"))
        else:
            qs, ks, vs = (cfg[n].float() for n in ("q", "k", "v"))
        del cfg
        qs = qs[:, :, :rows].contiguous()
        ts, rs = _median_time(lambda: O.sdpa_cpu(qs, ks, vs), 2.0, 5)
        others[name] = {"q_rows_measured": rows, "s_measured": round(ts, 4),
                        "tflops": round(attn_flops(1, Hs, rows, Ss, D) / ts / 1e12, 4),
                        "s_whole_shard_extrapolated": round(ts * Ss / rows, 2), "runs": rs,
                        "note": "fp32, first 2048 query rows x all keys of every shard head, the configuration's own tensors; whole-shard time is linear-in-Sq extrapolation, not measured"}
        del qs, ks, vs
    return {
        "value": round(attn_flops(B, H, S, S, D) / t / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": "torch CPU scaled_dot_product_attention (the call inside the reference's SDPA adapter), fp32 copies of "
                  "the same Flux-1024 tensors (B=1, H=%d, S=%d, D=%d), median of %d full-shape runs, "
                  "%.3f s per run; host has %d logical CPUs, torch uses %d threads"
                  % (H, S, D, runs, t, os.cpu_count(), torch.get_num_threads()),
        "others": others,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--model-shapes", action="store_true",
                    help="print a table of the reference's model shapes against torch's GPU flash attention, and exit")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 256 MiB device-to-device copy (a kernel of known traffic for scaling rocprof byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU only (no collectives / sharding code); --gpus %d is not supported" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)

    from xdit_amd import ops, ring, usp  # loads the HIP library; raises if it is not built

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.model_shapes:
        model_shapes(dev)
        return
    B, H, S, D = 1, 24, 4608, 128
    q, k, v = make_inputs(B, H, S, D, 1002, dev)
    out = torch.empty_like(q)

    def step():
        ops.attn_fwd(q, k, v, out=out)

    conditioning_calls = condition(step, 0.2)
    wall_ms, ev_ms = time_calls(step, args.steps, args.warmup)
    flops = attn_flops(B, H, S, S, D)
    tflops = flops / (wall_ms * 1e-3) / 1e12
    achieved = flops / (ev_ms * 1e-3) / 1e12

    traffic, traffic_commit = measured_traffic()
    plan = ops.launch_plan(q, k)   # what the library launches for this problem
    kernel_name = "attn_fwd_16_kernel<bf16, head_dim 128, %d wavefronts>: %d query tiles of %d rows, %d whole" % (
        plan["rows_per_workgroup"] // 32, plan["query_tiles"], plan["rows_per_workgroup"], plan["whole_tiles"])
    if plan["ranges"]:
        kernel_name += ", the other %d cut into %d ranges of %d KV iterations%s + attn_combine_kernel<bf16,128>" % (
            plan["query_tiles"] - plan["whole_tiles"], plan["ranges"], plan["range_len"], " (streamed)" if plan["streamed"] else "")
    result = {
        "metric": "joint-attn fwd ms/call + TFLOP/s (% MFMA peak) at Flux-1024 and HV-720p shard",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "c2_flux1024: joint attention forward (out, lse), B=1 H=24 S=4608 (512 text + 4096 image) D=128, "
                        "bf16, non-causal, BHSD-contiguous, RMSNorm'd q/k, single pass",
            "flops_per_step": flops,
            "options": "library defaults: fixed work geometry (results reproducible bit for bit); "
                       "streamed sharing (opt-in) is under also.c2_flux1024_streamed_sharing",
        },
        "conditioning": "%d untimed calls of the same step over 0.2 s before the %d warm-up calls, so that the chip's power "
                        "management is in its loaded state; the first calls of a fresh process are under also.c2_flux1024_first25"
                        % (conditioning_calls, args.warmup),
        "roofline": {
            "bound": "mfma",
            "achieved": round(achieved, 2),
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
            # HBM bytes per step from rocprofv3 FETCH_SIZE / WRITE_SIZE counters, each scaled by the
            # same counter's reading for a 256 MiB copy in the same run (--copy-calibration)
            "traffic": traffic,
            "traffic_source": "profiles/attn_fwd_bf16_flux1024_hbm_traffic.md, counters taken at commit %s" % traffic_commit,
            "kernel": kernel_name,
            "kernel_ms": round(ev_ms, 5),
        },
    }

    if not args.no_extras:
        also = {}
        n = max(20, args.steps)
        # The Flux step in a fresh process, per call: the first 25 calls and the steady state
        # (calls 101..300).  The first few dozen calls after start-up run slower than the steady
        # state (the chip's power management settles), which is where a short timed window lies.
        try:
            import subprocess
            r = subprocess.run([sys.executable, "-c", "import bench; bench._fresh_process_series(300)"], cwd=ROOT,
                               capture_output=True, text=True, timeout=300)
            us = json.loads(r.stdout.strip().splitlines()[-1])
            first, steady = sorted(us[:25]), sorted(us[100:])
            also["c2_flux1024_first25"] = {"us": first[len(first) // 2], "us_min": first[0], "us_max": first[-1],
                                           "us_mean": round(sum(first) / len(first), 1), "calls": "1-25 of a fresh process"}
            also["c2_flux1024_steady"] = {"us": steady[len(steady) // 2], "us_min": steady[0], "us_max": steady[-1],
                                          "us_mean": round(sum(steady) / len(steady), 1), "calls": "101-300 of the same process",
                                          "tflops": round(flops / steady[len(steady) // 2] / 1e6, 1),
                                          "frac_peak": round(flops / steady[len(steady) // 2] / 1e6 / PEAK_BF16_TFLOPS, 4)}
        except Exception as e:  # the series is a report, not a gate
            also["c2_flux1024_first25"] = {"error": str(e)[:160]}
        # host time of the calls (the Python wrapper + the C entry point; nothing waits for the GPU)
        lse = torch.empty(B, H, S, dtype=torch.float32, device=dev)
        also["host_us_per_call"] = {"attn_fwd": host_us_per_call(lambda: ops.attn_fwd(q, k, v, out=out, lse=lse)),
                                    "attn_fwd_allocating_out_and_lse": host_us_per_call(lambda: ops.attn_fwd(q, k, v))}
        # the opt-in launch that shares KV iterations of the last round's tiles dynamically (results reproducible to rounding only)
        also["c2_flux1024_streamed_sharing"] = with_rate(time_each(lambda: ops.attn_fwd(q, k, v, out=out, streamed=True), n, args.warmup), flops, PEAK_BF16_TFLOPS)
        # the plain launch (one workgroup per query tile, no shared last round, no combine kernel)
        also["c2_flux1024_plain_launch"] = with_rate(time_each(lambda: ops.attn_fwd(q, k, v, out=out, balance=False), n, args.warmup), flops)
        # same shape, BSHD-contiguous memory viewed as BHSD (what a single-GPU Flux block hands over)
        qb, kb, vb = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (q, k, v))
        ob = torch.empty(q.shape[0], q.shape[2], q.shape[1], q.shape[3], dtype=q.dtype, device=q.device).transpose(1, 2)
        also["c2_flux1024_bshd_view"] = with_rate(time_each(lambda: ops.attn_fwd(qb, kb, vb, out=ob), n, args.warmup), flops)
        # torch's GPU flash attention on the same tensors: what the reference's default backend runs
        try:
            also["c2_flux1024_torch_flash_same_gpu"] = with_rate(time_each(lambda: torch_flash(q, k, v), n, args.warmup), flops)
        except Exception as e:
            also["c2_flux1024_torch_flash_same_gpu"] = {"error": str(e)[:120]}
        # PixArt-512 self-attention in fp32 (the CPU-runnable configuration), fp32 matrix cores
        g1 = torch.Generator(device="cpu").manual_seed(1001)
        q1, k1, v1 = (torch.randn(1, 16, 1024, 72, generator=g1).to(dev) for _ in range(3))
        f1 = attn_flops(1, 16, 1024, 1024, 72)
        also["c1_pixart512_fp32"] = with_rate(time_each(lambda: ops.attn_fwd(q1, k1, v1), 50, 10), f1, PEAK_FP32_TFLOPS)
        del q1, k1, v1
        # ring of 4 KV chunks, merged in fp32 (the cast of the last fold is fused)
        fn = usp._get_attention_function()
        also["c3_flux_ring4"] = with_rate(time_each(lambda: usp.ring_attn(fn, q, k, v, ring_chunks=4), n, args.warmup), flops, PEAK_BF16_TFLOPS)
        also["host_us_per_call"]["ring4_four_fused_steps"] = host_us_per_call(lambda: usp.ring_attn(fn, q, k, v, ring_chunks=4), batch=10)
        # the same ring captured once in a HIP graph and replayed (shows whether the eager form is launch-bound)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            usp.ring_attn(fn, q, k, v, ring_chunks=4)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            usp.ring_attn(fn, q, k, v, ring_chunks=4)
        also["c3_flux_ring4_graph"] = with_rate(time_each(graph.replay, n, args.warmup), flops, PEAK_BF16_TFLOPS)
        del graph
        # the merge kernel alone: bytes per fold = 10*N*D + 12*N
        N = B * H * S
        acc = torch.randn(B, H, S, D, device=dev)
        acc_l = torch.randn(B, H, S, device=dev)
        blk_l = torch.randn(B, H, S, device=dev)
        st = time_each(lambda: ops.lse_merge(acc, acc_l, q, blk_l), 50, 5)
        mbytes = 10.0 * N * D + 12.0 * N
        also["lse_merge_fold"] = {"us": round(st["ms"] * 1e3, 2), "us_min": round(st["ms_min"] * 1e3, 2), "gbs": round(mbytes / st["ms"] / 1e6, 1),
                                  "frac_hbm_peak": round(mbytes / st["ms"] / 1e6 / PEAK_HBM_GBS, 4), "bytes": mbytes}
        # the last fold of a two-call ring, with the cast to bf16 fused: 12*N*D + 12*N bytes
        fin = torch.empty_like(q)
        st = time_each(lambda: ops.lse_merge(acc, acc_l, q, blk_l, final_out=fin), 50, 5)
        fbytes = 12.0 * N * D + 12.0 * N
        also["lse_merge_fold_with_cast"] = {"us": round(st["ms"] * 1e3, 2), "us_min": round(st["ms_min"] * 1e3, 2), "gbs": round(fbytes / st["ms"] / 1e6, 1),
                                            "frac_hbm_peak": round(fbytes / st["ms"] / 1e6 / PEAK_HBM_GBS, 4), "bytes": fbytes}
        del acc, qb, kb, vb, fin
        # HunyuanVideo 720p one-GPU head shard
        Bh, Hh, Sh = 1, 3, 118800 + 256
        qh, kh, vh = make_inputs(Bh, Hh, Sh, D, 1004, dev)
        fl = attn_flops(Bh, Hh, Sh, Sh, D)
        also["c4_hunyuan720p_shard"] = with_rate(time_each(lambda: ops.attn_fwd(qh, kh, vh), 5, 2), fl, PEAK_BF16_TFLOPS)
        try:
            also["c4_hunyuan720p_shard_torch_flash_same_gpu"] = with_rate(time_each(lambda: torch_flash(qh, kh, vh), 3, 1), fl)
        except Exception as e:
            also["c4_hunyuan720p_shard_torch_flash_same_gpu"] = {"error": str(e)[:120]}
        del qh, kh, vh
        # Wan2.1 720p head shard, fp8 e4m3fn + per-head scales -> bf16
        Bw, Hw, Sw = 1, 5, 75600
        qw, kw, vw = make_inputs(Bw, Hw, Sw, D, 1005, dev, rmsnorm=False)
        (q8, qd), (k8, kd), (v8, vd) = (ops.fp8_quant(t) for t in (qw, kw, vw))
        fl = attn_flops(Bw, Hw, Sw, Sw, D)
        also["c5_wan720p_shard_fp8"] = with_rate(time_each(lambda: ops.attn_fwd(q8, k8, v8, q_descale=qd, k_descale=kd, v_descale=vd), 5, 2), fl, PEAK_FP8_TFLOPS)
        st = time_each(lambda: ops.fp8_quant(qw), 20, 3)
        also["fp8_quant_wan_shard"] = {"us": round(st["ms"] * 1e3, 1), "us_min": round(st["ms_min"] * 1e3, 1),
                                       "gbs": round(qw.numel() * 5.0 / st["ms"] / 1e6, 1),
                                       "frac_hbm_peak": round(qw.numel() * 5.0 / st["ms"] / 1e6 / PEAK_HBM_GBS, 4)}
        del qw, kw, vw, q8, k8, v8
        # head_dim 64 (what the hybrid schedule hands the fp8 backend for SD3 and CogVideoX), fp8 beside bf16
        for name, (Bs, Hs, Ss) in (("sd3_1024_d64", (2, 24, 4250)), ("cogvideox_d64", (2, 48, 17776))):
            qs, ks, vs = make_inputs(Bs, Hs, Ss, 64, 1006, dev)
            (q8, qd), (k8, kd), (v8, vd) = (ops.fp8_quant(t) for t in (qs, ks, vs))
            fl = attn_flops(Bs, Hs, Ss, Ss, 64)
            n = 5 if Ss > 8192 else 40
            also[name + "_fp8"] = with_rate(time_each(lambda: ops.attn_fwd(q8, k8, v8, q_descale=qd, k_descale=kd, v_descale=vd), n, 3), fl, PEAK_FP8_TFLOPS)
            also[name + "_bf16"] = with_rate(time_each(lambda: ops.attn_fwd(qs, ks, vs), n, 3), fl, PEAK_BF16_TFLOPS)
            del qs, ks, vs, q8, k8, v8
        # pre-attention prologue (per-head RMSNorm + rotary embedding + BSHD -> BHSD), bf16:
        # bytes per call = 4*N*D (read + write) + 8*S*D (cos and sin rows, read once)
        from xdit_amd import prologue
        for name, (Bp, Sp, Hp) in (("prologue_flux_q", (1, 4608, 24)), ("prologue_hunyuan_q", (1, 119056, 24))):
            xp = torch.randn(Bp, Sp, Hp, D, device=dev).bfloat16()
            wp = torch.ones(D, device=dev).bfloat16()
            ang = torch.rand(Sp, D, device=dev)
            cs, sn = ang.cos(), ang.sin()
            yp = torch.empty(Bp, Hp, Sp, D, device=dev, dtype=torch.bfloat16)
            st = time_each(lambda: prologue.norm_rope(xp, weight=wp, freqs_cis=(cs, sn), sequence_dim=1, out=yp), 20, 3)
            pbytes = 4.0 * xp.numel() + 8.0 * Sp * D
            also[name] = {"us": round(st["ms"] * 1e3, 2), "us_min": round(st["ms_min"] * 1e3, 2), "gbs": round(pbytes / st["ms"] / 1e6, 1),
                          "frac_hbm_peak": round(pbytes / st["ms"] / 1e6 / PEAK_HBM_GBS, 4), "bytes": pbytes}
            del xp, yp, ang, cs, sn
        # the whole pre-attention step of a Flux block in one launch: norm + rotary + [text; image]
        # concatenation + BSHD -> BHSD of Q and K, re-layout of V (six jobs); bytes = 4 per element
        # of q, k, v plus the cos/sin rows read by the Q and K jobs
        S_txt, S_img = 512, 4096
        proj = [torch.randn(1, s, H * D, device=dev).bfloat16() for s in (S_img, S_img, S_img, S_txt, S_txt, S_txt)]
        gains = [torch.ones(D, device=dev).bfloat16() for _ in range(4)]
        ang = torch.rand(S_txt + S_img, D, device=dev)
        cs, sn = ang.cos(), ang.sin()
        est = time_each(lambda: prologue.flux_joint_qkv(*proj, H, *gains, (cs, sn)), 30, 5)
        also["host_us_per_call"]["flux_joint_qkv_six_jobs"] = host_us_per_call(lambda: prologue.flux_joint_qkv(*proj, H, *gains, (cs, sn)), batch=20)
        pbytes = 3 * 4.0 * H * D * (S_txt + S_img) + 2 * 8.0 * (S_txt + S_img) * D
        # replaying the call from a HIP graph shows the kernel itself
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            prologue.flux_joint_qkv(*proj, H, *gains, (cs, sn))
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            held = prologue.flux_joint_qkv(*proj, H, *gains, (cs, sn))
        gst = time_each(graph.replay, 30, 5)
        also["prologue_flux_block_qkv"] = {"us_eager_call": round(est["ms"] * 1e3, 2), "us": round(gst["ms"] * 1e3, 2), "us_min": round(gst["ms_min"] * 1e3, 2),
                                           "gbs": round(pbytes / gst["ms"] / 1e6, 1),
                                           "frac_hbm_peak": round(pbytes / gst["ms"] / 1e6 / PEAK_HBM_GBS, 4), "bytes": pbytes}
        del graph, held
        result["also"] = also

    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(q, k, v)

    print(json.dumps(result))


if __name__ == "__main__":
    main()
