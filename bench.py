#!/usr/bin/env python3
"""Benchmark of the mLSTM hot path on one MI355X.

A "step" is one TFLA forward + backward pass (mLSTMexp, upstream dH ~ N(0,1)) over the xLSTM-7B layer shape
B=4, S=16384, NH=8, DHQK=256, DHHV=512, chunk_size=128, bf16 inputs / fp32 states, synthetic N(0,1) data resident
in HBM before the timed region.  `value` is algorithmic TFLOP/s: 0.9964 TFLOP per step (matmul flops only,
causal work counted once, no recomputation) divided by the time per step.

Timing protocol (the reference's, mlstm_kernels/utils/benchmark/runtime.py:30-170): W untimed warm-up steps, then
exactly K timed steps; before every step a 512 MB buffer is zeroed to flush the L2 and the 256 MB memory-side cache,
gradients are reset, and the step is bracketed by a pair of HIP events on the launch stream; `ms_per_step` is the
MEDIAN of the K event times (the mean and the wall clock over the whole loop, flushes included, are reported next to
it).  Per-kernel durations come from a SEPARATE untimed pass over the same workload, in which the library records a
pair of HIP events around every kernel launch (mlstm_hip_profile_enable).

Objects on the JSON line besides the contract's keys:
  roofline      -- the chunkwise kernel with the largest share of the step against the bf16 MFMA peak: algorithmic
                   flops of one launch / its average duration; `traffic` = measured HBM bytes per launch, parsed from
                   the rocprofv3 counter summary under profiles/ (null when that file has no row for the kernel).
  peak_memory_gb -- peak device memory of one forward+backward pass (inputs, outputs, gradients, workspaces; without
                   the benchmark's own flush buffer); the reference's benchmark reports 9.0-9.9 GB for this workload.
  roofline_hbm  -- the same kernel against the HBM peak (algorithmic bytes per launch).
  roofline_step -- the whole forward+backward step against the HBM peak: algorithmic bytes if every operand moved once
                   and no chunk state travelled (4.31 GB), algorithmic bytes of this kernel decomposition (with the
                   kept chunk states), bytes measured by rocprofv3 (FETCH_SIZE + WRITE_SIZE summed over the five matrix
                   kernels, from profiles/), achieved GB/s = measured bytes / ms_per_step and its fraction of the
                   peak, and executed over algorithmic matrix flops (SQ_INSTS_VALU_MFMA_MOPS_BF16 x 512, from
                   profiles/).  `profile_kernel_ms` are the kernel durations of the profiled run: the counters describe
                   this run only where they agree with `kernels` (`profile_matches_run`).
  kernels       -- average duration, algorithmic TFLOP/s and GB/s of every kernel of the step.
  decode_step   -- fused decode step at B=256 after a chunkwise prefill of 2048 positions: ms per step, algorithmic
                   GB/s, its own HBM roofline; B=64 and B=16 (whose state fits the memory-side cache: "bound": "mall");
                   multi_token: 128 tokens per (batch, head) in ONE launch of the multi-token kernel.
  extra         -- the other benchmark configurations of the reference, same protocol: B=16/S=4096 and B=64/S=1024 (fwd+bwd), the
                   sigmoid gate with a non-zero initial state at B=4/S=16384, float16 operands at B=4/S=16384,
                   forward-only at B=4/S=16384 (without and with the last states returned), and the forward and the
                   forward+backward with the multi-head layer norm fused into the output kernel.
  cpu_baseline  -- the fp32 PyTorch oracle (restatement of the reference's native chunkwise forward + custom backward)
                   timed on this box's host cores on the same workload, plus the oracle's decode step.

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-extra]
"""
from __future__ import annotations

import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# ---- workload and algorithmic work (per token and head; DHQK=256, DHHV=512, L=128)
B, S, NH, DHQK, DHHV, CHUNK = 4, 16384, 8, 256, 512, 128
TOKEN_HEADS = B * S * NH
FLOPS_PER_TOKEN_HEAD = {
    # forward: 4*dqk*dhv + L*(dqk+dhv) = 622592
    "scan_fw": 2 * DHQK * DHHV,                         # K^T (a.V)
    "par_h": 2 * DHQK * DHHV + CHUNK * (DHQK + DHHV),   # Q C_prev, causal Q K^T and Sbar V
    # backward: 8*dqk*dhv + L*(3*dqk + 2*dhv) = 1277952
    "scan_bw": 2 * DHQK * DHHV,                         # Q^T dH
    "par_dv": 2 * DHQK * DHHV + CHUNK * (DHQK + DHHV),  # K dC, causal Q K^T and Sbar^T dH
    # dQ and dK run as one launch: dH C^T, causal dH V^T and dS K; V dC^T, causal dS^T Q
    "par_dqdk": 2 * DHQK * DHHV + CHUNK * (DHHV + DHQK) + 2 * DHQK * DHHV + CHUNK * DHQK,
}
# the fused sequential kernels do the work of a scan plus the chunk-parallel kernel that follows it
FLOPS_PER_TOKEN_HEAD["fused_fw"] = FLOPS_PER_TOKEN_HEAD["scan_fw"] + FLOPS_PER_TOKEN_HEAD["par_h"]
FLOPS_PER_TOKEN_HEAD["fused_dv"] = FLOPS_PER_TOKEN_HEAD["scan_bw"] + FLOPS_PER_TOKEN_HEAD["par_dv"]
FLOPS_PER_TOKEN_HEAD["scan_fw_recompute"] = FLOPS_PER_TOKEN_HEAD["scan_fw"]   # the state scan run again in the backward
FLOPS_FW = 4 * DHQK * DHHV + CHUNK * (DHQK + DHHV)
FLOPS_BW = 8 * DHQK * DHHV + CHUNK * (3 * DHQK + 2 * DHHV)
assert sum(FLOPS_PER_TOKEN_HEAD[n] for n in ("fused_fw", "fused_dv", "par_dqdk")) == FLOPS_FW + FLOPS_BW
PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E
FLUSH_BYTES = 512 << 20     # twice the memory-side cache
# decode step: bytes per (batch, head): C and n read+write fp32, m read+write, q,k,v in, h out (bf16), i,f
STEP_BYTES_PER_BH = 2 * DHQK * DHHV * 4 + 2 * DHQK * 4 + 2 * 4 + (2 * DHQK + DHHV) * 2 + DHHV * 2 + 2 * 2
DECODE_B, DECODE_PREFILL, DECODE_STEPS, DECODE_WARMUP = 256, 2048, 128, 10
MALL_BYTES = 256 << 20
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "tfla_fwbw_B4_S16384__pmc_hbm_traffic.md")
SQ_PROFILE = os.path.join(ROOT, "profiles", "tfla_fwbw_B4_S16384__pmc_sq_counters.md")
MATRIX_KERNELS = ("scan_fw", "par_h", "scan_bw", "par_dv", "par_dqdk")
# minimal HBM bytes per token and head: forward q, k, v in, H out, i, f (3076); backward q, k, v, dH, i, f in, dQ, dK,
# dV, dI, dF out (5136)
IO_ONCE_BYTES_PER_TOKEN_HEAD = 3076 + 5136


def algorithmic_bytes(stride: int) -> dict:
    """HBM bytes per launch if every operand moved once: bf16 q/k 268 MB each, v/dH/H/dV 537 MB each, bf16 chunk states
    (one per `stride` chunks of 128 positions) 1074 MB / stride per tensor."""
    qb, vb = B * NH * S * DHQK * 2, B * NH * S * DHHV * 2
    sb = B * NH * -(-(S // CHUNK) // stride) * DHQK * DHHV * 2
    return {
        "scan_fw": qb + vb + sb, "par_h": 2 * qb + 2 * vb + sb,
        "scan_bw": qb + vb + sb, "par_dv": 2 * qb + 2 * vb + sb,
        "par_dqdk": 4 * qb + 2 * vb + 2 * sb,   # Q, K, V, dH once for both gradients; C and dC states; dQ, dK out
    }


def measured_traffic() -> dict:
    """{kernel: HBM bytes per launch} parsed from the rocprofv3 FETCH_SIZE / WRITE_SIZE summary under profiles/
    (table rows `| kernel | fetched MB | written MB | total MB |`); empty when the file is absent."""
    out = {}
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return out
    for m in re.finditer(r"^\|\s*(\w+)\s*\|\s*([\d.]+)\s*\|\s*([\d.]+)\s*\|\s*([\d.]+)\s*\|\s*$", text, re.M):
        out[m.group(1)] = float(m.group(4)) * 1e6
    return out


def measured_mfma_flops() -> dict:
    """{kernel: executed matrix flops per launch} from the SQ counter summary under profiles/ (column MFMA MOPS, units
    of 512 flop), and {kernel: ms} the durations of that profiled run (row `profiled run, ms per launch`)."""
    flops, ms = {}, {}
    try:
        text = open(SQ_PROFILE).read()
    except OSError:
        return flops, ms
    for line in text.splitlines():
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if len(cells) >= 9 and cells[0] in MATRIX_KERNELS and cells[7].isdigit():
            flops[cells[0]] = int(cells[7]) * 512.0
    m = re.search(r"profiled run, ms per launch:\s*(\{.*\})", text)
    if m:
        ms = json.loads(m.group(1))
    return flops, ms


def cpu_model() -> str:
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(torch):
    """fp32 oracle on the host cores this process may use (the thread count the environment sets for one GPU's share of
    the box): chunkwise forward+backward on the whole workload (all 32 (batch, head) pairs at S=16384), and the decode
    step at B=16."""
    import oracle as O

    threads = torch.get_num_threads()
    g = torch.Generator().manual_seed(0)
    nh_s = B * NH  # every (batch, head) pair is independent, so one "batch" of 32 heads
    q = torch.randn(1, nh_s, S, DHQK, generator=g).bfloat16().float()
    k = torch.randn(1, nh_s, S, DHQK, generator=g).bfloat16().float()
    v = torch.randn(1, nh_s, S, DHHV, generator=g).bfloat16().float()
    dH = torch.randn(1, nh_s, S, DHHV, generator=g).bfloat16().float()
    i = torch.randn(1, nh_s, S, generator=g)
    f = 3 + torch.randn(1, nh_s, S, generator=g)
    O.chunkwise_bw(q[:, :1, :1024], k[:, :1, :1024], v[:, :1, :1024], i[:, :1, :1024], f[:, :1, :1024], dH[:, :1, :1024], chunk_size=CHUNK)
    times = []
    for _ in range(5):
        t0 = time.perf_counter()
        O.chunkwise_bw(q, k, v, i, f, dH, chunk_size=CHUNK)   # runs the forward (all states) and the backward
        times.append(time.perf_counter() - t0)
    t = sorted(times)[len(times) // 2]
    flops = (FLOPS_FW + FLOPS_BW) * nh_s * S
    del q, k, v, dH, i, f
    # decode step: python loop of the oracle step, fp32 state, B=16
    Bd, nsteps = 16, 12
    c, n, m = torch.randn(Bd, NH, DHQK, DHHV, generator=g), torch.randn(Bd, NH, DHQK, generator=g), torch.randn(Bd, NH, 1, generator=g)
    toks = [(torch.randn(Bd, NH, DHQK, generator=g), torch.randn(Bd, NH, DHQK, generator=g), torch.randn(Bd, NH, DHHV, generator=g),
             torch.randn(Bd, NH, 1, generator=g), 3 + torch.randn(Bd, NH, 1, generator=g)) for _ in range(nsteps + 2)]
    st = []
    for idx, tok in enumerate(toks):
        t0 = time.perf_counter()
        _, (c, n, m) = O.recurrent_step(*tok, c, n, m)
        if idx >= 2:
            st.append(time.perf_counter() - t0)
    ts = sorted(st)[len(st) // 2]
    return {
        "value": round(flops / t / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "cpu_model": cpu_model(), "host_logical_cpus": os.cpu_count(),
        "sample": f"fp32 oracle fwd+bwd on all {B * NH} (batch,head) pairs at S={S}: {t:.2f} s per pass, median of 5 after a "
                  f"warm-up; {threads} threads = this process's share of the host",
        "decode_step": {"value": round(STEP_BYTES_PER_BH * Bd * NH / ts / 1e9, 2), "unit": "GB/s", "ms_per_step": round(ts * 1e3, 3),
                        "sample": f"fp32 oracle step at B={Bd}, NH={NH}: median of {nsteps} consecutive steps after 2 warm-up steps"},
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip the other benchmark configurations and the small decode batches")
    ap.add_argument("--state-stride", type=int, default=0, help="chunk states kept every n-th chunk (0 = library default)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures the hot path on ONE GPU; --gpus > 1 is not supported "
              "(the path shards over batch and heads without communication).", file=sys.stderr)
        sys.exit(2)

    import torch

    from mlstm_kernels_amd import _lib
    from mlstm_kernels_amd.torch.chunkwise import mlstm_chunkwise__hip_xl_chunk, mlstm_siging_chunkwise__hip_xl_chunk
    from mlstm_kernels_amd.torch.recurrent import mlstm_recurrent_step__hip_fw

    _lib.get_lib()  # fail loudly if the HIP library is missing
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s: torch.randn(*s, device=dev, generator=gen)
    flush = torch.empty(FLUSH_BYTES, dtype=torch.uint8, device=dev)
    intra = {} if args.state_stride == 0 else {"chunk_size_intra": CHUNK * args.state_stride}
    stride = args.state_stride or _lib.default_state_stride(B, NH, S, DHQK, DHHV)

    def run_config(Bc, Sc, steps, warmup, sig=False, init=False, backward=True, profile_steps=3, head_norm="none",
                   dtype=torch.bfloat16, last_states=False, recompute=False):
        """Times `steps` passes of one configuration (median of per-step HIP-event times, caches flushed before every
        step), then profiles `profile_steps` further passes kernel by kernel."""
        q = rn(Bc, NH, Sc, DHQK).to(dtype).requires_grad_(backward)
        k = rn(Bc, NH, Sc, DHQK).to(dtype).requires_grad_(backward)
        v = rn(Bc, NH, Sc, DHHV).to(dtype).requires_grad_(backward)
        i = rn(Bc, NH, Sc).requires_grad_(backward)
        f = (3 + rn(Bc, NH, Sc)).requires_grad_(backward)
        dH = rn(Bc, NH, Sc, DHHV).to(dtype)
        kw = dict(chunk_size=CHUNK, autocast_kernel_dtype=dtype, head_norm=head_norm, return_last_states=last_states, **intra)
        if recompute:
            kw["recompute_states_in_bw"] = True   # the reference's default saved-state policy
        if init:
            kw.update(c_initial=0.1 * rn(Bc, NH, DHQK, DHHV), n_initial=0.1 * rn(Bc, NH, DHQK),
                      m_initial=torch.zeros(Bc, NH, 1, device=dev))
        op = mlstm_siging_chunkwise__hip_xl_chunk if sig else mlstm_chunkwise__hip_xl_chunk

        def step():
            if backward:
                out = op(q, k, v, i, f, **kw)
                (out[0] if last_states else out).backward(dH)
            else:
                with torch.no_grad():
                    op(q, k, v, i, f, **kw)

        def prepare():
            for t in (q, k, v, i, f):
                t.grad = None
            flush.zero_()

        for _ in range(warmup):
            prepare()
            step()
        torch.cuda.synchronize()
        # peak device memory of one pass beyond what is allocated before it (inputs, upstream gradient, flush buffer):
        # the output, the gradients and the library's workspaces -- the quantity the reference's benchmark reports
        prepare()
        torch.cuda.synchronize()
        base_mem = torch.cuda.memory_allocated()
        torch.cuda.reset_peak_memory_stats()
        step()
        torch.cuda.synchronize()
        peak_extra = torch.cuda.max_memory_allocated() - base_mem
        peak_total = torch.cuda.max_memory_allocated() - flush.numel()
        events = []
        t0 = time.perf_counter()
        for _ in range(steps):
            prepare()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            step()
            e1.record()
            events.append((e0, e1))
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        times = sorted(a.elapsed_time(b) for a, b in events)
        median, mean = times[len(times) // 2], sum(times) / len(times)
        # separate untimed pass: per-kernel durations
        _lib.profile_read()
        _lib.profile_enable(True)
        for _ in range(profile_steps):
            prepare()
            step()
        torch.cuda.synchronize()
        _lib.profile_enable(False)
        kern = {name: (ms / max(cnt, 1), cnt) for name, (ms, cnt) in _lib.profile_read().items()}
        return {"median_ms": median, "mean_ms": mean, "min_ms": times[0], "wall_ms_incl_flush": wall / steps * 1e3, "kernels": kern,
                "peak_memory_gb": round(peak_total / 1e9, 3), "peak_memory_beyond_inputs_gb": round(peak_extra / 1e9, 3)}

    def kernel_table(kern, token_heads, alg_bytes=None):
        table = {}
        for name, (avg, cnt) in kern.items():
            entry = {"avg_ms": round(avg, 4), "launches": cnt}
            if name in FLOPS_PER_TOKEN_HEAD:
                entry["alg_tflops"] = round(FLOPS_PER_TOKEN_HEAD[name] * token_heads / (avg * 1e-3) / 1e12, 2)
            if alg_bytes and name in alg_bytes:
                entry["alg_gbs"] = round(alg_bytes[name] / (avg * 1e-3) / 1e9, 1)
            table[name] = entry
        return table

    # ---- headline: mLSTMexp fwd+bwd, B=4, S=16384
    head = run_config(B, S, args.steps, args.warmup, profile_steps=5)
    ms_per_step = head["median_ms"]
    tflops = (FLOPS_FW + FLOPS_BW) * TOKEN_HEADS / (ms_per_step * 1e-3) / 1e12
    alg_bytes = algorithmic_bytes(stride)
    kernels = kernel_table(head["kernels"], TOKEN_HEADS, alg_bytes)
    traffic = measured_traffic()
    dom = max((n for n in kernels if n in FLOPS_PER_TOKEN_HEAD), key=lambda n: kernels[n]["avg_ms"])
    roofline = {
        "bound": "mfma", "kernel": dom, "achieved": kernels[dom]["alg_tflops"], "peak": PEAK_BF16_TFLOPS,
        "unit": "TFLOP/s", "frac": round(kernels[dom]["alg_tflops"] / PEAK_BF16_TFLOPS, 4),
        "traffic": traffic.get(dom), "avg_launch_ms": kernels[dom]["avg_ms"],
    }
    # the same kernel against the HBM roofline (with materialised chunk states the step is bandwidth-bound; both
    # fractions are reported)
    roofline_hbm = {"bound": "hbm", "kernel": dom, "achieved": kernels[dom]["alg_gbs"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "frac": round(kernels[dom]["alg_gbs"] / PEAK_HBM_GBS, 4), "traffic": traffic.get(dom)}
    for name, entry in kernels.items():
        if name in traffic:
            entry["hbm_bytes_measured"] = traffic[name]
            entry["measured_gbs"] = round(traffic[name] / (entry["avg_ms"] * 1e-3) / 1e9, 1)   # rocprofv3 bytes / this run's time

    # ---- the whole step against the HBM roofline
    mfma_flops, prof_ms = measured_mfma_flops()
    have_all = all(k in traffic for k in MATRIX_KERNELS)
    step_bytes_measured = sum(traffic[k] for k in MATRIX_KERNELS) if have_all else None
    io_once = IO_ONCE_BYTES_PER_TOKEN_HEAD * TOKEN_HEADS
    roofline_step = {
        "bound": "hbm", "algorithmic_bytes_io_once": io_once,
        "algorithmic_bytes_this_decomposition": sum(alg_bytes.values()),
        "measured_bytes": step_bytes_measured, "peak": PEAK_HBM_GBS, "unit": "GB/s",
        "achieved": None if step_bytes_measured is None else round(step_bytes_measured / (ms_per_step * 1e-3) / 1e9, 1),
        "frac": None if step_bytes_measured is None else round(step_bytes_measured / (ms_per_step * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
        "achieved_io_once": round(io_once / (ms_per_step * 1e-3) / 1e9, 1),
        "frac_io_once": round(io_once / (ms_per_step * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
        "mfma_flops_executed": sum(mfma_flops.values()) if all(k in mfma_flops for k in MATRIX_KERNELS) else None,
        "mfma_flops_algorithmic": (FLOPS_FW + FLOPS_BW) * TOKEN_HEADS,
        "profile_kernel_ms": prof_ms or None,
        "source": "profiles/tfla_fwbw_B4_S16384__pmc_hbm_traffic.md, profiles/tfla_fwbw_B4_S16384__pmc_sq_counters.md",
    }
    if roofline_step["mfma_flops_executed"]:
        roofline_step["executed_over_algorithmic_flops"] = round(roofline_step["mfma_flops_executed"] / roofline_step["mfma_flops_algorithmic"], 3)
    if prof_ms:
        roofline_step["profile_matches_run"] = all(
            k in kernels and abs(kernels[k]["avg_ms"] - prof_ms[k]) <= 0.2 * prof_ms[k] for k in MATRIX_KERNELS if k in prof_ms)

    extra = {}
    if not args.no_extra:
        n_extra = max(5, args.steps // 2)
        for tag, cfg in (("exp_fwbw_B16_S4096", dict(Bc=16, Sc=4096)), ("exp_fwbw_B64_S1024", dict(Bc=64, Sc=1024)),
                         ("sig_fwbw_B4_S16384_init", dict(Bc=4, Sc=16384, sig=True, init=True)),
                         ("exp_fwbw_B4_S16384_float16", dict(Bc=4, Sc=16384, dtype=torch.float16)),
                         ("exp_fwbw_B4_S16384_recompute_states_in_bw", dict(Bc=4, Sc=16384, recompute=True)),
                         ("exp_fw_B4_S16384", dict(Bc=4, Sc=16384, backward=False)),
                         ("exp_fw_B4_S16384_last_states", dict(Bc=4, Sc=16384, backward=False, last_states=True)),
                         ("exp_fw_B4_S16384_head_norm_layer", dict(Bc=4, Sc=16384, backward=False, head_norm="layer")),
                         ("exp_fwbw_B4_S16384_head_norm_layer", dict(Bc=4, Sc=16384, head_norm="layer"))):
            r = run_config(steps=n_extra, warmup=2, **cfg)
            fl = (FLOPS_FW + (FLOPS_BW if cfg.get("backward", True) else 0)) * TOKEN_HEADS
            extra[tag] = {"ms_per_step": round(r["median_ms"], 4), "steps": n_extra,
                          "value": round(fl / (r["median_ms"] * 1e-3) / 1e12, 2), "unit": "TFLOP/s",
                          "peak_memory_gb": r["peak_memory_gb"],
                          "kernels": kernel_table(r["kernels"], TOKEN_HEADS)}
            torch.cuda.empty_cache()
    del flush
    torch.cuda.empty_cache()

    # ---- decode step: chunkwise prefill, then consecutive in-place steps (state carried, n/m ping-pong)
    def bench_decode(Bd, graph):
        qp, kp, vp = rn(Bd, NH, DECODE_PREFILL, DHQK).bfloat16(), rn(Bd, NH, DECODE_PREFILL, DHQK).bfloat16(), rn(Bd, NH, DECODE_PREFILL, DHHV).bfloat16()
        ip, fp = rn(Bd, NH, DECODE_PREFILL), 3 + rn(Bd, NH, DECODE_PREFILL)
        with torch.no_grad():
            _, (c, n, m) = mlstm_chunkwise__hip_xl_chunk(qp, kp, vp, ip, fp, return_last_states=True, chunk_size=CHUNK)
        del qp, kp, vp, ip, fp
        total = DECODE_WARMUP + DECODE_STEPS
        qs, ks, vs = rn(total, Bd, NH, DHQK).bfloat16(), rn(total, Bd, NH, DHQK).bfloat16(), rn(total, Bd, NH, DHHV).bfloat16()
        is_, fs = rn(total, Bd, NH, 1), 3 + rn(total, Bd, NH, 1)
        n_alt, m_alt = torch.empty_like(n), torch.empty_like(m)
        step_bytes = STEP_BYTES_PER_BH * Bd * NH
        # a state that fits the memory-side cache is served from it step after step: not an HBM figure
        bound = "hbm" if c.numel() * 4 > MALL_BYTES else "mall"
        if graph:
            # two steps (n/m ping-pong) per graph, tokens in static buffers refreshed by device-side copies
            sq, sk, sv = qs[:2].clone(), ks[:2].clone(), vs[:2].clone()
            si, sf = is_[:2].clone(), fs[:2].clone()
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                mlstm_recurrent_step__hip_fw(c, n, m, sq[0], sk[0], sv[0], si[0], sf[0], matC_new=c, vecN_new=n_alt, scaM_new=m_alt)
                mlstm_recurrent_step__hip_fw(c, n_alt, m_alt, sq[1], sk[1], sv[1], si[1], sf[1], matC_new=c, vecN_new=n, scaM_new=m)
            torch.cuda.current_stream().wait_stream(side)
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                mlstm_recurrent_step__hip_fw(c, n, m, sq[0], sk[0], sv[0], si[0], sf[0], matC_new=c, vecN_new=n_alt, scaM_new=m_alt)
                mlstm_recurrent_step__hip_fw(c, n_alt, m_alt, sq[1], sk[1], sv[1], si[1], sf[1], matC_new=c, vecN_new=n, scaM_new=m)
            for t in range(0, total, 2):
                if t == DECODE_WARMUP:
                    torch.cuda.synchronize()
                    t_dec = time.perf_counter()
                sq.copy_(qs[t:t + 2]); sk.copy_(ks[t:t + 2]); sv.copy_(vs[t:t + 2]); si.copy_(is_[t:t + 2]); sf.copy_(fs[t:t + 2])
                g.replay()
            torch.cuda.synchronize()
            dec_ms = (time.perf_counter() - t_dec) / DECODE_STEPS * 1e3
            return {"batch": Bd, "mode": "hip graph (2 steps per replay, incl. token copies)", "ms_per_step": round(dec_ms, 4),
                    "value": round(step_bytes / (dec_ms * 1e-3) / 1e9, 1), "unit": "GB/s", "bound": bound}
        _lib.profile_read()
        t_dec = 0.0
        for t in range(total):
            if t == DECODE_WARMUP:
                torch.cuda.synchronize()
                _lib.profile_enable(True)
                t_dec = time.perf_counter()
            h, (c, n_new, m_new) = mlstm_recurrent_step__hip_fw(c, n, m, qs[t], ks[t], vs[t], is_[t], fs[t],
                                                               matC_new=c, vecN_new=n_alt, scaM_new=m_alt)
            n_alt, m_alt, n, m = n, m, n_new, m_new
        torch.cuda.synchronize()
        dec_ms = (time.perf_counter() - t_dec) / DECODE_STEPS * 1e3
        _lib.profile_enable(False)
        st_ms, st_cnt = _lib.profile_read().get("step", (0.0, 1))
        step_kernel_ms = st_ms / max(st_cnt, 1)
        return {
            "batch": Bd, "mode": "eager", "steps": DECODE_STEPS, "ms_per_step": round(dec_ms, 4), "kernel_ms": round(step_kernel_ms, 4),
            "value": round(step_bytes / (dec_ms * 1e-3) / 1e9, 1), "unit": "GB/s", "bound": bound,
            "roofline": {"bound": bound, "kernel": "step", "achieved": round(step_bytes / (step_kernel_ms * 1e-3) / 1e9, 1),
                         "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": round(step_bytes / (step_kernel_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                         "traffic": traffic.get("step") if Bd == DECODE_B else None},
        }

    # ---- multi-token decode: DECODE_STEPS tokens in one launch, the state stays on chip between tokens
    def bench_decode_sequence(Bd):
        from mlstm_kernels_amd.torch.recurrent import mlstm_recurrent_sequence__hip
        T = DECODE_STEPS
        qs, ks, vs = rn(Bd, NH, T, DHQK).bfloat16(), rn(Bd, NH, T, DHQK).bfloat16(), rn(Bd, NH, T, DHHV).bfloat16()
        is_, fs = rn(Bd, NH, T), 3 + rn(Bd, NH, T)
        c, n, m = rn(Bd, NH, DHQK, DHHV), rn(Bd, NH, DHQK), rn(Bd, NH, 1)
        times = []
        for rep in range(4):
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            mlstm_recurrent_sequence__hip(qs, ks, vs, is_, fs, c, n, m, return_last_states=True)
            e1.record()
            torch.cuda.synchronize()
            times.append(e0.elapsed_time(e1))
        ms = sorted(times[1:])[1]
        return {"batch": Bd, "tokens": T, "mode": "one launch for all tokens (state read and written once)",
                "ms_total": round(ms, 4), "us_per_token": round(ms / T * 1e3, 3),
                "tokens_per_s": round(Bd * T / (ms * 1e-3), 1),
                "state_bytes_moved": 2 * Bd * NH * DHQK * DHHV * 4}

    # ---- the step with its states kept in bfloat16 (half the bytes per step; arithmetic still fp32)
    def bench_decode_bf16_state(Bd):
        bf = torch.bfloat16
        c, n, m = rn(Bd, NH, DHQK, DHHV).to(bf), rn(Bd, NH, DHQK).to(bf), rn(Bd, NH, 1).to(bf)
        n_alt, m_alt = torch.empty_like(n), torch.empty_like(m)
        total = DECODE_WARMUP + DECODE_STEPS
        qs, ks, vs = rn(total, Bd, NH, DHQK).to(bf), rn(total, Bd, NH, DHQK).to(bf), rn(total, Bd, NH, DHHV).to(bf)
        is_, fs = rn(total, Bd, NH, 1), 3 + rn(total, Bd, NH, 1)
        _lib.profile_read()
        for t in range(total):
            if t == DECODE_WARMUP:
                torch.cuda.synchronize()
                _lib.profile_enable(True)
                t0 = time.perf_counter()
            _, (c, n_new, m_new) = mlstm_recurrent_step__hip_fw(c, n, m, qs[t], ks[t], vs[t], is_[t], fs[t], matC_new=c,
                                                               vecN_new=n_alt, scaM_new=m_alt, dtype_state=bf)
            n_alt, m_alt, n, m = n, m, n_new, m_new
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / DECODE_STEPS * 1e3
        _lib.profile_enable(False)
        st_ms, st_cnt = _lib.profile_read().get("step", (0.0, 1))
        nbytes = (2 * DHQK * DHHV * 2 + 2 * DHQK * 2 + 2 * 2 + (2 * DHQK + DHHV) * 2 + DHHV * 2 + 2 * 4) * Bd * NH
        return {"batch": Bd, "mode": "eager, bfloat16 states", "steps": DECODE_STEPS, "ms_per_step": round(ms, 4),
                "kernel_ms": round(st_ms / max(st_cnt, 1), 4), "bytes_per_step": nbytes,
                "value": round(nbytes / (ms * 1e-3) / 1e9, 1), "unit": "GB/s",
                "bound": "hbm" if c.numel() * 2 > MALL_BYTES else "mall"}

    decode = bench_decode(DECODE_B, graph=False)
    if not args.no_extra:
        decode["bf16_state"] = bench_decode_bf16_state(DECODE_B)
        decode["other_batches"] = [bench_decode(b, graph=g_) for b in (64, 16) for g_ in (False, True)]
        decode["multi_token"] = [bench_decode_sequence(b) for b in (DECODE_B, 64, 16)]
    torch.cuda.empty_cache()

    out = {
        "metric": "TFLA fwd+bwd TFLOP/s at B*S=65536 (NH8,256/512); decode-step HBM GB/s",
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "mLSTMexp TFLA fwd+bwd, B=4 S=16384 NH=8 DHQK=256 DHHV=512 chunk=128 (BASELINE configs[2]); "
                               "decode step B=256 (configs[4])", "state_stride": stride},
        "timing": {"protocol": "median of per-step HIP-event times, 512 MB cache flush and gradient reset before every step",
                   "mean_ms": round(head["mean_ms"], 4), "min_ms": round(head["min_ms"], 4),
                   "wall_ms_per_step_incl_flush": round(head["wall_ms_incl_flush"], 4)},
        "peak_memory_gb": head["peak_memory_gb"], "peak_memory_beyond_inputs_gb": head["peak_memory_beyond_inputs_gb"],
        "roofline": roofline, "roofline_hbm": roofline_hbm, "roofline_step": roofline_step, "kernels": kernels, "decode_step": decode, "extra": extra,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(torch)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
