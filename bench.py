#!/usr/bin/env python3
"""Benchmark of the mLSTM hot path on one MI355X.

A "step" is one TFLA forward + backward pass (mLSTMexp, upstream dH ~ N(0,1)) over the xLSTM-7B layer shape
B=4, S=16384, NH=8, DHQK=256, DHHV=512, chunk_size=128, bf16 inputs / fp32 states, synthetic N(0,1) data resident
in HBM before the timed region.  `value` is algorithmic TFLOP/s: 0.9964 TFLOP per step (matmul flops only,
causal work counted once, no recomputation) divided by the measured time per step.  The same run also times the
fused decode step (B=256, 128 consecutive steps after a chunkwise prefill) and reports it as algorithmic GB/s.

Extra objects on the JSON line:
  roofline      -- the chunkwise kernel with the largest share of the step (MFMA bound): algorithmic flops of one
                   launch / its average duration, measured with HIP events the library records around every
                   kernel launch on the launch stream during the timed region.
  kernels       -- the same figure for every kernel of the step.
  decode_step   -- ms per step, algorithmic GB/s and its own HBM roofline object.
  cpu_baseline  -- the fp32 PyTorch oracle (a restatement of the reference's native chunkwise forward + custom
                   backward) timed on this box's host cores on a bounded sample of the same workload.

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# ---- workload and algorithmic work (per token and head; DHQK=256, DHHV=512, L=128)
B, S, NH, DHQK, DHHV, CHUNK = 4, 16384, 8, 256, 512, 128
TOKEN_HEADS = B * S * NH
FLOPS_PER_TOKEN_HEAD = {
    # forward: 4*dqk*dhv + L*(dqk+dhv) = 622592
    "scan_fw": 2 * DHQK * DHHV,                       # K^T (a.V)
    "par_h": 2 * DHQK * DHHV + CHUNK * (DHQK + DHHV),  # Q C_prev, causal Q K^T and Sbar V
    # backward: 8*dqk*dhv + L*(3*dqk + 2*dhv) = 1277952
    "scan_bw": 2 * DHQK * DHHV,                       # Q^T dH
    "par_dv": 2 * DHQK * DHHV + CHUNK * (DHQK + DHHV),  # K dC, causal Q K^T and Sbar^T dH
    "par_dq": 2 * DHQK * DHHV + CHUNK * (DHHV + DHQK),  # dH C^T, causal dH V^T and dS K
    "par_dk": 2 * DHQK * DHHV + CHUNK * DHQK,           # V dC^T, causal dS^T Q
}
# the fused sequential kernels do the work of a scan plus the chunk-parallel kernel that follows it
FLOPS_PER_TOKEN_HEAD["fused_fw"] = FLOPS_PER_TOKEN_HEAD["scan_fw"] + FLOPS_PER_TOKEN_HEAD["par_h"]
FLOPS_PER_TOKEN_HEAD["fused_dv"] = FLOPS_PER_TOKEN_HEAD["scan_bw"] + FLOPS_PER_TOKEN_HEAD["par_dv"]
# dQ and dK run as one launch
FLOPS_PER_TOKEN_HEAD["par_dqdk"] = FLOPS_PER_TOKEN_HEAD.pop("par_dq") + FLOPS_PER_TOKEN_HEAD.pop("par_dk")
FLOPS_FW = 4 * DHQK * DHHV + CHUNK * (DHQK + DHHV)
FLOPS_BW = 8 * DHQK * DHHV + CHUNK * (3 * DHQK + 2 * DHHV)
assert sum(FLOPS_PER_TOKEN_HEAD[n] for n in ("fused_fw", "fused_dv", "par_dqdk")) == FLOPS_FW + FLOPS_BW
# algorithmic HBM bytes per launch at this workload: every operand once (bf16 q/k 268 MB, v/dH/H 537 MB, bf16 chunk
# states 1074 MB per tensor)
_QB, _VB = B * NH * S * DHQK * 2, B * NH * S * DHHV * 2
_SB = B * NH * (S // CHUNK) * DHQK * DHHV * 2
ALG_BYTES = {
    "scan_fw": _QB + _VB + _SB, "par_h": 2 * _QB + 2 * _VB + _SB,
    "scan_bw": _QB + _VB + _SB, "par_dv": 2 * _QB + 2 * _VB + _SB,
    "par_dqdk": 4 * _QB + 2 * _VB + 2 * _SB,   # Q, K, V, dH once for both gradients; C and dC states; dQ, dK out
}
# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on this workload (calibrated against a
# copy kernel of known size; summary in profiles/tfla_fwbw_B4_S16384__step_B256__pmc_hbm_traffic.md)
MEASURED_HBM_BYTES = {
    "scan_fw": 2122e6, "par_h": 2763e6, "scan_bw": 1883e6, "par_dv": 2890e6, "par_dqdk": 4319e6,
    "step": 2163e6,
}
PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E
# decode step: bytes per (batch, head): C and n read+write fp32, m read+write, q,k,v in, h out (bf16), i,f
STEP_BYTES_PER_BH = 2 * DHQK * DHHV * 4 + 2 * DHQK * 4 + 2 * 4 + (2 * DHQK + DHHV) * 2 + DHHV * 2 + 2 * 2
DECODE_B, DECODE_PREFILL, DECODE_STEPS, DECODE_WARMUP = 256, 2048, 128, 10


def cpu_baseline(torch):
    """fp32 oracle forward+backward on a bounded sample: 8 of the 32 (batch, head) pairs, full S."""
    import oracle as O

    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    g = torch.Generator().manual_seed(0)
    nh_s = 32  # the whole workload: every (batch, head) pair is independent, so one "batch" of 32 heads
    q = torch.randn(1, nh_s, S, DHQK, generator=g).bfloat16().float()
    k = torch.randn(1, nh_s, S, DHQK, generator=g).bfloat16().float()
    v = torch.randn(1, nh_s, S, DHHV, generator=g).bfloat16().float()
    dH = torch.randn(1, nh_s, S, DHHV, generator=g).bfloat16().float()
    i = torch.randn(1, nh_s, S, generator=g)
    f = 3 + torch.randn(1, nh_s, S, generator=g)
    O.chunkwise_bw(q[:, :1, :1024], k[:, :1, :1024], v[:, :1, :1024], i[:, :1, :1024], f[:, :1, :1024], dH[:, :1, :1024], chunk_size=CHUNK)
    times = []
    for _ in range(9):
        t0 = time.perf_counter()
        O.chunkwise_bw(q, k, v, i, f, dH, chunk_size=CHUNK)   # runs the forward (all states) and the backward
        times.append(time.perf_counter() - t0)
    t = sorted(times)[len(times) // 2]
    flops = (FLOPS_FW + FLOPS_BW) * nh_s * S
    return {
        "value": round(flops / t / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "sample": f"fp32 oracle fwd+bwd on all {B * NH} (batch,head) pairs at S={S}: {t:.2f} s per pass, median of 9 after a warm-up",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures the hot path on ONE GPU; --gpus > 1 is not supported "
              "(the path shards over batch and heads without communication).", file=sys.stderr)
        sys.exit(2)

    import torch

    from mlstm_kernels_amd import _lib
    from mlstm_kernels_amd.torch.chunkwise import mlstm_chunkwise__hip_xl_chunk
    from mlstm_kernels_amd.torch.recurrent import mlstm_recurrent_step__hip_fw

    _lib.get_lib()  # fail loudly if the HIP library is missing
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s: torch.randn(*s, device=dev, generator=gen)
    q = rn(B, NH, S, DHQK).bfloat16().requires_grad_(True)
    k = rn(B, NH, S, DHQK).bfloat16().requires_grad_(True)
    v = rn(B, NH, S, DHHV).bfloat16().requires_grad_(True)
    i = rn(B, NH, S).requires_grad_(True)
    f = (3 + rn(B, NH, S)).requires_grad_(True)
    dH = rn(B, NH, S, DHHV).bfloat16()

    def step():
        for t in (q, k, v, i, f):
            t.grad = None
        H = mlstm_chunkwise__hip_xl_chunk(q, k, v, i, f, chunk_size=CHUNK, autocast_kernel_dtype=torch.bfloat16)
        H.backward(dH)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    _lib.profile_enable(True)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    _lib.profile_enable(False)
    kern = _lib.profile_read()
    ms_per_step = elapsed / args.steps * 1e3
    tflops = (FLOPS_FW + FLOPS_BW) * TOKEN_HEADS / (ms_per_step * 1e-3) / 1e12

    kernels = {}
    for name, (ms, cnt) in kern.items():
        avg = ms / max(cnt, 1)
        entry = {"avg_ms": round(avg, 4), "launches": cnt}
        if name in FLOPS_PER_TOKEN_HEAD:
            entry["alg_tflops"] = round(FLOPS_PER_TOKEN_HEAD[name] * TOKEN_HEADS / (avg * 1e-3) / 1e12, 2)
        kernels[name] = entry
    dom = max((n for n in kernels if n in FLOPS_PER_TOKEN_HEAD), key=lambda n: kernels[n]["avg_ms"])
    roofline = {
        "bound": "mfma", "kernel": dom, "achieved": kernels[dom]["alg_tflops"], "peak": PEAK_BF16_TFLOPS,
        "unit": "TFLOP/s", "frac": round(kernels[dom]["alg_tflops"] / PEAK_BF16_TFLOPS, 4),
        "traffic": MEASURED_HBM_BYTES.get(dom), "avg_launch_ms": kernels[dom]["avg_ms"],
    }
    # the same kernel against the HBM roofline (at 65 flop per byte of materialised-state traffic the step is
    # bandwidth-bound; both fractions are reported)
    gbs = ALG_BYTES[dom] / (kernels[dom]["avg_ms"] * 1e-3) / 1e9
    roofline_hbm = {"bound": "hbm", "kernel": dom, "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": MEASURED_HBM_BYTES.get(dom)}
    for name, entry in kernels.items():
        if name in ALG_BYTES:
            entry["alg_gbs"] = round(ALG_BYTES[name] / (entry["avg_ms"] * 1e-3) / 1e9, 1)
    del q, k, v, i, f, dH
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
                    "value": round(step_bytes / (dec_ms * 1e-3) / 1e9, 1), "unit": "GB/s"}
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
            "value": round(step_bytes / (dec_ms * 1e-3) / 1e9, 1), "unit": "GB/s",
            "roofline": {"bound": "hbm", "kernel": "step", "achieved": round(step_bytes / (step_kernel_ms * 1e-3) / 1e9, 1),
                         "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": round(step_bytes / (step_kernel_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                         "traffic": MEASURED_HBM_BYTES["step"] if Bd == DECODE_B else None},
        }

    decode = bench_decode(DECODE_B, graph=False)
    decode["other_batches"] = [bench_decode(b, graph=g_) for b in (64, 16) for g_ in (False, True)]
    torch.cuda.empty_cache()

    out = {
        "metric": "TFLA fwd+bwd TFLOP/s at B*S=65536 (NH8,256/512); decode-step HBM GB/s",
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "mLSTMexp TFLA fwd+bwd, B=4 S=16384 NH=8 DHQK=256 DHHV=512 chunk=128 (BASELINE configs[2]); "
                               "decode step B=256 (configs[4])"},
        "roofline": roofline, "roofline_hbm": roofline_hbm, "kernels": kernels, "decode_step": decode,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(torch)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
