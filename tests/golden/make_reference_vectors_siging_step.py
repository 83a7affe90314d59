"""Writes tests/golden/reference_native_siging_step.npz: inputs and outputs of the reference's OWN
  * quadratic mLSTMsig forward and backward (mlstm_kernels/torch/parallel/native_siging/fw.py:14
    `mlstm_siging_parallel_fw`, native_siging/bw.py:9 `mlstm_siging_parallel_bw`), zero initial state, with and
    without normalisation -- the only native implementation of the sigmoid input gate the reference has, and
  * native decode step (mlstm_kernels/torch/recurrent/native_step.py:8 `mlstm_recurrent_step__native_fw`) from random
    non-zero states
on small seeded inputs.  The oracle's counterparts are pinned mathematically as well (recurrent == quadratic ==
chunkwise, fp64 autograd with detached normaliser, a hand-computed step); these vectors add the reference's own
numbers on top.

The three source files import only torch; they are loaded by file path (no package __init__, no Triton module is
executed).  This script runs only where /root/reference exists; the fixture it writes is plain data.

Usage:  python tests/golden/make_reference_vectors_siging_step.py
"""
import importlib.util
import os

import numpy as np
import torch

REF = "/root/reference/mlstm_kernels/torch"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_native_siging_step.npz")


def load(path, name):
    spec = importlib.util.spec_from_file_location(name, os.path.join(REF, path))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def bf16_round(t):
    return t.to(torch.bfloat16).to(torch.float64)


def siging_case(fw, bw, seed, B, NH, S, DQK, DHV, normalize):
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    q, k, v, dH = bf16_round(rn(B, NH, S, DQK)), bf16_round(rn(B, NH, S, DQK)), bf16_round(rn(B, NH, S, DHV)), bf16_round(rn(B, NH, S, DHV))
    i, f = rn(B, NH, S).float().double(), (3.0 + rn(B, NH, S)).float().double()
    H, n = fw.mlstm_siging_parallel_fw(q, k, v, i, f, eps=1e-6, stable_fgate=True, normalize=normalize)
    dQ, dK, dV, dI, dF = bw.mlstm_siging_parallel_bw(dH, q, k, v, i, f, n, eps=1e-6, stable_fgate=True, normalize=normalize)
    out = dict(q=q, k=k, v=v, i=i, f=f, dH=dH, H=H, dQ=dQ, dK=dK, dV=dV, dI=dI, dF=dF,
               meta=torch.tensor([B, NH, S, DQK, DHV, int(normalize)]))
    if normalize:
        out["n"] = n
    return out


def step_case(step, seed, B, NH, DQK, DHV, steps):
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    c, n, m = rn(B, NH, DQK, DHV).float().double(), rn(B, NH, DQK).float().double(), rn(B, NH, 1).float().double()
    out = dict(c0=c, n0=n, m0=m, meta=torch.tensor([B, NH, DQK, DHV, steps]))
    for t in range(steps):
        q, k, v = bf16_round(rn(B, NH, DQK)), bf16_round(rn(B, NH, DQK)), bf16_round(rn(B, NH, DHV))
        i, f = rn(B, NH, 1).float().double(), (3.0 + rn(B, NH, 1)).float().double()
        h, (c, n, m) = step.mlstm_recurrent_step__native_fw(c, n, m, q, k, v, i, f, eps=1e-6, dtype_state=torch.float64)
        out.update({f"q{t}": q, f"k{t}": k, f"v{t}": v, f"i{t}": i, f"f{t}": f, f"h{t}": h})
    out.update(c_last=c, n_last=n, m_last=m)
    return out


def main():
    fw = load("parallel/native_siging/fw.py", "ref_siging_fw")
    bw = load("parallel/native_siging/bw.py", "ref_siging_bw")
    step = load("recurrent/native_step.py", "ref_native_step")
    cases = {
        "sigA": siging_case(fw, bw, 0, 1, 1, 256, 64, 128, True),
        "sigB": siging_case(fw, bw, 1, 1, 2, 128, 128, 64, False),
        "stepA": step_case(step, 3, 2, 2, 64, 128, 3),
        "stepB": step_case(step, 4, 1, 3, 128, 64, 2),
    }
    flat = {}
    for name, d in cases.items():
        for key, t in d.items():
            arr = t.detach().numpy()
            flat[f"{name}_{key}"] = arr.astype(np.float32) if arr.dtype == np.float64 else arr
    np.savez_compressed(OUT, **flat)
    print("wrote", OUT, len(flat), "arrays,", os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
