"""Writes tests/golden/reference_native_chunkwise.npz: inputs and outputs of the reference's OWN native chunkwise
forward and backward (mlstm_kernels/torch/chunkwise/native/fw.py:224 `mlstm_chunkwise_fw`,
native/bw.py:206 `mlstm_chunkwise_bw`) on small seeded inputs.

Why these two functions and nothing else: everything the oracle computes is pinned by mathematics (three
formulations agreeing, fp64 autograd, invariances) EXCEPT two conventions that only the reference can state and a
misreading of which no such check would notice:
  * what the forward stores as vecN_out / vecM_out (where the exp(-m) floor and eps enter the stored normaliser),
  * which terms the hand-written backward treats as constants and over which span dF is accumulated.

The two source files are loaded by file path (torch + einops only; the package __init__ files, which pull in the
Triton wrappers, are not executed).  This script runs only where /root/reference exists; the fixture it writes is
plain data (inputs and expected outputs) and is what the tests read.

Usage:  python tests/golden/make_reference_vectors.py
"""
import importlib.util
import os
import sys
import types

import numpy as np
import torch

REF = "/root/reference/mlstm_kernels/torch/chunkwise/native"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_native_chunkwise.npz")


def load_native():
    pkg = types.ModuleType("refnative")
    pkg.__path__ = [REF]
    sys.modules["refnative"] = pkg
    mods = {}
    for name in ("fw", "bw"):
        spec = importlib.util.spec_from_file_location(f"refnative.{name}", os.path.join(REF, f"{name}.py"))
        mod = importlib.util.module_from_spec(spec)
        sys.modules[f"refnative.{name}"] = mod
        spec.loader.exec_module(mod)
        mods[name] = mod
    return mods["fw"], mods["bw"]


def bf16_round(t):
    return t.to(torch.bfloat16).to(torch.float64)


def case(fw, bw, seed, B, NH, S, DQK, DHV, L, init, dcl):
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    # q, k, v, dH are bf16-representable so that the HIP kernels consume exactly these values
    q, k, v, dH = bf16_round(rn(B, NH, S, DQK)), bf16_round(rn(B, NH, S, DQK)), bf16_round(rn(B, NH, S, DHV)), bf16_round(rn(B, NH, S, DHV))
    i, f = rn(B, NH, S).float().double(), (3.0 + rn(B, NH, S)).float().double()
    c0 = n0 = m0 = dCl = None
    if init:
        c0, n0 = (0.1 * rn(B, NH, DQK, DHV)).float().double(), (0.1 * rn(B, NH, DQK)).float().double()
        m0 = (0.5 * rn(B, NH, 1)).float().double()
    if dcl:
        dCl = (0.1 * rn(B, NH, DQK, DHV)).float().double()
    H, n_out, m_out, last, _ = fw.mlstm_chunkwise_fw(
        q, k, v, i, f, matC_initial=c0, vecN_initial=n0, scaM_initial=m0, return_last_states=True,
        chunk_size=L, eps=1e-6)
    dQ, dK, dV, dI, dF, dC0, _, _ = bw.mlstm_chunkwise_bw(
        q, k, v, i, f, matC_initial=c0, vecN_initial=n0, scaM_initial=m0, vecN_out=n_out, vecM_out=m_out,
        matDeltaH=dH, matDeltaC_last=dCl, CHUNK_SIZE=L, EPS=1e-6)
    out = dict(q=q, k=k, v=v, i=i, f=f, dH=dH, H=H, n_out=n_out, m_out=m_out, C_last=last[0], n_last=last[1],
               m_last=last[2], dQ=dQ, dK=dK, dV=dV, dI=dI, dF=dF)
    if init:
        out.update(c0=c0, n0=n0, m0=m0, dC0=dC0)
    if dcl:
        out.update(dC_last=dCl)
    out["meta"] = torch.tensor([B, NH, S, DQK, DHV, L, int(init), int(dcl)])
    return out


def main():
    fw, bw = load_native()
    cases = {
        "a": case(fw, bw, 0, 1, 2, 256, 64, 64, 64, False, False),    # the small fp32 shape, zero initial state
        "b": case(fw, bw, 1, 1, 2, 128, 64, 128, 32, True, True),     # initial states and an upstream dC_last
    }
    flat = {}
    for name, d in cases.items():
        for key, t in d.items():
            arr = t.detach().numpy()
            flat[f"{name}_{key}"] = arr.astype(np.float32) if arr.dtype == np.float64 else arr
    np.savez_compressed(OUT, **flat)
    print("wrote", OUT, {k: v.shape for k, v in flat.items() if k.startswith("a_")})


if __name__ == "__main__":
    main()
