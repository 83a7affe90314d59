"""Writes tests/golden/chunkwise_small.npz: seeded bf16-representable inputs and the fp64 oracle's outputs
(forward, last states, gradients) for mLSTMexp and mLSTMsig at B=1, NH=1, S=128, DHQK=64, DHHV=64 with
non-zero initial states.  The reference ships no golden vectors for this path (its tests compare live
implementations), so this fixture is a regression anchor for the oracle -- whose correctness is pinned
separately by tests/test_oracle.py -- and a fixed known-answer case for the HIP kernels.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle as O  # noqa: E402


def main():
    B, NH, S, DQK, DHV = 1, 1, 128, 64, 64
    g = torch.Generator().manual_seed(20240611)
    rb = lambda *s: torch.randn(*s, generator=g).bfloat16().double()  # values exactly representable in bf16
    q, k, v, dH = rb(B, NH, S, DQK), rb(B, NH, S, DQK), rb(B, NH, S, DHV), rb(B, NH, S, DHV)
    i = torch.randn(B, NH, S, generator=g).double()
    f = (3.0 + torch.randn(B, NH, S, generator=g)).double()
    c0 = (0.1 * torch.randn(B, NH, DQK, DHV, generator=g)).double()
    n0 = (0.1 * torch.randn(B, NH, DQK, generator=g)).double()
    m0 = torch.zeros(B, NH, 1).double()
    out = dict(q=q, k=k, v=v, i=i, f=f, dH=dH, c0=c0, n0=n0, m0=m0)
    for tag, sig in (("exp", False), ("sig", True)):
        fw = O.chunkwise_fw(q, k, v, i, f, c0, n0, m0, chunk_size=32, siging=sig)
        bw = O.chunkwise_bw(q, k, v, i, f, dH, c0, n0, m0, None, chunk_size=32, siging=sig)
        out.update({f"{tag}_H": fw["H"], f"{tag}_C": fw["C_last"], f"{tag}_n": fw["n_last"], f"{tag}_m": fw["m_last"]})
        for name, t in zip(["dQ", "dK", "dV", "dI", "dF", "dC0"], bw):
            out[f"{tag}_{name}"] = t
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "chunkwise_small.npz")
    np.savez_compressed(path, **{k_: v_.numpy().astype(np.float32) for k_, v_ in out.items()})
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
