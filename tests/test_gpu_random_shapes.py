"""Randomised parity sweep: shapes (ragged sequence lengths, head dimensions that are multiples of 64 only), both
gates, initial states, an upstream dC_last, both chunkwise paths, every state stride and both saved-state policies
(chunk states kept for the backward or recomputed in it), each against the fp64 oracle.  Tolerances are
norm-relative (bf16 operands): H 6e-3, gradients 8e-3, final C 1e-3 of its scale, gate gradients 5e-2 of theirs."""
import random

import pytest
import torch

import oracle as O
from helpers import rel_norm, rel_to_scale

pytestmark = pytest.mark.gpu


def _case(seed):
    rnd = random.Random(seed)
    cfg = dict(
        B=rnd.choice([1, 2, 3]), NH=rnd.choice([1, 2, 5]),
        S=rnd.choice([7, 64, 100, 128, 130, 255, 256, 300, 513, 777]),
        DQ=rnd.choice([64, 128, 192, 256, 320, 512]), DV=rnd.choice([64, 128, 192, 256, 320, 512, 768]),
        sig=rnd.random() < 0.3, init=rnd.random() < 0.5, dcl=rnd.random() < 0.4,
        f_offset=rnd.choice([0.0, 3.0, 5.0]), fused=rnd.random() < 0.5)
    cfg["normalize"] = (not cfg["sig"]) or rnd.random() < 0.7
    cfg["stride"] = rnd.choice([1, 2, 3, 4, 8])
    if cfg["DQ"] not in (128, 256):
        cfg["fused"] = False   # the fused path supports these two head dimensions only
    cfg["recompute"] = rnd.random() < 0.35
    return cfg


@pytest.mark.parametrize("seed", list(range(32)))
def test_random_shape_forward_backward(seed):
    from mlstm_kernels_amd.torch.chunkwise import mlstm_chunkwise__hip_xl_chunk, mlstm_siging_chunkwise__hip_xl_chunk

    c = _case(seed)
    B, NH, S, DQ, DV, sig, normalize = c["B"], c["NH"], c["S"], c["DQ"], c["DV"], c["sig"], c["normalize"]
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g)
    q, k, v, dH = rn(B, NH, S, DQ).bfloat16(), rn(B, NH, S, DQ).bfloat16(), rn(B, NH, S, DV).bfloat16(), rn(B, NH, S, DV).bfloat16()
    i, f = rn(B, NH, S), c["f_offset"] + rn(B, NH, S)
    c0 = n0 = m0 = dCl = None
    if c["init"]:
        c0, n0, m0 = 0.1 * rn(B, NH, DQ, DV), 0.1 * rn(B, NH, DQ), 0.3 * rn(B, NH, 1)
    if c["dcl"]:
        dCl = 0.1 * rn(B, NH, DQ, DV)
    d = lambda t: None if t is None else t.double()
    L = next(x for x in (64, 32, 16, 8, 4, 2, 1) if S % x == 0)
    m0_o = None if sig else d(m0)
    fw = O.chunkwise_fw(d(q), d(k), d(v), d(i), d(f), d(c0), d(n0), m0_o, chunk_size=L, siging=sig, normalize=normalize)
    bw = O.chunkwise_bw(d(q), d(k), d(v), d(i), d(f), d(dH), d(c0), d(n0), m0_o, d(dCl), chunk_size=L, siging=sig,
                        normalize=normalize)
    cu = lambda t: None if t is None else t.cuda()
    leaves = [cu(t).requires_grad_(True) for t in (q, k, v, i, f)]
    c0l = None if c0 is None else cu(c0).requires_grad_(True)
    kw = dict(c_initial=c0l, n_initial=cu(n0), m_initial=cu(m0), return_last_states=True, chunk_size=128,
              any_sequence_length=True, kernel_path="fused" if c["fused"] else "split",
              chunk_size_intra=128 * c["stride"], recompute_states_in_bw=c["recompute"])
    print(f"case {c}", flush=True)
    if sig:
        H, st = mlstm_siging_chunkwise__hip_xl_chunk(*leaves, normalize=normalize, **kw)
    else:
        H, st = mlstm_chunkwise__hip_xl_chunk(*leaves, **kw)
    loss = (H.float() * cu(dH).float()).sum()
    if c["dcl"]:
        loss = loss + (st[0] * cu(dCl)).sum()
    loss.backward()
    err = dict(H=rel_norm(H, fw["H"]), C=rel_to_scale(st[0], fw["C_last"]), dQ=rel_norm(leaves[0].grad, bw[0]),
               dK=rel_norm(leaves[1].grad, bw[1]), dV=rel_norm(leaves[2].grad, bw[2]),
               dI=rel_to_scale(leaves[3].grad, bw[3]), dF=rel_to_scale(leaves[4].grad, bw[4]))
    if c["init"]:
        err["dC0"] = rel_norm(c0l.grad, bw[5])
    lim = dict(H=6e-3, C=1e-3, dQ=8e-3, dK=8e-3, dV=8e-3, dI=5e-2, dF=5e-2, dC0=8e-3)
    bad = {name: e for name, e in err.items() if not e <= lim[name]}
    assert not bad, f"{c}: {bad}"
