"""fp64 emulation of the chunkwise kernels' arithmetic with their 16-bit roundings made explicit (test infrastructure).

The HIP kernels multiply 16-bit operands on the matrix cores with fp32 accumulation.  Besides the inputs, four
intermediate operands are rounded to the 16-bit format: the gated score blocks, the chunk states the scans write
out, the row-scaled value-side operand of the scans, and the outputs.  This module restates the chunkwise formulation
of `oracle/mlstm_ref.py` (same equations, same reference lines) with a rounding function applied at exactly those
points and everything else in fp64.  With the identity as rounding function it reproduces the oracle (checked on the
CPU); with the kernels' format it predicts their output up to fp32 accumulation noise, so a GPU test can hold EVERY
element of H, dQ, dK, dV to the plain 2e-2/2e-2 bound against it: what separates the kernels from the exact oracle on
rows whose terms nearly cancel is then shown to be the operand format, not the kernels.

Grouping of the products (what decides which values get rounded): the state recurrences run in chunks of 128
positions; outputs are formed per window of `stride` chunks from the state kept at the window's boundary and the
score blocks of the whole window (stride 1: the plain chunkwise form).  The sequence length must be a multiple of the
window.  The training call is emulated (no last state returned: the forward scan rounds its value operand once)."""
from __future__ import annotations

import torch
import torch.nn.functional as F

L0 = 128  # chunk of the state recurrences


def _identity(x):
    return x


def rounder(dtype):
    """x -> x rounded to `dtype` (round to nearest even), returned in float64."""
    return lambda x: x.to(dtype).to(torch.float64)


def _scan_gates(i, f, siging):
    """Per 128-chunk gate quantities (oracle/mlstm_ref.py::_chunk_gates): b inclusive cumsum of logsig(f), g its last
    entry, a = g - b + itilde."""
    B, NH, S = i.shape
    NC = S // L0
    lf = F.logsigmoid(f).reshape(B, NH, NC, L0)
    it = (F.logsigmoid(i) if siging else i).reshape(B, NH, NC, L0)
    b = lf.cumsum(-1)
    g = b[..., -1]
    return lf, it, b, g, (g[..., None] - b) + it


def chunkwise_fw_rounded(q, k, v, i, f, c_initial=None, n_initial=None, m_initial=None, stride=1, eps=1e-6,
                         siging=False, normalize=True, rnd=_identity, nmax_given=None):
    """Forward.  Returns H (rounded like the kernel's output), nmax (B,NH,S), the per-chunk states (unrounded fp64
    accumulators) C_all (B,NH,NC+1,DQK,DHV), n_all, m_all, the per-position combined stabiliser m_comb, nmax_own (the
    emulation's own row normalisers) and den_abs, the sum of the magnitudes of the terms of every denominator.  `nmax_given` (B,NH,S): row normalisers to divide by
    instead of the emulation's own (a denominator whose terms nearly cancel is, summed in fp32, uncertain by about
    1e-6 of den_abs; a caller that has checked a kernel's normalisers to that accuracy passes them in so that the
    comparison of the outputs is about the matrix arithmetic alone)."""
    B, NH, S, DQK = q.shape
    DHV = v.shape[-1]
    W = L0 * stride
    assert S % W == 0, "the emulation needs a sequence length that is a multiple of the window"
    NC = S // L0
    s = DQK ** -0.5
    dt = torch.float64
    lf, it, b, g, a = _scan_gates(i, f, siging)
    # ---- state scan in chunks of 128 (native/fw.py:88-121): the value operand is scaled in fp32 and rounded once
    C = torch.zeros(B, NH, DQK, DHV, dtype=dt) if c_initial is None else c_initial.to(dt)
    n = torch.zeros(B, NH, DQK, dtype=dt) if n_initial is None else n_initial.to(dt)
    m = torch.zeros(B, NH, dtype=dt) if (m_initial is None or siging) else m_initial.to(dt).reshape(B, NH)
    C_all, n_all, m_all = [C], [n], [m]
    track_n = not (siging and not normalize)
    for c in range(NC):
        sl = slice(c * L0, (c + 1) * L0)
        m_next = torch.zeros_like(m) if siging else torch.maximum(g[:, :, c] + m, a[:, :, c].max(-1).values)
        abar = torch.exp(a[:, :, c] - m_next[..., None])
        gbar = torch.exp(g[:, :, c] + m - m_next)
        C = gbar[..., None, None] * C + k[:, :, sl].transpose(-1, -2) @ rnd(v[:, :, sl] * abar[..., None])
        if track_n:
            n = gbar[..., None] * n + (k[:, :, sl] * abar[..., None]).sum(-2)
        m = m_next
        C_all.append(C), n_all.append(n), m_all.append(m)
    # ---- outputs per window from the state kept at its boundary (native/fw.py:171-212)
    H = torch.empty(B, NH, S, DHV, dtype=dt)
    nmax_all = torch.ones(B, NH, S, dtype=dt)
    mcomb_all = torch.zeros(B, NH, S, dtype=dt)
    den_abs = torch.zeros(B, NH, S, dtype=dt)
    causal = torch.ones(W, W, dtype=torch.bool).tril()
    lfw, itw = lf.reshape(B, NH, S // W, W), it.reshape(B, NH, S // W, W)
    for w in range(S // W):
        sl = slice(w * W, (w + 1) * W)
        c0 = w * stride
        qc, kc, vc = q[:, :, sl], k[:, :, sl], v[:, :, sl]
        bw_ = lfw[:, :, w].cumsum(-1)
        logD = (bw_[..., :, None] - bw_[..., None, :]).masked_fill(~causal, float("-inf")) + itw[:, :, w][..., None, :]
        m_prev = m_all[c0]
        m_comb = torch.zeros_like(bw_) if siging else torch.maximum(bw_ + m_prev[..., None], logD.max(-1).values)
        Sbar = (qc @ kc.transpose(-1, -2)) * s * torch.exp(logD - m_comb[..., None])
        bbar = torch.exp(bw_ + m_prev[..., None] - m_comb)
        num = (qc @ rnd(C_all[c0])) * (bbar * s)[..., None] + rnd(Sbar) @ vc
        if track_n:
            den = (bbar * s) * (qc * n_all[c0][..., None, :]).sum(-1) + Sbar.sum(-1)
            floor = torch.ones_like(den) if siging else torch.exp(-m_comb)
            nmax = torch.maximum(den.abs(), floor)
            nmax_all[:, :, sl] = nmax
            den_abs[:, :, sl] = (bbar * s) * (qc.abs() * n_all[c0][..., None, :].abs()).sum(-1) + Sbar.abs().sum(-1)
            if nmax_given is not None:
                nmax = nmax_given[:, :, sl].to(dt)
            H[:, :, sl] = rnd(num / (nmax[..., None] + eps))
        else:
            H[:, :, sl] = rnd(num)
        mcomb_all[:, :, sl] = m_comb
    nmax_used = nmax_given.to(dt) if (nmax_given is not None and track_n) else nmax_all
    return {"H": H, "nmax": nmax_used, "nmax_own": nmax_all, "m_comb": mcomb_all, "C_all": C_all, "n_all": n_all,
            "m_all": m_all, "den_abs": den_abs}


def chunkwise_bw_rounded(q, k, v, i, f, dH, c_initial=None, n_initial=None, m_initial=None, stride=1, eps=1e-6,
                         siging=False, normalize=True, rnd=_identity, nmax_given=None):
    """Backward (native/bw.py:67-198): returns dQ, dK, dV rounded like the kernels' outputs."""
    B, NH, S, DQK = q.shape
    W = L0 * stride
    NC = S // L0
    s = DQK ** -0.5
    fw = chunkwise_fw_rounded(q, k, v, i, f, c_initial, n_initial, m_initial, stride, eps, siging, normalize, rnd,
                              nmax_given)
    C_all, m_all = fw["C_all"], fw["m_all"]
    track_n = not (siging and not normalize)
    rho = 1.0 / (fw["nmax"] + eps) if track_n else torch.ones_like(fw["nmax"])
    lf, it, b, g, a = _scan_gates(i, f, siging)
    m_comb128 = fw["m_comb"].reshape(B, NH, NC, L0)
    # ---- dC scan in chunks of 128 (bw.py:67-98): the dH rows are scaled in fp32 and rounded once; dC_all[c] is the
    # gradient of the state after chunk c-1 (= before chunk c)
    dC = torch.zeros_like(C_all[0])
    dC_all = [None] * (NC + 1)
    dC_all[NC] = dC
    for c in range(NC - 1, -1, -1):
        sl = slice(c * L0, (c + 1) * L0)
        bbar = torch.exp(b[:, :, c] + m_all[c][..., None] - m_comb128[:, :, c])
        gbar = torch.exp(g[:, :, c] + m_all[c] - m_all[c + 1])
        sc = bbar * s * rho[:, :, sl]
        dC = gbar[..., None, None] * dC + q[:, :, sl].transpose(-1, -2) @ rnd(dH[:, :, sl] * sc[..., None])
        dC_all[c] = dC
    # ---- gradients per window (bw.py:153-198)
    dQ, dK, dV = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    causal = torch.ones(W, W, dtype=torch.bool).tril()
    lfw, itw = lf.reshape(B, NH, S // W, W), it.reshape(B, NH, S // W, W)
    for w in range(S // W):
        sl = slice(w * W, (w + 1) * W)
        c0, c1 = w * stride, (w + 1) * stride
        qc, kc, vc, dhc, rc = q[:, :, sl], k[:, :, sl], v[:, :, sl], dH[:, :, sl], rho[:, :, sl]
        bw_ = lfw[:, :, w].cumsum(-1)
        gw = bw_[..., -1]
        logD = (bw_[..., :, None] - bw_[..., None, :]).masked_fill(~causal, float("-inf")) + itw[:, :, w][..., None, :]
        m_comb = fw["m_comb"][:, :, sl]
        D = torch.exp(logD - m_comb[..., None])
        bbar = torch.exp(bw_ + m_all[c0][..., None] - m_comb)
        abar = torch.exp((gw[..., None] - bw_) + itw[:, :, w] - m_all[c1][..., None])
        Pv = rnd((qc @ kc.transpose(-1, -2)) * s * D * rc[..., None])      # score block of the dV kernel (rho folded in)
        dS = rnd((dhc @ vc.transpose(-1, -2)) * s * D * rc[..., None])     # score block of the dQ/dK kernel
        dCn, Cp = rnd(dC_all[c1]), rnd(C_all[c0])
        dV[:, :, sl] = rnd(Pv.transpose(-1, -2) @ dhc + (kc @ dCn) * abar[..., None])
        dK[:, :, sl] = rnd(dS.transpose(-1, -2) @ qc + (vc @ dCn.transpose(-1, -2)) * abar[..., None])
        dQ[:, :, sl] = rnd(dS @ kc + (dhc @ Cp.transpose(-1, -2)) * (bbar * s * rc)[..., None])
    return dQ, dK, dV
