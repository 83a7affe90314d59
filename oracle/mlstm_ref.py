"""fp32/fp64 PyTorch restatement of the reference's native mLSTM formulations (TEST INFRASTRUCTURE ONLY).

Every function works in the dtype of its inputs (feed fp64 for a tight oracle, fp32 for the CPU baseline).
Shapes: q, k (B, NH, S, DQK); v (B, NH, S, DHV); i, f (B, NH, S); C (B, NH, DQK, DHV); n (B, NH, DQK);
m (B, NH, 1).  ``siging=True`` selects the sigmoid-input-gate cell (mLSTMsig), otherwise the exponential
input gate (mLSTMexp).

Reference files each part follows (paths relative to the reference checkout):
  recurrent_step            mlstm_kernels/torch/recurrent/native_step.py:8-101
  recurrent_sequence        mlstm_kernels/torch/recurrent/native_sequence.py:13-122
  parallel_stablef_fw/_bw   mlstm_kernels/torch/parallel/native_stablef/fw.py:12-63, bw.py:9-82
  parallel_siging_fw/_bw    mlstm_kernels/torch/parallel/native_siging/fw.py:14-78, bw.py:9-103
  chunkwise_fw              mlstm_kernels/torch/chunkwise/native/fw.py:29-309
  chunkwise_bw              mlstm_kernels/torch/chunkwise/native/bw.py:31-349
  chunkwise sig variants    mlstm_kernels/triton/chunkwise/xl_chunk_siging/fw_kernel_recurrent.py:137-186,
                            fw_kernel_parallel.py:76-256 and
                            mlstm_kernels/torch/chunkwise/triton_xl_chunk_siging/chunkwise_gates.py:72-100
                            (no native chunkwise sig implementation exists in the reference).

How each part is pinned (tests/test_oracle.py, tests/test_golden.py): the decode step by its closed form and a
hand-computed vector; the forward by three independent formulations (recurrent, quadratic, chunkwise) agreeing in
fp64 for both gates, plus chunk-size, state-passing and stabiliser-shift invariance; the backward by fp64 autograd
through an independently written forward and by sum_d k*dK == sum_d v*dV; and the two conventions that only the
reference can state -- what the forward stores as n_out / m_out, and what the hand-written backward treats as
constant -- by outputs of the reference's own mlstm_chunkwise_fw / mlstm_chunkwise_bw on seeded inputs
(tests/golden/reference_native_chunkwise.npz, written by tests/golden/make_reference_vectors.py).  The sigmoid-gate
chunkwise variant has no native counterpart in the reference to take vectors from; it is pinned by the first two
groups of checks only.  No function here is "parity unpinned".
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

__all__ = [
    "recurrent_step",
    "recurrent_step_siging",
    "recurrent_sequence",
    "parallel_stablef_fw",
    "parallel_stablef_bw",
    "parallel_siging_fw",
    "parallel_siging_bw",
    "chunkwise_fw",
    "chunkwise_bw",
    "head_normalize",
    "head_normalize_bw",
    "mlstm_chunkwise__native_autograd",
    "mlstm_chunkwise__native_custbw",
    "mlstm_siging_chunkwise__native_custbw",
    "mlstm_recurrent_step__native",
    "mlstm_recurrent_sequence__native_fw",
]


# --------------------------------------------------------------------------------------------------
# recurrent formulation
# --------------------------------------------------------------------------------------------------
def recurrent_step(q, k, v, i, f, c, n, m, eps: float = 1e-6, dtype_state=None):
    """One decode step of mLSTMexp.  q,k (B,NH,DQK); v (B,NH,DHV); i,f,m (B,NH,1).

    Follows native_step.py:69-95: m' = max(logsig(f)+m, i); C' = exp(logsig(f)+m-m') C + exp(i-m') k v^T;
    n' likewise; h = (q/sqrt(d))^T C' / (max(|q/sqrt(d) . n'|, exp(-m')) + eps).
    Returns h in q's dtype and the new states in ``dtype_state`` (default: the dtype of ``c``).
    """
    dt_s = c.dtype if dtype_state is None else dtype_state
    dt_in = q.dtype
    c, n, m = c.to(dt_s), n.to(dt_s), m.to(dt_s)
    dqk = q.shape[-1]
    lf = F.logsigmoid(f.to(dt_s))
    ii = i.to(dt_s)
    m_new = torch.maximum(lf + m, ii)
    fa = torch.exp(lf + m - m_new)
    ia = torch.exp(ii - m_new)
    qs = q.to(dt_s) * dqk ** -0.5
    kk, vv = k.to(dt_s), v.to(dt_s)
    c_new = fa[..., None] * c + ia[..., None] * (kk[..., :, None] * vv[..., None, :])
    n_new = fa * n + ia * kk
    num = torch.einsum("bhd,bhde->bhe", qs, c_new)
    qn = (qs * n_new).sum(-1, keepdim=True)
    den = torch.maximum(qn.abs(), torch.exp(-m_new)) + eps
    h = (num / den).to(dt_in)
    return h, (c_new, n_new, m_new)


def recurrent_step_siging(q, k, v, i, f, c, n, eps: float = 1e-6, normalize: bool = True):
    """One decode step of mLSTMsig: C' = sig(f) C + sig(i) k v^T, n' likewise,
    h = q_s^T C' / (max(|q_s . n'|, 1) + eps)  (or the numerator alone when ``normalize`` is False)."""
    dqk = q.shape[-1]
    fa, ia = torch.sigmoid(f), torch.sigmoid(i)
    c_new = fa[..., None] * c + ia[..., None] * (k[..., :, None] * v[..., None, :])
    n_new = fa * n + ia * k
    qs = q * dqk ** -0.5
    num = torch.einsum("bhd,bhde->bhe", qs, c_new)
    if normalize:
        qn = (qs * n_new).sum(-1, keepdim=True)
        num = num / (torch.maximum(qn.abs(), torch.ones_like(qn)) + eps)
    return num, (c_new, n_new)


def recurrent_sequence(q, k, v, i, f, c_initial=None, n_initial=None, m_initial=None, eps: float = 1e-6,
                       siging: bool = False, normalize: bool = True, dtype_state=None):
    """Token-by-token loop over the step (native_sequence.py:13-122).  Returns H and the last states
    ((C, n, m) for mLSTMexp, (C, n) for mLSTMsig)."""
    B, NH, S, DQK = q.shape
    DHV = v.shape[-1]
    dt = q.dtype if dtype_state is None else dtype_state
    c = torch.zeros(B, NH, DQK, DHV, dtype=dt, device=q.device) if c_initial is None else c_initial.to(dt)
    n = torch.zeros(B, NH, DQK, dtype=dt, device=q.device) if n_initial is None else n_initial.to(dt)
    m = torch.zeros(B, NH, 1, dtype=dt, device=q.device) if m_initial is None else m_initial.to(dt)
    hs = []
    for t in range(S):
        it, ft = i[:, :, t, None], f[:, :, t, None]
        if siging:
            h, (c, n) = recurrent_step_siging(q[:, :, t], k[:, :, t], v[:, :, t], it, ft, c, n, eps, normalize)
        else:
            h, (c, n, m) = recurrent_step(q[:, :, t], k[:, :, t], v[:, :, t], it, ft, c, n, m, eps, dtype_state=dt)
        hs.append(h)
    H = torch.stack(hs, dim=2)
    return (H, (c, n)) if siging else (H, (c, n, m))


# --------------------------------------------------------------------------------------------------
# quadratic (parallel) formulation
# --------------------------------------------------------------------------------------------------
def _log_decay_matrix(lf: torch.Tensor) -> torch.Tensor:
    """(B,NH,S) log forget gates -> (B,NH,S,S) matrix with entry [t,j] = sum_{u=j+1..t} lf_u for j<=t and
    -inf above the diagonal.  Built by a column-wise cumulative sum of the strictly-lower-triangular
    broadcast (no subtraction of two large cumsums)."""
    S = lf.shape[-1]
    lower = lf[..., :, None].expand(*lf.shape, S).tril(-1)
    acc = lower.cumsum(-2)
    keep = torch.ones(S, S, dtype=torch.bool, device=lf.device).tril()
    return acc.masked_fill(~keep, float("-inf"))


def parallel_stablef_fw(q, k, v, i, f, eps: float = 1e-6):
    """Quadratic mLSTMexp forward from zero state.  Returns (H, n, m) with n, m of shape (B,NH,S)."""
    dqk = q.shape[-1]
    logD = _log_decay_matrix(F.logsigmoid(f)) + i[..., None, :]
    m = logD.max(-1, keepdim=True).values
    D = torch.exp(logD - m)
    Ct = (q @ k.transpose(-1, -2)) * dqk ** -0.5 * D
    n = torch.maximum(Ct.sum(-1, keepdim=True).abs(), torch.exp(-m))
    H = (Ct / (n + eps)) @ v
    return H, n.squeeze(-1), m.squeeze(-1)


def parallel_stablef_bw(dH, q, k, v, i, f, n, m, eps: float = 1e-6):
    """Quadratic mLSTMexp backward with the normaliser n and stabiliser m held constant."""
    dqk = q.shape[-1]
    s = dqk ** -0.5
    logD = _log_decay_matrix(F.logsigmoid(f)) + i[..., None, :]
    D = torch.exp(logD - m[..., None])
    dHn = dH / (n[..., None] + eps)
    dCt = dHn @ v.transpose(-1, -2)
    S = (q @ k.transpose(-1, -2)) * s
    P = dCt * D
    dI = (P * S).sum(-2)
    dQ = (P @ k) * s
    dK = (P.transpose(-1, -2) @ q) * s
    dV = (S * D).transpose(-1, -2) @ dHn
    acc = (q * dQ - k * dK).sum(-1)
    dF = acc.flip(-1).cumsum(-1).flip(-1) * torch.sigmoid(-f)
    return dQ, dK, dV, dI, dF


def parallel_siging_fw(q, k, v, i, f, eps: float = 1e-6, normalize: bool = True):
    """Quadratic mLSTMsig forward from zero state.  Returns (H, n) (n is None without normalisation)."""
    dqk = q.shape[-1]
    D = torch.exp(_log_decay_matrix(F.logsigmoid(f)) + F.logsigmoid(i)[..., None, :])
    Ct = (q @ k.transpose(-1, -2)) * dqk ** -0.5 * D
    if not normalize:
        return Ct @ v, None
    n = torch.maximum(Ct.sum(-1, keepdim=True).abs(), torch.ones_like(Ct[..., :1]))
    return (Ct / (n + eps)) @ v, n.squeeze(-1)


def parallel_siging_bw(dH, q, k, v, i, f, n, eps: float = 1e-6, normalize: bool = True):
    """Quadratic mLSTMsig backward, normaliser held constant."""
    dqk = q.shape[-1]
    s = dqk ** -0.5
    D = torch.exp(_log_decay_matrix(F.logsigmoid(f)) + F.logsigmoid(i)[..., None, :])
    dHn = dH / (n[..., None] + eps) if normalize else dH
    dCt = dHn @ v.transpose(-1, -2)
    S = (q @ k.transpose(-1, -2)) * s
    P = dCt * D
    dIbar = (P * S).sum(-2)
    dQ = (P @ k) * s
    dK = (P.transpose(-1, -2) @ q) * s
    dV = (S * D).transpose(-1, -2) @ dHn
    acc = (q * dQ - k * dK).sum(-1)
    dF = acc.flip(-1).cumsum(-1).flip(-1) * torch.sigmoid(-f)
    dI = dIbar * torch.sigmoid(-i)
    return dQ, dK, dV, dI, dF


# --------------------------------------------------------------------------------------------------
# chunkwise formulation
# --------------------------------------------------------------------------------------------------
def _chunk_gates(i, f, L: int, siging: bool):
    """b = inclusive within-chunk cumsum of logsig(f); g = b[-1]; a = (g - b) + itilde,
    itilde = i (exp gate) or logsig(i) (sig gate).  All (B,NH,NC,L) except g (B,NH,NC)."""
    B, NH, S = i.shape
    NC = S // L
    lf = F.logsigmoid(f).reshape(B, NH, NC, L)
    it = (F.logsigmoid(i) if siging else i).reshape(B, NH, NC, L)
    b = lf.cumsum(-1)
    g = b[..., -1]
    a = (g[..., None] - b) + it
    return b, g, a, it


def chunkwise_fw(q, k, v, i, f, c_initial=None, n_initial=None, m_initial=None, chunk_size: int = 64,
                 eps: float = 1e-6, siging: bool = False, normalize: bool = True,
                 return_all_states: bool = False, return_bounds: bool = False):
    """Chunkwise-parallel forward.  Returns a dict with H (B,NH,S,DHV), n_out/m_out (B,NH,S) (the per-row
    denominator max(|den|, floor) *without* eps and the combined stabiliser), the last states and,
    on request, the per-chunk states C_all (B,NH,NC+1,DQK,DHV), n_all (B,NH,NC+1,DQK), m_all (B,NH,NC+1)
    where index k holds the state *before* chunk k.

    ``return_bounds`` adds H_abs (B,NH,S,DHV): the sum of the MAGNITUDES of all products that enter an output element
    in this chunk decomposition, (|qbar| |C_prev| + |Sbar| |V|) / (nmax + eps).  An implementation that rounds one
    operand of every product to a p-bit significand deviates from the exact H by at most 2^-p H_abs (first order);
    tests use it to bound the elements whose normaliser nearly cancels.  Not part of the reference's algorithm."""
    B, NH, S, DQK = q.shape
    DHV = v.shape[-1]
    L = chunk_size
    assert S % L == 0, f"sequence length {S} is not divisible by the chunk size {L}"
    NC = S // L
    dt, dev = q.dtype, q.device
    s = DQK ** -0.5
    b, g, a, it = _chunk_gates(i, f, L, siging)
    C = torch.zeros(B, NH, DQK, DHV, dtype=dt, device=dev) if c_initial is None else c_initial.to(dt)
    n = torch.zeros(B, NH, DQK, dtype=dt, device=dev) if n_initial is None else n_initial.to(dt)
    m = torch.zeros(B, NH, dtype=dt, device=dev) if (m_initial is None or siging) else m_initial.to(dt).reshape(B, NH)
    causal = torch.ones(L, L, dtype=torch.bool, device=dev).tril()
    H = torch.empty(B, NH, S, DHV, dtype=dt, device=dev)
    H_abs = torch.empty(B, NH, S, DHV, dtype=dt, device=dev) if return_bounds else None
    n_out = torch.ones(B, NH, S, dtype=dt, device=dev)
    m_out = torch.zeros(B, NH, S, dtype=dt, device=dev)
    C_all, n_all, m_all = [], [], []
    for c_idx in range(NC):
        sl = slice(c_idx * L, (c_idx + 1) * L)
        qc, kc, vc = q[:, :, sl], k[:, :, sl], v[:, :, sl]
        bc, ac, gc, ic = b[:, :, c_idx], a[:, :, c_idx], g[:, :, c_idx], it[:, :, c_idx]
        if return_all_states:
            C_all.append(C), n_all.append(n), m_all.append(m)
        # ---- outputs of this chunk from the incoming state (fw.py:171-212)
        logD = (bc[..., :, None] - bc[..., None, :]).masked_fill(~causal, float("-inf")) + ic[..., None, :]
        if siging:
            m_comb = torch.zeros_like(bc)
        else:
            m_comb = torch.maximum(bc + m[..., None], logD.max(-1).values)
        D = torch.exp(logD - m_comb[..., None])
        Sbar = (qc @ kc.transpose(-1, -2)) * s * D
        bbar = torch.exp(bc + m[..., None] - m_comb)
        qbar = qc * (bbar * s)[..., None]
        num = qbar @ C + Sbar @ vc
        num_abs = qbar.abs() @ C.abs() + Sbar.abs() @ vc.abs() if return_bounds else None
        if siging and not normalize:
            H[:, :, sl] = num
            if return_bounds:
                H_abs[:, :, sl] = num_abs
        else:
            den = (qbar * n[..., None, :]).sum(-1) + Sbar.sum(-1)
            floor = torch.ones_like(den) if siging else torch.exp(-m_comb)
            nmax = torch.maximum(den.abs(), floor)
            H[:, :, sl] = num / (nmax[..., None] + eps)
            if return_bounds:
                H_abs[:, :, sl] = num_abs / (nmax[..., None] + eps)
            n_out[:, :, sl] = nmax
        m_out[:, :, sl] = m_comb
        # ---- state update over this chunk (fw.py:88-121)
        m_next = torch.zeros_like(m) if siging else torch.maximum(gc + m, ac.max(-1).values)
        abar = torch.exp(ac - m_next[..., None])
        gbar = torch.exp(gc + m - m_next)
        kbar = kc * abar[..., None]
        C = gbar[..., None, None] * C + kbar.transpose(-1, -2) @ vc
        if not (siging and not normalize):
            n = gbar[..., None] * n + kbar.sum(-2)
        m = m_next
    out = {"H": H, "n_out": n_out, "m_out": m_out, "C_last": C, "n_last": n, "m_last": m[..., None]}
    if return_bounds:
        out["H_abs"] = H_abs
    if return_all_states:
        C_all.append(C), n_all.append(n), m_all.append(m)
        out["C_all"] = torch.stack(C_all, 2)
        out["n_all"] = torch.stack(n_all, 2)
        out["m_all"] = torch.stack(m_all, 2)
    return out


def chunkwise_bw(q, k, v, i, f, dH, c_initial=None, n_initial=None, m_initial=None, dC_last=None,
                 chunk_size: int = 64, eps: float = 1e-6, siging: bool = False, normalize: bool = True,
                 return_bounds: bool = False):
    """Chunkwise backward with the reference's convention: n_out and every stabiliser are constants
    (bw.py:44-46), dI = sum_d v*dV (bw.py:326, times sig(-i) for the sig gate), dF is the reverse
    cumulative sum over the WHOLE sequence of sum_d(q*dQ - k*dK) times sig(-f) (bw.py:320-323).
    Returns dQ, dK, dV, dI, dF, dC_initial (None unless c_initial was given).

    ``return_bounds`` appends a dict with dQ_abs, dK_abs, dV_abs: the sums of the magnitudes of all products entering
    a gradient element in this chunk decomposition (the dC recurrence carried in magnitudes too, since an
    implementation that rounds the operands of the dC update carries that error along).  See chunkwise_fw."""
    B, NH, S, DQK = q.shape
    DHV = v.shape[-1]
    L = chunk_size
    NC = S // L
    s = DQK ** -0.5
    dev = q.device
    fw = chunkwise_fw(q, k, v, i, f, c_initial, n_initial, m_initial, L, eps, siging, normalize, True)
    b, g, a, it = _chunk_gates(i, f, L, siging)
    C_all, m_all = fw["C_all"], fw["m_all"]
    m_comb = fw["m_out"].reshape(B, NH, NC, L)
    if siging and not normalize:
        dHn = dH
    else:
        dHn = dH / (fw["n_out"][..., None] + eps)
    causal = torch.ones(L, L, dtype=torch.bool, device=dev).tril()
    dQ, dK, dV = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    dC = torch.zeros_like(C_all[:, :, 0]) if dC_last is None else dC_last.to(q.dtype)
    if return_bounds:
        dQa, dKa, dVa = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        dCa = dC.abs()
    for c_idx in range(NC - 1, -1, -1):
        sl = slice(c_idx * L, (c_idx + 1) * L)
        qc, kc, vc, dhc = q[:, :, sl], k[:, :, sl], v[:, :, sl], dHn[:, :, sl]
        bc, ac, gc, ic, mc = b[:, :, c_idx], a[:, :, c_idx], g[:, :, c_idx], it[:, :, c_idx], m_comb[:, :, c_idx]
        m_prev, m_next = m_all[:, :, c_idx], m_all[:, :, c_idx + 1]
        logD = (bc[..., :, None] - bc[..., None, :]).masked_fill(~causal, float("-inf")) + ic[..., None, :]
        D = torch.exp(logD - mc[..., None])
        Sbar = (qc @ kc.transpose(-1, -2)) * s * D
        dS = (dhc @ vc.transpose(-1, -2)) * D
        bbar = torch.exp(bc + m_prev[..., None] - mc)[..., None]
        abar = torch.exp(ac - m_next[..., None])[..., None]
        gbar = torch.exp(gc + m_prev - m_next)[..., None, None]
        C_prev = C_all[:, :, c_idx]
        dV[:, :, sl] = Sbar.transpose(-1, -2) @ dhc + (kc * abar) @ dC
        dK[:, :, sl] = (dS.transpose(-1, -2) @ qc) * s + (vc * abar) @ dC.transpose(-1, -2)
        dQ[:, :, sl] = (dS @ kc) * s + (dhc * bbar) @ (C_prev * s).transpose(-1, -2)
        if return_bounds:
            dVa[:, :, sl] = Sbar.abs().transpose(-1, -2) @ dhc.abs() + (kc.abs() * abar) @ dCa
            dKa[:, :, sl] = (dS.abs().transpose(-1, -2) @ qc.abs()) * s + (vc.abs() * abar) @ dCa.transpose(-1, -2)
            dQa[:, :, sl] = (dS.abs() @ kc.abs()) * s + (dhc.abs() * bbar) @ (C_prev.abs() * s).transpose(-1, -2)
            dCa = gbar * dCa + (qc.abs() * bbar * s).transpose(-1, -2) @ dhc.abs()
        dC = gbar * dC + (qc * bbar * s).transpose(-1, -2) @ dhc
    acc = (q * dQ - k * dK).sum(-1)
    dF = acc.flip(-1).cumsum(-1).flip(-1) * torch.sigmoid(-f)
    dI = (v * dV).sum(-1)
    if siging:
        dI = dI * torch.sigmoid(-i)
    if return_bounds:
        return dQ, dK, dV, dI, dF, (dC if c_initial is not None else None), {"dQ_abs": dQa, "dK_abs": dKa, "dV_abs": dVa}
    return dQ, dK, dV, dI, dF, (dC if c_initial is not None else None)


# --------------------------------------------------------------------------------------------------
# head norm (the op that follows the cell in the xLSTM block)
# --------------------------------------------------------------------------------------------------
def head_normalize(x, norm_specifier: str = "layer", eps: float = 1e-6):
    """Normalisation over the last dimension without scale parameters, as the reference states it in
    mlstm_kernels/utils/analysis/transfer_behavior/_norm_layers.py:11-64 (``apply_normalize``):
    "layer": (x - mean) * rsqrt(biased var + eps)  (:23-34);  "rms": x * rsqrt(mean(x^2) + eps)  (:11-20);
    "none": x.  Computed in the dtype of x (the tests feed fp64)."""
    if norm_specifier == "none":
        return x
    if norm_specifier == "rms":
        return x * torch.rsqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)
    if norm_specifier == "layer":
        xc = x - x.mean(dim=-1, keepdim=True)
        return xc * torch.rsqrt(x.var(dim=-1, keepdim=True, unbiased=False) + eps)
    raise ValueError(f"Unsupported norm specifier {norm_specifier}.")


def head_normalize_bw(dy, x, norm_specifier: str = "layer", eps: float = 1e-6):
    """Gradient of ``head_normalize`` with respect to x, in closed form (checked against autograd in the tests):
    with y = head_normalize(x) and rstd the reciprocal root above,
    "layer": rstd * (dy - mean(dy) - y * mean(dy * y));  "rms": rstd * (dy - y * mean(dy * y))."""
    if norm_specifier == "none":
        return dy
    y = head_normalize(x, norm_specifier, eps)
    if norm_specifier == "rms":
        rstd = torch.rsqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)
        return rstd * (dy - y * (dy * y).mean(dim=-1, keepdim=True))
    rstd = torch.rsqrt(x.var(dim=-1, keepdim=True, unbiased=False) + eps)
    return rstd * (dy - dy.mean(dim=-1, keepdim=True) - y * (dy * y).mean(dim=-1, keepdim=True))


# --------------------------------------------------------------------------------------------------
# operator-level wrappers with the reference's call signatures (used to exercise the boundary on CPU)
# --------------------------------------------------------------------------------------------------
def _pack_fw(out, return_last_states, siging):
    if not return_last_states:
        return out["H"]
    if siging:
        return out["H"], (out["C_last"], out["n_last"])
    return out["H"], (out["C_last"], out["n_last"], out["m_last"])


def mlstm_chunkwise__native_autograd(q, k, v, i, f, c_initial=None, n_initial=None, m_initial=None,
                                     return_last_states=False, eps=1e-6, chunk_size=64, **kwargs):
    """Forward only; gradients (if any) come from torch.autograd through the forward itself."""
    out = chunkwise_fw(q, k, v, i, f, c_initial, n_initial, m_initial, chunk_size, eps)
    return _pack_fw(out, return_last_states, False)


class _ChunkwiseCustBw(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, i, f, c0, n0, m0, return_last_states, chunk_size, eps, siging, normalize):
        out = chunkwise_fw(q, k, v, i, f, c0, n0, m0, chunk_size, eps, siging, normalize)
        ctx.save_for_backward(q, k, v, i, f, c0, n0, m0)
        ctx.cfg = (chunk_size, eps, siging, normalize)
        if return_last_states:
            return out["H"], out["C_last"], out["n_last"], out["m_last"]
        return out["H"], None, None, None

    @staticmethod
    def backward(ctx, dH, dC_last, dn_last, dm_last):
        q, k, v, i, f, c0, n0, m0 = ctx.saved_tensors
        L, eps, siging, normalize = ctx.cfg
        dQ, dK, dV, dI, dF, dC0 = chunkwise_bw(q, k, v, i, f, dH, c0, n0, m0, dC_last, L, eps, siging, normalize)
        dn0 = torch.zeros_like(n0) if n0 is not None else None
        dm0 = torch.zeros_like(m0) if m0 is not None else None
        return dQ, dK, dV, dI, dF, dC0, dn0, dm0, None, None, None, None, None


def mlstm_chunkwise__native_custbw(q, k, v, i, f, c_initial=None, n_initial=None, m_initial=None,
                                   return_last_states=False, eps=1e-6, chunk_size=64, autocast_kernel_dtype=None,
                                   **kwargs):
    H, C, n, m = _ChunkwiseCustBw.apply(q, k, v, i, f, c_initial, n_initial, m_initial, return_last_states,
                                        chunk_size, eps, False, True)
    return (H, (C, n, m)) if return_last_states else H


def mlstm_siging_chunkwise__native_custbw(q, k, v, i, f, c_initial=None, n_initial=None, m_initial=None,
                                          return_last_states=False, eps=1e-6, normalize=True, chunk_size=64,
                                          autocast_kernel_dtype=None, **kwargs):
    H, C, n, _ = _ChunkwiseCustBw.apply(q, k, v, i, f, c_initial, n_initial, None, return_last_states,
                                        chunk_size, eps, True, normalize)
    return (H, (C, n)) if return_last_states else H


def mlstm_recurrent_step__native(q, k, v, i, f, c, n, m, eps=1e-6, dtype_state=torch.float32, **kwargs):
    return recurrent_step(q, k, v, i, f, c, n, m, eps, dtype_state)


def mlstm_recurrent_sequence__native_fw(q, k, v, i, f, c_initial=None, n_initial=None, m_initial=None,
                                        return_last_states=False, eps=1e-6, dtype_state=torch.float32, **kwargs):
    H, states = recurrent_sequence(q, k, v, i, f, c_initial, n_initial, m_initial, eps, dtype_state=dtype_state)
    return (H, states) if return_last_states else H
