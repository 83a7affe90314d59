"""Pins the CPU oracle (oracle/mlstm_ref.py) by relations the mathematics fixes, not by its own formulas:
three independent formulations agree, invariances hold, and the custom backward equals fp64 autograd
through an independently written forward whose normaliser/stabiliser are detached."""
import math

import pytest
import torch
import torch.nn.functional as F

import oracle as O

torch.set_default_dtype(torch.float32)


def make_inputs(B=1, NH=2, S=64, DQK=16, DHV=24, seed=0, dtype=torch.float64, f_offset=3.0):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, NH, S, DQK, generator=g, dtype=dtype)
    k = torch.randn(B, NH, S, DQK, generator=g, dtype=dtype)
    v = torch.randn(B, NH, S, DHV, generator=g, dtype=dtype)
    i = torch.randn(B, NH, S, generator=g, dtype=dtype)
    f = f_offset + torch.randn(B, NH, S, generator=g, dtype=dtype)
    return q, k, v, i, f


# ---------------------------------------------------------------- decode step: closed form from zero state
def test_step_closed_form_zero_state():
    B, NH, DQK, DHV = 2, 3, 8, 5
    g = torch.Generator().manual_seed(3)
    q, k = torch.randn(B, NH, DQK, generator=g, dtype=torch.float64), torch.randn(B, NH, DQK, generator=g, dtype=torch.float64)
    v = torch.randn(B, NH, DHV, generator=g, dtype=torch.float64)
    i, f = torch.randn(B, NH, 1, generator=g, dtype=torch.float64), torch.randn(B, NH, 1, generator=g, dtype=torch.float64)
    z = torch.zeros
    h, (c, n, m) = O.recurrent_step(q, k, v, i, f, z(B, NH, DQK, DHV, dtype=torch.float64), z(B, NH, DQK, dtype=torch.float64), z(B, NH, 1, dtype=torch.float64), eps=1e-6)
    for b in range(B):
        for hh in range(NH):
            lf = -math.log1p(math.exp(-f[b, hh, 0].item()))
            mm = max(lf, i[b, hh, 0].item())
            w = math.exp(i[b, hh, 0].item() - mm)
            s = w * float(q[b, hh] @ k[b, hh]) / math.sqrt(DQK)
            den = max(abs(s), math.exp(-mm)) + 1e-6
            assert abs(m[b, hh, 0].item() - mm) < 1e-12
            torch.testing.assert_close(h[b, hh], v[b, hh] * s / den, rtol=1e-10, atol=1e-12)
            torch.testing.assert_close(c[b, hh], w * torch.outer(k[b, hh], v[b, hh]), rtol=1e-10, atol=1e-12)
            torch.testing.assert_close(n[b, hh], w * k[b, hh], rtol=1e-10, atol=1e-12)


def test_step_known_answer_scalar():
    # d=1 hand-computed: f=0 -> logsig=-ln2, m=1, i=0.5: m'=max(-ln2+1, .5)=.5 ; f'=exp(-ln2+1-.5), i'=1
    one = lambda x: torch.tensor([[[x]]], dtype=torch.float64)
    h, (c, n, m) = O.recurrent_step(one(2.0), one(3.0), one(5.0), one(0.5), one(0.0),
                                    one(4.0)[..., None], one(-1.0), one(1.0), eps=0.0)
    fp = math.exp(-math.log(2) + 0.5)
    c_ref = fp * 4.0 + 15.0
    n_ref = fp * -1.0 + 3.0
    assert abs(c.item() - c_ref) < 1e-12 and abs(n.item() - n_ref) < 1e-12 and abs(m.item() - 0.5) < 1e-15
    assert abs(h.item() - (2.0 * c_ref) / max(abs(2.0 * n_ref), math.exp(-0.5))) < 1e-12


# ---------------------------------------------------------------- three formulations agree (mLSTMexp)
@pytest.mark.parametrize("dtype,tol", [(torch.float64, 1e-10), (torch.float32, 2e-5)])
@pytest.mark.parametrize("f_offset", [3.0, 0.0, -2.0])
def test_three_way_agreement_exp(dtype, tol, f_offset):
    q, k, v, i, f = make_inputs(dtype=dtype, f_offset=f_offset)
    H_par, n_par, m_par = O.parallel_stablef_fw(q, k, v, i, f)
    H_rec, (C_r, n_r, m_r) = O.recurrent_sequence(q, k, v, i, f)
    out = O.chunkwise_fw(q, k, v, i, f, chunk_size=16)
    for H in (H_rec, out["H"]):
        torch.testing.assert_close(H, H_par, rtol=tol, atol=tol)
    # the chunkwise/recurrent stabiliser also sees the (zero) initial m, the quadratic one does not:
    # only the unstabilised normaliser n*exp(m) is common to both
    torch.testing.assert_close(out["n_out"] * torch.exp(out["m_out"]), n_par * torch.exp(m_par), rtol=10 * tol, atol=tol)
    assert (out["m_out"] >= m_par - tol).all()
    scale = C_r.abs().max()
    assert (out["C_last"] - C_r).abs().max() <= tol * scale
    torch.testing.assert_close(out["n_last"], n_r, rtol=tol, atol=tol * float(n_r.abs().max()))
    torch.testing.assert_close(out["m_last"], m_r, rtol=tol, atol=tol)


def test_parallel_m_is_recurrent_m_except_zero_init_floor():
    # recurrent m starts from m0=0 and so is max(running, decayed 0); the quadratic form has no m0 term.
    # H nevertheless agrees (checked above) because n and the floor rescale together.
    q, k, v, i, f = make_inputs(S=32)
    out16, out8 = O.chunkwise_fw(q, k, v, i, f, chunk_size=16), O.chunkwise_fw(q, k, v, i, f, chunk_size=8)
    torch.testing.assert_close(out16["m_out"], out8["m_out"], rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("L", [8, 16, 32, 64])
def test_chunk_size_invariance(L):
    q, k, v, i, f = make_inputs(S=64)
    ref = O.chunkwise_fw(q, k, v, i, f, chunk_size=64)
    out = O.chunkwise_fw(q, k, v, i, f, chunk_size=L)
    torch.testing.assert_close(out["H"], ref["H"], rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(out["C_last"], ref["C_last"], rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(out["n_last"], ref["n_last"], rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(out["m_last"], ref["m_last"], rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("siging", [False, True])
def test_state_passing_invariance(siging):
    q, k, v, i, f = make_inputs(S=96, seed=5)
    g = torch.Generator().manual_seed(9)
    C0 = 0.1 * torch.randn(1, 2, 16, 24, generator=g, dtype=torch.float64)
    n0 = 0.1 * torch.randn(1, 2, 16, generator=g, dtype=torch.float64)
    m0 = torch.randn(1, 2, 1, generator=g, dtype=torch.float64)
    full = O.chunkwise_fw(q, k, v, i, f, C0, n0, m0, chunk_size=32, siging=siging)
    Hs, st = [], (C0, n0, m0)
    for lo, hi in ((0, 32), (32, 48), (48, 96)):
        part = O.chunkwise_fw(q[:, :, lo:hi], k[:, :, lo:hi], v[:, :, lo:hi], i[:, :, lo:hi], f[:, :, lo:hi],
                              *st, chunk_size=16, siging=siging)
        Hs.append(part["H"])
        st = (part["C_last"], part["n_last"], part["m_last"])
    torch.testing.assert_close(torch.cat(Hs, 2), full["H"], rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(st[0], full["C_last"], rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(st[1], full["n_last"], rtol=1e-10, atol=1e-10)
    # and against the token loop with the same initial state
    H_rec, st_rec = O.recurrent_sequence(q, k, v, i, f, C0, n0, m0, siging=siging)
    torch.testing.assert_close(full["H"], H_rec, rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(full["C_last"], st_rec[0], rtol=1e-10, atol=1e-10)


def test_stabiliser_shift_invariance():
    # (C0, n0, m0) and (e^-d C0, e^-d n0, m0 + d) describe the same unnormalised state
    q, k, v, i, f = make_inputs(S=32, seed=2)
    g = torch.Generator().manual_seed(1)
    C0 = torch.randn(1, 2, 16, 24, generator=g, dtype=torch.float64)
    n0 = torch.randn(1, 2, 16, generator=g, dtype=torch.float64)
    m0 = torch.zeros(1, 2, 1, dtype=torch.float64)
    d = 1.7
    a = O.chunkwise_fw(q, k, v, i, f, C0, n0, m0, chunk_size=16, eps=0.0)  # eps breaks the exact invariance
    b = O.chunkwise_fw(q, k, v, i, f, math.exp(-d) * C0, math.exp(-d) * n0, m0 + d, chunk_size=16, eps=0.0)
    torch.testing.assert_close(a["H"], b["H"], rtol=1e-9, atol=1e-9)
    sa = a["C_last"] * torch.exp(a["m_last"])[..., None]
    sb = b["C_last"] * torch.exp(b["m_last"])[..., None]
    torch.testing.assert_close(sa, sb, rtol=1e-9, atol=1e-9)


# ---------------------------------------------------------------- backward
def _quadratic_detached(q, k, v, i, f, C0=None, n0=None, m0=None, siging=False, normalize=True, eps=1e-6):
    """Independent quadratic forward with optional initial state; stabiliser and normaliser are detached,
    which is exactly the reference's gradient convention.  Also returns the (detached-m) last C."""
    S, DQK = q.shape[-2], q.shape[-1]
    s = DQK ** -0.5
    lf = F.logsigmoid(f)
    it = F.logsigmoid(i) if siging else i
    Bc = lf.cumsum(-1)                                            # B_t
    logD = Bc[..., :, None] - Bc[..., None, :] + it[..., None, :]
    mask = torch.ones(S, S, dtype=torch.bool).tril()
    logD = logD.masked_fill(~mask, float("-inf"))
    if siging:
        m = torch.zeros_like(Bc)
        m0v = torch.zeros_like(Bc[..., :1])
    else:
        m0v = torch.zeros_like(Bc[..., :1]) if m0 is None else m0
        m = torch.maximum(logD.max(-1).values, Bc + m0v).detach()
    W = torch.exp(logD - m[..., None])
    Sb = (q @ k.transpose(-1, -2)) * s * W
    num = Sb @ v
    den = Sb.sum(-1)
    if C0 is not None:
        qb = q * (torch.exp(Bc + m0v - m) * s)[..., None]
        num = num + qb @ C0
        den = den + (qb * n0[..., None, :]).sum(-1)
    if siging and not normalize:
        H = num
    else:
        floor = torch.ones_like(den) if siging else torch.exp(-m)
        H = num / (torch.maximum(den.abs(), floor).detach()[..., None] + eps)
    # last C with the final stabiliser held constant
    mS = m[..., -1:]
    wl = torch.exp(Bc[..., -1:] - Bc + it - mS)
    C_last = (k * wl[..., None]).transpose(-1, -2) @ v
    if C0 is not None:
        C_last = C_last + torch.exp(Bc[..., -1:] + m0v - mS)[..., None] * C0
    return H, C_last


@pytest.mark.parametrize("siging,normalize", [(False, True), (True, True), (True, False)])
def test_backward_equals_detached_autograd(siging, normalize):
    q, k, v, i, f = make_inputs(S=48, seed=11)
    g = torch.Generator().manual_seed(4)
    dH = torch.randn(v.shape, generator=g, dtype=torch.float64)
    leaves = [t.clone().requires_grad_(True) for t in (q, k, v, i, f)]
    H, _ = _quadratic_detached(*leaves, siging=siging, normalize=normalize)
    grads = torch.autograd.grad((H * dH).sum(), leaves)
    mine = O.chunkwise_bw(q, k, v, i, f, dH, chunk_size=16, siging=siging, normalize=normalize)
    for name, a, b in zip("QKVIF", mine[:5], grads):
        torch.testing.assert_close(a, b, rtol=1e-8, atol=1e-9, msg=lambda s: f"d{name}: {s}")
    # both expressions for the input-gate gradient coincide
    torch.testing.assert_close((k * mine[1]).sum(-1), (v * mine[2]).sum(-1), rtol=1e-8, atol=1e-9)
    # and the quadratic restatement of the same convention
    if siging:
        _, n_par = O.parallel_siging_fw(q, k, v, i, f, normalize=normalize)
        par = O.parallel_siging_bw(dH, q, k, v, i, f, n_par, normalize=normalize)
    else:
        _, n_par, m_par = O.parallel_stablef_fw(q, k, v, i, f)
        par = O.parallel_stablef_bw(dH, q, k, v, i, f, n_par, m_par)
    # (the quadratic stabiliser lacks the zero initial m, so eps=1e-6 enters at a different scale: 1e-5 here)
    for name, a, b in zip("QKVIF", mine[:5], par):
        torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-5, msg=lambda s: f"d{name} (parallel): {s}")


@pytest.mark.parametrize("siging", [False, True])
def test_backward_with_initial_state_and_dC_last(siging):
    q, k, v, i, f = make_inputs(S=32, seed=21)
    g = torch.Generator().manual_seed(8)
    C0 = 0.3 * torch.randn(1, 2, 16, 24, generator=g, dtype=torch.float64)
    n0 = 0.3 * torch.randn(1, 2, 16, generator=g, dtype=torch.float64)
    m0 = 0.5 * torch.randn(1, 2, 1, generator=g, dtype=torch.float64)
    dH = torch.randn(v.shape, generator=g, dtype=torch.float64)
    dCl = torch.randn(C0.shape, generator=g, dtype=torch.float64)
    # (a) initial state only: every gradient incl. dF and dC0 is the detached-autograd gradient
    leaves = [t.clone().requires_grad_(True) for t in (q, k, v, i, f, C0)]
    H, _ = _quadratic_detached(*leaves[:5], C0=leaves[5], n0=n0, m0=m0, siging=siging)
    grads = torch.autograd.grad((H * dH).sum(), leaves)
    mine = O.chunkwise_bw(q, k, v, i, f, dH, C0, n0, m0, None, chunk_size=8, siging=siging)
    for name, a, b in zip(["dQ", "dK", "dV", "dI", "dF", "dC0"], mine, grads):
        torch.testing.assert_close(a, b, rtol=1e-8, atol=1e-9, msg=lambda s: f"{name}: {s}")
    # (b) plus a gradient arriving through the last C state: dQ, dK, dV, dI, dC0 are true gradients
    # (the reference's dF formula drops a constant in this case and is followed as is, so dF is not compared)
    leaves = [t.clone().requires_grad_(True) for t in (q, k, v, i, f, C0)]
    H, C_last = _quadratic_detached(*leaves[:5], C0=leaves[5], n0=n0, m0=m0, siging=siging)
    grads = torch.autograd.grad((H * dH).sum() + (C_last * dCl).sum(), leaves)
    mine = O.chunkwise_bw(q, k, v, i, f, dH, C0, n0, m0, dCl, chunk_size=8, siging=siging)
    for idx, name in ((0, "dQ"), (1, "dK"), (2, "dV"), (3, "dI"), (5, "dC0")):
        torch.testing.assert_close(mine[idx], grads[idx], rtol=1e-8, atol=1e-9, msg=lambda s: f"{name}: {s}")


# ---------------------------------------------------------------- mLSTMsig: three formulations agree
@pytest.mark.parametrize("normalize", [True, False])
def test_three_way_agreement_sig(normalize):
    q, k, v, i, f = make_inputs(S=64, seed=13)
    H_par, n_par = O.parallel_siging_fw(q, k, v, i, f, normalize=normalize)
    H_rec, (C_r, n_r) = O.recurrent_sequence(q, k, v, i, f, siging=True, normalize=normalize)
    out = O.chunkwise_fw(q, k, v, i, f, chunk_size=16, siging=True, normalize=normalize)
    torch.testing.assert_close(H_rec, H_par, rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(out["H"], H_par, rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(out["C_last"], C_r, rtol=1e-10, atol=1e-10)
    if normalize:
        torch.testing.assert_close(out["n_out"], n_par, rtol=1e-10, atol=1e-10)
        torch.testing.assert_close(out["n_last"], n_r, rtol=1e-10, atol=1e-10)


# ---------------------------------------------------------------- operator wrappers
def test_custbw_wrapper_autograd_plumbing():
    q, k, v, i, f = make_inputs(S=32)
    leaves = [t.clone().requires_grad_(True) for t in (q, k, v, i, f)]
    H, (C, n, m) = O.mlstm_chunkwise__native_custbw(*leaves, return_last_states=True, chunk_size=16)
    assert C.shape == (1, 2, 16, 24) and n.shape == (1, 2, 16) and m.shape == (1, 2, 1)
    dH = torch.randn_like(H)
    (H * dH).sum().backward()
    ref = O.chunkwise_bw(q, k, v, i, f, dH, chunk_size=16)
    for leaf, r in zip(leaves, ref[:5]):
        torch.testing.assert_close(leaf.grad, r)


# ------------------------------------------------------------------ head norm
@pytest.mark.parametrize("spec", ["layer", "rms"])
def test_head_normalize_matches_library_routine_and_autograd(spec):
    """The oracle's head norm against torch's own layer_norm (rms: the textbook formula on a hand-made row), and its
    closed-form gradient against fp64 autograd."""
    g = torch.Generator().manual_seed(0)
    x = torch.randn(2, 3, 5, 64, generator=g, dtype=torch.float64) * 2 + 0.3
    y = O.head_normalize(x, spec, eps=1e-6)
    if spec == "layer":
        torch.testing.assert_close(y, torch.nn.functional.layer_norm(x, (64,), eps=1e-6), rtol=1e-12, atol=1e-12)
    else:
        row = torch.tensor([[3.0, -4.0]], dtype=torch.float64)           # rms = sqrt(12.5)
        torch.testing.assert_close(O.head_normalize(row, "rms", eps=0.0), row / 12.5 ** 0.5, rtol=1e-14, atol=1e-14)
        torch.testing.assert_close((y * y).mean(-1), torch.ones(2, 3, 5, dtype=torch.float64), rtol=1e-5, atol=1e-5)
    xr = x.clone().requires_grad_(True)
    dy = torch.randn(2, 3, 5, 64, generator=g, dtype=torch.float64)
    (O.head_normalize(xr, spec, eps=1e-6) * dy).sum().backward()
    torch.testing.assert_close(O.head_normalize_bw(dy, x, spec, eps=1e-6), xr.grad, rtol=1e-10, atol=1e-10)
    assert O.head_normalize(x, "none") is x
    with pytest.raises(ValueError):
        O.head_normalize(x, "batch")


# ---------------------------------------------------------------- the rounding emulation used by the GPU tests
@pytest.mark.parametrize("stride", [1, 2, 4])
@pytest.mark.parametrize("siging,normalize,init", [(False, True, False), (False, True, True), (True, True, True),
                                                   (True, False, False)])
def test_rounding_emulation_without_rounding_is_the_oracle(stride, siging, normalize, init):
    """tests/rounding_emulation.py restates the chunkwise forward and backward with explicit rounding points and its
    own grouping (scans in chunks of 128, outputs per window of `stride` chunks).  With the identity as rounding
    function it must reproduce the oracle's H, row normaliser, dQ, dK and dV to fp64 accuracy."""
    sys_path_has_tests()
    import rounding_emulation as R

    q, k, v, i, f = make_inputs(B=1, NH=2, S=512, DQK=16, DHV=24, seed=31)
    g = torch.Generator().manual_seed(32)
    dH = torch.randn(1, 2, 512, 24, generator=g, dtype=torch.float64)
    c0 = n0 = m0 = None
    if init:
        c0 = 0.1 * torch.randn(1, 2, 16, 24, generator=g, dtype=torch.float64)
        n0 = 0.1 * torch.randn(1, 2, 16, generator=g, dtype=torch.float64)
        m0 = torch.zeros(1, 2, 1, dtype=torch.float64)
    fw = O.chunkwise_fw(q, k, v, i, f, c0, n0, m0, chunk_size=64, siging=siging, normalize=normalize)
    bw = O.chunkwise_bw(q, k, v, i, f, dH, c0, n0, m0, chunk_size=64, siging=siging, normalize=normalize)
    em = R.chunkwise_fw_rounded(q, k, v, i, f, c0, n0, m0, stride=stride, siging=siging, normalize=normalize)
    dQ, dK, dV = R.chunkwise_bw_rounded(q, k, v, i, f, dH, c0, n0, m0, stride=stride, siging=siging, normalize=normalize)
    assert torch.allclose(em["H"], fw["H"], rtol=1e-9, atol=1e-10)
    assert torch.allclose(em["nmax"], fw["n_out"], rtol=1e-9, atol=1e-12)
    for name, x, r in zip(["dQ", "dK", "dV"], [dQ, dK, dV], bw[:3]):
        assert torch.allclose(x, r, rtol=1e-8, atol=1e-9), name


def sys_path_has_tests():
    import os
    import sys

    here = os.path.dirname(os.path.abspath(__file__))
    if here not in sys.path:
        sys.path.insert(0, here)
