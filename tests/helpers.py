"""Seeded inputs and comparison metrics shared by the GPU parity tests and the smoke/bench checks."""
from __future__ import annotations

import torch


def make_qkvif(B, NH, S, DHQK, DHHV, seed=0, f_offset=3.0, dtype=torch.bfloat16):
    """q,k,v,i ~ N(0,1), f = f_offset + N(0,1), drawn in fp32 on the CPU and rounded to `dtype`
    (gates stay fp32).  The oracle is fed the same rounded values up-cast, so only compute error is measured."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, NH, S, DHQK, generator=g).to(dtype)
    k = torch.randn(B, NH, S, DHQK, generator=g).to(dtype)
    v = torch.randn(B, NH, S, DHHV, generator=g).to(dtype)
    i = torch.randn(B, NH, S, generator=g)
    f = f_offset + torch.randn(B, NH, S, generator=g)
    return q, k, v, i, f


def rel_to_scale(a: torch.Tensor, ref: torch.Tensor) -> float:
    """max |a - ref| / max |ref|  (error relative to the scale of the tensor)."""
    a, ref = a.detach().double().cpu(), ref.detach().double().cpu()
    return float((a - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


def rel_norm(a: torch.Tensor, ref: torch.Tensor) -> float:
    """||a - ref|| / ||ref||."""
    a, ref = a.detach().double().cpu(), ref.detach().double().cpu()
    return float((a - ref).norm() / ref.norm().clamp_min(1e-30))


def allclose_frac(a: torch.Tensor, ref: torch.Tensor, rtol: float, atol: float) -> float:
    """Fraction of elements violating |a - ref| <= atol + rtol |ref|."""
    a, ref = a.detach().double().cpu(), ref.detach().double().cpu()
    bad = (a - ref).abs() > atol + rtol * ref.abs()
    return float(bad.double().mean())


def assert_state_close(a, ref, tol=1e-3, name="state"):
    e1, e2 = rel_to_scale(a, ref), rel_norm(a, ref)
    assert e1 <= tol and e2 <= tol, f"{name}: max-rel-to-scale {e1:.3e}, norm-rel {e2:.3e} exceed {tol}"


def assert_h_close(a, ref, tol=2e-2, name="H"):
    a64, r64 = a.detach().double().cpu(), ref.detach().double().cpu()
    torch.testing.assert_close(a64, r64, rtol=tol, atol=tol, msg=lambda s: f"{name}: {s}")
