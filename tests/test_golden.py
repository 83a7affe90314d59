"""Golden vectors: a hand-computed decode step and the committed chunkwise fixture.  On the CPU they pin the
oracle (regression); on the GPU the HIP kernels are checked against the same files."""
import json
import os

import numpy as np
import pytest
import torch

import oracle as O
from helpers import allclose_frac, assert_state_close, rel_norm, rel_to_scale

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _kat():
    return json.load(open(os.path.join(GOLD, "step_kat.json")))


def _fixture():
    z = np.load(os.path.join(GOLD, "chunkwise_small.npz"))
    return {k: torch.from_numpy(z[k]) for k in z.files}


def test_step_kat_oracle():
    kat = _kat()
    t = lambda x, *s: torch.full(s, x, dtype=torch.float64)
    h, (c, n, m) = O.recurrent_step(t(kat["q"], 1, 1, 1), t(kat["k"], 1, 1, 1), t(kat["v"], 1, 1, 1), t(kat["i"], 1, 1, 1),
                                    t(kat["f"], 1, 1, 1), t(kat["c"], 1, 1, 1, 1), t(kat["n"], 1, 1, 1), t(kat["m"], 1, 1, 1),
                                    eps=kat["eps"])
    assert abs(h.item() - kat["h"]) < 1e-12 and abs(c.item() - kat["c_new"]) < 1e-12
    assert abs(n.item() - kat["n_new"]) < 1e-12 and abs(m.item() - kat["m_new"]) < 1e-15


@pytest.mark.parametrize("tag,sig", [("exp", False), ("sig", True)])
def test_chunkwise_fixture_oracle(tag, sig):
    z = {k: v.double() for k, v in _fixture().items()}
    fw = O.chunkwise_fw(z["q"], z["k"], z["v"], z["i"], z["f"], z["c0"], z["n0"], z["m0"], chunk_size=64, siging=sig)
    bw = O.chunkwise_bw(z["q"], z["k"], z["v"], z["i"], z["f"], z["dH"], z["c0"], z["n0"], z["m0"], None, chunk_size=16, siging=sig)
    torch.testing.assert_close(fw["H"], z[f"{tag}_H"], rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(fw["C_last"], z[f"{tag}_C"], rtol=1e-5, atol=1e-5)
    for name, t in zip(["dQ", "dK", "dV", "dI", "dF", "dC0"], bw):
        torch.testing.assert_close(t, z[f"{tag}_{name}"], rtol=1e-4, atol=1e-4, msg=lambda s: f"{name}: {s}")


def _reference_vectors(case):
    """Outputs of the reference's own native chunkwise forward/backward (tests/golden/make_reference_vectors.py)."""
    z = np.load(os.path.join(GOLD, "reference_native_chunkwise.npz"))
    d = {k[len(case) + 1:]: torch.from_numpy(z[k]) for k in z.files if k.startswith(case + "_")}
    B, NH, S, DQK, DHV, L, init, dcl = (int(x) for x in d.pop("meta"))
    return d, L, bool(init), bool(dcl)


@pytest.mark.parametrize("case", ["a", "b"])
def test_oracle_matches_reference_native_vectors(case):
    """Pins the two conventions only the reference can state: the stored normaliser / stabiliser rows (n_out, m_out)
    and the hand-written backward (constants of the gradient, span of the dF sum).  fp32-stored vectors: 1e-5."""
    z, L, init, dcl = _reference_vectors(case)
    z = {k: v.double() for k, v in z.items()}
    ini = (z["c0"], z["n0"], z["m0"]) if init else (None, None, None)
    fw = O.chunkwise_fw(z["q"], z["k"], z["v"], z["i"], z["f"], *ini, chunk_size=L)
    for name in ("H", "n_out", "m_out", "C_last", "n_last", "m_last"):
        torch.testing.assert_close(fw[name].reshape(z[name].shape), z[name], rtol=1e-5, atol=1e-5, msg=lambda s: f"{name}: {s}")
    # the chunk size must not matter (the vectors were made with L, the HIP kernels use 128)
    fw2 = O.chunkwise_fw(z["q"], z["k"], z["v"], z["i"], z["f"], *ini, chunk_size=2 * L)
    torch.testing.assert_close(fw2["H"], z["H"], rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(fw2["n_out"], z["n_out"], rtol=1e-5, atol=1e-5)
    bw = O.chunkwise_bw(z["q"], z["k"], z["v"], z["i"], z["f"], z["dH"], *ini, z.get("dC_last"), chunk_size=L)
    names = ["dQ", "dK", "dV", "dI", "dF"] + (["dC0"] if init else [])
    for name, t in zip(names, bw):
        torch.testing.assert_close(t, z[name], rtol=1e-5, atol=2e-5, msg=lambda s: f"{name}: {s}")


@pytest.mark.gpu
@pytest.mark.parametrize("case", ["a", "b"])
def test_hip_matches_reference_native_vectors(case):
    from mlstm_kernels_amd.torch.chunkwise import mlstm_chunkwise__hip_xl_chunk

    z, L, init, dcl = _reference_vectors(case)
    dev = "cuda"
    q, k, v = (z[x].bfloat16().to(dev).requires_grad_(True) for x in "qkv")
    i, f = z["i"].to(dev).requires_grad_(True), z["f"].to(dev).requires_grad_(True)
    kw = {}
    if init:
        c0 = z["c0"].to(dev).requires_grad_(True)
        kw = dict(c_initial=c0, n_initial=z["n0"].to(dev), m_initial=z["m0"].to(dev))
    H, (C, n, m) = mlstm_chunkwise__hip_xl_chunk(q, k, v, i, f, return_last_states=True, chunk_size=L, **kw)
    loss = (H.float() * z["dH"].to(dev)).sum()
    if dcl:
        loss = loss + (C * z["dC_last"].to(dev)).sum()
    loss.backward()
    # tolerances: outputs / gradients 2e-2 (bf16 operands), states 1e-3, gate gradients 5e-2 of their scale
    assert allclose_frac(H, z["H"], 2e-2, 2e-2) <= 1e-3 and rel_to_scale(H, z["H"]) <= 1e-2
    assert_state_close(C, z["C_last"], 1e-3, "C_last")
    assert_state_close(n, z["n_last"], 1e-3, "n_last")
    assert (m.cpu() - z["m_last"]).abs().max() <= 1e-3
    for name, t in (("dQ", q), ("dK", k), ("dV", v)):
        assert allclose_frac(t.grad, z[name], 2e-2, 2e-2) <= 1e-3, name
        assert rel_to_scale(t.grad, z[name]) <= 1e-2 and rel_norm(t.grad, z[name]) <= 5e-3, name
    for name, t in (("dI", i), ("dF", f)):
        assert rel_to_scale(t.grad, z[name]) <= 5e-2, name
    if init:
        assert rel_norm(c0.grad, z["dC0"]) <= 5e-3


@pytest.mark.gpu
@pytest.mark.parametrize("case", ["a", "b"])
def test_hip_stored_rows_match_reference_native_vectors(case):
    """The optional n_out / m_out outputs of the C entry point (the rows the reference's forward returns as vecN_out and
    vecM_out, native/fw.py:208-212) against the reference-made vectors: m_out depends on the gates only (1e-4), n_out
    carries the bf16 rounding of the scores (2e-2)."""
    from mlstm_kernels_amd import _lib
    from mlstm_kernels_amd.torch.utils import current_stream_ptr, ptr

    z, L, init, dcl = _reference_vectors(case)
    dev = torch.device("cuda")
    q, k, v = (z[x].bfloat16().to(dev).contiguous() for x in "qkv")
    i, f = z["i"].to(dev).contiguous(), z["f"].to(dev).contiguous()
    B, NH, S, DHQK = q.shape
    DHHV = v.shape[-1]
    c0 = n0 = m0 = None
    if init:
        c0, n0, m0 = z["c0"].to(dev).contiguous(), z["n0"].to(dev).contiguous(), z["m0"].reshape(B, NH).to(dev).contiguous()
    lib = _lib.get_lib()
    ws_bytes = lib.mlstm_hip_chunkwise_fw_workspace_bytes(B, NH, S, DHQK, DHHV, 0, _lib.PATH_AUTO, 0)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    H = torch.empty(B, NH, S, DHHV, dtype=torch.bfloat16, device=dev)
    n_out = torch.empty(B, NH, S, dtype=torch.float32, device=dev)
    m_out = torch.empty(B, NH, S, dtype=torch.float32, device=dev)
    rc = lib.mlstm_hip_chunkwise_fw(ptr(q), ptr(k), ptr(v), ptr(i), ptr(f), ptr(c0), ptr(n0), ptr(m0), ptr(H), ptr(n_out),
                                    ptr(m_out), None, None, None, ptr(ws), ws_bytes, 0, B, NH, S, DHQK, DHHV, 1e-6,
                                    _lib.BF16, _lib.F32, _lib.GATE_EXP, 1, _lib.PATH_AUTO, 0, _lib.NORM_NONE, 0.0, None, None,
                                    current_stream_ptr(dev))
    _lib.check(rc, "mlstm_hip_chunkwise_fw")
    torch.cuda.synchronize()
    assert (m_out.cpu() - z["m_out"]).abs().max() <= 1e-4
    torch.testing.assert_close(n_out.cpu(), z["n_out"], rtol=2e-2, atol=2e-2)
    assert allclose_frac(H, z["H"], 2e-2, 2e-2) <= 1e-3


@pytest.mark.gpu
def test_step_kat_hip():
    from mlstm_kernels_amd.torch.recurrent import mlstm_recurrent_step__hip

    kat = _kat()
    # the kernel needs DHHV % 4 == 0: embed the scalar problem in column 0 / row 0 of zero-padded operands
    dev = "cuda"
    q = torch.zeros(1, 1, 4, device=dev); k = torch.zeros(1, 1, 4, device=dev); v = torch.zeros(1, 1, 4, device=dev)
    q[..., 0], k[..., 0], v[..., 0] = kat["q"] * 2.0, kat["k"], kat["v"]   # q/sqrt(4) = kat q
    c = torch.zeros(1, 1, 4, 4, device=dev); n = torch.zeros(1, 1, 4, device=dev)
    c[..., 0, 0], n[..., 0] = kat["c"], kat["n"]
    i = torch.full((1, 1, 1), kat["i"], device=dev); f = torch.full((1, 1, 1), kat["f"], device=dev)
    m = torch.full((1, 1, 1), kat["m"], device=dev)
    h, (c2, n2, m2) = mlstm_recurrent_step__hip(q, k, v, i, f, c, n, m, eps=kat["eps"])
    assert abs(h[0, 0, 0].item() - kat["h"]) < 1e-5 * abs(kat["h"])
    assert abs(c2[0, 0, 0, 0].item() - kat["c_new"]) < 1e-5 * kat["c_new"]
    assert abs(n2[0, 0, 0].item() - kat["n_new"]) < 1e-6 and abs(m2.item() - kat["m_new"]) < 1e-6
    assert h[0, 0, 1:].abs().max().item() == 0.0 and c2[0, 0, 1:, :].abs().max().item() == 0.0


@pytest.mark.gpu
@pytest.mark.parametrize("tag,sig", [("exp", False), ("sig", True)])
def test_chunkwise_fixture_hip(tag, sig):
    from mlstm_kernels_amd.torch.chunkwise import mlstm_chunkwise__hip_xl_chunk, mlstm_siging_chunkwise__hip_xl_chunk

    z = _fixture()
    dev = "cuda"
    q, k, v = (z[x].bfloat16().to(dev).requires_grad_(True) for x in "qkv")
    i, f = z["i"].to(dev).requires_grad_(True), z["f"].to(dev).requires_grad_(True)
    c0 = z["c0"].to(dev).requires_grad_(True)
    fn = mlstm_siging_chunkwise__hip_xl_chunk if sig else mlstm_chunkwise__hip_xl_chunk
    H, st = fn(q, k, v, i, f, c_initial=c0, n_initial=z["n0"].to(dev), m_initial=z["m0"].to(dev), return_last_states=True, chunk_size=128)
    H.backward(z["dH"].bfloat16().to(dev))
    # tolerances: outputs / gradients 2e-2 (bf16 operands), states 1e-3, gate gradients 5e-2 of their scale
    assert allclose_frac(H, z[f"{tag}_H"], 2e-2, 2e-2) <= 1e-3 and rel_to_scale(H, z[f"{tag}_H"]) <= 1e-2
    assert_state_close(st[0], z[f"{tag}_C"], 1e-3, "C_last")
    assert_state_close(st[1], z[f"{tag}_n"], 1e-3, "n_last")
    if not sig:
        assert (st[2].cpu() - z["exp_m"]).abs().max() <= 1e-3
    for name, t in (("dQ", q), ("dK", k), ("dV", v)):
        assert allclose_frac(t.grad, z[f"{tag}_{name}"], 2e-2, 2e-2) <= 1e-3, name
        assert rel_to_scale(t.grad, z[f"{tag}_{name}"]) <= 1e-2 and rel_norm(t.grad, z[f"{tag}_{name}"]) <= 5e-3, name
    for name, t in (("dI", i), ("dF", f)):
        assert rel_to_scale(t.grad, z[f"{tag}_{name}"]) <= 5e-2, name
    assert rel_norm(c0.grad, z[f"{tag}_dC0"]) <= 5e-3


# ------------------------------------------------------------------ reference-made vectors: sigmoid gate, decode step
def _reference_siging_step(case):
    """Outputs of the reference's own native_siging forward/backward and native decode step
    (tests/golden/make_reference_vectors_siging_step.py)."""
    z = np.load(os.path.join(GOLD, "reference_native_siging_step.npz"))
    d = {k[len(case) + 1:]: torch.from_numpy(z[k]) for k in z.files if k.startswith(case + "_")}
    return d, [int(x) for x in d.pop("meta")]


@pytest.mark.parametrize("case", ["sigA", "sigB"])
def test_oracle_matches_reference_siging_vectors(case):
    """The oracle's quadratic AND chunkwise mLSTMsig (forward and hand-written backward) against the reference's
    native_siging numbers (fp32-stored vectors: 1e-5)."""
    z, (B, NH, S, DQK, DHV, normalize) = _reference_siging_step(case)
    z = {k: v.double() for k, v in z.items()}
    H, n = O.parallel_siging_fw(z["q"], z["k"], z["v"], z["i"], z["f"], normalize=bool(normalize))
    torch.testing.assert_close(H, z["H"], rtol=1e-5, atol=1e-5)
    if normalize:
        torch.testing.assert_close(n, z["n"], rtol=1e-5, atol=1e-5)
    grads = O.parallel_siging_bw(z["dH"], z["q"], z["k"], z["v"], z["i"], z["f"], n, normalize=bool(normalize))
    for name, t in zip(["dQ", "dK", "dV", "dI", "dF"], grads):
        torch.testing.assert_close(t, z[name], rtol=1e-5, atol=1e-5, msg=lambda s: f"{name}: {s}")
    fw = O.chunkwise_fw(z["q"], z["k"], z["v"], z["i"], z["f"], chunk_size=32, siging=True, normalize=bool(normalize))
    torch.testing.assert_close(fw["H"], z["H"], rtol=1e-5, atol=1e-5)
    bw = O.chunkwise_bw(z["q"], z["k"], z["v"], z["i"], z["f"], z["dH"], chunk_size=32, siging=True, normalize=bool(normalize))
    for name, t in zip(["dQ", "dK", "dV", "dI", "dF"], bw[:5]):
        torch.testing.assert_close(t, z[name], rtol=2e-5, atol=2e-5, msg=lambda s: f"chunkwise {name}: {s}")


@pytest.mark.parametrize("case", ["stepA", "stepB"])
def test_oracle_matches_reference_step_vectors(case):
    """The oracle's decode step, from random non-zero (C, n, m), against the reference's native step over a few
    consecutive steps (fp32-stored vectors: 1e-5)."""
    z, (B, NH, DQK, DHV, steps) = _reference_siging_step(case)
    z = {k: v.double() for k, v in z.items()}
    c, n, m = z["c0"], z["n0"], z["m0"]
    for t in range(steps):
        h, (c, n, m) = O.recurrent_step(z[f"q{t}"], z[f"k{t}"], z[f"v{t}"], z[f"i{t}"], z[f"f{t}"], c, n, m)
        torch.testing.assert_close(h, z[f"h{t}"], rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(c, z["c_last"], rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(n, z["n_last"], rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(m, z["m_last"], rtol=1e-5, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("case", ["sigA", "sigB"])
def test_hip_matches_reference_siging_vectors(case):
    """The HIP mLSTMsig operator against the reference's native_siging numbers (bf16 operand bounds: outputs and
    gradients 2e-2 on >= 99.9 % of the elements, 1e-2 of the scale, 5e-3 norm-wise; gate gradients 5e-2 of their scale)."""
    from mlstm_kernels_amd.torch.chunkwise import mlstm_siging_chunkwise__hip_xl_chunk

    z, (B, NH, S, DQK, DHV, normalize) = _reference_siging_step(case)
    dev = "cuda"
    q, k, v = (z[x].bfloat16().to(dev).requires_grad_(True) for x in "qkv")
    i, f = z["i"].to(dev).requires_grad_(True), z["f"].to(dev).requires_grad_(True)
    H = mlstm_siging_chunkwise__hip_xl_chunk(q, k, v, i, f, normalize=bool(normalize), chunk_size=128)
    (H.float() * z["dH"].to(dev)).sum().backward()
    for name, t in (("H", H), ("dQ", q.grad), ("dK", k.grad), ("dV", v.grad)):
        assert allclose_frac(t, z[name], 2e-2, 2e-2) <= 1e-3, name
        assert rel_to_scale(t, z[name]) <= 1e-2 and rel_norm(t, z[name]) <= 5e-3, name
    for name, t in (("dI", i.grad), ("dF", f.grad)):
        assert rel_to_scale(t, z[name]) <= 5e-2, name


@pytest.mark.gpu
@pytest.mark.parametrize("case", ["stepA", "stepB"])
def test_hip_step_matches_reference_step_vectors(case):
    """The HIP decode step, state carried over a few consecutive steps, against the reference's native step: fp32
    states 1e-5 relative, h within bf16 rounding of the output (5e-3 of the scale)."""
    from mlstm_kernels_amd.torch.recurrent import mlstm_recurrent_step__hip

    z, (B, NH, DQK, DHV, steps) = _reference_siging_step(case)
    dev = "cuda"
    c, n, m = z["c0"].to(dev), z["n0"].to(dev), z["m0"].to(dev)
    for t in range(steps):
        h, (c, n, m) = mlstm_recurrent_step__hip(z[f"q{t}"].bfloat16().to(dev), z[f"k{t}"].bfloat16().to(dev),
                                                 z[f"v{t}"].bfloat16().to(dev), z[f"i{t}"].to(dev), z[f"f{t}"].to(dev), c, n, m)
        assert rel_to_scale(h, z[f"h{t}"]) <= 5e-3, f"h at step {t}"
    assert_state_close(c, z["c_last"], 1e-5, "C")
    assert_state_close(n, z["n_last"], 1e-5, "n")
    assert (m.cpu() - z["m_last"]).abs().max() <= 1e-5
