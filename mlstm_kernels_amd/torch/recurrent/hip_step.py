"""Fused recurrent decode step on the HIP kernel, plus the token loop built on it.

Mirrors mlstm_kernels/torch/recurrent/triton_step.py:15-158 (``mlstm_recurrent_step__triton_fw`` /
``mlstm_recurrent_step__triton``) and mlstm_kernels/torch/recurrent/native_sequence.py:13-122 of the
reference: same argument names, shapes, return structure and shape assertions."""
from __future__ import annotations

import torch

from ... import _lib
from ..utils import current_stream_ptr, dtype_code, ptr, require_gpu, state_dtype_code


def _check_state_dtype(dtype_state: torch.dtype) -> torch.dtype:
    """The states are kept in float32, bfloat16 or float16 -- the choices of the reference's inference_state_dtype
    (mlstm_kernels/torch/backend_module.py:38,75); the arithmetic is float32 either way."""
    if dtype_state not in (torch.float32, torch.bfloat16, torch.float16):
        raise NotImplementedError(f"the HIP step kernels keep the recurrent state in float32, bfloat16 or float16, not {dtype_state}")
    return dtype_state


def mlstm_recurrent_step__hip_fw(
    matC_old: torch.Tensor,  # (B, NH, DHQK, DHHV)
    vecN_old: torch.Tensor,  # (B, NH, DHQK)
    scaM_old: torch.Tensor,  # (B, NH, 1)
    vecQ: torch.Tensor,  # (B, NH, DHQK)
    vecK: torch.Tensor,  # (B, NH, DHQK)
    vecV: torch.Tensor,  # (B, NH, DHHV)
    scaI: torch.Tensor,  # (B, NH, 1)
    scaF: torch.Tensor,  # (B, NH, 1)
    matC_new: torch.Tensor = None,
    vecN_new: torch.Tensor = None,
    scaM_new: torch.Tensor = None,
    qk_scale: float = None,
    eps: float = 1e-6,
    dtype_state: torch.dtype = torch.float32,
    **kwargs,
):
    """One step.  ``matC_new`` may be ``matC_old`` itself (in-place state update, the step then moves the
    state through HBM exactly once each way); ``vecN_new``/``scaM_new`` must be distinct buffers."""
    B, NH, DHQK = vecQ.shape
    DHHV = vecV.shape[-1]
    assert vecQ.shape == vecK.shape, "q and k must have the same shape"
    assert matC_old.shape == (B, NH, DHQK, DHHV), f"matC_old has wrong shape, got {matC_old.shape}"
    assert vecN_old.shape == (B, NH, DHQK), f"vecN_old has wrong shape, got {vecN_old.shape}"
    assert scaM_old.shape == (B, NH, 1), f"scaM_old has wrong shape, got {scaM_old.shape}"
    assert scaI.shape == (B, NH, 1), f"scaI has wrong shape, got {scaI.shape}"
    assert scaF.shape == (B, NH, 1), f"scaF has wrong shape, got {scaF.shape}"
    if qk_scale is not None and abs(qk_scale - DHQK ** -0.5) > 1e-12:
        raise NotImplementedError("the HIP step kernel uses qk_scale = DHQK**-0.5")
    dtype_state = _check_state_dtype(dtype_state)
    dev = require_gpu(vecQ, vecK, vecV, scaI, scaF, matC_old, vecN_old, scaM_old)
    qdt, gdt = vecQ.dtype, scaI.dtype   # float32, bfloat16 or float16 each; the arithmetic is float32
    q, k, v = vecQ.contiguous(), vecK.to(qdt).contiguous(), vecV.to(qdt).contiguous()
    i, f = scaI.to(gdt).contiguous(), scaF.to(gdt).contiguous()
    c_old = matC_old.to(dtype_state).contiguous()
    n_old = vecN_old.to(dtype_state).contiguous()
    m_old = scaM_old.to(dtype_state).contiguous()
    if matC_new is None:
        assert vecN_new is None and scaM_new is None, "Initial states must be provided together."
        matC_new = torch.empty_like(c_old)
        vecN_new = torch.empty_like(n_old)
        scaM_new = torch.empty_like(m_old)
    else:
        assert vecN_new is not None and scaM_new is not None, "Initial states must be provided together."
        for t in (matC_new, vecN_new, scaM_new):
            assert t.dtype == dtype_state and t.is_contiguous(), f"state outputs must be contiguous {dtype_state}"
    h = torch.empty_like(v)
    lib = _lib.get_lib()
    rc = lib.mlstm_hip_step(
        ptr(q), ptr(k), ptr(v), ptr(i), ptr(f), ptr(c_old), ptr(n_old), ptr(m_old),
        ptr(h), ptr(matC_new), ptr(vecN_new), ptr(scaM_new),
        B, NH, DHQK, DHHV, float(eps), dtype_code(q), dtype_code(i), state_dtype_code(c_old), current_stream_ptr(dev),
    )
    _lib.check(rc, "mlstm_hip_step")
    return h, (matC_new, vecN_new, scaM_new)


def mlstm_recurrent_step__hip(
    q: torch.Tensor,  # (B, NH, DHQK)
    k: torch.Tensor,  # (B, NH, DHQK)
    v: torch.Tensor,  # (B, NH, DHHV)
    i: torch.Tensor,  # (B, NH, 1)
    f: torch.Tensor,  # (B, NH, 1)
    c: torch.Tensor,  # (B, NH, DHQK, DHHV)
    n: torch.Tensor,  # (B, NH, DHQK)
    m: torch.Tensor,  # (B, NH, 1)
    eps: float = 1e-6,
    dtype_state: torch.dtype = torch.float32,
    **kwargs,
):
    """Single mLSTM step: returns ``h (B,NH,DHHV)`` in q's dtype and ``(C', n', m')`` in ``dtype_state`` (float32 unless
    asked otherwise; the arithmetic is float32 either way and h is formed from the unrounded new state)."""
    return mlstm_recurrent_step__hip_fw(
        matC_old=c, vecN_old=n, scaM_old=m, vecQ=q, vecK=k, vecV=v, scaI=i, scaF=f,
        eps=eps, dtype_state=dtype_state, **kwargs,
    )


def mlstm_recurrent_sequence__hip(
    q: torch.Tensor,  # (B, NH, S, DHQK)
    k: torch.Tensor,
    v: torch.Tensor,  # (B, NH, S, DHHV)
    i: torch.Tensor,  # (B, NH, S)
    f: torch.Tensor,
    c_initial: torch.Tensor = None,
    n_initial: torch.Tensor = None,
    m_initial: torch.Tensor = None,
    return_last_states: bool = False,
    eps: float = 1e-6,
    dtype_state: torch.dtype = torch.float32,
    **kwargs,
):
    """All S tokens in one launch of the multi-token kernel: the state stays on chip between tokens and moves
    through HBM once each way for the whole sequence (a loop of single steps moves it once each way per token).
    Used for multi-token decode and for the short remainder of a prefill.  Same arguments and return structure
    as mlstm_recurrent_sequence__triton_step_fused_fw (mlstm_kernels/torch/recurrent/native_sequence.py:86-122), with
    two differences that are stated here rather than hidden: ``return_all_states=True`` (the state after every token,
    native_sequence.py:20,64-83) is not implemented and raises; with a 16-bit ``dtype_state`` the state is rounded
    once per call -- it stays float32 in registers between the tokens -- where the reference's token loop rounds it
    after every step (the results of that mode are therefore closer to the float32 recurrence, not bit-equal)."""
    if kwargs.pop("return_all_states", False):
        raise NotImplementedError("mlstm_recurrent_sequence__hip does not return the state after every token "
                                  "(return_all_states=True); loop over mlstm_recurrent_step__hip for that")
    if kwargs:
        raise TypeError(f"mlstm_recurrent_sequence__hip() got unexpected keyword arguments {sorted(kwargs)}")
    B, NH, S, DHQK = q.shape
    DHHV = v.shape[-1]
    assert k.shape == q.shape, "q and k must have the same shape"
    assert v.shape[:3] == (B, NH, S), f"v has wrong shape, got {v.shape}"
    assert i.shape == (B, NH, S) and f.shape == (B, NH, S), "i and f must have shape (B, NH, S)"
    dtype_state = _check_state_dtype(dtype_state)
    dev = require_gpu(q, k, v, i, f)
    if c_initial is not None:
        assert n_initial is not None and m_initial is not None, "Initial states must be provided together."
        c = c_initial.to(dtype_state).contiguous()
        n = n_initial.to(dtype_state).contiguous()
        m = m_initial.to(dtype_state).contiguous().reshape(B, NH, 1)
        assert c.shape == (B, NH, DHQK, DHHV), f"c_initial has wrong shape, got {c.shape}"
        assert n.shape == (B, NH, DHQK), f"n_initial has wrong shape, got {n.shape}"
    else:
        c = torch.zeros(B, NH, DHQK, DHHV, dtype=dtype_state, device=dev)
        n = torch.zeros(B, NH, DHQK, dtype=dtype_state, device=dev)
        m = torch.zeros(B, NH, 1, dtype=dtype_state, device=dev)
    if S == 0:
        H = torch.empty(B, NH, 0, DHHV, dtype=q.dtype, device=dev)
        return (H, (c.clone(), n.clone(), m.clone())) if return_last_states else H
    qdt, gdt = q.dtype, i.dtype
    qc, kc, vc = q.contiguous(), k.to(qdt).contiguous(), v.to(qdt).contiguous()
    ic, fc = i.to(gdt).contiguous(), f.to(gdt).contiguous()
    H = torch.empty(B, NH, S, DHHV, dtype=qdt, device=dev)
    c_out, n_out, m_out = torch.empty_like(c), torch.empty_like(n), torch.empty_like(m)
    lib = _lib.get_lib()
    rc = lib.mlstm_hip_recurrent_sequence(
        ptr(qc), ptr(kc), ptr(vc), ptr(ic), ptr(fc), ptr(c), ptr(n), ptr(m),
        ptr(H), ptr(c_out), ptr(n_out), ptr(m_out),
        B, NH, S, DHQK, DHHV, float(eps), dtype_code(qc), dtype_code(ic), state_dtype_code(c), current_stream_ptr(dev),
    )
    _lib.check(rc, "mlstm_hip_recurrent_sequence")
    if return_last_states:
        return H, (c_out, n_out, m_out)
    return H
