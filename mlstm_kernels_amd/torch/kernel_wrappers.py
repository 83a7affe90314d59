"""Sequence-length adapters around a chunkwise kernel, with the semantics of
mlstm_kernels/torch/kernel_wrappers.py:12-273 in the reference."""
from __future__ import annotations

from collections.abc import Callable

import torch


def wrap_chunkwise__arbitrary_sequence_length(
    mlstm_chunkwise_kernel: Callable,
    mlstm_sequence_kernel: Callable,
    mlstm_step_kernel: Callable,
    q: torch.Tensor,  # (B, NH, S, DHQK)
    k: torch.Tensor,  # (B, NH, S, DHQK)
    v: torch.Tensor,  # (B, NH, S, DHHV)
    f: torch.Tensor,  # (B, NH, S)
    i: torch.Tensor,  # (B, NH, S)
    c_initial: torch.Tensor = None,
    n_initial: torch.Tensor = None,
    m_initial: torch.Tensor = None,
    return_last_states: bool = True,
    eps: float = 1e-6,
    autocast_kernel_dtype: torch.dtype = torch.bfloat16,
    chunk_size: int = 64,
    dtype_state: torch.dtype = torch.float32,
    enable_logging: bool = False,
):
    """Process a sequence of any length S >= 1: the chunkwise kernel consumes the longest prefix that is a
    multiple of chunk_size, then of chunk_size/2, ... down to 16; the last < 16 tokens go through the token
    loop; S == 1 goes straight to the step kernel.  States are threaded through all parts.

    A chunkwise kernel that masks a ragged tail itself announces it with the function attribute
    ``supports_any_sequence_length``; it then gets the whole sequence in ONE call (keyword
    ``any_sequence_length=True``) instead of the chunk-halving loop plus the per-token loop."""
    B, NH, S, DHQK = k.shape
    DHHV = v.shape[-1]
    dev = k.device
    c_state = c_initial if c_initial is not None else torch.zeros(B, NH, DHQK, DHHV, device=dev, dtype=dtype_state)
    n_state = n_initial if n_initial is not None else torch.zeros(B, NH, DHQK, device=dev, dtype=dtype_state)
    m_state = m_initial if m_initial is not None else torch.zeros(B, NH, 1, device=dev, dtype=dtype_state)

    if S == 1:
        h_out, (c_state, n_state, m_state) = mlstm_step_kernel(
            q=q.squeeze(2), k=k.squeeze(2), v=v.squeeze(2), i=i, f=f, c=c_state, n=n_state, m=m_state, eps=eps
        )
        h_out = h_out[:, :, None, :]
    elif getattr(mlstm_chunkwise_kernel, "supports_any_sequence_length", False):
        h_out, (c_state, n_state, m_state) = mlstm_chunkwise_kernel(
            q=q.contiguous(), k=k.contiguous(), v=v.contiguous(), f=f.contiguous(), i=i.contiguous(),
            c_initial=c_state, n_initial=n_state, m_initial=m_state,
            chunk_size=chunk_size, return_last_states=True, autocast_kernel_dtype=autocast_kernel_dtype, eps=eps,
            any_sequence_length=True,
        )
    else:
        assert S > 1, f"Received empty sequence (S={S}), require at least single element in the sequence."
        pieces = []
        pos = 0
        cs = chunk_size
        while cs >= 16 and pos < S:
            n_chunks = (S - pos) // cs
            if n_chunks > 0:
                end = pos + n_chunks * cs
                h_part, (c_state, n_state, m_state) = mlstm_chunkwise_kernel(
                    q=q[..., pos:end, :].contiguous(),
                    k=k[..., pos:end, :].contiguous(),
                    v=v[..., pos:end, :].contiguous(),
                    f=f[..., pos:end].contiguous(),
                    i=i[..., pos:end].contiguous(),
                    c_initial=c_state,
                    n_initial=n_state,
                    m_initial=m_state,
                    chunk_size=cs,
                    return_last_states=True,
                    autocast_kernel_dtype=autocast_kernel_dtype,
                    eps=eps,
                )
                pieces.append(h_part)
                pos = end
            cs //= 2
        if pos < S:
            h_part, (c_state, n_state, m_state) = mlstm_sequence_kernel(
                q=q[..., pos:S, :].contiguous(),
                k=k[..., pos:S, :].contiguous(),
                v=v[..., pos:S, :].contiguous(),
                i=i[..., pos:S].contiguous(),
                f=f[..., pos:S].contiguous(),
                c_initial=c_state,
                n_initial=n_state,
                m_initial=m_state,
                return_last_states=True,
                eps=eps,
            )
            pieces.append(h_part)
        h_out = torch.concatenate(pieces, dim=2)

    if return_last_states:
        return h_out, (c_state, n_state, m_state)
    return h_out


def wrap_chunkwise__pad_zeros(
    mlstm_chunkwise_kernel: Callable,
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    f: torch.Tensor,
    i: torch.Tensor,
    c_initial: torch.Tensor = None,
    n_initial: torch.Tensor = None,
    m_initial: torch.Tensor = None,
    return_last_states: bool = False,
    eps: float = 1e-6,
    autocast_kernel_dtype: torch.dtype = torch.bfloat16,
    chunk_size: int = 64,
    **kwargs,
):
    """Zero-pad the sequence to a multiple of chunk_size, run the kernel, cut H back.  Last states of a
    padded sequence would not be the true last states, so they cannot be requested."""
    assert not return_last_states, "We are padding zeros, so we cannot return last states, as they would be not the true last states."
    B, NH, S, _ = q.shape
    if S % chunk_size != 0:
        S_pad = -(-S // chunk_size) * chunk_size

        def pad(t):
            out = t.new_zeros(*t.shape[:2], S_pad, *t.shape[3:])
            out[:, :, :S] = t
            return out

        q, k, v, i, f = pad(q), pad(k), pad(v), pad(i), pad(f)
    H = mlstm_chunkwise_kernel(
        q=q, k=k, v=v, i=i, f=f, c_initial=c_initial, n_initial=n_initial, m_initial=m_initial,
        return_last_states=return_last_states, eps=eps, autocast_kernel_dtype=autocast_kernel_dtype,
        chunk_size=chunk_size, **kwargs,
    )
    return H[:, :, :S, :]
