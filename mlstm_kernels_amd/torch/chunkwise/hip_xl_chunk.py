"""TFLA chunkwise mLSTM (forward + backward) on the HIP kernels: mLSTMexp and mLSTMsig.

Mirrors the public operators of the reference,
  mlstm_kernels/torch/chunkwise/triton_xl_chunk/fwbw.py:244-300          (``mlstm_chunkwise__xl_chunk``)
  mlstm_kernels/torch/chunkwise/triton_xl_chunk_siging/fwbw.py:211-269   (``mlstm_siging_chunkwise__xl_chunk``)
with the same argument names, defaults, return structure and shape rules
(mlstm_kernels/triton/chunkwise/kernel_param_heuristics.py:42-128).  The HIP kernels always scan the sequence in
internal chunks of 128 positions (the reference's ``chunk_size_inter``), which leaves H and the last states unchanged
because the chunkwise formulation is exact for every chunk length.  ``chunk_size_intra`` (a multiple of 128, at most
1024) selects how far apart the kept chunk states are, as in the reference (``save_states_every_nth_chunk`` =
``chunk_size_intra // chunk_size_inter``); ``chunk_size_inter`` is checked and otherwise has no effect;
``recompute_states_in_bw=True`` makes the autograd function drop the chunk states after the forward and run the state
scan again in the backward, as the reference does (default here: ``False``, the states are kept -- the reference's
default is ``True``); the Triton tile-size and launch keywords are accepted and ignored.

Arithmetic: the matrix cores multiply bfloat16 or float16 operands -- the dtype of q after the autocast cast to
``autocast_kernel_dtype`` -- and accumulate in fp32; gates, stabilisers, normalisers and states are fp32.  float32
inputs are rounded to bfloat16 at the boundary -- unlike the reference's Triton kernels, which then multiply in
tf32 -- and a warning says so once."""
from __future__ import annotations

import warnings

import torch
from torch.amp import custom_bwd, custom_fwd

from ... import _lib
from ..utils import current_stream_ptr, dtype_code, ptr, require_gpu

_IGNORED_TUNING_KWARGS = (
    "siz_b_L_parallel", "siz_b_L_loop", "siz_b_DH_parallel", "siz_b_DH_loop", "num_warps_intra", "num_warps_inter",
    "num_stages_intra", "num_stages_inter",
)
_POLICY_KWARGS = ("chunk_size_inter", "chunk_size_intra", "recompute_states_in_bw")
_INTERNAL_CHUNK = 128
_warned_rounding: set = set()


def _warn_rounding_once(dtype: torch.dtype) -> None:
    if dtype not in _warned_rounding:
        _warned_rounding.add(dtype)
        warnings.warn(
            f"mlstm_kernels_amd: {dtype} operands are rounded to bfloat16 for the HIP chunkwise kernels (16-bit matrix "
            "cores with fp32 accumulation; gates, normalisers and states stay fp32). "
            "Pass bfloat16 or float16 tensors to choose the operand format yourself.",
            stacklevel=4,
        )


def _state_stride(tuning_kwargs: dict, who: str, chunk_size: int = 128) -> int:
    """chunk_size_inter / chunk_size_intra of the reference (kernel_param_heuristics.py:118-121) -> state stride.

    The reference scans in chunks of chunk_size_inter and keeps a state every chunk_size_intra positions.  The HIP
    scan always runs in chunks of 128 positions -- the results do not depend on the chunk of the scan -- so
    chunk_size_inter only has to be a value the reference would take (a power of two from 16 to 128 that divides
    chunk_size_intra); chunk_size_intra sets the distance between kept states, in units of 128 positions (a smaller
    value keeps a state per internal chunk)."""
    for key in tuning_kwargs:
        if key not in _IGNORED_TUNING_KWARGS and key not in _POLICY_KWARGS:
            raise TypeError(f"{who}() got an unexpected keyword argument '{key}'")
    inter = tuning_kwargs.get("chunk_size_inter")
    intra = tuning_kwargs.get("chunk_size_intra")
    if inter is not None and inter not in (16, 32, 64, _INTERNAL_CHUNK):
        raise ValueError(f"chunk_size_inter must be 16, 32, 64 or {_INTERNAL_CHUNK} (or None), got {inter}")
    if intra is None:
        # the reference takes chunk_size as chunk_size_intra when the latter is not given
        # (kernel_param_heuristics.py:96-121): a caller who asks for chunks of 256 positions or more gets a kept state
        # every chunk_size positions (at most every 1024); the reference's default of 128 leaves the choice to the
        # library (a state every 256 positions, the measured optimum on MI355X: same results, half the workspace)
        if isinstance(chunk_size, int) and chunk_size >= 2 * _INTERNAL_CHUNK and chunk_size % _INTERNAL_CHUNK == 0:
            return min(chunk_size // _INTERNAL_CHUNK, 8)
        return 0
    if inter is not None and (intra < inter or intra % inter != 0):
        raise ValueError(f"chunk_size_intra ({intra}) must be a multiple of chunk_size_inter ({inter})")
    if intra in (16, 32, 64):
        return 1
    if intra <= 0 or intra % _INTERNAL_CHUNK != 0 or intra // _INTERNAL_CHUNK > 8:
        raise ValueError(f"chunk_size_intra must be 16, 32, 64 or a multiple of {_INTERNAL_CHUNK} up to "
                         f"{8 * _INTERNAL_CHUNK}, got {intra}")
    return intra // _INTERNAL_CHUNK


def _recompute_states(tuning_kwargs: dict) -> bool:
    """recompute_states_in_bw of the reference (triton_xl_chunk/fwbw.py:45,62): True = keep no chunk states between
    forward and backward and run the state scan again in the backward.  Unlike the reference the default is False."""
    flag = tuning_kwargs.get("recompute_states_in_bw")
    if flag is not None and not isinstance(flag, bool):
        raise ValueError(f"recompute_states_in_bw must be True, False or None, got {flag!r}")
    return bool(flag)


def _is_pow2(x: int) -> bool:
    return x > 0 and (x & (x - 1)) == 0


def validate_xl_chunk_shapes(S: int, chunk_size: int) -> None:
    """Shape rules of the reference's xl_chunk kernels (kernel_param_heuristics.py:74-116)."""
    assert S % 16 == 0, "Sequence length must be divisible by 16."
    if S < 128:
        assert _is_pow2(S), "Sequence length must be a power of 2."
        return
    if chunk_size >= 64:
        assert chunk_size % 64 == 0, "Target chunk size must be divisible by the default chunk block size 64."
    assert S % chunk_size == 0, f"Sequence length must be divisible by the target chunk size {chunk_size}."


def _fw_launch(q, k, v, i, f, c0, n0, m0, eps, siging, normalize, want_last, keep, path, stride, norm=0, norm_eps=1e-6,
               n_out=None, m_out=None):
    """One forward launch.  n_out / m_out: optional fp32 (B,NH,S) tensors that receive the row normaliser
    max(|den|, floor) and the combined stabiliser (vecN_out / vecM_out of the reference's mlstm_chunkwise_fw,
    mlstm_kernels/torch/chunkwise/triton_xl_chunk/fw.py:150-170)."""
    B, NH, S, DHQK = q.shape
    DHHV = v.shape[-1]
    dev = q.device
    lib = _lib.get_lib()
    if path == _lib.PATH_FUSED and q.dtype != torch.bfloat16:
        raise RuntimeError(f"the fused kernel path supports bfloat16 operands only, got {q.dtype}")
    ws_bytes = lib.mlstm_hip_chunkwise_fw_workspace_bytes(B, NH, S, DHQK, DHHV, int(keep), path, stride)
    if ws_bytes == 0:
        if DHQK % 64 == 0 and DHQK > 896:
            raise RuntimeError(f"DHQK too large for the HIP chunkwise kernels: {DHQK} (at most 896)")
        if path == _lib.PATH_FUSED and DHQK not in (128, 256) and DHQK % 64 == 0 and DHHV % 64 == 0:
            raise RuntimeError(f"the fused kernel path supports DHQK = 128 or 256 only, got {DHQK}")
        raise ValueError(
            f"unsupported shape for the HIP chunkwise kernels: B={B}, NH={NH}, S={S}, DHQK={DHQK}, DHHV={DHHV} "
            "(head dimensions must be multiples of 64, DHQK <= 896, B*NH <= 65535)"
        )
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    H = torch.empty(B, NH, S, DHHV, dtype=q.dtype, device=dev)
    if norm != _lib.NORM_NONE:
        if DHHV not in (64, 128, 256, 512):
            raise ValueError(f"the fused head norm needs DHHV = 64, 128, 256 or 512, got {DHHV}")
        norm_mean = torch.empty(B, NH, S, dtype=torch.float32, device=dev)
        norm_rstd = torch.empty(B, NH, S, dtype=torch.float32, device=dev)
    else:
        norm_mean = norm_rstd = None
    if want_last:
        c_last = torch.empty(B, NH, DHQK, DHHV, dtype=torch.float32, device=dev)
        n_last = torch.empty(B, NH, DHQK, dtype=torch.float32, device=dev)
        m_last = torch.empty(B, NH, 1, dtype=torch.float32, device=dev)
    else:
        c_last = n_last = m_last = None
    rc = lib.mlstm_hip_chunkwise_fw(
        ptr(q), ptr(k), ptr(v), ptr(i), ptr(f), ptr(c0), ptr(n0), ptr(m0),
        ptr(H), ptr(n_out), ptr(m_out), ptr(c_last), ptr(n_last), ptr(m_last),
        ptr(ws), ws_bytes, int(keep), B, NH, S, DHQK, DHHV, float(eps),
        dtype_code(q), dtype_code(i), _lib.GATE_SIG if siging else _lib.GATE_EXP, int(normalize), path, stride,
        norm, float(norm_eps), ptr(norm_mean), ptr(norm_rstd), current_stream_ptr(dev),
    )
    _lib.check(rc, "mlstm_hip_chunkwise_fw")
    return H, c_last, n_last, m_last, ws, norm_rstd


def _prep_inputs(q, k, v, i, f, c0, n0, m0, siging, f32_as_f16=False):
    dev = require_gpu(q, k, v, i, f)
    B, NH, S, DHQK = q.shape
    assert k.shape == (B, NH, S, DHQK), f"k has wrong shape {tuple(k.shape)}"
    assert v.shape[:3] == (B, NH, S), f"v has wrong shape {tuple(v.shape)}"
    assert i.shape == (B, NH, S) and f.shape == (B, NH, S), "i and f must have shape (B, NH, S)"
    # operand format of the matrix kernels: float16 when q is float16 (or float32 and the caller asked for float16
    # operands), bfloat16 otherwise
    kd = torch.float16 if (q.dtype == torch.float16 or (q.dtype == torch.float32 and f32_as_f16)) else torch.bfloat16
    for t in (q, k, v):
        if t.dtype == torch.float32 and not f32_as_f16:
            _warn_rounding_once(t.dtype)
    qb, kb, vb = (t.to(kd).contiguous() for t in (q, k, v))
    gate_dt = i.dtype if (i.dtype == f.dtype and i.dtype in (torch.bfloat16, torch.float16)) else torch.float32
    ib, fb = i.to(gate_dt).contiguous(), f.to(gate_dt).contiguous()
    if c0 is not None:
        assert n0 is not None, "Initial states must be provided together."
        if not siging:
            assert m0 is not None, "Initial states must be provided together."
        c0 = c0.to(torch.float32).contiguous()
        n0 = n0.to(torch.float32).contiguous()
        m0 = None if (siging or m0 is None) else m0.to(torch.float32).reshape(B, NH).contiguous()
    else:
        n0 = m0 = None
    return dev, qb, kb, vb, ib, fb, c0, n0, m0


def _make_fwbw(autocast_kernel_dtype, siging: bool, normalize: bool, path: int, stride: int, norm: int, norm_eps: float,
               recompute: bool, f32_as_f16: bool = False):
    class _HipChunkwiseFwBw(torch.autograd.Function):
        @staticmethod
        @custom_fwd(device_type="cuda", cast_inputs=autocast_kernel_dtype)
        def forward(ctx, q, k, v, i, f, c0, n0, m0, return_last_states, eps):
            # outputs nobody differentiates (the last states in most losses) arrive as None in backward instead of as
            # freshly allocated zero tensors the size of the state
            ctx.set_materialize_grads(False)
            out_dtype = q.dtype
            dev, qb, kb, vb, ib, fb, c0f, n0f, m0f = _prep_inputs(q, k, v, i, f, c0, n0, m0, siging, f32_as_f16)
            needs_bw = any(ctx.needs_input_grad[:6])
            H, c_last, n_last, m_last, ws, norm_rstd = _fw_launch(
                qb, kb, vb, ib, fb, c0f, n0f, m0f, eps, siging, normalize, return_last_states, needs_bw, path, stride,
                norm, norm_eps
            )
            c0s = None
            if recompute and needs_bw:
                # keep only what lies in front of the chunk states (gate vectors, normaliser states, row normalisers);
                # the backward runs the state scan again, from the initial state when there is one
                B_, NH_, S_, DHQK_ = qb.shape
                saved_bytes = _lib.get_lib().mlstm_hip_chunkwise_fw_saved_bytes(B_, NH_, S_, DHQK_, vb.shape[-1])
                if ws.numel() > saved_bytes:
                    ws = ws[:saved_bytes].clone()
                c0s = c0f
            if norm != _lib.NORM_NONE and needs_bw:
                ctx.save_for_backward(qb, kb, vb, ib, fb, ws, c0s, H, norm_rstd)   # H holds the normalised rows
            else:
                ctx.save_for_backward(qb, kb, vb, ib, fb, ws, c0s)
            ctx.cfg = (eps, q.dtype, k.dtype, v.dtype, i.dtype, f.dtype,
                       None if c0 is None else c0.dtype, n0 is not None, m0 is not None)
            H = H if out_dtype == H.dtype else H.to(out_dtype)
            return H, c_last, n_last, m_last

        @staticmethod
        @custom_bwd(device_type="cuda")
        def backward(ctx, dH, dC_last, dn_last, dm_last):
            qb, kb, vb, ib, fb, ws, c0s, *normed = ctx.saved_tensors
            eps, qdt, kdt, vdt, idt, fdt, c0dt, has_n0, has_m0 = ctx.cfg
            B, NH, S, DHQK = qb.shape
            DHHV = vb.shape[-1]
            dev = qb.device
            lib = _lib.get_lib()
            bw_bytes = lib.mlstm_hip_chunkwise_bw_workspace_bytes(B, NH, S, DHQK, DHHV, stride)
            bws = torch.empty(bw_bytes, dtype=torch.uint8, device=dev)
            if recompute:
                full_bytes = lib.mlstm_hip_chunkwise_fw_workspace_bytes(B, NH, S, DHQK, DHHV, 1, path, stride)
                full = torch.empty(full_bytes, dtype=torch.uint8, device=dev)
                full[:ws.numel()].copy_(ws)
                rc = lib.mlstm_hip_chunkwise_recompute_states(
                    ptr(kb), ptr(vb), ptr(c0s), ptr(full), full_bytes, B, NH, S, DHQK, DHHV, dtype_code(qb), stride,
                    current_stream_ptr(dev),
                )
                _lib.check(rc, "mlstm_hip_chunkwise_recompute_states")
                ws = full
            if dH is None:  # only the last states are differentiated
                dH = torch.zeros(B, NH, S, DHHV, dtype=qb.dtype, device=dev)
            dHb = dH.to(qb.dtype).contiguous()
            if normed:
                # gradient of the normalised rows -> gradient of H (the un-normalised rows were never stored)
                Hn, rstd = normed
                dHraw = torch.empty_like(dHb)
                rc = lib.mlstm_hip_head_norm_bw(ptr(dHb), ptr(Hn), ptr(rstd), ptr(dHraw), B * NH * S, DHHV, norm,
                                                dtype_code(dHb), current_stream_ptr(dev))
                _lib.check(rc, "mlstm_hip_head_norm_bw")
                dHb = dHraw
            dCl = None if dC_last is None else dC_last.to(torch.float32).contiguous()
            dQ, dK, dV = torch.empty_like(qb), torch.empty_like(kb), torch.empty_like(vb)
            dI = torch.empty(B, NH, S, dtype=torch.float32, device=dev)
            dF = torch.empty(B, NH, S, dtype=torch.float32, device=dev)
            dC0 = torch.empty(B, NH, DHQK, DHHV, dtype=torch.float32, device=dev) if c0dt is not None else None
            rc = lib.mlstm_hip_chunkwise_bw(
                ptr(qb), ptr(kb), ptr(vb), ptr(ib), ptr(fb), ptr(dHb), ptr(dCl),
                ptr(dQ), ptr(dK), ptr(dV), ptr(dI), ptr(dF), ptr(dC0),
                ptr(ws), ws.numel(), ptr(bws), bw_bytes, B, NH, S, DHQK, DHHV, float(eps),
                dtype_code(qb), dtype_code(ib), _lib.GATE_SIG if siging else _lib.GATE_EXP, int(normalize), path, stride,
                current_stream_ptr(dev),
            )
            _lib.check(rc, "mlstm_hip_chunkwise_bw")
            dn0 = torch.zeros(B, NH, DHQK, dtype=torch.float32, device=dev) if has_n0 else None
            dm0 = torch.zeros(B, NH, 1, dtype=torch.float32, device=dev) if has_m0 else None
            return (dQ.to(qdt), dK.to(kdt), dV.to(vdt), dI.to(idt), dF.to(fdt),
                    None if dC0 is None else dC0.to(c0dt), dn0, dm0, None, None)

    return _HipChunkwiseFwBw


_FWBW_CACHE: dict = {}


def _get_fwbw(autocast_kernel_dtype: torch.dtype, siging: bool, normalize: bool, kernel_path: str, stride: int,
              head_norm: str = "none", head_norm_eps: float = 1e-6, recompute: bool = False,
              float32_operands: str = "bfloat16"):
    if autocast_kernel_dtype not in (torch.float32, torch.float16, torch.bfloat16):
        raise ValueError(f"Unsupported kernel dtype {autocast_kernel_dtype}.")
    path = _lib.path_code(kernel_path)
    norm = _lib.norm_code(head_norm)
    if norm != _lib.NORM_NONE and path == _lib.PATH_FUSED:
        raise ValueError("head_norm is fused into the split kernel path only (kernel_path='auto' or 'split')")
    if float32_operands not in ("bfloat16", "float16"):
        raise ValueError(f"float32_operands must be 'bfloat16' or 'float16', got {float32_operands!r}")
    f32_as_f16 = float32_operands == "float16"
    if f32_as_f16 and path == _lib.PATH_FUSED:
        raise ValueError("the fused kernel path multiplies bfloat16 operands only")
    key = (autocast_kernel_dtype, siging, normalize, path, stride, norm, float(head_norm_eps), bool(recompute), f32_as_f16)
    if key not in _FWBW_CACHE:
        _FWBW_CACHE[key] = _make_fwbw(autocast_kernel_dtype, siging, normalize, path, stride, norm, float(head_norm_eps),
                                      bool(recompute), f32_as_f16)
    return _FWBW_CACHE[key]


def mlstm_chunkwise__hip_xl_chunk(
    q: torch.Tensor,  # (B, NH, S, DHQK)
    k: torch.Tensor,  # (B, NH, S, DHQK)
    v: torch.Tensor,  # (B, NH, S, DHHV)
    i: torch.Tensor,  # (B, NH, S)
    f: torch.Tensor,  # (B, NH, S)
    c_initial: torch.Tensor = None,  # (B, NH, DHQK, DHHV)
    n_initial: torch.Tensor = None,  # (B, NH, DHQK)
    m_initial: torch.Tensor = None,  # (B, NH, 1)
    return_last_states: bool = False,
    eps: float = 1e-6,
    chunk_size: int = 128,
    autocast_kernel_dtype: torch.dtype = torch.float32,
    any_sequence_length: bool = False,
    kernel_path: str = "auto",
    head_norm: str = "none",
    head_norm_eps: float = 1e-6,
    float32_operands: str = "bfloat16",
    **tuning_kwargs,
):
    """mLSTMexp TFLA forward (+ autograd backward).  Returns ``H`` (dtype of q) or
    ``(H, (C_last fp32 (B,NH,DHQK,DHHV), n_last fp32 (B,NH,DHQK), m_last fp32 (B,NH,1)))``.
    Two defaults differ from the reference behind the same signature (the results do not): ``recompute_states_in_bw``
    defaults to False here (True in mlstm_kernels/torch/chunkwise/triton_xl_chunk/fwbw.py:266; keeping the states
    holds 0.56 GB more between the passes at the benchmark shape and is 0.35 ms faster), and
    ``autocast_kernel_dtype=torch.float32`` -- the reference's default, for which it instantiates a float32 kernel
    (fwbw.py:222-241) -- means bfloat16 OPERANDS here: the matrix kernels multiply in the dtype of q, bfloat16 or
    float16, with fp32 accumulation, gates, normalisers and states; float32 inputs are rounded to bfloat16 with a
    one-time warning (about 1e-2 relative error in H against the float32 recurrence on the unrounded inputs).
    ``float32_operands="float16"`` (not in the reference) rounds float32 inputs to float16 instead: the 11-bit
    significand of the TF32 arithmetic the reference's float32 kernels run in on NVIDIA GPUs (about 1e-3 relative
    error in H and the gradients), but float16's range -- values above 65504 overflow and gradients below 6e-8 vanish, which is why it
    is not the default.
    ``chunk_size`` is validated like the reference does; 256 or more also sets the distance between kept states
    (as the reference's chunk_size_intra default does), 128 leaves it to the library.
    ``any_sequence_length=True`` (not in the reference) skips the reference's shape rules: the kernels mask a ragged
    tail themselves, so every S >= 1 is one call.  ``kernel_path`` ("auto", "split", "stream", "fused"; not in the
    reference) selects the kernels of the chunk-parallel passes.  ``chunk_size_intra`` (reference keyword) sets the distance between
    kept chunk states; ``recompute_states_in_bw=True`` (reference keyword) keeps none of them between forward and
    backward.  ``head_norm`` ("none", "layer", "rms"; not in the reference's operator) fuses the multi-head
    norm that follows the cell in the xLSTM block -- the reference's ``apply_normalize(norm_specifier, x, eps)``,
    mlstm_kernels/utils/analysis/transfer_behavior/_norm_layers.py:11-64, over the DHHV columns of every row, without
    scale parameters -- into the output kernel: the returned ``H`` is then the normalised one and the un-normalised
    output never goes to memory (DHHV = 64, 128, 256 or 512)."""
    stride = _state_stride(tuning_kwargs, "mlstm_chunkwise__hip_xl_chunk", chunk_size)
    if not any_sequence_length:
        validate_xl_chunk_shapes(q.shape[2], chunk_size)
    fn = _get_fwbw(autocast_kernel_dtype, False, True, kernel_path, stride, head_norm, head_norm_eps,
                   _recompute_states(tuning_kwargs), float32_operands)
    H, c_last, n_last, m_last = fn.apply(q, k, v, i, f, c_initial, n_initial, m_initial, return_last_states, eps)
    if return_last_states:
        return H, (c_last, n_last, m_last)
    return H


def mlstm_siging_chunkwise__hip_xl_chunk(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    i: torch.Tensor,
    f: torch.Tensor,
    c_initial: torch.Tensor = None,
    n_initial: torch.Tensor = None,
    m_initial: torch.Tensor = None,  # unused: placeholder to match the mLSTMexp interface
    return_last_states: bool = False,
    eps: float = 1e-6,
    normalize: bool = True,
    chunk_size: int = 128,
    autocast_kernel_dtype: torch.dtype = torch.float32,
    any_sequence_length: bool = False,
    kernel_path: str = "auto",
    head_norm: str = "none",
    head_norm_eps: float = 1e-6,
    float32_operands: str = "bfloat16",
    **tuning_kwargs,
):
    """mLSTMsig (sigmoid input gate) TFLA forward (+ autograd backward).  Returns ``H`` or ``(H, (C_last, n_last))``.
    ``any_sequence_length``, ``kernel_path``, ``chunk_size_intra``, ``head_norm`` and ``float32_operands`` as for the
    exp gate."""
    stride = _state_stride(tuning_kwargs, "mlstm_siging_chunkwise__hip_xl_chunk", chunk_size)
    if not any_sequence_length:
        validate_xl_chunk_shapes(q.shape[2], chunk_size)
    fn = _get_fwbw(autocast_kernel_dtype, True, bool(normalize), kernel_path, stride, head_norm, head_norm_eps,
                   _recompute_states(tuning_kwargs), float32_operands)
    H, c_last, n_last, _ = fn.apply(q, k, v, i, f, c_initial, n_initial, None, return_last_states, eps)
    if return_last_states:
        return H, (c_last, n_last)
    return H


# the kernels mask a ragged last chunk themselves: sequence-length adapters may hand over any S >= 1 in one call
mlstm_chunkwise__hip_xl_chunk.supports_any_sequence_length = True
mlstm_siging_chunkwise__hip_xl_chunk.supports_any_sequence_length = True
