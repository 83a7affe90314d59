"""CPU-side checks of the operator boundary: registries, config validation, sequence-length adapters (driven
with the oracle kernels registered under their reference names), the C-ABI library's exported symbols, and
the absence of any CPU fallback behind the 'hip' names."""
import os
import re

import pytest
import torch

import oracle as O
from helpers import make_qkvif
from mlstm_kernels_amd import _lib
from mlstm_kernels_amd.torch import (
    get_available_mlstm_kernels,
    get_available_mlstm_sequence_kernels,
    get_available_mlstm_step_kernels,
    get_mlstm_kernel,
    get_mlstm_sequence_kernel,
    get_mlstm_step_kernel,
    register_mlstm_kernel,
    register_mlstm_sequence_kernel,
    register_mlstm_step_kernel,
)
from mlstm_kernels_amd.torch.backend_module import mLSTMBackend, mLSTMBackendConfig
from mlstm_kernels_amd.torch.chunkwise.hip_xl_chunk import validate_xl_chunk_shapes
from mlstm_kernels_amd.torch.kernel_wrappers import wrap_chunkwise__arbitrary_sequence_length, wrap_chunkwise__pad_zeros

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module", autouse=True)
def _register_oracle_kernels():
    # tests may use the oracle; the package itself never imports it
    register_mlstm_kernel("chunkwise--native_custbw", O.mlstm_chunkwise__native_custbw)
    register_mlstm_kernel("chunkwise--native_autograd", O.mlstm_chunkwise__native_autograd)
    register_mlstm_step_kernel("native", O.mlstm_recurrent_step__native)
    register_mlstm_sequence_kernel("native_sequence__native", O.mlstm_recurrent_sequence__native_fw)


def test_registry_names_and_errors():
    assert {"chunkwise--hip_xl_chunk", "chunkwise--hip_xl_chunk_siging"} <= set(get_available_mlstm_kernels())
    assert "hip" in get_available_mlstm_step_kernels()
    assert "native_sequence__hip" in get_available_mlstm_sequence_kernels()
    assert callable(get_mlstm_kernel("chunkwise--hip_xl_chunk"))
    assert callable(get_mlstm_step_kernel("hip"))
    assert callable(get_mlstm_sequence_kernel("native_sequence__hip"))
    with pytest.raises(ValueError):
        get_mlstm_kernel("chunkwise--does_not_exist")
    with pytest.raises(ValueError):
        get_mlstm_kernel("nomodule--hip_xl_chunk")
    with pytest.raises(ValueError):
        get_mlstm_step_kernel("triton")
    with pytest.raises(ValueError):
        get_mlstm_sequence_kernel("nope")


def test_config_defaults_and_validation():
    cfg = mLSTMBackendConfig()
    assert (cfg.chunk_size, cfg.return_last_states, cfg.autocast_kernel_dtype, cfg.eps) == (64, True, "bfloat16", 1e-6)
    assert (cfg.inference_state_dtype, cfg.normalize_siging, cfg.mode) == ("float32", True, "train")
    with pytest.raises(ValueError):
        mLSTMBackendConfig(mode="train_with_padding", return_last_states=True)
    with pytest.raises(ValueError):
        mLSTMBackendConfig(chunkwise_kernel="parallel--native_custbw", return_last_states=True)
    mLSTMBackendConfig(mode="train_with_padding", return_last_states=False)


def test_shape_rules_of_the_xl_chunk_operator():
    validate_xl_chunk_shapes(256, 128)
    validate_xl_chunk_shapes(64, 128)   # short power-of-two sequences are one chunk
    validate_xl_chunk_shapes(16, 64)
    with pytest.raises(AssertionError):
        validate_xl_chunk_shapes(250, 128)      # not a multiple of 16
    with pytest.raises(AssertionError):
        validate_xl_chunk_shapes(48, 64)        # < 128 and not a power of two
    with pytest.raises(AssertionError):
        validate_xl_chunk_shapes(384, 256)      # not divisible by the chunk size


def test_operator_options_are_validated_on_the_host():
    """The options this package adds to or honours from the reference's keyword set: chunk_size_intra -> state stride
    (mlstm_kernels/triton/chunkwise/kernel_param_heuristics.py:118-121), kernel path, head norm, state dtype."""
    from mlstm_kernels_amd.torch.chunkwise.hip_xl_chunk import _recompute_states, _state_stride
    from mlstm_kernels_amd.torch.recurrent.hip_step import _check_state_dtype

    # recompute_states_in_bw (mlstm_kernels/torch/chunkwise/triton_xl_chunk/fwbw.py:45,62): honoured, default False here
    assert _recompute_states({}) is False and _recompute_states({"recompute_states_in_bw": None}) is False
    assert _recompute_states({"recompute_states_in_bw": True}) is True
    assert _recompute_states({"recompute_states_in_bw": False}) is False
    with pytest.raises(ValueError):
        _recompute_states({"recompute_states_in_bw": "yes"})
    assert _state_stride({}, "op") == 0                                   # library default
    assert _state_stride({"chunk_size_intra": 128}, "op") == 1
    assert _state_stride({"chunk_size_inter": 128, "chunk_size_intra": 512}, "op") == 4
    assert _state_stride({"siz_b_L_parallel": 64, "num_warps_intra": 4, "recompute_states_in_bw": True}, "op") == 0
    assert _state_stride({"chunk_size_inter": 64, "chunk_size_intra": 256}, "op") == 2   # the scan's own chunk stays 128
    assert _state_stride({"chunk_size_inter": 64, "chunk_size_intra": 64}, "op") == 1
    for bad in ({"chunk_size_inter": 96}, {"chunk_size_inter": 256}, {"chunk_size_intra": 192}, {"chunk_size_intra": 2048},
                {"chunk_size_intra": 0}, {"chunk_size_inter": 128, "chunk_size_intra": 64}):
        with pytest.raises(ValueError):
            _state_stride(bad, "op")
    with pytest.raises(TypeError, match="unexpected keyword"):
        _state_stride({"chunk_size_itnra": 256}, "op")
    assert [_lib.path_code(n) for n in ("auto", "split", "fused")] == [_lib.PATH_AUTO, _lib.PATH_SPLIT, _lib.PATH_FUSED]
    with pytest.raises(ValueError):
        _lib.path_code("triton")
    assert [_lib.norm_code(n) for n in ("none", "layer", "rms")] == [_lib.NORM_NONE, _lib.NORM_LAYER, _lib.NORM_RMS]
    with pytest.raises(ValueError):
        _lib.norm_code("group")
    for ok in (torch.float32, torch.bfloat16, torch.float16):
        assert _check_state_dtype(ok) is ok
    with pytest.raises(NotImplementedError):
        _check_state_dtype(torch.float64)


def test_hip_kernels_have_no_cpu_fallback():
    q, k, v, i, f = make_qkvif(1, 1, 128, 64, 64)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        get_mlstm_kernel("chunkwise--hip_xl_chunk")(q, k, v, i, f)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        get_mlstm_step_kernel("hip")(q[:, :, 0], k[:, :, 0], v[:, :, 0], i[:, :, :1], f[:, :, :1],
                                     torch.zeros(1, 1, 64, 64), torch.zeros(1, 1, 64), torch.zeros(1, 1, 1))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "mlstm_hip.h")).read()
    declared = sorted(set(re.findall(r"\b(mlstm_hip_\w+)\s*\(", header)))
    assert declared, "no declarations found in include/mlstm_hip.h"
    assert declared == _lib.exported_symbols(), "ctypes signature table and header disagree"
    if not os.path.exists(_lib.lib_path()):
        pytest.skip("libmlstm_hip.so not built (run `python -m mlstm_kernels_amd.build`)")
    lib = _lib.get_lib()
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in the header but not exported by the library"
    assert lib.mlstm_hip_abi_version() == _lib.ABI_VERSION
    # size queries and argument validation work without a GPU (no kernel is launched)
    assert lib.mlstm_hip_chunkwise_fw_workspace_bytes(1, 2, 256, 64, 128, 1, _lib.PATH_AUTO, 0) > 0
    assert lib.mlstm_hip_chunkwise_fw_workspace_bytes(1, 2, 256, 60, 128, 1, _lib.PATH_AUTO, 0) == 0
    assert lib.mlstm_hip_chunkwise_fw_workspace_bytes(1, 2, 256, 960, 128, 1, _lib.PATH_AUTO, 0) == 0   # DHQK limit: 896
    assert lib.mlstm_hip_chunkwise_fw_workspace_bytes(1, 2, 256, 896, 128, 1, _lib.PATH_AUTO, 0) > 0
    assert lib.mlstm_hip_chunkwise_fw_workspace_bytes(1, 2, 256, 64, 128, 1, _lib.PATH_FUSED, 0) == 0  # fused: 128/256 only
    assert lib.mlstm_hip_chunkwise_fw_workspace_bytes(1, 2, 256, 64, 128, 1, _lib.PATH_AUTO, 9) == 0   # stride 1 .. 8
    # a chunk state kept every second chunk halves the state part of the workspace
    full = lib.mlstm_hip_chunkwise_fw_workspace_bytes(1, 2, 4096, 256, 512, 1, _lib.PATH_SPLIT, 1)
    half = lib.mlstm_hip_chunkwise_fw_workspace_bytes(1, 2, 4096, 256, 512, 1, _lib.PATH_SPLIT, 2)
    assert full - half == 2 * 16 * 256 * 512 * 2
    assert lib.mlstm_hip_chunkwise_bw_workspace_bytes(1, 2, 256, 64, 128, 0) > 0
    rc = lib.mlstm_hip_step(None, None, None, None, None, None, None, None, None, None, None, None,
                            1, 1, 64, 64, 1e-6, 1, 0, 0, None)
    assert rc != 0 and b"null pointer" in lib.mlstm_hip_last_error()


# ------------------------------------------------------------------ the small fp32 shape: CPU plumbing check
def test_backend_module_train_mode_cpu_plumbing():
    # B=1, NH=4, S=256, DHQK=64, DHHV=64, chunk_size=64, fp32, zero initial states, return_last_states=True
    q, k, v, i, f = make_qkvif(1, 4, 256, 64, 64, seed=0, dtype=torch.float32)
    backend = mLSTMBackend(mLSTMBackendConfig(chunkwise_kernel="chunkwise--native_custbw", sequence_kernel="native_sequence__native",
                                              step_kernel="native", chunk_size=64, autocast_kernel_dtype="float32"))
    H, (C, n, m) = backend(q, k, v, i, f)
    assert H.shape == (1, 4, 256, 64) and H.dtype == q.dtype
    assert C.shape == (1, 4, 64, 64) and n.shape == (1, 4, 64) and m.shape == (1, 4, 1)
    H_par, _, _ = O.parallel_stablef_fw(q.double(), k.double(), v.double(), i.double(), f.double())
    H_rec, (C_r, n_r, m_r) = O.recurrent_sequence(q.double(), k.double(), v.double(), i.double(), f.double())
    torch.testing.assert_close(H.double(), H_par, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(H.double(), H_rec, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(C.double(), C_r, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(m.double(), m_r, rtol=1e-5, atol=1e-5)
    assert backend(q, k, v, i, f, return_last_states=False).shape == H.shape


@pytest.mark.parametrize("S", [1, 7, 65, 93, 500])
def test_arbitrary_sequence_length_wrapper(S):
    q, k, v, i, f = make_qkvif(1, 2, S, 32, 32, seed=S, dtype=torch.float64)
    i, f = i.double(), f.double()
    H, (C, n, m) = wrap_chunkwise__arbitrary_sequence_length(
        mlstm_chunkwise_kernel=O.mlstm_chunkwise__native_custbw,
        mlstm_sequence_kernel=lambda **kw: O.mlstm_recurrent_sequence__native_fw(dtype_state=torch.float64, **kw),
        mlstm_step_kernel=lambda **kw: O.mlstm_recurrent_step__native(dtype_state=torch.float64, **kw),
        q=q, k=k, v=v, f=f, i=i, chunk_size=64, dtype_state=torch.float64)
    H_ref, (C_r, n_r, m_r) = O.recurrent_sequence(q, k, v, i, f)
    torch.testing.assert_close(H, H_ref, rtol=1e-9, atol=1e-9)
    torch.testing.assert_close(C, C_r, rtol=1e-9, atol=1e-9)
    torch.testing.assert_close(n, n_r, rtol=1e-9, atol=1e-9)
    torch.testing.assert_close(m, m_r, rtol=1e-9, atol=1e-9)


def test_arbitrary_sequence_length_wrapper_hands_whole_sequence_to_a_capable_kernel():
    """A chunkwise kernel that announces `supports_any_sequence_length` gets ONE call with the whole sequence."""
    calls = []

    def kernel(**kw):
        calls.append(kw)
        return O.mlstm_chunkwise__native_custbw(**{k_: v_ for k_, v_ in kw.items() if k_ != "any_sequence_length"}, )

    kernel.supports_any_sequence_length = True
    S = 96   # a length the oracle's chunkwise formulation accepts in one piece (chunk 32), so the fake can delegate
    q, k, v, i, f = make_qkvif(1, 2, S, 32, 32, seed=5, dtype=torch.float64)
    i, f = i.double(), f.double()

    def fail(**kw):
        raise AssertionError("token loop must not run")

    H, (C, n, m) = wrap_chunkwise__arbitrary_sequence_length(
        mlstm_chunkwise_kernel=kernel, mlstm_sequence_kernel=fail, mlstm_step_kernel=fail,
        q=q, k=k, v=v, f=f, i=i, chunk_size=32, dtype_state=torch.float64)
    assert len(calls) == 1 and calls[0]["any_sequence_length"] is True and calls[0]["q"].shape[2] == S
    H_ref, (C_r, n_r, m_r) = O.recurrent_sequence(q, k, v, i, f)
    torch.testing.assert_close(H, H_ref, rtol=1e-9, atol=1e-9)
    torch.testing.assert_close(C, C_r, rtol=1e-9, atol=1e-9)


def test_backend_inference_mode_threads_states():
    q, k, v, i, f = make_qkvif(1, 2, 100, 32, 32, seed=3, dtype=torch.float32)
    backend = mLSTMBackend(mLSTMBackendConfig(chunkwise_kernel="chunkwise--native_custbw", sequence_kernel="native_sequence__native",
                                              step_kernel="native", chunk_size=32, mode="inference", autocast_kernel_dtype="float32"))
    H, st = backend(q, k, v, i, f)
    H1, st1 = backend(q[:, :, :63], k[:, :, :63], v[:, :, :63], i[:, :, :63], f[:, :, :63])
    outs = [H1]
    for t in range(63, 100):   # generation: one token at a time through the step kernel
        h, st1 = backend(q[:, :, t:t + 1], k[:, :, t:t + 1], v[:, :, t:t + 1], i[:, :, t:t + 1], f[:, :, t:t + 1], *st1)
        outs.append(h)
    torch.testing.assert_close(torch.cat(outs, 2), H, rtol=1e-4, atol=1e-4)
    for a, b in zip(st1, st):
        torch.testing.assert_close(a, b, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("S", [128, 65, 1, 400])
def test_pad_zeros_wrapper(S):
    q, k, v, i, f = make_qkvif(1, 2, S, 32, 32, seed=S, dtype=torch.float64)
    i, f = i.double(), f.double()
    H = wrap_chunkwise__pad_zeros(O.mlstm_chunkwise__native_custbw, q=q, k=k, v=v, f=f, i=i, chunk_size=64)
    H_ref, _ = O.recurrent_sequence(q, k, v, i, f)
    assert H.shape == H_ref.shape
    torch.testing.assert_close(H, H_ref, rtol=1e-8, atol=1e-8)
    with pytest.raises(AssertionError):
        wrap_chunkwise__pad_zeros(O.mlstm_chunkwise__native_custbw, q=q, k=k, v=v, f=f, i=i, return_last_states=True)


def test_reference_kernel_names_are_opt_in_aliases():
    """A configuration written for the reference (its Triton kernel names) selects the HIP kernels once
    use_reference_kernel_names() has been called; before that the names are unknown, and the reference's other
    kernels (native, limit_chunk, parallel) stay unknown afterwards: nothing falls back to another implementation."""
    import mlstm_kernels_amd.torch as T

    saved = ({m: dict(e) for m, e in T._extra_kernels.items()}, dict(T._extra_step), dict(T._extra_sequence))
    before = (set(get_available_mlstm_kernels()), set(get_available_mlstm_step_kernels()),
              set(get_available_mlstm_sequence_kernels()))
    try:
        with pytest.raises(ValueError):
            get_mlstm_kernel("chunkwise--triton_xl_chunk")
        T.use_reference_kernel_names()
        assert get_mlstm_kernel("chunkwise--triton_xl_chunk") is get_mlstm_kernel("chunkwise--hip_xl_chunk")
        assert get_mlstm_kernel("chunkwise--triton_xl_chunk_siging") is get_mlstm_kernel("chunkwise--hip_xl_chunk_siging")
        assert get_mlstm_step_kernel("triton") is get_mlstm_step_kernel("hip")
        assert get_mlstm_sequence_kernel("native_sequence__triton") is get_mlstm_sequence_kernel("native_sequence__hip")
        cfg = mLSTMBackendConfig(chunkwise_kernel="chunkwise--triton_xl_chunk", sequence_kernel="native_sequence__triton",
                                 step_kernel="triton", chunk_size=128, mode="inference")
        backend = mLSTMBackend(cfg)
        assert backend.chunkwise_kernel_fn is get_mlstm_kernel("chunkwise--hip_xl_chunk")
        # exactly these four names were added (other tests may have registered stand-ins of their own before)
        assert set(get_available_mlstm_kernels()) - before[0] == {"chunkwise--triton_xl_chunk", "chunkwise--triton_xl_chunk_siging"}
        assert set(get_available_mlstm_step_kernels()) - before[1] == {"triton"}
        assert set(get_available_mlstm_sequence_kernels()) - before[2] == {"native_sequence__triton"}
        with pytest.raises(ValueError):
            get_mlstm_kernel("chunkwise--triton_limit_chunk")
    finally:
        T._extra_kernels.clear(), T._extra_kernels.update(saved[0])
        T._extra_step.clear(), T._extra_step.update(saved[1])
        T._extra_sequence.clear(), T._extra_sequence.update(saved[2])


def test_noalloc_scratch_size_matches_the_header():
    """_lib.NOALLOC_SCRATCH_BYTES mirrors MLSTM_NOALLOC_SCRATCH_BYTES of include/mlstm_hip.h: parsed here, not retyped."""
    import os
    import re

    from mlstm_kernels_amd import _lib

    header = open(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "mlstm_hip.h")).read()
    m = re.search(r"#define\s+MLSTM_NOALLOC_SCRATCH_BYTES\s+\((\d+)u\s*<<\s*(\d+)\)", header)
    assert m, "MLSTM_NOALLOC_SCRATCH_BYTES not found in the header"
    assert int(m.group(1)) << int(m.group(2)) == _lib.NOALLOC_SCRATCH_BYTES
    for name, code in (("MLSTM_PATH_AUTO", _lib.PATH_AUTO), ("MLSTM_PATH_SPLIT", _lib.PATH_SPLIT),
                       ("MLSTM_PATH_FUSED", _lib.PATH_FUSED), ("MLSTM_PATH_STREAM", _lib.PATH_STREAM)):
        m = re.search(r"#define\s+" + name + r"\s+(\d+)", header)
        assert m and int(m.group(1)) == code, name


def test_chunk_size_sets_the_state_stride_like_the_reference_default():
    """chunk_size_intra defaults to the target chunk size in the reference (kernel_param_heuristics.py:96-121): 256 or
    more therefore names the distance between kept states here too; 128 leaves it to the library."""
    from mlstm_kernels_amd.torch.chunkwise.hip_xl_chunk import _state_stride

    assert _state_stride({}, "op", 128) == 0
    assert _state_stride({}, "op", 64) == 0
    assert _state_stride({}, "op", 256) == 2
    assert _state_stride({}, "op", 512) == 4
    assert _state_stride({}, "op", 2048) == 8
    assert _state_stride({"chunk_size_intra": 128}, "op", 512) == 1   # an explicit value wins


def test_recurrent_sequence_rejects_what_it_does_not_implement():
    import pytest
    import torch

    from mlstm_kernels_amd.torch.recurrent import mlstm_recurrent_sequence__hip

    t = torch.zeros(1, 1, 2, 64)
    g = torch.zeros(1, 1, 2)
    with pytest.raises(NotImplementedError, match="return_all_states"):
        mlstm_recurrent_sequence__hip(t, t, t, g, g, return_all_states=True)
    with pytest.raises(TypeError, match="unexpected keyword"):
        mlstm_recurrent_sequence__hip(t, t, t, g, g, no_such_option=1)


def test_float32_operand_option_is_validated_before_anything_runs():
    """float32_operands: "bfloat16" (default) or "float16" for float32 inputs; anything else, or float16 on the fused
    path (which multiplies bfloat16 operands only), is rejected when the operator is built."""
    import pytest
    import torch
    from mlstm_kernels_amd.torch.chunkwise.hip_xl_chunk import _get_fwbw

    a = _get_fwbw(torch.float32, False, True, "auto", 0)
    b = _get_fwbw(torch.float32, False, True, "auto", 0, float32_operands="float16")
    assert a is not b and a is _get_fwbw(torch.float32, False, True, "auto", 0, float32_operands="bfloat16")
    with pytest.raises(ValueError, match="float32_operands"):
        _get_fwbw(torch.float32, False, True, "auto", 0, float32_operands="float32")
    with pytest.raises(ValueError, match="bfloat16 operands only"):
        _get_fwbw(torch.float32, False, True, "fused", 0, float32_operands="float16")
