"""ctypes binding of libmlstm_hip.so (C ABI in include/mlstm_hip.h).  Loading fails loudly."""
from __future__ import annotations

import ctypes
import os
import threading

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libmlstm_hip.so")
_lock = threading.Lock()
_lib = None

F32, BF16 = 0, 1
F16 = 2
GATE_EXP, GATE_SIG = 0, 1
PATH_AUTO, PATH_SPLIT, PATH_FUSED, PATH_STREAM = 0, 1, 2, 3
NORM_NONE, NORM_LAYER, NORM_RMS = 0, 1, 2
ABI_VERSION = 6
NOALLOC_SCRATCH_BYTES = 64 << 20  # MLSTM_NOALLOC_SCRATCH_BYTES of include/mlstm_hip.h

_vp, _i, _f, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t

_SIGNATURES = {
    "mlstm_hip_abi_version": (_i, []),
    "mlstm_hip_last_error": (ctypes.c_char_p, []),
    "mlstm_hip_profile_enable": (_i, [_i]),
    "mlstm_hip_profile_read": (_i, [_i, ctypes.c_char_p, _sz, ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_int)]),
    "mlstm_hip_step": (_i, [_vp] * 12 + [_i, _i, _i, _i, _f, _i, _i, _i, _vp]),
    "mlstm_hip_recurrent_sequence": (_i, [_vp] * 12 + [_i, _i, _i, _i, _i, _f, _i, _i, _i, _vp]),
    "mlstm_hip_chunkwise_fw_workspace_bytes": (_sz, [_i] * 8),
    "mlstm_hip_chunkwise_fw": (_i, [_vp] * 15 + [_sz, _i] + [_i] * 5 + [_f] + [_i] * 7 + [_f, _vp, _vp] + [_vp]),
    "mlstm_hip_chunkwise_fw_saved_bytes": (_sz, [_i] * 5),
    "mlstm_hip_chunkwise_recompute_states": (_i, [_vp] * 4 + [_sz] + [_i] * 7 + [_vp]),
    "mlstm_hip_head_norm_bw": (_i, [_vp] * 4 + [_sz, _i, _i, _i, _vp]),
    "mlstm_hip_chunkwise_fw_noalloc": (_i, [_vp] * 14 + [_i] * 5 + [_f] + [_i] * 4 + [_vp]),
    "mlstm_hip_chunkwise_bw_workspace_bytes": (_sz, [_i] * 6),
    "mlstm_hip_chunkwise_bw": (_i, [_vp] * 14 + [_sz, _vp, _sz] + [_i] * 5 + [_f] + [_i] * 6 + [_vp]),
}


def lib_path() -> str:
    return _LIB_PATH


def exported_symbols() -> list[str]:
    return sorted(_SIGNATURES)


def get_lib() -> ctypes.CDLL:
    """Return the loaded library; raise RuntimeError if it was not built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(_LIB_PATH):
                raise RuntimeError(
                    f"{_LIB_PATH} not found. The HIP kernels are the only implementation of this package; "
                    "build them with `python -m mlstm_kernels_amd.build` (needs hipcc, targets gfx950)."
                )
            # The host process shares ONE HIP runtime between torch (which owns the device memory and the streams
            # passed in) and this library: torch is imported first so that its runtime is the one the library binds
            # to.  Loaded in the other order, two runtimes end up in the process and the second sees no device.
            import torch  # noqa: F401

            lib = ctypes.CDLL(_LIB_PATH)
            for name, (res, args) in _SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype = res
                fn.argtypes = args
            if lib.mlstm_hip_abi_version() != ABI_VERSION:
                raise RuntimeError(
                    f"libmlstm_hip.so has ABI version {lib.mlstm_hip_abi_version()}, expected {ABI_VERSION}; rebuild it."
                )
            _lib = lib
    return _lib


_PATH_CODES = {"auto": PATH_AUTO, "split": PATH_SPLIT, "fused": PATH_FUSED, "stream": PATH_STREAM}
_NORM_CODES = {"none": NORM_NONE, "layer": NORM_LAYER, "rms": NORM_RMS}


def norm_code(name: str) -> int:
    """'none' / 'layer' / 'rms' (the norm specifiers of the reference's apply_normalize) -> the C ABI's code."""
    try:
        return _NORM_CODES[name]
    except KeyError:
        raise ValueError(f"Unsupported norm specifier {name}.") from None


def path_code(name: str) -> int:
    """'auto' / 'split' / 'fused' / 'stream' -> the C ABI's kernel path code."""
    try:
        return _PATH_CODES[name]
    except KeyError:
        raise ValueError(f"unknown kernel path {name!r}; expected one of {sorted(_PATH_CODES)}") from None


def default_state_stride(B: int, NH: int, S: int, DHQK: int, DHHV: int) -> int:
    """The state stride the library picks for this shape when asked for 0 (read off its own workspace sizes)."""
    lib = get_lib()
    size = lambda s: lib.mlstm_hip_chunkwise_fw_workspace_bytes(B, NH, S, DHQK, DHHV, 1, PATH_SPLIT, s)
    chosen = size(0)
    for s in range(1, 9):
        if size(s) == chosen:
            return s
    raise RuntimeError("cannot determine the default state stride")


def profile_enable(on: bool) -> None:
    get_lib().mlstm_hip_profile_enable(int(on))


def profile_read() -> dict[str, tuple[float, int]]:
    """{kernel name: (summed milliseconds, launches)} of everything recorded since the last read."""
    lib = get_lib()
    out: dict[str, tuple[float, int]] = {}
    buf = ctypes.create_string_buffer(64)
    ms, cnt = ctypes.c_float(0.0), ctypes.c_int(0)
    n = lib.mlstm_hip_profile_read(0, buf, 64, ctypes.byref(ms), ctypes.byref(cnt))  # index 0 aggregates
    for idx in range(n):
        if idx > 0:
            lib.mlstm_hip_profile_read(idx, buf, 64, ctypes.byref(ms), ctypes.byref(cnt))
        out[buf.value.decode()] = (ms.value, cnt.value)
    return out


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = get_lib().mlstm_hip_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed: {msg}")
