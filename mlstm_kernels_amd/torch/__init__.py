"""Name -> callable registries of the HIP mLSTM operators, with the lookup functions of the reference
(mlstm_kernels/torch/__init__.py:7-120): kernel names are ``"<module>--<backend>"`` for sequence kernels
(``"chunkwise--hip_xl_chunk"``, ``"chunkwise--hip_xl_chunk_siging"``), plain backend names for step
(``"hip"``) and token-loop kernels (``"native_sequence__hip"``).  Unknown names raise ``ValueError``.

``register_mlstm_kernel`` / ``register_mlstm_step_kernel`` / ``register_mlstm_sequence_kernel`` let a host
application add further callables under its own names (the package itself ships HIP kernels only).
``use_reference_kernel_names()`` additionally answers to the reference's own Triton names, so that a configuration
written for NX-AI/mlstm_kernels (e.g. ``chunkwise_kernel="chunkwise--triton_xl_chunk"``, ``step_kernel="triton"``)
selects the HIP kernels unchanged."""
from __future__ import annotations

from collections.abc import Callable

_extra_kernels: dict[str, dict[str, Callable]] = {}
_extra_step: dict[str, Callable] = {}
_extra_sequence: dict[str, Callable] = {}


def _module_registry() -> dict[str, dict[str, Callable]]:
    from .chunkwise import registry as chunkwise_registry

    reg: dict[str, dict[str, Callable]] = {"chunkwise": dict(chunkwise_registry)}
    for module, entries in _extra_kernels.items():
        reg.setdefault(module, {}).update(entries)
    return reg


def _step_registry() -> dict[str, Callable]:
    from .recurrent import registry_step

    return {**registry_step, **_extra_step}


def _sequence_registry() -> dict[str, Callable]:
    from .recurrent import registry_sequence

    return {**registry_sequence, **_extra_sequence}


def register_mlstm_kernel(name: str, fn: Callable) -> None:
    module, backend = name.split("--")
    _extra_kernels.setdefault(module, {})[backend] = fn


def register_mlstm_step_kernel(name: str, fn: Callable) -> None:
    _extra_step[name] = fn


def register_mlstm_sequence_kernel(name: str, fn: Callable) -> None:
    _extra_sequence[name] = fn


# reference name -> name here (mlstm_kernels/torch/chunkwise/__init__.py:9-15, recurrent/__init__.py:13-24)
_REFERENCE_CHUNKWISE = {"chunkwise--triton_xl_chunk": "chunkwise--hip_xl_chunk",
                        "chunkwise--triton_xl_chunk_siging": "chunkwise--hip_xl_chunk_siging"}
_REFERENCE_STEP = {"triton": "hip"}
_REFERENCE_SEQUENCE = {"native_sequence__triton": "native_sequence__hip"}


def use_reference_kernel_names() -> None:
    """Opt-in: registers the HIP kernels under the reference's Triton kernel names as well (the TFLA chunkwise
    kernels, the fused step and the step-fused sequence kernel -- the ones this package replaces).  The reference's
    other names (native_*, limit_chunk, parallel--*) stay unknown and raise ``ValueError``: there is no fallback."""
    for ref, own in _REFERENCE_CHUNKWISE.items():
        register_mlstm_kernel(ref, get_mlstm_kernel(own))
    for ref, own in _REFERENCE_STEP.items():
        register_mlstm_step_kernel(ref, get_mlstm_step_kernel(own))
    for ref, own in _REFERENCE_SEQUENCE.items():
        register_mlstm_sequence_kernel(ref, get_mlstm_sequence_kernel(own))


def get_available_mlstm_kernels() -> list[str]:
    return [f"{m}--{b}" for m, entries in _module_registry().items() for b in entries]


def get_mlstm_kernel(name: str) -> Callable:
    reg = _module_registry()
    module, backend = name.split("--")
    if module not in reg:
        raise ValueError(f"Unknown module name: {module}. Available module names: {list(reg.keys())}")
    if backend not in reg[module]:
        raise ValueError(
            f"Unknown mlstm kernel backend name: {backend}. Available backend names: {list(reg[module].keys())}"
        )
    return reg[module][backend]


def get_available_mlstm_step_kernels() -> list[str]:
    return list(_step_registry().keys())


def get_mlstm_step_kernel(name: str) -> Callable:
    reg = _step_registry()
    if name not in reg:
        raise ValueError(f"Unknown step kernel backend name: {name}. Available backend names: {list(reg.keys())}")
    return reg[name]


def get_available_mlstm_sequence_kernels() -> list[str]:
    return list(_sequence_registry().keys())


def get_mlstm_sequence_kernel(name: str) -> Callable:
    reg = _sequence_registry()
    if name not in reg:
        raise ValueError(f"Unknown backend name: {name}. Available backend names: {list(reg.keys())}")
    return reg[name]
