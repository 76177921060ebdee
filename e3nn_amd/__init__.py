"""MI355X-native implementation of e3nn's equivariant message-passing hot path.

``e3nn_amd.o3`` mirrors the API of ``e3nn.o3`` for ``Irreps``, ``wigner_3j``,
``TensorProduct``, ``FullyConnectedTensorProduct`` and ``spherical_harmonics``; the
arithmetic runs in hand-written HIP kernels (gfx950) reached through a C ABI.
"""
from typing import Any, Dict

__version__ = "0.1.0"

# Accepted for API compatibility with e3nn.set_optimization_defaults / get_optimization_defaults
# (reference e3nn/__init__.py:12,53-82); the HIP path has a single code path, so the flags only
# round-trip.
_OPT_DEFAULTS: Dict[str, Any] = dict(specialized_code=True, optimize_einsums=True, jit_script_fx=True, jit_mode="eager")


def set_optimization_defaults(**kwargs) -> None:
    for k, v in kwargs.items():
        if k not in _OPT_DEFAULTS:
            raise ValueError(f"Unknown optimization option: {k}")
        _OPT_DEFAULTS[k] = v


def get_optimization_defaults() -> Dict[str, Any]:
    return dict(_OPT_DEFAULTS)


from . import o3  # noqa: E402,F401
