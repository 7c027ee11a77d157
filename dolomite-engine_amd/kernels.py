"""Global kernel allow-set and the ``enable_kernels`` context manager.

Behaviour follows lm_engine/kernels.py:21-49: a module-global set; entering a context REPLACES the
set (it does not merge with an outer context) and the previous set is put back on exit.  Unlike the
reference the restore sits in a ``finally`` so an exception inside the block cannot leak the
inner set.

``ENABLE_ALL_CUTE_KERNELS`` (lm_engine/kernels.py:14-19, 75-76): when the variable is set to a true value
at import time and the kernels can run at all (a GPU is visible and the library is built -- the counterpart
of the reference's ``is_cute_kernels_available()``), every kernel is switched on for the life of the process,
as if the whole program ran inside ``enable_all_kernels()``.
"""

import os
from contextlib import contextmanager

from .enums import Kernel


def _boolean_env_variable(name: str, default: bool) -> bool:
    """"1" / "true" (any case) are true, "0" / "false" false; anything else is an error."""
    value = os.environ.get(name)
    if value is None:
        return default
    value = value.strip().lower()
    if value in ("1", "true"):
        return True
    if value in ("0", "false", ""):
        return False
    raise ValueError(f"{name} must be one of 1 / true / 0 / false, got {value!r}")


def _kernels_available() -> bool:
    import torch

    from . import _lib

    return torch.cuda.is_available() and _lib.is_built()


_KERNELS: set[Kernel] = set()


def is_kernel_allowed(kernel: Kernel) -> bool:
    return kernel in _KERNELS


@contextmanager
def enable_kernels(kernels: set[Kernel] | list[Kernel]):
    if not isinstance(kernels, set):
        kernels = set(kernels)

    global _KERNELS
    previous = _KERNELS
    _KERNELS = kernels
    try:
        yield
    finally:
        _KERNELS = previous


@contextmanager
def enable_all_kernels():
    with enable_kernels([k for k in Kernel if k != Kernel.ladder_residual_overlapped_layer]):
        yield


def _enable_all_from_environment() -> bool:
    """The import-time switch (lm_engine/kernels.py:14-19, 75-76).  Returns whether it switched anything on."""
    global _KERNELS
    if not _boolean_env_variable("ENABLE_ALL_CUTE_KERNELS", False) or not _kernels_available():
        return False
    _KERNELS = {k for k in Kernel if k != Kernel.ladder_residual_overlapped_layer}
    return True


_ENABLE_ALL_KERNELS = _enable_all_from_environment()
