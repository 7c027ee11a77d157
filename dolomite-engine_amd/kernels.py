"""Global kernel allow-set and the ``enable_kernels`` context manager.

Behaviour follows lm_engine/kernels.py:21-49: a module-global set; entering a context REPLACES the
set (it does not merge with an outer context) and the previous set is put back on exit.  Unlike the
reference the restore sits in a ``finally`` so an exception inside the block cannot leak the
inner set.
"""

from contextlib import contextmanager

from .enums import Kernel


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
