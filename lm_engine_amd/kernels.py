"""Kernel flag registry in the reference's convention.

The reference switches every accelerated kernel with a module-global table read at forward
time (lm_engine/kernels.py:15-63, enum at lm_engine/enums.py:61-93): ``is_kernel_allowed``,
the ``enable_kernels`` context manager and the ``ENABLE_KERNELS`` / ``ENABLE_ALL_KERNELS``
environment variables.  Its GatedDeltaNet layer is the one mixer without an entry there; this
module adds that entry, ``Kernel.gated_delta_rule``, with the same interface so the layer can
guard the HIP operator the way the other mixers guard theirs.

Difference from the reference: ``gated_delta_rule`` is ON by default, and switching it off makes
the operator raise: this package ships no second implementation to fall back to.

``Kernel.gated_delta_rule_fused_launch`` (on by default as well) lets the chunked forward run its prepare and
scan steps as one launch for the shapes where that is the faster way (``GDN_FLAG_FUSED_LAUNCH`` of the C ABI:
fixed-length batches whose scan fills about half of the GPU).  Results stay within the same parity gates, but
they are not bit-identical to the two-kernel path, which every other batch takes (packed, left-padded, few or
many sequences): switch it off - ``enable_kernels([Kernel.gated_delta_rule], reset=True)`` or
``ENABLE_KERNELS=gated_delta_rule`` - where runs of different batch shapes are compared bit for bit.
"""

from __future__ import annotations

import os
from contextlib import contextmanager
from enum import Enum


class Kernel(Enum):
    gated_delta_rule = "gated_delta_rule"
    gated_delta_rule_fused_launch = "gated_delta_rule_fused_launch"


_ON_BY_DEFAULT = (Kernel.gated_delta_rule, Kernel.gated_delta_rule_fused_launch)
_KERNELS: dict[Kernel, bool] = {kernel: kernel in _ON_BY_DEFAULT for kernel in Kernel}


def enable_kernels_from_env_variable() -> None:
    """``ENABLE_KERNELS`` is a comma-separated allow-list as in the reference; when set, kernels
    it does not name are switched off.  ``ENABLE_ALL_KERNELS`` switches everything on."""
    if os.getenv("ENABLE_ALL_KERNELS", "False").lower() in ("1", "true"):
        assert not os.getenv("ENABLE_KERNELS", "")
        for kernel in Kernel:
            _KERNELS[kernel] = True
        return

    names = [name.strip() for name in os.getenv("ENABLE_KERNELS", "").split(",") if name.strip()]
    if not names:
        return
    known = {kernel.value for kernel in Kernel}
    listed = {name for name in names if name in known}  # names of the reference's other kernels are ignored
    for kernel in Kernel:
        _KERNELS[kernel] = kernel.value in listed


enable_kernels_from_env_variable()


def is_kernel_allowed(kernel: Kernel) -> bool:
    return _KERNELS[kernel]


@contextmanager
def enable_kernels(kernels: list[Kernel], reset: bool = False):
    """Inside the block the listed kernels are on; with ``reset=True`` every other one is off.
    The previous table is restored on exit (same contract as lm_engine/kernels.py:47-63)."""
    global _KERNELS

    original = dict(_KERNELS)
    updated = {} if reset else dict(original)
    for kernel in Kernel:
        if reset or not original[kernel]:
            updated[kernel] = kernel in kernels
    _KERNELS = updated

    try:
        yield
    finally:
        _KERNELS = original


@contextmanager
def enable_all_kernels():
    with enable_kernels(list(Kernel)):
        yield
