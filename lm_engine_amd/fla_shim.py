"""Makes the unmodified reference layer resolve its two imports to this package.

The reference imports ``chunk_gated_delta_rule`` and ``fused_recurrent_gated_delta_rule`` from
``fla.ops.gated_delta_rule`` when ``import fla`` succeeds
(lm_engine/modeling_utils/sequence_mixer_blocks/gated_deltanet/module.py:24-25,
lm_engine/utils/packages.py:56-65).  ``install_as_fla()`` registers stand-in modules of those
names in ``sys.modules`` *before* lm_engine is imported, so the layer binds to the HIP
operator without any edit.  It refuses to shadow a real ``fla`` installation.
"""

from __future__ import annotations

import importlib.util
import sys
import types

from . import ops


_MODULE_NAMES = ("fla", "fla.ops", "fla.ops.gated_delta_rule")


def install_as_fla(force: bool = False) -> types.ModuleType:
    """Registers ``fla.ops.gated_delta_rule`` backed by lm_engine_amd.ops; returns that module."""
    already_ours = getattr(sys.modules.get("fla"), "__lm_engine_amd_shim__", False)
    if not already_ours and not force:
        if "fla" in sys.modules or importlib.util.find_spec("fla") is not None:
            raise RuntimeError("a real `fla` package is installed; pass force=True to shadow it")

    modules = {}
    for name in _MODULE_NAMES:
        module = types.ModuleType(name)
        module.__lm_engine_amd_shim__ = True
        module.__path__ = []  # mark as package so sub-imports resolve through sys.modules
        modules[name] = module

    leaf = modules["fla.ops.gated_delta_rule"]
    leaf.chunk_gated_delta_rule = ops.chunk_gated_delta_rule
    leaf.fused_recurrent_gated_delta_rule = ops.fused_recurrent_gated_delta_rule
    modules["fla"].ops = modules["fla.ops"]
    modules["fla.ops"].gated_delta_rule = leaf

    sys.modules.update(modules)
    return leaf


def uninstall_fla_shim() -> None:
    for name in _MODULE_NAMES:
        if getattr(sys.modules.get(name), "__lm_engine_amd_shim__", False):
            del sys.modules[name]
