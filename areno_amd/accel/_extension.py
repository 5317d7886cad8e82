"""Lazy loader for the compiled ``areno_amd.accel._areno_accel`` PyTorch-ROCm extension.

Same contract as the reference's loader (``areno/accel/_extension.py:21-41``): the module is
imported on first use, there is no Python fallback, and a missing build raises a
``RuntimeError`` that says what to do.
"""

from __future__ import annotations

import importlib
import os
from types import ModuleType

_EXT: ModuleType | None = None


def extension() -> ModuleType:
    """Return the compiled HIP extension module, importing it on first call."""
    global _EXT
    if _EXT is None:
        try:
            _EXT = importlib.import_module("areno_amd.accel._areno_accel")
        except ImportError as exc:
            skipped = os.environ.get("ARENO_BUILD_EXT", "").strip().lower() in {"0", "false", "no", "off"}
            build_hint = " ARENO_BUILD_EXT is set to skip the native build in this environment." if skipped else ""
            raise RuntimeError(
                "AReno runtime setup failed: the compiled `areno_accel` extension is not installed."
                f"{build_hint}\n"
                "Why: the paged attention ops run only as HIP kernels on an AMD GPU; there is no Python fallback.\n"
                "Next steps: build it in-tree with `python setup.py build_ext --inplace` (needs ROCm's hipcc and a "
                f"ROCm build of PyTorch). Import error: {exc}"
            ) from exc
    return _EXT


def library_path() -> str:
    """Path of the C-ABI shared library (``include/areno_hip.h``) that sits beside this file."""
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), "libareno_hip.so")
