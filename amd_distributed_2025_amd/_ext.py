"""Loader of the torch extension built by `build.build_extension()`.

The module `_ext/moe_a2a_torch.so` holds the torch::Tensor wrappers of
`csrc/moe_a2a_torch.cpp` (the binding idiom of the reference's submissions,
all2all/hipv8.py:230-252) and is linked against `libmoe_a2a.so`. It is loaded
as built; nothing is compiled here and there is no fallback.
"""
from __future__ import annotations

import importlib.util

from . import _lib
from .build import EXT_DIR, EXT_NAME

MODULE = EXT_DIR / f"{EXT_NAME}.so"
_mod = None


def load():
    """Import the built extension once. Raises if it has not been built."""
    global _mod
    if _mod is not None:
        return _mod
    if not MODULE.exists():
        raise _lib.MoeA2AError(
            f"{MODULE} is missing: build it with `python -m amd_distributed_2025_amd.build` "
            "(or use binding='ctypes')"
        )
    import torch  # noqa: F401  the module links against torch's libraries

    _lib.load()  # the C ABI library the wrappers call into
    spec = importlib.util.spec_from_file_location(EXT_NAME, str(MODULE))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    if mod.a2a_version() != _lib.load().moe_a2a_version().decode():
        raise _lib.MoeA2AError("the extension and libmoe_a2a.so were built from different versions of the ABI")
    _mod = mod
    return mod
