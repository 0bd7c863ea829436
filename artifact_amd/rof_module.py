"""Loader of the compiled operator module `artifact_amd/_ROF*.so` (csrc/rof_torch.cpp): upstream's seven `ROF`
functions (ROF/reuse_conv/reuse_conv.cpp:353-365) as a C++ extension over librof.so's C ABI.

    from artifact_amd import rof_module
    ROF = rof_module.compiled()          # or: rof_module.install()  ->  `import ROF` finds the compiled module

`artifact_amd.ROF` is the same interface written in Python over ctypes (it additionally accepts a prebuilt
layout); both produce the same bits.  There is no fallback: a missing module raises.
"""
from __future__ import annotations

import importlib
import os
import sys

from . import _lib

_HERE = os.path.dirname(os.path.abspath(__file__))


def compiled():
    """The compiled module; raises ImportError naming the build command if it has not been built."""
    import torch  # noqa: F401  (the module links against PyTorch's libraries: load them first)

    _lib.lib()    # librof.so, with the HIP runtime PyTorch brought
    try:
        return importlib.import_module("artifact_amd._ROF")
    except ImportError as ex:
        raise ImportError(f"artifact_amd/_ROF*.so is not built or does not load ({ex}); run "
                          f"`python -m artifact_amd.build`") from ex


def install(name="ROF"):
    """Register the compiled module under upstream's module name, so that `import ROF` (reuse_conv.py:2) finds it."""
    mod = compiled()
    sys.modules[name] = mod
    return mod
