"""The reference's import root: ``fast_moe.kernels.moe``, ``fast_moe.kernels.moe_fp8``,
``fast_moe.kernels.utils``, ``fast_moe.modules.fast_moe_module``, ``fast_moe.utils.utils`` and
``fast_moe.utils.configs`` resolve to the modules of ``fast_moe_amd`` (the same module objects, no
second copy), so that code written against meta-recsys/fast_moe's operator path imports
unchanged.  Nothing else of the reference's package is provided here.
"""
import importlib
import sys

import fast_moe_amd
from fast_moe_amd import FastMoELayer, GatingNetwork, KernelType, __version__

for _name in ("kernels", "kernels.utils", "kernels.moe", "kernels.moe_fp8", "modules", "modules.fast_moe_module",
              "utils", "utils.utils", "utils.configs"):
    _mod = importlib.import_module("fast_moe_amd." + _name)
    sys.modules[__name__ + "." + _name] = _mod
    if "." not in _name:
        globals()[_name] = _mod

__all__ = ["FastMoELayer", "GatingNetwork", "KernelType", "__version__"]
