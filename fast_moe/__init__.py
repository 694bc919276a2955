"""The reference's import root.  ``fast_moe.kernels.moe``, ``fast_moe.kernels.moe_fp8``,
``fast_moe.kernels.utils``, ``fast_moe.modules.fast_moe_module``, ``fast_moe.utils.utils`` and
``fast_moe.dev_settings`` resolve to the modules of ``fast_moe_amd`` (the same module objects, no
second copy), so that code written against meta-recsys/fast_moe's operator path imports
unchanged.  Three more paths name types that live elsewhere in ``fast_moe_amd``:
``fast_moe.kernels.triton.triton_moe`` the two option dataclasses the reference's callers import
from it (the HIP operators accept and ignore them), ``fast_moe.utils.enums`` the three option
enumerations, ``fast_moe.utils.configs`` the SGMoE configuration and output types.  Nothing else
of the reference's package is provided here.
"""
import importlib
import sys
import types

import fast_moe_amd
from fast_moe_amd import FastMoELayer, GatingNetwork, KernelType, __version__

for _name in ("kernels", "kernels.utils", "kernels.moe", "kernels.moe_fp8", "modules", "modules.fast_moe_module",
              "utils", "utils.utils", "dev_settings"):
    _mod = importlib.import_module("fast_moe_amd." + _name)
    sys.modules[__name__ + "." + _name] = _mod
    if "." not in _name:
        globals()[_name] = _mod

# the option types under the module path the reference's tests import them from
_triton = types.ModuleType(__name__ + ".kernels.triton")
_triton_moe = types.ModuleType(__name__ + ".kernels.triton.triton_moe")
_triton_moe.__doc__ = "Option dataclasses of the operator API (defined in fast_moe_amd.kernels.moe); no Triton here."
_triton_moe.IndexSelectJaggedBmmOption = kernels.moe.IndexSelectJaggedBmmOption
_triton_moe.SiluJaggedBmmCombineOption = kernels.moe.SiluJaggedBmmCombineOption
_triton.triton_moe = _triton_moe
sys.modules[_triton.__name__] = _triton
sys.modules[_triton_moe.__name__] = _triton_moe

# the SGMoE configuration and output types under the module path the reference keeps them at
# (utils/configs.py:13-33); they are defined next to the layer that uses them
_configs = types.ModuleType(__name__ + ".utils.configs")
_configs.__doc__ = "SGConfig, MRNOutput (defined in fast_moe_amd.modules.sgmoe)."
from fast_moe_amd.modules.sgmoe import MRNOutput, SGConfig  # noqa: E402
_configs.SGConfig, _configs.MRNOutput = SGConfig, MRNOutput
sys.modules[_configs.__name__] = _configs

# the option enumerations under the module path the reference keeps them at (utils/enums.py)
_enums = types.ModuleType(__name__ + ".utils.enums")
_enums.__doc__ = "ExpertType, RouterChoice, LossType (defined in fast_moe_amd.utils)."
from fast_moe_amd.utils import ExpertType, LossType, RouterChoice  # noqa: E402
_enums.ExpertType, _enums.RouterChoice, _enums.LossType = ExpertType, RouterChoice, LossType
sys.modules[_enums.__name__] = _enums

__all__ = ["FastMoELayer", "GatingNetwork", "KernelType", "ExpertType", "RouterChoice", "LossType", "__version__"]
