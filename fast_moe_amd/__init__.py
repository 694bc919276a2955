"""fast_moe_amd: the MoE-forward hot path of meta-recsys/fast_moe as hand-written
gfx950 (MI355X) HIP kernels behind the reference's operator API."""
from .kernels.utils import KernelType
from .modules.fast_moe_module import FastMoELayer, GatingNetwork
from .modules.sgmoe import MRNOutput, SGConfig, SGMoE

__version__ = "0.1.0"
__all__ = ["FastMoELayer", "GatingNetwork", "KernelType", "MRNOutput", "SGConfig", "SGMoE", "__version__"]
