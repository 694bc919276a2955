"""Import path of the reference's utils/configs.py: the SGMoE configuration and output types,
defined next to the layer that uses them."""
from ..modules.sgmoe import MRNOutput, SGConfig

__all__ = ["MRNOutput", "SGConfig"]
