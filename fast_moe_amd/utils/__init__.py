"""Router front-end helpers of the SGMoE / MRN layer (reference: utils/utils.py), and the three
option enumerations callers of the reference import beside them (reference: utils/enums.py:10-26,
re-exported by utils/__init__.py:8 and the package root).  Nothing on the MoE forward path reads the
enumerations; they are here so that such imports resolve, with the reference's member names and values."""
from enum import Enum, unique

ExpertType = unique(Enum("ExpertType", {"MLP": "MLP", "FFN": "FFN", "FFNBIAS": "FFN_WITH_BIAS"}, module=__name__))
RouterChoice = unique(Enum("RouterChoice", {"TopK": "TOP_K", "Vanilla": "VANILLA"}, module=__name__))
LossType = unique(Enum("LossType", {"LB": "LOAD_BALANCE", "MI": "MUTAL_INFORMATION"}, module=__name__))

__all__ = ["ExpertType", "RouterChoice", "LossType"]
