"""Router front-end helpers of the SGMoE / MRN layer (reference: utils/utils.py)."""
