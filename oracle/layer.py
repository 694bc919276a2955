"""FastMoELayer forward oracle (PYTORCH-kernel path) and the dense every-expert
MoE used as its independent end-to-end check.

TEST INFRASTRUCTURE ONLY -- never imported by the product package.

Restates /root/reference/modules/fast_moe_module.py:188-225 (gate softmax, top-k,
routing metadata, GEMM1, SiLU + GEMM2 + weighted merge) and the dense
formulation of /root/reference/modules/moe_base.py:79-94.
"""
from __future__ import annotations

from typing import Dict

import numpy as np
import torch
from torch.nn import functional as F

from . import moe as _moe
from . import routing as _routing


def _dtype_name(dt: torch.dtype) -> str:
    return {torch.bfloat16: "bf16", torch.float32: "fp32"}[dt]


def gate_scores(x: torch.Tensor, gate_w: torch.Tensor, gate_b) -> torch.Tensor:
    """fast_moe_module.py:21-27: ``softmax(x @ Wg.T + bg)`` over experts, in x's dtype."""
    return F.softmax(F.linear(x, gate_w, gate_b), dim=-1)


def route_scores(scores: torch.Tensor, k: int) -> Dict[str, torch.Tensor]:
    """fast_moe_module.py:93-144 on [T, E] scores -> torch tensors (int64 / scores' dtype)."""
    meta = _routing.route(scores.float().numpy(), k, dtype=_dtype_name(scores.dtype))
    out = {}
    for name, v in meta.items():
        if name == "max_seq_len":
            out[name] = v
        elif name == "gates":
            out[name] = torch.from_numpy(v).to(scores.dtype)
        else:
            out[name] = torch.from_numpy(np.ascontiguousarray(v))
    return out


def moe_layer_forward(x, gate_w, gate_b, w_hidden, b_hidden, w_out, b_out, k: int):
    """fast_moe_module.py:188-225 with the PYTORCH kernel.

    x [B, S, D]; gate_w [E, D]; w_hidden [E, H, D]; b_hidden [E, H];
    w_out [E, O, H]; b_out [E, O] -- the parameter layouts of :64-91.
    Returns ``(y [B, S, O], routing dict)``."""
    B, S, D = x.shape
    E = w_hidden.shape[0]
    scores = gate_scores(x, gate_w, gate_b).reshape(-1, E)
    r = route_scores(scores, k)
    x_flat = x.reshape(-1, D)
    hidden = _moe.index_select_jagged_bmm(
        r["offsets"], r["gate_index"].view(-1, k), x_flat,
        w_hidden.permute(0, 2, 1).to(x.dtype), b_hidden.to(x.dtype))
    y = _moe.silu_jagged_bmm_combine(
        r["offsets"], hidden, w_out.permute(0, 2, 1).to(x.dtype), b_out.to(x.dtype),
        r["token_index"], k, r["gates"], r["gate_index"], has_silu=True)
    return y.view(B, S, -1), r


def dense_moe_forward(x, gate_w, gate_b, w_hidden, b_hidden, w_out, b_out, k: int):
    """moe_base.py:79-94 with SiLU experts: every expert runs on every token, the
    masked, L1-normalised gate matrix weights the outputs."""
    scores = gate_scores(x, gate_w, gate_b)
    _, topk = scores.topk(k, dim=-1, sorted=False)
    mask = torch.zeros_like(scores).scatter_(-1, topk, 1)
    gates = F.normalize(scores * mask, p=1, dim=-1)
    outs = torch.stack(
        [F.linear(F.silu(F.linear(x, w_hidden[e], b_hidden[e])), w_out[e], b_out[e])
         for e in range(w_hidden.shape[0])], dim=-2)          # [B, S, E, O]
    return torch.einsum("bte,bteo->bto", gates, outs)
