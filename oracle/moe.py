"""bf16 / fp32 operator oracle (torch on CPU).

TEST INFRASTRUCTURE ONLY -- never imported by the product package.

Restates the semantics of /root/reference/kernels/pytorch/moe.py.  Shapes use the
reference's letters: L tokens, E experts, A (=K_top) activated experts per token,
K input dim, N output dim.  Every function keeps the reference's rounding
points: a per-expert ``F.linear`` result is rounded to the input dtype before
the next element-wise op.
"""
from __future__ import annotations

from typing import List, Optional

import torch
from torch.nn import functional as F


def _sizes(offsets: torch.Tensor) -> List[int]:
    return (offsets[1:] - offsets[:-1]).tolist()


def _gather_split(offsets, index, jagged):
    """moe.py:66-73: rows of ``jagged`` in expert-sorted order, split per expert."""
    token = index.reshape(-1) // index.shape[-1]
    return list(jagged[token].contiguous().split(_sizes(offsets)))


def _linear_per_expert(rows: List[torch.Tensor], weight_kn: torch.Tensor, bias):
    """moe.py:75-82: ``rows[e] @ weight[e] + bias[e]`` with weight given [E, K, N]."""
    w_t = weight_kn.permute(0, 2, 1)
    return [
        F.linear(rows[e], w_t[e], bias[e] if bias is not None else None)
        for e in range(len(rows))
    ]


def index_select_jagged_bmm(offsets, index, jagged, weight, bias):
    """moe.py:40-84 -> [L*A, N]."""
    rows = _gather_split(offsets, index, jagged)
    return torch.cat(_linear_per_expert(rows, weight, bias), dim=0)


def index_select_jagged_bmm_swiglu(offsets, index, jagged, weight, bias, weight_p, bias_p):
    """moe.py:87-146: ``silu(x W + b) * (x Wp + bp)`` per expert."""
    rows = _gather_split(offsets, index, jagged)
    a = _linear_per_expert(rows, weight, bias)
    b = _linear_per_expert(rows, weight_p, bias_p)
    return torch.cat([F.silu(x) * y for x, y in zip(a, b)], dim=0)


def index_select_jagged_gating_bmm(
    offsets, index, jagged_a, jagged_b, weight_a, weight_b, bias_a, bias_b
):
    """moe.py:149-221: ``silu(A Wa + ba) * (B Wb + bb)`` with two inputs."""
    rows_a = _gather_split(offsets, index, jagged_a)
    rows_b = rows_a if jagged_a is jagged_b else _gather_split(offsets, index, jagged_b)
    alpha = torch.cat(_linear_per_expert(rows_a, weight_a, bias_a), dim=0)
    beta = torch.cat(_linear_per_expert(rows_b, weight_b, bias_b), dim=0)
    return F.silu(alpha) * beta


def index_select_jagged_bmm_3D(offsets, index, jagged, weight, bias):
    """moe.py:224-252: jagged [L, E, K]; expert e reads slice ``[:, e, :]``."""
    rows = _gather_split(offsets, index, jagged)
    w_t = weight.permute(0, 2, 1)
    out = [
        F.linear(rows[e][:, e, :], w_t[e], bias[e] if bias is not None else None)
        for e in range(len(rows))
    ]
    return torch.cat(out, dim=0)


def silu_jagged_bmm(offsets, jagged, weight, bias, has_silu: bool = True):
    """moe.py:255-275 composed with the permute of :287: weight given [E, K, N],
    rows already expert-sorted."""
    if has_silu:
        jagged = F.silu(jagged)
    rows = list(jagged.split(_sizes(offsets)))
    return torch.cat(_linear_per_expert(rows, weight, bias), dim=0)


def mul_merge_k_add(index, value, k: int, weight: Optional[torch.Tensor] = None,
                    weight_index: Optional[torch.Tensor] = None):
    """moe.py:14-37: product in the promoted dtype of (value, weight), fp32
    ``index_add`` in ascending row order, cast back to the product's dtype."""
    if weight is not None:
        assert weight_index is not None
        assert weight.numel() == weight_index.numel() == value.shape[0]
        value = value.mul(weight.contiguous().view(-1)[weight_index].view(-1, 1))
    acc = torch.zeros(index.shape[0] // k, value.shape[1], dtype=torch.float32)
    return acc.index_add(0, index, value.float()).to(value.dtype)


def silu_jagged_bmm_combine(offsets, jagged, weight, bias, index, k,
                            gating_scores=None, gates_index=None, has_silu=True):
    """moe.py:278-303."""
    bmm_out = silu_jagged_bmm(offsets, jagged, weight, bias, has_silu)
    return mul_merge_k_add(index, bmm_out, k, gating_scores, gates_index)


def fused_jagged_bmm_swiglu_combine(offsets, index, jagged, weight, bias, weight_p, bias_p,
                                    weight_out, bias_out, k, gates=None, gates_index=None):
    """moe.py:306-391: SwiGLU GEMM, down GEMM and combine in one call."""
    hidden = index_select_jagged_bmm_swiglu(offsets, index, jagged, weight, bias, weight_p, bias_p)
    token = index.reshape(-1) // index.shape[-1]
    rows = list(hidden.split(_sizes(offsets)))
    out = torch.cat(_linear_per_expert(rows, weight_out, bias_out), dim=0)
    return mul_merge_k_add(token, out, k, gates, gates_index)
