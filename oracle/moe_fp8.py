"""FP8 operator oracle (torch on CPU; quantisation through oracle.fp8).

TEST INFRASTRUCTURE ONLY -- never imported by the product package.

Restates /root/reference/kernels/pytorch/moe_fp8.py:78-139 and composes the
same emulation into the SwiGLU / down-projection / combine chain that the
fp8 configurations run (the reference has no single fp8 SwiGLU function; the
composition follows its fp8 gather-GEMM for every GEMM and its bf16 rounding
points for the element-wise steps).
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import numpy as np
import torch
from torch.nn import functional as F

from . import fp8 as _fp8
from .moe import _sizes, mul_merge_k_add


def _dtype_name(t: torch.Tensor) -> str:
    return {torch.bfloat16: "bf16", torch.float32: "fp32"}[t.dtype]


def rowwise_quant_fp8(a: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """quant_fp8.py:27-34 on a torch tensor: returns (uint8 codes, fp32 multiplier scale)."""
    codes, scale = _fp8.rowwise_quant_fp8(a.contiguous().float().numpy(), _dtype_name(a))
    return torch.from_numpy(codes), torch.from_numpy(scale)


def dequant(codes: torch.Tensor) -> torch.Tensor:
    """uint8 e4m3fn codes -> fp32 values."""
    return torch.from_numpy(_fp8.e4m3fn_decode(codes.numpy()))


def index_select_jagged_bmm_raw(offsets, index, jagged, weight, bias):
    """moe_fp8.py:78-95: the unquantised form of the same op."""
    E = weight.shape[0]
    A = index.shape[-1]
    flat = index.reshape(-1)
    return torch.cat(
        [
            jagged[flat[offsets[e]: offsets[e + 1]] // A] @ weight[e]
            + (bias[e] if bias is not None else 0)
            for e in range(E)
        ],
        dim=0,
    )


def fp8_linear_per_expert(q_rows: List[torch.Tensor], s_rows: List[torch.Tensor],
                          q_w: torch.Tensor, s_w: torch.Tensor, bias, out_dtype):
    """moe_fp8.py:127-137: ``(bf16(qa) @ bf16(qw).T) / (sa x sw)`` cast, plus bias.

    q_rows[e] : [m_e, K] fp32 holding e4m3 values; s_rows[e] : [m_e] multiplier scales
    q_w       : [E, N, K] fp32 holding e4m3 values; s_w : [E, N]
    """
    out = []
    for e in range(len(q_rows)):
        acc = torch.matmul(q_rows[e].to(torch.bfloat16), q_w[e].T.to(torch.bfloat16))
        y = (acc / (s_rows[e][:, None] * s_w[e][None, :])).to(out_dtype)
        out.append(y + (bias[e] if bias is not None else 0))
    return out


def index_select_jagged_bmm_fp8(offsets, index, jagged, weight, bias):
    """moe_fp8.py:98-139 -> [L*A, N] in the input dtype."""
    assert jagged.dtype == weight.dtype and (bias is None or bias.dtype == jagged.dtype)
    qw_c, s_w = rowwise_quant_fp8(weight.permute(0, 2, 1))       # [E, N, K], [E, N]
    qa_c, s_a = rowwise_quant_fp8(jagged)                        # [L, K], [L]
    q_w, q_a = dequant(qw_c), dequant(qa_c)
    token = index.reshape(-1) // index.shape[-1]
    sizes = _sizes(offsets)
    q_rows = list(q_a[token].split(sizes))
    s_rows = list(s_a[token].split(sizes))
    return torch.cat(fp8_linear_per_expert(q_rows, s_rows, q_w, s_w, bias, jagged.dtype), dim=0)


def index_select_jagged_bmm_fp8_backward(offsets, index, jagged, weight, bias, d_out):
    """Backward of the fp8 gather-GEMM as the Triton operator runs it
    (kernels/triton/triton_moe_fp8.py:1201-1340): every GEMM operand re-quantised to e4m3,

    * d_jagged: d_out quantised per row, weight [E, K, N] per (e, k) row along N; the products
      are dequantised with the two reciprocal scales (:971-979), land at their [L, A] position
      in fp32 and are summed over A, then cast (:1244-1249, 1337);
    * d_weight: jagged and d_out quantised per COLUMN over all their rows
      (transpose_rowwise_quant, :1281-1286), contracted over the rows of each expert, the
      left operand gathered by token (:1075-1087), dequantised the same way (:1094-1103);
    * d_bias: plain per-expert column sums of d_out (:1320-1335).

    Parity pinned by tests/test_oracle_moe.py: on inputs whose quantisation is lossless the three
    results equal torch autograd through the unquantised operator.
    Returns (d_jagged [L, K], d_weight [E, K, N], d_bias [E, N] or None)."""
    L, A = index.shape
    E, K, N = weight.shape
    flat = index.reshape(-1)
    token = flat // A
    sizes = _sizes(offsets)
    bounds = [(int(offsets[e]), int(offsets[e + 1])) for e in range(E)]

    qd_c, s_d = rowwise_quant_fp8(d_out)                    # [R, N], [R]
    qw_c, s_w = rowwise_quant_fp8(weight)                   # [E, K, N], [E, K]
    qd, qw = dequant(qd_c), dequant(qw_c)
    expanded = torch.zeros((L * A, K), dtype=torch.float32)
    for e, (lo, hi) in enumerate(bounds):
        acc = qd[lo:hi] @ qw[e].T                           # [m_e, K]
        acc = (acc * (1.0 / s_d[lo:hi])[:, None]) * (1.0 / s_w[e])[None, :]
        expanded[flat[lo:hi]] = acc
    d_jagged = expanded.view(L, A, K).sum(dim=1).to(jagged.dtype)

    qjt_c, s_j = (torch.from_numpy(t) for t in _fp8.transpose_rowwise_quant_fp8(
        jagged.contiguous().float().numpy(), _dtype_name(jagged)))      # [K, L], [K]
    qdt_c, s_t = (torch.from_numpy(t) for t in _fp8.transpose_rowwise_quant_fp8(
        d_out.contiguous().float().numpy(), _dtype_name(d_out)))        # [N, R], [N]
    qjt, qdt = dequant(qjt_c), dequant(qdt_c)
    d_weight = torch.zeros((E, K, N), dtype=weight.dtype)
    for e, (lo, hi) in enumerate(bounds):
        if hi > lo:
            acc = qjt[:, token[lo:hi]] @ qdt[:, lo:hi].T    # [K, N]
            d_weight[e] = ((acc * (1.0 / s_j)[:, None]) * (1.0 / s_t)[None, :]).to(weight.dtype)
    d_bias = None
    if bias is not None:
        d_bias = torch.stack([d_out[lo:hi].float().sum(dim=0) for lo, hi in bounds]).to(bias.dtype)
    return d_jagged, d_weight, d_bias


def swiglu_moe_fp8(offsets, index, jagged, w_gate, b_gate, w_up, b_up, w_down, b_down,
                   token_index, k, gates=None, gates_index=None):
    """The fp8 SwiGLU MoE forward as a composition of the emulated fp8 GEMM:
    tokens quantised per row before the gather, gate/up weights per output row,
    ``silu(g) * u`` with the bf16 rounding points of moe.py:125-139, hidden
    re-quantised per row, down projection, weighted merge (moe.py:14-37).
    Weights are given [E, K, N] like every operator.  Returns (out, hidden)."""
    dt = jagged.dtype
    qa_c, s_a = rowwise_quant_fp8(jagged)
    q_a = dequant(qa_c)
    token = index.reshape(-1) // index.shape[-1]
    sizes = _sizes(offsets)
    q_rows = list(q_a[token].split(sizes))
    s_rows = list(s_a[token].split(sizes))

    def w_quant(w):
        c, s = rowwise_quant_fp8(w.permute(0, 2, 1))
        return dequant(c), s

    qg, sg = w_quant(w_gate)
    qu, su = w_quant(w_up)
    g = fp8_linear_per_expert(q_rows, s_rows, qg, sg, b_gate, dt)
    u = fp8_linear_per_expert(q_rows, s_rows, qu, su, b_up, dt)
    hidden = torch.cat([F.silu(x) * y for x, y in zip(g, u)], dim=0)

    qh_c, s_h = rowwise_quant_fp8(hidden)
    q_h = dequant(qh_c)
    qd, sd = w_quant(w_down)
    y = torch.cat(
        fp8_linear_per_expert(list(q_h.split(sizes)), list(s_h.split(sizes)), qd, sd, b_down, dt),
        dim=0,
    )
    return mul_merge_k_add(token_index, y, k, gates, gates_index), hidden
