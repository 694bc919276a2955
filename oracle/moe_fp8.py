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


# rows x cols above which rowwise_quant_fp8 takes the library cast instead of the bit-level encoder
_BITS_LIMIT = 1 << 21


def rowwise_quant_fp8(a: torch.Tensor, cast: Optional[str] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """quant_fp8.py:27-34 on a torch tensor: returns (uint8 codes, fp32 multiplier scale).

    ``cast="bits"``: the numpy bit-level encoder of oracle.fp8 (about 1 us per element).
    ``cast="torch"``: the same scale formula, then ``Tensor.to(torch.float8_e4m3fn)``, the
    library routine quant_fp8.py:33 itself calls; for the operands of the large configurations
    (10^9 weight elements).  Default: by size.  tests/test_oracle_fp8.py pins the two against
    each other (random rows, outliers, zeros, subnormal results, inf / NaN rows)."""
    if cast is None:
        cast = "bits" if a.numel() <= _BITS_LIMIT else "torch"
    if cast == "bits":
        codes, scale = _fp8.rowwise_quant_fp8(a.contiguous().float().numpy(), _dtype_name(a))
        return torch.from_numpy(codes), torch.from_numpy(scale)
    assert cast == "torch", cast
    amax = a.abs().amax(dim=-1).float()
    scale = torch.from_numpy(_fp8.calculate_scale(amax.numpy(), _dtype_name(a)))
    codes = torch.empty(a.shape, dtype=torch.uint8)
    flat_a, flat_c, flat_s = a.reshape(-1, a.shape[-1]), codes.view(-1, a.shape[-1]), scale.reshape(-1)
    step = max(1, (1 << 24) // a.shape[-1])         # bounded fp32 temporaries
    for lo in range(0, flat_a.shape[0], step):
        scaled = flat_a[lo: lo + step].float() * flat_s[lo: lo + step, None]
        flat_c[lo: lo + step] = scaled.to(torch.float8_e4m3fn).view(torch.uint8)
    return codes, scale


def dequant(codes: torch.Tensor) -> torch.Tensor:
    """uint8 e4m3fn codes -> fp32 values (large operands: the library's decode, equal to the
    table of oracle.fp8 for all 256 codes by tests/test_oracle_fp8.py)."""
    if codes.numel() > _BITS_LIMIT:
        return codes.contiguous().view(torch.float8_e4m3fn).to(torch.float32)
    return torch.from_numpy(_fp8.e4m3fn_decode(codes.numpy()))


class LazyDequant:
    """``q_w[e]`` -> fp32 values [N, K] of expert e's e4m3 codes, decoded on demand: the weight
    operand of ``fp8_linear_per_expert`` for configurations whose decoded weights would not be
    worth holding (10^9 elements)."""

    def __init__(self, codes: torch.Tensor):
        self.codes = codes

    def __getitem__(self, e):
        return dequant(self.codes[e])

    def __len__(self):
        return self.codes.shape[0]


def quantize_weight(w: torch.Tensor):
    """Weight [E, K, N] (any strides) -> (LazyDequant over codes [E, N, K], scale [E, N]): one scale
    per (expert, output row), the quantisation moe_fp8.py:111 applies to ``weight.permute(0, 2, 1)``."""
    codes, scale = rowwise_quant_fp8(w.permute(0, 2, 1))
    return LazyDequant(codes), scale


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
        if q_rows[e].shape[0] == 0:                 # an expert without rows: nothing to decode
            out.append(torch.empty((0, s_w.shape[1]), dtype=out_dtype))
            continue
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
                   token_index, k, gates=None, gates_index=None, quantized=None):
    """The fp8 SwiGLU MoE forward as a composition of the emulated fp8 GEMM:
    tokens quantised per row before the gather, gate/up weights per output row,
    ``silu(g) * u`` with the bf16 rounding points of moe.py:125-139, hidden
    re-quantised per row, down projection, weighted merge (moe.py:14-37).
    Weights are given [E, K, N] like every operator.  ``quantized``: the three
    ``quantize_weight`` results of (w_gate, w_up, w_down) when the caller holds them already
    (then the weight arguments are not read).  Returns (out, hidden)."""
    dt = jagged.dtype
    qa_c, s_a = rowwise_quant_fp8(jagged)
    q_a = dequant(qa_c)
    token = index.reshape(-1) // index.shape[-1]
    sizes = _sizes(offsets)
    q_rows = list(q_a[token].split(sizes))
    s_rows = list(s_a[token].split(sizes))

    if quantized is None:
        quantized = (quantize_weight(w_gate), quantize_weight(w_up), quantize_weight(w_down))
    (qg, sg), (qu, su), (qd, sd) = quantized
    g = fp8_linear_per_expert(q_rows, s_rows, qg, sg, b_gate, dt)
    u = fp8_linear_per_expert(q_rows, s_rows, qu, su, b_up, dt)
    hidden = torch.cat([F.silu(x) * y for x, y in zip(g, u)], dim=0)

    qh_c, s_h = rowwise_quant_fp8(hidden)
    q_h = dequant(qh_c)
    y = torch.cat(
        fp8_linear_per_expert(list(q_h.split(sizes)), list(s_h.split(sizes)), qd, sd, b_down, dt),
        dim=0,
    )
    return mul_merge_k_add(token_index, y, k, gates, gates_index), hidden
