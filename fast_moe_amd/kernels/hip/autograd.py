"""Backward of the MoE operators on the HIP back-end (torch.autograd.Function wrappers).

What the reference's Triton autograd functions compute
(/root/reference/kernels/triton/triton_moe.py:606-804 index_select_jagged_bmm backward,
:62-141 fused SwiGLU backward, :922-983 merge backward, :3790-4027 silu_jagged_bmm_combine
backward), built from the library's kernels:

* input gradient  = grouped GEMM of the output gradient with the transposed weight (read in
  place; the two branches of a SwiGLU layer summed in one GEMM, fmoe_gemm_desc.a2), then the
  deterministic gather-form sum of the K routed rows of every token (fmoe_combine);
* weight gradient = grouped GEMM over the rows of each expert as its contraction window
  (fmoe_grouped_gemm + k_window), on the row-major tensors themselves (a_stride_k; the token
  rows first put in expert order by fmoe_gather_rows; both matrices of a SwiGLU layer from one
  launch, out2), or, for operands that do not qualify, on copies that fmoe_jagged_transpose
  laid out K-contiguous and zero padded;
* bias gradient   = fmoe_segment_colsum; activation and merge backward = fmoe_swiglu_bwd,
  fmoe_combine_bwd;
* the e4m3 operators: backward in bf16 for silu_jagged_bmm_combine_fp8, on re-quantised e4m3
  operands for index_select_jagged_bmm(fp8=True), as the reference's operators do.

Besides these kernels torch does index bookkeeping only, on [E]-, [R]-, [T, K]- and (3D variant)
[T, E, K]-sized integer tensors.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import ops
from ._lib import EPI_NONE, EPI_SWIGLU


_WINDOW_MULTIPLE = 64    # two 64-byte K-slices of bf16: what the LDS-ring GEMM steps by


def _pad_layout(offsets: torch.Tensor, total_rows: int) -> Tuple[torch.Tensor, int]:
    """Per-expert row counts rounded up to whole multiples of 64, at least 128 -> (padded prefix
    [E+1], host-side bound of its end)."""
    m = _WINDOW_MULTIPLE
    lengths = (offsets[1:] - offsets[:-1]).clamp_min(0)
    padded = ((lengths + m - 1) // m * m).clamp_min(2 * m)
    pad_offsets = torch.zeros_like(offsets)
    pad_offsets[1:] = torch.cumsum(padded, 0)
    E = offsets.numel() - 1
    bound = (total_rows + 2 * m * E + m - 1) // m * m
    return pad_offsets, bound


def _reverse_from_index(index: torch.Tensor) -> torch.Tensor:
    """index [T, K] (sorted position -> flat token*K+slot) -> [T, K] sorted positions of each
    token's rows, ascending (the order a sequential index_add meets them in)."""
    T, K = index.shape
    flat = index.reshape(-1)
    inv = torch.empty_like(flat)
    inv[flat] = torch.arange(flat.numel(), device=flat.device, dtype=flat.dtype)
    return inv.view(T, K).sort(dim=1).values


class _WgradOperand:
    """The input rows of the routed rows as the weight-gradient GEMM wants them, shared by the
    weight gradients of every weight that multiplied the same input (SwiGLU's gate and up
    projections).  Preferred form: the rows themselves in expert order with slack behind them
    (one gather copy when they are indexed), contracted in place with the row gradients.
    Otherwise: transposed and zero padded per expert ([K_in, bound])."""

    def __init__(self, a_src: torch.Tensor, offsets: torch.Tensor, total_rows: int, *,
                 row_index: Optional[torch.Tensor] = None, index_div: int = 1, apply_silu: bool = False):
        self.offsets = offsets
        self.args = (a_src, total_rows, row_index, index_div, apply_silu)
        self.rows = None            # [total_rows, K_in] in expert order, with slack
        self.a_t = None
        if a_src.dtype == torch.bfloat16 and a_src.ndim == 2 and a_src.shape[1] % 8 == 0:
            if row_index is None and not apply_silu:
                self.rows = a_src
            elif row_index is None:             # SiLU rounded as the forward GEMM rounds it on load
                self.rows = ops.silu_mul(a_src, None, with_slack=True)
            elif not apply_silu:
                self.rows = ops.gather_rows(a_src, row_index, index_div)

    def _transposed(self):
        if self.a_t is None:
            a_src, total_rows, row_index, index_div, apply_silu = self.args
            self.pad_offsets, self.bound = _pad_layout(self.offsets, total_rows)
            self.a_t = ops.jagged_transpose(a_src, self.offsets, self.pad_offsets, self.bound, row_index, index_div,
                                            apply_silu)

    def weight_grad_pair(self, both: torch.Tensor):
        """The weight gradients of two matrices whose row gradients lie side by side in ``both``
        [rows, 2 N], from one GEMM: ([E, N, K_in], [E, N, K_in]), or None when the operands do not
        qualify for the in-place kernel."""
        if self.rows is None:
            return None
        return ops.jagged_weight_grad(both, self.rows, self.offsets, halves=True)

    def weight_grad(self, dout: torch.Tensor) -> torch.Tensor:
        """dW[e, n, k] = sum over the rows r of expert e of dout[r, n] * a(r)[k] -> [E, N, K_in]."""
        if self.rows is not None:
            dw = ops.jagged_weight_grad(dout, self.rows, self.offsets)
            if dw is not None:
                return dw
        self._transposed()
        N = dout.shape[1]
        Kin = self.a_t.shape[0]
        E = self.offsets.numel() - 1
        dout_t = ops.jagged_transpose(dout, self.offsets, self.pad_offsets, self.bound)        # [N, bound]
        dev = dout.device
        seg = torch.arange(E + 1, device=dev, dtype=torch.int64) * N
        rows = torch.arange(E * N, device=dev, dtype=torch.int64) % N
        b = self.a_t.t().unsqueeze(0).expand(E, self.bound, Kin)                               # B[e, k, n'] = a_t[n', k]
        dw = ops.grouped_gemm(seg, dout_t, b, total_rows=E * N, row_index=rows, index_div=1, epilogue=EPI_NONE,
                              k_window=self.pad_offsets, k_window_multiple=_WINDOW_MULTIPLE)
        return dw.view(E, N, Kin)


def _input_grad(drow_list, weights, offsets, reverse_index) -> torch.Tensor:
    """sum over branches and over the K rows of a token of drow @ W^T -> [T, K_in]."""
    R = drow_list[0].shape[0]
    n = len(drow_list)
    Kin = weights[0].shape[1]
    if n == 2:      # both branches of a SwiGLU layer in one GEMM where the kernel allows
        w0, w1 = (w.permute(0, 2, 1) for w in weights)
        value = ops.grouped_gemm_sum2(offsets, drow_list[0], w0, drow_list[1], w1, total_rows=R)
        if value is not None:
            return ops.combine(value, reverse_index)
    value = torch.empty((n * R, Kin), dtype=drow_list[0].dtype, device=drow_list[0].device)
    for i, (d, w) in enumerate(zip(drow_list, weights)):
        ops.grouped_gemm(offsets, d, w.permute(0, 2, 1), total_rows=R, out=value[i * R:(i + 1) * R])
    if n == 1:
        return ops.combine(value, reverse_index)
    rev = torch.cat([reverse_index + i * R for i in range(n)], dim=1)
    return ops.combine(value, rev)


class IndexSelectJaggedBmm(torch.autograd.Function):
    """index_select_jagged_bmm and index_select_jagged_bmm_swiglu (weight_p is None or not)."""

    @staticmethod
    def forward(ctx, offsets, index, jagged, weight, bias, weight_p, bias_p):
        swiglu = weight_p is not None
        pre = None
        if swiglu:   # both pre-activations are kept for the backward pass, as the reference does
            out_dtype = torch.float32 if jagged.dtype == torch.float32 else torch.bfloat16
            pre = tuple(torch.empty((index.numel(), weight.shape[2]), dtype=out_dtype, device=jagged.device)
                        for _ in range(2))
        out = ops.grouped_gemm(offsets, jagged, weight, total_rows=index.numel(), row_index=index,
                               index_div=index.shape[-1], bias=bias, b2=weight_p, bias2=bias_p,
                               epilogue=EPI_SWIGLU if swiglu else EPI_NONE, aux=pre)
        ctx.save_for_backward(offsets, index, jagged, weight, bias, weight_p, bias_p, *(pre or (None, None)))
        return out

    @staticmethod
    def backward(ctx, dout):
        offsets, index, jagged, weight, bias, weight_p, bias_p, g, u = ctx.saved_tensors
        K = index.shape[-1]
        R = index.numel()
        dout = dout.contiguous()
        swiglu = weight_p is not None
        both = None
        if swiglu:      # dg | du side by side in one buffer: the GEMMs that need both read one operand
            dg, du = ops.swiglu_bwd(g, u, dout, joint=True)
            del g, u
            drows, weights = [dg, du], [weight, weight_p]
            both = ops.joint_rows(dg, du)
        else:
            drows, weights = [dout], [weight]
        need = ctx.needs_input_grad
        d_jagged = d_w = d_b = d_wp = d_bp = None
        if need[2]:
            d_jagged = _input_grad(drows, weights, offsets, _reverse_from_index(index)).view_as(jagged)
        operand = None
        if need[3] or (swiglu and need[5]):
            operand = _WgradOperand(jagged, offsets, R, row_index=index.reshape(-1), index_div=K)
        H = drows[0].shape[1]
        pair = None
        if both is not None and need[3] and need[5]:
            # one GEMM for both weight gradients (2H = 2816 rows per expert fill whole 256-row tiles
            # where H = 1408 leaves every sixth one half empty), each into its own tensor
            pair = operand.weight_grad_pair(both)
        if pair is not None:
            d_w, d_wp = pair[0].permute(0, 2, 1), pair[1].permute(0, 2, 1)
        else:
            if need[3]:
                d_w = operand.weight_grad(drows[0]).permute(0, 2, 1)
            if swiglu and need[5]:
                d_wp = operand.weight_grad(drows[1]).permute(0, 2, 1)
        if both is not None and bias is not None and bias_p is not None and need[4] and need[6]:
            d_sum = ops.segment_colsum(both, offsets)
            d_b, d_bp = d_sum[:, :H], d_sum[:, H:]
        else:
            if bias is not None and need[4]:
                d_b = ops.segment_colsum(drows[0], offsets)
            if swiglu and bias_p is not None and need[6]:
                d_bp = ops.segment_colsum(drows[1], offsets)
        return None, None, d_jagged, d_w, d_b, d_wp, d_bp


class IndexSelectJaggedBmmFp8(torch.autograd.Function):
    """index_select_jagged_bmm(fp8=True): forward and both backward GEMMs on e4m3 operands
    (kernels/triton/triton_moe_fp8.py:1114-1340).

    Backward, as the reference quantises: d_out per row and the weight per (expert, input row)
    along the output dimension for the input gradient; the gathered inputs and d_out per
    COLUMN for the weight gradient.  The column scales are taken over the routed rows in expert
    order, which hold every token at least once, so they are the reference's scales over all
    tokens.  The input gradient's rows are rounded to bf16 before the K rows of a token are
    summed (the reference sums them in fp32)."""

    @staticmethod
    def forward(ctx, offsets, index, jagged, weight, bias, fp8_weight):
        qa, sa = ops.quant_rows_fp8(jagged)
        ctx.save_for_backward(offsets, index, jagged, weight, bias)
        return ops.grouped_gemm(offsets, qa, fp8_weight[0], total_rows=index.numel(), row_index=index,
                                index_div=index.shape[-1], bias=bias, scales_pow2=ops.scales_are_pow2(sa, fp8_weight[1]),
                                a_scale=sa, b_scale=fp8_weight[1], epilogue=EPI_NONE)

    @staticmethod
    def backward(ctx, dout):
        offsets, index, jagged, weight, bias = ctx.saved_tensors
        E, Kin, N = weight.shape
        R, K = index.numel(), index.shape[-1]
        dout = dout.contiguous()
        need = ctx.needs_input_grad
        d_jagged = d_w = d_b = None
        if need[2]:
            qd, sd = ops.quant_rows_fp8(dout)                           # [R, N], [R]
            w_rows = weight
            if weight.stride(2) != 1 and weight.stride(1) == 1:         # rows along N strided: one transposing copy
                w_rows = ops.to_k_contiguous(weight.permute(0, 2, 1)).permute(0, 2, 1)
            qw, sw = ops.quant_rows_fp8(w_rows)                         # [E, Kin, N], [E, Kin]
            d_rows = ops.grouped_gemm(offsets, qd, qw.permute(0, 2, 1), total_rows=R, scales_pow2=True, a_scale=sd, b_scale=sw)
            d_jagged = ops.combine(d_rows, _reverse_from_index(index)).view_as(jagged)
        if need[3]:
            pad_offsets, bound = _pad_layout(offsets, R)
            a_t = ops.jagged_transpose(jagged, offsets, pad_offsets, bound, index.reshape(-1), K)   # [Kin, bound]
            d_t = ops.jagged_transpose(dout, offsets, pad_offsets, bound)                          # [N, bound]
            qa, sa = ops.quant_rows_fp8(a_t)                            # scales [Kin]
            qt, st = ops.quant_rows_fp8(d_t)                            # scales [N]
            # the gradient in the parameter's own memory order: [E, N, Kin] rows for K-contiguous storage
            by_n = weight.stride(1) == 1 and weight.stride(2) != 1
            (q_l, s_l, M), (q_r, s_r, C) = ((qt, st, N), (qa, sa, Kin)) if by_n else ((qa, sa, Kin), (qt, st, N))
            dev = dout.device
            seg = torch.arange(E + 1, device=dev, dtype=torch.int64) * M
            rows = torch.arange(E * M, device=dev, dtype=torch.int64) % M
            b = q_r.t().unsqueeze(0).expand(E, bound, C)                # B[e, r, c] = q_r[c, r]
            d_w = ops.grouped_gemm(seg, q_l, b, total_rows=E * M, row_index=rows, index_div=1,
                                   scales_pow2=True, a_scale=s_l, b_scale=s_r.unsqueeze(0).expand(E, C).contiguous(),
                                   k_window=pad_offsets, k_window_multiple=_WINDOW_MULTIPLE)
            d_w = d_w.view(E, M, C).to(weight.dtype)
            if by_n:
                d_w = d_w.permute(0, 2, 1)
        if bias is not None and need[4]:
            d_b = ops.segment_colsum(dout, offsets)
        return None, None, d_jagged, d_w, d_b, None


class IndexSelectJaggedGatingBmm(torch.autograd.Function):
    """index_select_jagged_gating_bmm with two different inputs: silu(A Wa + ba) * (B Wb + bb)
    (backward of kernels/triton/triton_moe.py:2839-2990)."""

    @staticmethod
    def forward(ctx, offsets, index, jagged_a, jagged_b, weight_a, weight_b, bias_a, bias_b):
        R, K = index.numel(), index.shape[-1]
        pre_a = ops.grouped_gemm(offsets, jagged_a, weight_a, total_rows=R, row_index=index, index_div=K, bias=bias_a)
        pre_b = ops.grouped_gemm(offsets, jagged_b, weight_b, total_rows=R, row_index=index, index_div=K, bias=bias_b)
        ctx.save_for_backward(offsets, index, jagged_a, jagged_b, weight_a, weight_b, bias_a, bias_b, pre_a, pre_b)
        return ops.silu_mul(pre_a, pre_b)

    @staticmethod
    def backward(ctx, dout):
        offsets, index, jagged_a, jagged_b, weight_a, weight_b, bias_a, bias_b, pre_a, pre_b = ctx.saved_tensors
        R, K = index.numel(), index.shape[-1]
        d_a, d_b = ops.swiglu_bwd(pre_a, pre_b, dout.contiguous())
        need = ctx.needs_input_grad
        reverse = _reverse_from_index(index) if need[2] or need[3] else None
        grads = []
        for pos, (src, w, bias, d) in enumerate(((jagged_a, weight_a, bias_a, d_a), (jagged_b, weight_b, bias_b, d_b))):
            d_src = d_w = d_bias = None
            if need[2 + pos]:
                d_src = _input_grad([d], [w], offsets, reverse).view_as(src)
            if need[4 + pos]:
                operand = _WgradOperand(src, offsets, R, row_index=index.reshape(-1), index_div=K)
                d_w = operand.weight_grad(d).permute(0, 2, 1)
            if bias is not None and need[6 + pos]:
                d_bias = ops.segment_colsum(d, offsets)
            grads.append((d_src, d_w, d_bias))
        (da, dwa, dba), (db, dwb, dbb) = grads
        return None, None, da, db, dwa, dwb, dba, dbb


class IndexSelectJaggedBmm3D(torch.autograd.Function):
    """index_select_jagged_bmm_3D: jagged [L, E, K], expert e reads slice [:, e, :] (backward of
    kernels/triton/triton_moe.py:1399-1476)."""

    @staticmethod
    def forward(ctx, offsets, index, jagged, weight, bias):
        jagged = ops._rows_contiguous(jagged)
        ctx.save_for_backward(offsets, index, jagged, weight, bias)
        return ops.grouped_gemm(offsets, jagged, weight, total_rows=index.numel(), row_index=index,
                                index_div=index.shape[-1], bias=bias, epilogue=EPI_NONE,
                                a_expert_stride=jagged.stride(1))

    @staticmethod
    def backward(ctx, dout):
        offsets, index, jagged, weight, bias = ctx.saved_tensors
        L, E, Kin = jagged.shape
        R, K = index.numel(), index.shape[-1]
        dout = dout.contiguous()
        need = ctx.needs_input_grad
        d_jagged = d_w = d_b = None
        if need[2] or need[3]:
            # sorted row r reads slice (token(r), expert(r)) of the input
            lengths = (offsets[1:] - offsets[:-1]).clamp_min(0)
            expert = torch.repeat_interleave(torch.arange(E, device=index.device), lengths, output_size=R)
            cell = torch.div(index.reshape(-1), K, rounding_mode="floor") * E + expert
        if need[2]:
            d_rows = ops.grouped_gemm(offsets, dout, weight.permute(0, 2, 1), total_rows=R)
            # every (token, expert) cell receives the rows routed there, most cells none (the
            # reference adds into an fp32 [L, A, E, K] tensor of zeros and sums it, :1412-1416, 1470).
            # Gather form instead: slot j of cell (l, e) names the j-th routed row of token l if
            # that row went to expert e, else nothing; the merge kernel adds a cell's rows in
            # ascending order in fp32 and writes zeros where there are none.
            rows_of_token = _reverse_from_index(index)                                  # [L, K] ascending
            experts_of = expert[rows_of_token]                                          # [L, K]
            here = experts_of[:, None, :] == torch.arange(E, device=index.device)[None, :, None]
            slots = torch.where(here, rows_of_token[:, None, :], rows_of_token.new_full((), -1))
            d_jagged = ops.combine(d_rows, slots.view(L * E, K)).view(L, E, Kin).to(jagged.dtype)
        if need[3]:
            src = jagged.contiguous().view(L * E, Kin)
            d_w = _WgradOperand(src, offsets, R, row_index=cell, index_div=1).weight_grad(dout).permute(0, 2, 1)
        if bias is not None and need[4]:
            d_b = ops.segment_colsum(dout, offsets)
        return None, None, d_jagged, d_w, d_b


class MulMergeKAdd(torch.autograd.Function):
    """mul_merge_k_add: weighted deterministic merge."""

    @staticmethod
    def forward(ctx, index, reverse_index, value, weight, weight_index):
        out = ops.combine(value, reverse_index, weight, weight_index)
        ctx.save_for_backward(index, value, weight, weight_index)
        ctx.K = reverse_index.shape[1]
        return out

    @staticmethod
    def backward(ctx, dy):
        index, value, weight, weight_index = ctx.saved_tensors
        need_w = weight is not None and ctx.needs_input_grad[3]
        dy = dy.to(value.dtype)
        d_value, d_gate = ops.combine_bwd(dy, value, index, ctx.K, weight, weight_index, need_gate_grad=need_w)
        d_weight = d_gate.view(weight.shape).to(weight.dtype) if need_w else None
        return None, None, d_value if ctx.needs_input_grad[2] else None, d_weight, None


class SiluJaggedBmmCombine(torch.autograd.Function):
    """silu_jagged_bmm_combine: (SiLU,) grouped GEMM + bias, weighted merge.

    With ``fp8_weight`` = (e4m3 weight [E, D_in, D_out] view, scales): the mixed-precision form of
    silu_jagged_bmm_combine_fp8, forward GEMM on row-quantised e4m3 operands, backward in bf16 on
    the original tensors; ``recompute`` drops the GEMM output after the forward and computes it
    again in bf16 for the gate gradient (SiluJaggedBmmFp8MixedGemmCombine and its
    activation_checkpointing, kernels/triton/triton_moe_fp8.py:1373-1720)."""

    @staticmethod
    def forward(ctx, offsets, jagged, weight, bias, index, reverse_index, gating_scores, gates_index, has_silu,
                fp8_weight=None, recompute=False):
        silu_rows = None
        if fp8_weight is None:
            if has_silu and not recompute and jagged.dtype == torch.bfloat16 and jagged.ndim == 2:
                # SiLU once, kept for the weight gradient (the reference saves silu_jagged as well,
                # kernels/triton/triton_moe.py:3770-3776); with recompute it is made again in backward
                silu_rows = ops.silu_mul(jagged, None, with_slack=True)
                bmm_out = ops.grouped_gemm(offsets, silu_rows, weight, total_rows=jagged.shape[0], bias=bias,
                                           epilogue=EPI_NONE)
            else:
                bmm_out = ops.grouped_gemm(offsets, jagged, weight, total_rows=jagged.shape[0], bias=bias,
                                           epilogue=EPI_NONE, a_silu=has_silu)
        else:
            qa, sa = ops.quant_rows_fp8(jagged, apply_silu=has_silu)
            bmm_out = ops.grouped_gemm(offsets, qa, fp8_weight[0], total_rows=jagged.shape[0], bias=bias,
                                       scales_pow2=ops.scales_are_pow2(sa, fp8_weight[1]), a_scale=sa,
                                       b_scale=fp8_weight[1], epilogue=EPI_NONE)
        out = ops.combine(bmm_out, reverse_index, gating_scores, gates_index)
        ctx.save_for_backward(offsets, jagged, weight, bias, index, gating_scores, gates_index,
                              None if recompute else bmm_out, silu_rows)
        ctx.has_silu = has_silu
        ctx.K = reverse_index.shape[1]
        return out

    @staticmethod
    def backward(ctx, dy):
        offsets, jagged, weight, bias, index, gating_scores, gates_index, bmm_out, silu_rows = ctx.saved_tensors
        if bmm_out is None:
            bmm_out = ops.grouped_gemm(offsets, jagged, weight, total_rows=jagged.shape[0], bias=bias,
                                       epilogue=EPI_NONE, a_silu=ctx.has_silu)
        need = ctx.needs_input_grad
        need_g = gating_scores is not None and need[6]
        dy = dy.to(bmm_out.dtype)
        d_bmm, d_gate = ops.combine_bwd(dy, bmm_out, index, ctx.K, gating_scores, gates_index,
                                        need_gate_grad=need_g)
        d_jagged = d_w = d_b = d_g = None
        if need[1]:
            d_h = ops.grouped_gemm(offsets, d_bmm, weight.permute(0, 2, 1), total_rows=d_bmm.shape[0])
            d_jagged = ops.swiglu_bwd(jagged, None, d_h)[0] if ctx.has_silu else d_h
        if need[2]:
            if silu_rows is not None:
                operand = _WgradOperand(silu_rows, offsets, jagged.shape[0])
            else:
                operand = _WgradOperand(jagged, offsets, jagged.shape[0], apply_silu=ctx.has_silu)
            d_w = operand.weight_grad(d_bmm).permute(0, 2, 1)
        if bias is not None and need[3]:
            d_b = ops.segment_colsum(d_bmm, offsets)
        if need_g:
            d_g = d_gate.view(gating_scores.shape).to(gating_scores.dtype)
        return None, d_jagged, d_w, d_b, None, None, d_g, None, None, None, None


def needs_grad(*tensors: Optional[torch.Tensor]) -> bool:
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)
