"""Tensor-level wrappers over the C ABI: argument checks, output allocation,
stride marshalling and the current-stream hand-off.  PyTorch is used for device
memory and streams only; every computation below happens in libfastmoe_hip.so.
"""
from __future__ import annotations

import ctypes
import os
from typing import Dict, Optional, Tuple

import torch

from . import _lib
from ._lib import EPI_GATED, EPI_NONE, EPI_SILU, EPI_SWIGLU, FMOE_BF16, FMOE_E4M3, FMOE_F32, GemmDesc

_DTYPE_CODE = {torch.float32: FMOE_F32, torch.bfloat16: FMOE_BF16}
FP8_DTYPE = torch.float8_e4m3fn


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _need_cuda(name: str, *tensors: Optional[torch.Tensor]) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise ValueError(f"{name}: all tensors must live on the GPU (got a {t.device} tensor); "
                             f"fast_moe_amd has no CPU path")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise ValueError(f"{name}: tensors on different devices ({dev} and {t.device})")
    return dev


def _forward_only(name: str, *tensors: Optional[torch.Tensor]) -> None:
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors):
        raise RuntimeError(f"{name}: the HIP back-end is forward-only; call it under torch.no_grad() "
                           f"or detach the inputs")


def _i64(name: str, t: torch.Tensor) -> torch.Tensor:
    if t.dtype != torch.int64:
        raise ValueError(f"{name} must be int64, got {t.dtype}")
    return t.contiguous()


def _rows_contiguous(t: torch.Tensor) -> torch.Tensor:
    """Last dimension contiguous (the reference's switch_to_contiguous_if_needed)."""
    return t if t.stride(-1) == 1 else t.contiguous()


# ------------------------------------------------------------------- routing
GATE_RAW, GATE_L1, GATE_SOFTMAX_ALL, GATE_SOFTMAX_TOPK = 0, 1, 2, 3


def route_topk(scores: torch.Tensor, k: int, renorm=True, static_scratch: bool = False,
               out: Optional[Dict[str, torch.Tensor]] = None) -> Dict[str, torch.Tensor]:
    """scores [T, E] (fp32 / bf16 gate probabilities, or router logits for the softmax modes)
    -> routing tensors, see fmoe_route_topk.  ``renorm``: bool, or one of the GATE_* modes.
    ``static_scratch``: fmoe_route_topk_static, whose scratch is built into the library (no
    workspace allocation; T*k <= 2^20, E <= 512).  ``out``: a dict of a previous call with the
    same shapes, written in place (with static_scratch the call then allocates nothing)."""
    dev = _need_cuda("route_topk", scores)
    if scores.ndim != 2:
        raise ValueError("route_topk: scores must be [T, E]")
    if scores.dtype not in _DTYPE_CODE:
        raise ValueError(f"route_topk: scores must be fp32 or bf16, got {scores.dtype}")
    scores = scores.contiguous()
    T, E = scores.shape
    i64 = dict(dtype=torch.int64, device=dev)
    if out is None:
        out = {
            "topk_idx": torch.empty((T, k), **i64),
            "gates": torch.empty((T, k), dtype=scores.dtype, device=dev),
            "lengths": torch.empty((E,), **i64),
            "offsets": torch.empty((E + 1,), **i64),
            "gate_index": torch.empty((T * k,), **i64),
            "token_index": torch.empty((T * k,), **i64),
            "reverse_index": torch.empty((T, k), **i64),
        }
    else:
        # the kernels write every one of these through raw pointers: shape, dtype, device and
        # contiguity of each are checked, not only of the first few
        want = {"topk_idx": ((T, k), torch.int64), "gates": ((T, k), scores.dtype), "lengths": ((E,), torch.int64),
                "offsets": ((E + 1,), torch.int64), "gate_index": ((T * k,), torch.int64),
                "token_index": ((T * k,), torch.int64), "reverse_index": ((T, k), torch.int64)}
        for name, (shape, dtype) in want.items():
            t = out.get(name)
            if (t is None or tuple(t.shape) != shape or t.dtype != dtype or t.device != dev
                    or not t.is_contiguous()):
                raise ValueError(f"route_topk: out[{name!r}] must be a contiguous {dtype} tensor of shape {shape} on "
                                 f"{dev} (a dict of a previous call with the same T, E, k and score dtype)")
    lib = _lib.load()
    if static_scratch:
        rc = lib.fmoe_route_topk_static(
            scores.data_ptr(), _DTYPE_CODE[scores.dtype], T, E, k, int(renorm),
            out["topk_idx"].data_ptr(), out["gates"].data_ptr(), out["lengths"].data_ptr(),
            out["offsets"].data_ptr(), out["gate_index"].data_ptr(), out["token_index"].data_ptr(),
            out["reverse_index"].data_ptr(), _stream(scores))
        _lib.check(rc, "fmoe_route_topk_static")
        return out
    ws_bytes = lib.fmoe_route_workspace_bytes(T, E, k)
    ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=dev)
    rc = lib.fmoe_route_topk(
        scores.data_ptr(), _DTYPE_CODE[scores.dtype], T, E, k, int(renorm),
        out["topk_idx"].data_ptr(), out["gates"].data_ptr(), out["lengths"].data_ptr(),
        out["offsets"].data_ptr(), out["gate_index"].data_ptr(), out["token_index"].data_ptr(),
        out["reverse_index"].data_ptr(), ws.data_ptr(), ws_bytes, _stream(scores))
    _lib.check(rc, "fmoe_route_topk")
    return out


def route_from_topk(topk_idx: torch.Tensor, num_experts: int) -> Dict[str, torch.Tensor]:
    """topk_idx [T, K] int64 expert ids -> routing tensors, see fmoe_route_from_topk.  Ids outside
    [0, num_experts) are dropped and counted in ``bad_count`` (a device tensor: reading it
    synchronises); with FMOE_CHECK_ROUTING=1 in the environment the call checks it and raises."""
    dev = _need_cuda("route_from_topk", topk_idx)
    if topk_idx.ndim != 2:
        raise ValueError("route_from_topk: topk_idx must be [T, K]")
    topk_idx = _i64("topk_idx", topk_idx)
    T, k = topk_idx.shape
    E = num_experts
    i64 = dict(dtype=torch.int64, device=dev)
    out = {
        "lengths": torch.empty((E,), **i64),
        "offsets": torch.empty((E + 1,), **i64),
        "gate_index": torch.empty((T * k,), **i64),
        "token_index": torch.empty((T * k,), **i64),
        "reverse_index": torch.empty((T, k), **i64),
        "bad_count": torch.empty((1,), **i64),
    }
    lib = _lib.load()
    ws_bytes = lib.fmoe_route_workspace_bytes(T, E, k)
    ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=dev)
    rc = lib.fmoe_route_from_topk(
        topk_idx.data_ptr(), T, E, k, out["lengths"].data_ptr(), out["offsets"].data_ptr(),
        out["gate_index"].data_ptr(), out["token_index"].data_ptr(), out["reverse_index"].data_ptr(),
        out["bad_count"].data_ptr(), ws.data_ptr(), ws_bytes, _stream(topk_idx))
    _lib.check(rc, "fmoe_route_from_topk")
    if os.environ.get("FMOE_CHECK_ROUTING") == "1":     # debugging aid: costs a host synchronisation
        bad = int(out["bad_count"])
        if bad:
            raise ValueError(f"route_from_topk: {bad} expert ids outside [0, {E})")
    return out


# ---------------------------------------------------------------- fp8 quant
def quant_rows_fp8(a: torch.Tensor, apply_silu: bool = False, reciprocal_scale: bool = False,
                   out_like_input: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """Row-wise (last dim) e4m3fn quantisation of ``a`` [..., rows, cols] read through its strides.

    Returns ``(q, scale)``: q is float8_e4m3fn, contiguous in a's logical shape (or laid out
    with a's own strides when ``out_like_input``), scale is fp32 with a's leading shape."""
    dev = _need_cuda("quant_rows_fp8", a)
    if a.dtype not in _DTYPE_CODE:
        raise ValueError(f"quant_rows_fp8: input must be fp32 or bf16, got {a.dtype}")
    if a.ndim < 1 or a.shape[-1] < 1:
        raise ValueError("quant_rows_fp8: need at least one column")
    shape = tuple(a.shape)
    if a.ndim == 1:
        a3 = a.view(1, 1, -1)
    elif a.ndim == 2:
        a3 = a.unsqueeze(0)
    elif a.ndim == 3:
        a3 = a
    else:
        a3 = a.reshape(-1, shape[-2], shape[-1])     # may copy for exotic >3-D strides
    B, Rr, C = a3.shape
    if out_like_input:
        q3 = torch.empty_strided(a3.shape, a3.stride(), dtype=torch.uint8, device=dev)
    else:
        q3 = torch.empty(a3.shape, dtype=torch.uint8, device=dev)
    scale = torch.empty((B, Rr), dtype=torch.float32, device=dev)
    lib = _lib.load()
    rc = lib.fmoe_quant_rows_e4m3(
        a3.data_ptr(), _DTYPE_CODE[a.dtype], B, Rr, C, a3.stride(0), a3.stride(1), a3.stride(2),
        int(apply_silu), q3.data_ptr(), q3.stride(0), q3.stride(1), q3.stride(2), scale.data_ptr(),
        int(reciprocal_scale), _stream(a))
    _lib.check(rc, "fmoe_quant_rows_e4m3")
    q = q3.view(FP8_DTYPE)
    if a.ndim == 1:
        q = q[0, 0]
    elif a.ndim == 2:
        q = q[0]
    elif a.ndim > 3:
        q = q.view(shape)
    scale = scale.view(shape[:-1])
    scale._fmoe_pow2 = scale._version       # (see scales_are_pow2)
    return q, scale


def scales_are_pow2(*scales: torch.Tensor) -> bool:
    """True when every scale tensor is one this module's quantiser returned (that very tensor object):
    those hold exact powers of two (kernels/pytorch/quant_fp8.py:13-24), which is what
    ``grouped_gemm(scales_pow2=True)`` relies on.  A tensor of any other origin (a caller's own
    quantisation handed in as ``fp8_weight``, a slice, a copy) is not vouched for, and the GEMM then
    divides the scales out in its epilogue, which is right for any positive scale."""
    return all(getattr(s, "_fmoe_pow2", None) == s._version for s in scales)      # (and not written to since)


def to_k_contiguous(w: torch.Tensor) -> torch.Tensor:
    """[E, K, N] weight with N contiguous -> the same logical tensor as a view of [E, N, K]
    storage (one transposing copy by fmoe_transpose_last2).  Other layouts are returned as is."""
    if w.ndim != 3 or w.stride(2) != 1 or w.stride(1) == 1 or w.element_size() not in (1, 2):
        return w
    E, K, N = w.shape
    if w.stride(1) < N:
        return w
    dst = torch.empty((E, N, K), dtype=w.dtype, device=w.device)
    rc = _lib.load().fmoe_transpose_last2(w.data_ptr(), dst.data_ptr(), w.element_size(), E, K, N,
                                          w.stride(0), w.stride(1), _stream(w))
    _lib.check(rc, "fmoe_transpose_last2")
    return dst.permute(0, 2, 1)


# ------------------------------------------------------- rows with slack
SLACK_ROWS = 128    # what fmoe_grouped_gemm asks for behind row-indexed operands


def empty_rows(rows: int, cols: int, dtype: torch.dtype, device) -> torch.Tensor:
    """[rows, cols] view of a buffer with SLACK_ROWS more rows behind it: what the weight-gradient
    GEMM may read (and masks out, whatever they hold) past an expert's last row."""
    return torch.empty((rows + SLACK_ROWS, cols), dtype=dtype, device=device)[:rows]


def slack_rows(t: torch.Tensor) -> int:
    """Rows of t's row pitch that its storage holds behind its last row."""
    if t.ndim != 2 or t.stride(1) != 1 or t.stride(0) < t.shape[1]:
        return 0
    have = t.untyped_storage().nbytes() // t.element_size() - t.storage_offset()
    return max(0, (have - t.shape[1]) // t.stride(0) + 1 - t.shape[0]) if t.stride(0) > 0 else 0


def jagged_weight_grad(dout: torch.Tensor, a_rows: torch.Tensor, offsets: torch.Tensor, halves: bool = False):
    """dW[e, n, k] = sum over the rows r of expert e of dout[r, n] * a_rows[r, k] -> [E, N, K_in],
    both operands read in place (fmoe_grouped_gemm with a_stride_k).  Returns None when the
    operands do not qualify (dtype, alignment, no slack behind them): the caller then takes the
    route over transposed copies.  ``halves``: dout holds the row gradients of two matrices side
    by side; the result is two tensors [E, N/2, K_in] (fmoe_gemm_desc.out2)."""
    if dout.dtype != torch.bfloat16 or a_rows.dtype != torch.bfloat16 or dout.shape[0] != a_rows.shape[0]:
        return None
    R, N = dout.shape
    Kin = a_rows.shape[1]
    E = offsets.numel() - 1
    ok = (dout.stride(1) == 1 and a_rows.stride(1) == 1 and N % 8 == 0 and Kin % 8 == 0 and E <= 256
          and dout.stride(0) % 8 == 0 and a_rows.stride(0) % 8 == 0 and dout.data_ptr() % 16 == 0
          and a_rows.data_ptr() % 16 == 0 and R >= 128 and E * N < (1 << 31)
          and slack_rows(dout) >= SLACK_ROWS and slack_rows(a_rows) >= SLACK_ROWS
          and (not halves or N % 64 == 0))
    if not ok:
        return None
    dev = dout.device
    offsets = _i64("offsets", offsets)
    seg = torch.arange(E + 1, device=dev, dtype=torch.int64) * N
    if halves:
        out = torch.empty((E * (N // 2), Kin), dtype=torch.bfloat16, device=dev)
        out2 = torch.empty_like(out)
    else:
        out = torch.empty((E * N, Kin), dtype=torch.bfloat16, device=dev)
    d = GemmDesc()
    d.num_experts, d.n, d.k, d.index_div = E, Kin, R, 1
    if halves:
        d.out2 = out2.data_ptr()
    d.total_rows, d.a_rows = E * N, N
    d.offsets = seg.data_ptr()
    d.a, d.a_dtype, d.a_stride_row, d.a_stride_k = dout.data_ptr(), _DTYPE_CODE[dout.dtype], 1, dout.stride(0)
    d.b, d.b_stride_e, d.b_stride_k, d.b_stride_n = a_rows.data_ptr(), 0, a_rows.stride(0), 1
    d.epilogue, d.out_dtype = EPI_NONE, _DTYPE_CODE[torch.bfloat16]
    d.out, d.out_stride_row = out.data_ptr(), Kin
    d.k_window, d.k_slack_rows = offsets.data_ptr(), SLACK_ROWS
    rc = _lib.load().fmoe_grouped_gemm(ctypes.byref(d), _stream(dout))
    _lib.check(rc, "fmoe_grouped_gemm")
    if halves:
        return out.view(E, N // 2, Kin), out2.view(E, N // 2, Kin)
    return out.view(E, N, Kin)


# -------------------------------------------------------------- grouped GEMM
def grouped_gemm(offsets: torch.Tensor, a: torch.Tensor, b: torch.Tensor, *, total_rows: int,
                 row_index: Optional[torch.Tensor] = None, index_div: int = 1,
                 bias: Optional[torch.Tensor] = None, b2: Optional[torch.Tensor] = None,
                 bias2: Optional[torch.Tensor] = None, epilogue: int = EPI_NONE, a_silu: bool = False,
                 a_scale: Optional[torch.Tensor] = None, b_scale: Optional[torch.Tensor] = None,
                 b2_scale: Optional[torch.Tensor] = None, a_expert_stride: int = 0,
                 k_window: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                 k_window_multiple: int = 0,
                 aux: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                 gate: Optional[torch.Tensor] = None,
                 plan_only: bool = False, scales_pow2: bool = False) -> torch.Tensor:
    """Jagged GEMM, see fmoe_grouped_gemm.  ``b`` (and ``b2``) are [E, K, N] tensors of any
    strides, bf16 / fp32 / float8_e4m3fn; ``a`` is [rows, K] with contiguous rows.  Returns
    [total_rows, N] in bf16 (fp32 for fp32 operands).  ``aux`` = two tensors like the output
    that receive the SWIGLU pre-activations.  ``gate`` (bf16 [total_rows, N], with
    ``epilogue=EPI_GATED``): the result is ``silu(gate) * (A B + bias)``.  ``plan_only``: launch nothing and return the
    _lib.PLAN_* code of the kernel this call would run (fmoe_grouped_gemm_plan).  ``scales_pow2``
    (e4m3): a promise that every scale is an exact power of two, as ``quant_rows_fp8`` writes them;
    the ring kernel then folds them into its MFMAs (fmoe_gemm_desc.scale_pow2)."""
    dev = _need_cuda("grouped_gemm", offsets, a, b, row_index, bias, b2, bias2, a_scale, b_scale, b2_scale)
    fp8 = a.dtype == FP8_DTYPE
    if not fp8 and a.dtype not in (torch.bfloat16, torch.float32):
        raise NotImplementedError(
            f"grouped_gemm: the HIP kernels take bf16, fp32 or float8_e4m3fn operands, got {a.dtype}")
    out_dtype = torch.float32 if a.dtype == torch.float32 else torch.bfloat16
    if b.dtype != a.dtype or (b2 is not None and b2.dtype != a.dtype):
        raise ValueError("grouped_gemm: A and B must share a dtype")
    if b.ndim != 3:
        raise ValueError("grouped_gemm: B must be [E, K, N]")
    E, K, N = b.shape
    if a.ndim not in (2, 3) or a.shape[-1] != K:
        raise ValueError(f"grouped_gemm: A must be [rows, {K}] (or [rows, E, {K}]), got {tuple(a.shape)}")
    if (a.ndim == 3) != (a_expert_stride != 0):
        raise ValueError("grouped_gemm: a 3-D A needs a_expert_stride and vice versa")
    if b2 is not None and (tuple(b2.shape) != (E, K, N) or b2.stride() != b.stride()):
        raise ValueError("grouped_gemm: b2 must match b in shape and strides")
    if offsets.numel() != E + 1:
        raise ValueError(f"grouped_gemm: offsets must have E+1={E + 1} entries")
    a = _rows_contiguous(a)
    if k_window is not None:
        k_window = _i64("k_window", k_window)
        if k_window.numel() != E + 1:
            raise ValueError(f"grouped_gemm: k_window must have E+1={E + 1} entries")
    offsets = _i64("offsets", offsets)
    if row_index is not None:
        row_index = _i64("row_index", row_index).view(-1)
        if row_index.numel() != total_rows:
            raise ValueError("grouped_gemm: row_index must have total_rows entries")
    if out is None:    # (with slack: the output may become an operand of a weight-gradient GEMM)
        out = empty_rows(total_rows, N, out_dtype, dev)
    elif (tuple(out.shape) != (total_rows, N) or out.dtype != out_dtype or out.device != dev
          or out.stride(1) != 1):
        raise ValueError(f"grouped_gemm: out must be {out_dtype} [{total_rows}, {N}] with contiguous rows")
    if aux is not None:
        if epilogue != EPI_SWIGLU:
            raise ValueError("grouped_gemm: aux outputs exist for the SWIGLU epilogue only")
        for t in aux:
            if (tuple(t.shape) != (total_rows, N) or t.dtype != out_dtype or t.device != dev or t.stride(1) != 1
                    or t.stride(0) != aux[0].stride(0)):
                raise ValueError(f"grouped_gemm: aux tensors must be {out_dtype} [{total_rows}, {N}] with "
                                 "contiguous rows and one row stride")
    if (gate is not None) != (epilogue == EPI_GATED):
        raise ValueError("grouped_gemm: gate and EPI_GATED come together")
    if gate is not None:
        if a.dtype != torch.bfloat16:
            raise NotImplementedError("grouped_gemm: the gated epilogue is built for bf16 operands")
        if (tuple(gate.shape) != (total_rows, N) or gate.dtype != out_dtype or gate.device != dev
                or gate.stride(1) != 1 or aux is not None):
            raise ValueError(f"grouped_gemm: gate must be {out_dtype} [{total_rows}, {N}] with contiguous rows "
                             "(and no aux outputs)")
    if total_rows == 0:
        return _lib.PLAN_NONE if plan_only else out

    def bias_ok(t):
        if t is None:
            return None
        if t.dtype != out_dtype or tuple(t.shape) != (E, N):
            raise ValueError(f"grouped_gemm: bias must be {out_dtype} [E, N]")
        return _rows_contiguous(t)

    bias, bias2 = bias_ok(bias), bias_ok(bias2)
    if bias is not None and bias2 is not None and bias.stride(0) != bias2.stride(0):
        bias2 = bias2.contiguous()
        bias = bias.contiguous()
    if fp8:
        for name, s, n in (("a_scale", a_scale, a.shape[0] if a_expert_stride == 0 else None),
                           ("b_scale", b_scale, E * N), ("b2_scale", b2_scale, E * N)):
            if s is None:
                if name == "b2_scale" and b2 is None:
                    continue
                raise ValueError(f"grouped_gemm: fp8 operands need {name}")
            if s.dtype != torch.float32 or not s.is_contiguous() or (n is not None and s.numel() != n):
                raise ValueError(f"grouped_gemm: {name} must be contiguous fp32 with one entry per row")

    d = GemmDesc()
    d.num_experts, d.n, d.k, d.index_div = E, N, K, index_div
    d.total_rows = total_rows
    d.a_rows = a.shape[0]
    d.offsets = offsets.data_ptr()
    d.row_index = _ptr(row_index)
    d.a = a.data_ptr()
    d.a_dtype = FMOE_E4M3 if fp8 else _DTYPE_CODE[a.dtype]
    d.a_silu = int(a_silu)
    d.a_stride_row = a.stride(0)
    d.a_stride_e = a_expert_stride
    d.a_scale = _ptr(a_scale)
    d.b = b.data_ptr()
    d.b2 = _ptr(b2)
    d.b_stride_e, d.b_stride_k, d.b_stride_n = b.stride()
    d.b_scale = _ptr(b_scale)
    d.b2_scale = _ptr(b2_scale)
    d.scale_pow2 = int(bool(scales_pow2) and fp8)
    d.bias = _ptr(bias)
    d.bias2 = _ptr(bias2)
    d.bias_stride_e = bias.stride(0) if bias is not None else (bias2.stride(0) if bias2 is not None else 0)
    d.epilogue = epilogue
    d.out_dtype = _DTYPE_CODE[out_dtype]
    d.out = out.data_ptr()
    d.out_stride_row = out.stride(0)
    d.k_window = _ptr(k_window)
    d.k_window_multiple = k_window_multiple if k_window is not None else 0
    if aux is not None:
        d.aux, d.aux2, d.aux_stride_row = aux[0].data_ptr(), aux[1].data_ptr(), aux[0].stride(0)
    if gate is not None:
        d.aux, d.aux_stride_row = gate.data_ptr(), gate.stride(0)
    lib = _lib.load()
    # N-contiguous weights of a useful size that only the element-load kernel would read in
    # place (correct, but an order of magnitude slower): one transposing copy buys a streaming kernel
    if (k_window is None and b.stride(2) == 1 and b.stride(1) != 1 and K % 16 == 0 and N % 8 == 0
            and gemm_plan(d) == _lib.PLAN_ELEMENT and total_rows * N >= (1 << 22)):
        b = to_k_contiguous(b)
        d.b = b.data_ptr()
        d.b_stride_e, d.b_stride_k, d.b_stride_n = b.stride()
        if b2 is not None:
            b2 = to_k_contiguous(b2)
            d.b2 = b2.data_ptr()
    # SiLU on load exists in the register-staged kernel only.  Where the LDS-ring kernel would take
    # the same call without it, one element-wise pass over the source rows (same rounding: SiLU in
    # fp32, rounded to bf16 before it multiplies) and the ring kernel are faster together.
    if a_silu and a.dtype == torch.bfloat16 and a.ndim == 2 and total_rows * N >= (1 << 22):
        d.a_silu = 0
        if gemm_plan(d) == _lib.PLAN_RING:
            a = silu_mul(a, None)
            d.a, d.a_stride_row = a.data_ptr(), a.stride(0)
        else:
            d.a_silu = 1
    if plan_only:
        return gemm_plan(d)
    rc = lib.fmoe_grouped_gemm(ctypes.byref(d), _stream(a))
    _lib.check(rc, "fmoe_grouped_gemm")
    return out


def grouped_gemm_sum2(offsets: torch.Tensor, a: torch.Tensor, b: torch.Tensor, a2: torch.Tensor,
                      b2: torch.Tensor, *, total_rows: int,
                      out: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """``a @ b[e] + a2 @ b2[e]`` per expert in one pass, accumulated in fp32 and rounded once
    (fmoe_gemm_desc.a2): a, a2 [rows, K], [rows, K2] bf16; b, b2 [E, K, N], [E, K2, N] with N
    contiguous.  None when the operands do not qualify: the caller runs two GEMMs and adds."""
    dev = _need_cuda("grouped_gemm_sum2", offsets, a, b, a2, b2)
    E, K, N = b.shape
    K2 = b2.shape[1]
    if (any(t.dtype != torch.bfloat16 for t in (a, b, a2, b2)) or a.ndim != 2 or a2.ndim != 2
            or a.shape != (total_rows, K) or a2.shape != (total_rows, K2) or b2.shape != (E, K2, N)
            or a.stride(1) != 1 or a2.stride() != a.stride() or b2.stride() != b.stride() or total_rows == 0):
        return None
    offsets = _i64("offsets", offsets)
    if out is None:
        out = empty_rows(total_rows, N, torch.bfloat16, dev)
    d = GemmDesc()
    d.num_experts, d.n, d.k, d.index_div = E, N, K, 1
    d.total_rows = d.a_rows = total_rows
    d.offsets = offsets.data_ptr()
    d.a, d.a2, d.k2 = a.data_ptr(), a2.data_ptr(), K2
    d.a_dtype = d.out_dtype = _DTYPE_CODE[torch.bfloat16]
    d.a_stride_row = a.stride(0)
    d.b, d.b2 = b.data_ptr(), b2.data_ptr()
    d.b_stride_e, d.b_stride_k, d.b_stride_n = b.stride()
    d.epilogue = EPI_NONE
    d.out, d.out_stride_row = out.data_ptr(), out.stride(0)
    lib = _lib.load()
    plan = ctypes.c_int(0)
    if lib.fmoe_grouped_gemm_plan(ctypes.byref(d), ctypes.byref(plan)) != 0:
        return None
    _lib.check(lib.fmoe_grouped_gemm(ctypes.byref(d), _stream(a)), "fmoe_grouped_gemm")
    return out


def gemm_plan(d: GemmDesc) -> int:
    """The kernel fmoe_grouped_gemm would run for this descriptor (one of _lib.PLAN_*)."""
    plan = ctypes.c_int(0)
    _lib.check(_lib.load().fmoe_grouped_gemm_plan(ctypes.byref(d), ctypes.byref(plan)), "fmoe_grouped_gemm_plan")
    return plan.value


# ------------------------------------------------------------------ combine
def combine(value: torch.Tensor, reverse_index: torch.Tensor, gates: Optional[torch.Tensor] = None,
            gates_index: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Weighted merge, see fmoe_combine.  value [T*K, D]; reverse_index [T, K]."""
    dev = _need_cuda("combine", value, reverse_index, gates, gates_index)
    if value.dtype not in _DTYPE_CODE:
        raise NotImplementedError(f"combine: value must be fp32 or bf16, got {value.dtype}")
    T, K = reverse_index.shape
    D = value.shape[1]
    value = _rows_contiguous(value)
    reverse_index = _i64("reverse_index", reverse_index)
    out_dtype = value.dtype
    g_code, g_cols, g_sr, g_sc = FMOE_F32, 1, 1, 1
    if gates is not None:
        if gates.dtype not in _DTYPE_CODE:
            raise NotImplementedError(f"combine: gates must be fp32 or bf16, got {gates.dtype}")
        if gates.numel() != T * K:
            raise ValueError(f"combine: gates has {gates.numel()} entries, expected {T * K}")
        if gates.ndim == 1:
            gates = gates.view(-1, 1)
        if gates.ndim != 2:
            gates = gates.contiguous().view(-1, 1)
        out_dtype = torch.promote_types(value.dtype, gates.dtype)
        g_code, g_cols, g_sr, g_sc = _DTYPE_CODE[gates.dtype], gates.shape[1], gates.stride(0), gates.stride(1)
        if gates_index is not None:
            gates_index = _i64("gates_index", gates_index).view(-1)
            if gates_index.numel() != T * K:
                raise ValueError("combine: gates_index must have T*K entries")
    else:
        gates_index = None
    out = torch.empty((T, D), dtype=out_dtype, device=dev)
    rc = _lib.load().fmoe_combine(
        value.data_ptr(), _DTYPE_CODE[value.dtype], T, K, D, value.stride(0), reverse_index.data_ptr(),
        _ptr(gates), g_code, g_cols, g_sr, g_sc, _ptr(gates_index), out.data_ptr(), _DTYPE_CODE[out_dtype],
        _stream(value))
    _lib.check(rc, "fmoe_combine")
    return out


def gather_rows(src: torch.Tensor, index: torch.Tensor, index_div: int = 1) -> torch.Tensor:
    """``src[index // index_div]`` for a 2-D src with contiguous rows of whole 16-byte chunks
    (fmoe_gather_rows); the result has slack rows behind it."""
    dev = _need_cuda("gather_rows", src, index)
    if src.ndim != 2:
        raise ValueError("gather_rows: src must be 2-D")
    src = _rows_contiguous(src)
    index = _i64("index", index).view(-1)
    out = empty_rows(index.numel(), src.shape[1], src.dtype, dev)
    es = src.element_size()
    rc = _lib.load().fmoe_gather_rows(src.data_ptr(), src.shape[0], src.shape[1] * es, src.stride(0) * es,
                                      index.data_ptr(), index_div, index.numel(), out.data_ptr(),
                                      out.stride(0) * es, _stream(src))
    _lib.check(rc, "fmoe_gather_rows")
    return out


def silu_mul(a: torch.Tensor, b: Optional[torch.Tensor], with_slack: bool = False) -> torch.Tensor:
    """``silu(a) * b`` element-wise (bf16 or fp32, same shape); ``silu(a)`` when b is None.
    ``with_slack`` (2-D a): the result has SLACK_ROWS readable rows behind it."""
    _need_cuda("silu_mul", a, b)
    if a.dtype not in _DTYPE_CODE or (b is not None and (b.dtype != a.dtype or a.shape != b.shape)):
        raise ValueError("silu_mul: two bf16 (or two fp32) tensors of one shape expected")
    a = a.contiguous()
    b = None if b is None else b.contiguous()
    out = empty_rows(a.shape[0], a.shape[1], a.dtype, a.device) if with_slack and a.ndim == 2 else torch.empty_like(a)
    rc = _lib.load().fmoe_silu_mul(a.data_ptr(), _ptr(b), out.data_ptr(), _DTYPE_CODE[a.dtype], a.numel(),
                                   _stream(a))
    _lib.check(rc, "fmoe_silu_mul")
    return out


# ----------------------------------------------------------------- backward
def jagged_transpose(src: torch.Tensor, offsets: torch.Tensor, pad_offsets: torch.Tensor, padded_cols: int,
                     row_index: Optional[torch.Tensor] = None, index_div: int = 1,
                     apply_silu: bool = False) -> torch.Tensor:
    """[rows, C] jagged rows (optionally gathered) -> [C, padded_cols] transposed and zero padded per
    expert, see fmoe_jagged_transpose."""
    dev = _need_cuda("jagged_transpose", src, offsets, pad_offsets, row_index)
    if src.ndim != 2 or src.dtype not in _DTYPE_CODE:
        raise ValueError("jagged_transpose: src must be a 2-D bf16 or fp32 tensor")
    src = _rows_contiguous(src)
    offsets, pad_offsets = _i64("offsets", offsets), _i64("pad_offsets", pad_offsets)
    if row_index is not None:
        row_index = _i64("row_index", row_index).view(-1)
    E = offsets.numel() - 1
    C = src.shape[1]
    dst = torch.empty((C, padded_cols), dtype=src.dtype, device=dev)
    rc = _lib.load().fmoe_jagged_transpose(
        src.data_ptr(), _DTYPE_CODE[src.dtype], src.shape[0], C, src.stride(0), _ptr(row_index), index_div,
        offsets.data_ptr(), pad_offsets.data_ptr(), E, dst.data_ptr(), dst.stride(0), padded_cols,
        int(apply_silu), _stream(src))
    _lib.check(rc, "fmoe_jagged_transpose")
    return dst


def segment_colsum(src: torch.Tensor, offsets: torch.Tensor) -> torch.Tensor:
    """Per-expert column sums [E, C] of jagged rows [R, C], see fmoe_segment_colsum."""
    dev = _need_cuda("segment_colsum", src, offsets)
    if src.ndim != 2 or src.dtype not in _DTYPE_CODE:
        raise ValueError("segment_colsum: src must be a 2-D bf16 or fp32 tensor")
    src = _rows_contiguous(src)
    offsets = _i64("offsets", offsets)
    E = offsets.numel() - 1
    out = torch.empty((E, src.shape[1]), dtype=src.dtype, device=dev)
    rc = _lib.load().fmoe_segment_colsum(src.data_ptr(), _DTYPE_CODE[src.dtype], src.shape[0], src.shape[1],
                                         src.stride(0), offsets.data_ptr(), E, out.data_ptr(), _stream(src))
    _lib.check(rc, "fmoe_segment_colsum")
    return out


def swiglu_bwd(g: torch.Tensor, u: Optional[torch.Tensor], dh: torch.Tensor, joint: bool = False):
    """Backward of ``silu(g) * u`` (or of ``silu(g)`` when u is None): returns (dg, du).
    ``joint`` (gated form, 2-D bf16, columns a multiple of 8): dg and du are the two halves of one
    [rows, 2 * cols] buffer, ``torch.cat([dg, du], 1)`` without the copy, so that the GEMMs that
    consume both can take them as one operand (``dg._base`` is that buffer's storage)."""
    _need_cuda("swiglu_bwd", g, u, dh)
    if g.dtype not in _DTYPE_CODE or dh.dtype != g.dtype or dh.shape != g.shape or (
            u is not None and (u.dtype != g.dtype or u.shape != g.shape)):
        raise ValueError("swiglu_bwd: bf16 (or fp32) tensors of one shape expected")
    g, dh = g.contiguous(), dh.contiguous()
    u = None if u is None else u.contiguous()
    cols = g.shape[-1] if g.ndim >= 1 else 1
    pitch = 0
    if (joint and u is not None and g.ndim == 2 and g.dtype == torch.bfloat16 and cols % 8 == 0 and cols >= 8
            and g.numel() > 0):
        both = empty_rows(g.shape[0], 2 * cols, g.dtype, g.device)
        dg, du, pitch = both[:, :cols], both[:, cols:], 2 * cols
    else:
        dg = empty_rows(g.shape[0], g.shape[1], g.dtype, g.device) if g.ndim == 2 else torch.empty_like(g)
        du = None if u is None else (empty_rows(g.shape[0], g.shape[1], g.dtype, g.device) if g.ndim == 2
                                     else torch.empty_like(g))
    rc = _lib.load().fmoe_swiglu_bwd(g.data_ptr(), _ptr(u), dh.data_ptr(), dg.data_ptr(), _ptr(du),
                                     _DTYPE_CODE[g.dtype], g.numel(), cols, pitch, _stream(g))
    _lib.check(rc, "fmoe_swiglu_bwd")
    return dg, du


def joint_rows(left: torch.Tensor, right: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    """[rows, 2 * cols] view over two [rows, cols] tensors that are the halves of one buffer (what
    ``swiglu_bwd(joint=True)`` returns), else None."""
    if (right is None or left.ndim != 2 or left.shape != right.shape or left.dtype != right.dtype
            or left.untyped_storage().data_ptr() != right.untyped_storage().data_ptr()):
        return None
    rows, cols = left.shape
    if (left.stride() != (2 * cols, 1) or right.stride() != (2 * cols, 1)
            or right.storage_offset() != left.storage_offset() + cols):
        return None
    return torch.as_strided(left, (rows, 2 * cols), (2 * cols, 1))


def combine_bwd(dy: torch.Tensor, value: Optional[torch.Tensor], token_index: torch.Tensor, K: int,
                gates: Optional[torch.Tensor] = None, gates_index: Optional[torch.Tensor] = None,
                need_gate_grad: bool = False):
    """Backward of ``combine``: (d_value [T*K, D], d_gates fp32 [T*K] in the gates' flat layout or None)."""
    dev = _need_cuda("combine_bwd", dy, value, token_index, gates, gates_index)
    if dy.ndim != 2 or dy.dtype not in _DTYPE_CODE:
        raise ValueError("combine_bwd: dy must be a 2-D bf16 or fp32 tensor")
    dy = dy.contiguous()
    T, D = dy.shape
    R = T * K
    token_index = _i64("token_index", token_index).view(-1)
    if token_index.numel() != R:
        raise ValueError("combine_bwd: token_index must have T*K entries")
    g_code, g_cols, g_sr, g_sc = FMOE_F32, 1, 1, 1
    if gates is not None:
        if gates.dtype not in _DTYPE_CODE or gates.numel() != R:
            raise ValueError("combine_bwd: gates must be bf16 / fp32 with T*K entries")
        if gates.ndim != 2:
            gates = gates.contiguous().view(-1, 1)
        g_code, g_cols, g_sr, g_sc = _DTYPE_CODE[gates.dtype], gates.shape[1], gates.stride(0), gates.stride(1)
        if gates_index is not None:
            gates_index = _i64("gates_index", gates_index).view(-1)
    else:
        gates_index = None
    d_gates = None
    v_stride = D
    if need_gate_grad:
        if value is None or value.dtype != dy.dtype or tuple(value.shape) != (R, D):
            raise ValueError("combine_bwd: the gate gradient needs value [T*K, D] in dy's dtype")
        value = _rows_contiguous(value)
        v_stride = value.stride(0)
        d_gates = torch.zeros((R,), dtype=torch.float32, device=dev)
    d_value = empty_rows(R, D, dy.dtype, dev)
    rc = _lib.load().fmoe_combine_bwd(
        dy.data_ptr(), _ptr(value) if need_gate_grad else None, _DTYPE_CODE[dy.dtype], T, K, D, v_stride,
        token_index.data_ptr(), _ptr(gates), g_code, g_cols, g_sr, g_sc, _ptr(gates_index), d_value.data_ptr(),
        _ptr(d_gates), _stream(dy))
    _lib.check(rc, "fmoe_combine_bwd")
    return d_value, d_gates
