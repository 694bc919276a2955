"""Routing oracle (numpy): top-k selection, L1-normalised gates, jagged offsets,
stable expert permutation and its inverse.

TEST INFRASTRUCTURE ONLY -- never imported by the product package.

Restates /root/reference/modules/fast_moe_module.py:93-144 with the two
implementation-defined points of that code fixed to one canonical answer:

* ``topk(sorted=False)`` (fast_moe_module.py:98) leaves the slot order inside a
  token row and the winner among equal scores unspecified.  Canonical here:
  slots in descending score order, equal scores -> lower expert id first.  Any
  such choice is a valid ``topk`` answer; ``token_index``, ``lengths``,
  ``offsets``, ``reverse_token_index`` and the layer output do not depend on
  the slot order, ``gate_index`` and ``gates[T, K]`` do (consistently).
* ``lengths`` is the histogram of the selected expert ids, where the reference
  counts ``scores > 0`` (fast_moe_module.py:120,126).  The two agree whenever
  every selected probability is positive (a softmax output that did not
  underflow), and the histogram is what its own sort and offsets need.
"""
from __future__ import annotations

import numpy as np

_EPS = 1e-12  # F.normalize default eps (fast_moe_module.py:103)


def round_to_bf16(x: np.ndarray) -> np.ndarray:
    """Round float32 to the nearest bfloat16 (ties to even), returned as float32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32).astype(np.uint64)
    lsb = (bits >> 16) & 1
    rounded = ((bits + 0x7FFF + lsb) >> 16) << 16
    out = rounded.astype(np.uint32).view(np.float32).copy()
    nan = np.isnan(x)
    out[nan] = np.float32(np.nan)
    return out


def _round(x: np.ndarray, dtype: str) -> np.ndarray:
    if dtype == "bf16":
        return round_to_bf16(x)
    if dtype == "fp32":
        return np.asarray(x, dtype=np.float32)
    raise ValueError(f"unsupported score dtype {dtype!r}")


def complete_cumsum(lengths: np.ndarray) -> np.ndarray:
    """``[E] -> [E+1]``: ``out[0] = 0``, ``out[i+1] = sum(lengths[:i+1])``.

    Closed form of ``torch.ops.fbgemm.asynchronous_complete_cumsum`` as called at
    fast_moe_module.py:131 (third-party op, absent from the reference tree).
    """
    lengths = np.asarray(lengths, dtype=np.int64)
    out = np.zeros(lengths.shape[0] + 1, dtype=np.int64)
    np.cumsum(lengths, out=out[1:])
    return out


def order_key(scores: np.ndarray) -> np.ndarray:
    """int64 key whose order is the order torch.topk ranks float32 scores by: increasing value,
    -0 == +0, every NaN equal and above +inf."""
    scores = np.ascontiguousarray(scores, dtype=np.float32)
    bits = scores.view(np.uint32).astype(np.int64)
    mag = bits & 0x7FFFFFFF
    key = np.where(bits & 0x80000000 != 0, 0x7FFFFFFF - mag, 0x80000000 + mag)
    key = np.where(mag == 0, 0x80000000, key)
    return np.where(mag > 0x7F800000, 0xFFFFFFFF, key)


def select_top_k(scores: np.ndarray, k: int, dtype: str = "fp32", renorm: bool = True):
    """Canonical top-k + L1 renormalisation (fast_moe_module.py:93-105).

    scores : [T, E] float32 holding values representable in ``dtype``.
    Returns ``(topk_idx [T, k] int64, gates [T, k] float32 rounded to dtype)``.

    The gate of slot j is ``v_j / max(sum_j |v_j|, eps)`` as ``F.normalize(p=1)``
    computes it in the scores' dtype: the L1 norm is accumulated in fp32 (in slot
    order, i.e. descending score), rounded to ``dtype``, clamped, and the
    quotient is rounded to ``dtype`` again.  ``renorm=False`` returns the raw
    selected scores.
    """
    scores = np.asarray(scores, dtype=np.float32)
    T, E = scores.shape
    assert 1 <= k <= E
    # stable descending sort on a total order: NaN above +inf (torch.topk / torch.sort treat NaN as
    # the largest value), -0 equal to +0, ties -> lower index
    order = np.argsort(-order_key(scores), axis=1, kind="stable")[:, :k].astype(np.int64)
    vals = np.take_along_axis(scores, order, axis=1)
    if not renorm:
        return order, vals
    s = np.zeros(T, dtype=np.float32)
    for j in range(k):  # sequential fp32 accumulation in slot order
        s = (s + np.abs(vals[:, j])).astype(np.float32)
    denom = np.maximum(_round(s, dtype), _round(np.float32(_EPS), dtype)).astype(np.float32)
    with np.errstate(invalid="ignore", divide="ignore"):
        gates = _round((vals / denom[:, None]).astype(np.float32), dtype)
    return order, gates


def routing_metadata(topk_idx: np.ndarray, num_experts: int):
    """Jagged routing tensors from selected expert ids (fast_moe_module.py:107-144).

    topk_idx : [T, K] integer expert ids.
    Returns a dict of int64 arrays:
      gate_index    [T*K]  stable argsort of the flattened expert ids (:122)
      token_index   [T*K]  gate_index // K (:124)
      lengths       [E]    rows per expert (:126, see module docstring)
      offsets       [E+1]  complete cumsum of lengths (:131)
      reverse_index [T, K] stable argsort of token_index, viewed [T, K] (:132-134)
      max_seq_len   int    max(lengths) (:135)
    """
    topk_idx = np.asarray(topk_idx, dtype=np.int64)
    T, K = topk_idx.shape
    flat = topk_idx.reshape(-1)
    assert flat.size == 0 or (flat.min() >= 0 and flat.max() < num_experts)
    gate_index = np.argsort(flat, kind="stable").astype(np.int64)
    token_index = gate_index // K
    lengths = np.bincount(flat, minlength=num_experts).astype(np.int64)
    offsets = complete_cumsum(lengths)
    reverse_index = np.argsort(token_index, kind="stable").astype(np.int64).reshape(T, K)
    return {
        "gate_index": gate_index,
        "token_index": token_index,
        "lengths": lengths,
        "offsets": offsets,
        "reverse_index": reverse_index,
        "max_seq_len": int(lengths.max()) if lengths.size else 0,
    }


def route(scores: np.ndarray, k: int, dtype: str = "fp32", renorm: bool = True):
    """select_top_k + routing_metadata in one call; adds ``topk_idx`` and ``gates``."""
    topk_idx, gates = select_top_k(scores, k, dtype=dtype, renorm=renorm)
    meta = routing_metadata(topk_idx, scores.shape[1])
    meta["topk_idx"] = topk_idx
    meta["gates"] = gates
    return meta
