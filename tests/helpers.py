"""Shared input generators and comparison helpers for the parity tests."""
import numpy as np
import torch

from oracle import routing as o_routing

BF16 = torch.bfloat16


def make_routing(L, E, K, seed=0):
    """The generator of kernels/tests/moe_test.py:191-197,241 on the CPU: random top-k ->
    stable sort -> lengths -> complete cumsum."""
    g = torch.Generator().manual_seed(seed)
    topk = torch.randn(L, E, generator=g).topk(K, dim=1).indices
    meta = o_routing.routing_metadata(topk.numpy(), E)
    return {
        "topk_idx": topk,
        "index": torch.from_numpy(meta["gate_index"]).view(-1, K),
        "gate_index": torch.from_numpy(meta["gate_index"]),
        "token_index": torch.from_numpy(meta["token_index"]),
        "reverse_index": torch.from_numpy(meta["reverse_index"]),
        "offsets": torch.from_numpy(meta["offsets"]),
        "lengths": torch.from_numpy(meta["lengths"]),
    }


def skewed_topk(T, E, K, seed=0, s=1.1, empty=2):
    """Zipf(s)-biased distinct expert choices per token; the last `empty` experts get no row."""
    g = torch.Generator().manual_seed(seed)
    p = (torch.arange(E, dtype=torch.float64) + 1) ** -s
    if empty:
        p[E - empty:] = 0
    logits = torch.log(p.clamp_min(1e-300)).float()[None, :] + torch.randn(T, E, generator=g) * 0.5
    logits[:, E - empty:] = -1e30 if empty else logits[:, E - empty:]
    return logits.topk(K, dim=1).indices


def uniform(shape, seed, dtype=BF16, lo=-1.0, hi=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.empty(shape).uniform_(lo, hi, generator=g).to(dtype)


def randn(shape, seed, dtype=BF16, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def dev(t):
    return None if t is None else t.cuda()


def assert_bf16_close(got, ref_fp32, rtol=1e-2, atol=1e-2, what=""):
    """max-abs / rel check of a bf16 result against an fp32-accumulated oracle."""
    got = got.float().cpu()
    ref = ref_fp32.float().cpu()
    assert got.shape == ref.shape, f"{what}: shape {got.shape} vs {ref.shape}"
    err = (got - ref).abs()
    bound = atol + rtol * ref.abs()
    bad = err > bound
    assert not bad.any(), (f"{what}: {int(bad.sum())} of {bad.numel()} elements out of tolerance; "
                           f"max err {err.max().item():.4g} at ref {ref.flatten()[err.argmax()].item():.4g}")


def special_scores(T=64, E=16, seed=3):
    """Rows with NaN, +-inf, +-0 and all-equal values among ordinary ones (distinct otherwise)."""
    g = torch.Generator().manual_seed(seed)
    s = torch.rand(T, E, generator=g)
    s[1] = float("nan")                       # the usual divergence case: a row of NaN
    s[2, 3] = float("nan")
    s[2, 9] = float("nan")
    s[3, 5] = float("inf")
    s[4, 7] = float("-inf")
    s[5] = 0.25                               # all equal
    s[6, :4] = 0.0
    s[6, 4:8] = -0.0
    s[7, 2] = float("nan")
    s[7, 11] = float("inf")
    return s
