"""Pins oracle.routing: library routines, brute force on tiny inputs, invariants."""
import numpy as np
import pytest
import torch
from torch.nn import functional as F

from oracle import routing
from tests.helpers import special_scores


def brute_force_routing(topk, E):
    """Counting sort written as plain loops: the definition of a stable sort by expert."""
    T, K = len(topk), len(topk[0])
    buckets = [[] for _ in range(E)]
    for t in range(T):
        for j in range(K):
            buckets[topk[t][j]].append(t * K + j)
    gate_index = [p for b in buckets for p in b]
    lengths = [len(b) for b in buckets]
    token_index = [p // K for p in gate_index]
    per_token = [[] for _ in range(T)]
    for pos, t in enumerate(token_index):
        per_token[t].append(pos)
    return gate_index, token_index, lengths, per_token


@pytest.mark.parametrize("T,E,K", [(1, 4, 1), (5, 4, 2), (7, 8, 3), (16, 3, 3), (33, 16, 4)])
def test_metadata_matches_brute_force(T, E, K):
    rng = np.random.default_rng(T * 100 + E)
    topk = np.stack([rng.permutation(E)[:K] for _ in range(T)])
    meta = routing.routing_metadata(topk, E)
    g, t, l, r = brute_force_routing(topk.tolist(), E)
    assert meta["gate_index"].tolist() == g
    assert meta["token_index"].tolist() == t
    assert meta["lengths"].tolist() == l
    assert meta["reverse_index"].tolist() == r
    assert meta["offsets"].tolist() == [0] + np.cumsum(l).tolist()


@pytest.mark.parametrize("T,E,K", [(64, 8, 2), (300, 64, 8), (100, 128, 8), (17, 5, 5)])
def test_metadata_matches_torch_stable_sort_and_invariants(T, E, K):
    g = torch.Generator().manual_seed(T + E + K)
    topk = torch.randn(T, E, generator=g).topk(K, dim=1).indices
    meta = routing.routing_metadata(topk.numpy(), E)
    # the library routines the reference calls (fast_moe_module.py:122-134)
    _, gate_index = topk.reshape(-1).sort(stable=True)
    token_index = gate_index // K
    reverse = token_index.sort(stable=True)[1].view(T, K)
    assert torch.equal(torch.from_numpy(meta["gate_index"]), gate_index)
    assert torch.equal(torch.from_numpy(meta["token_index"]), token_index)
    assert torch.equal(torch.from_numpy(meta["reverse_index"]), reverse)
    lengths = torch.zeros(E, dtype=torch.int64).scatter_add(
        0, topk.reshape(-1), torch.ones(T * K, dtype=torch.int64))
    assert torch.equal(torch.from_numpy(meta["lengths"]), lengths)
    # invariants
    off = meta["offsets"]
    assert off[0] == 0 and off[-1] == T * K and np.all(np.diff(off) == meta["lengths"])
    sorted_e = topk.reshape(-1).numpy()[meta["gate_index"]]
    assert np.all(np.diff(sorted_e) >= 0)
    for e in range(E):
        seg = meta["token_index"][off[e]:off[e + 1]]
        assert np.all(np.diff(seg) > 0)
    assert np.all(meta["token_index"][meta["reverse_index"]] == np.arange(T)[:, None])
    assert np.all(np.diff(meta["reverse_index"], axis=1) > 0)


def test_complete_cumsum_closed_form():
    assert routing.complete_cumsum(np.array([], dtype=np.int64)).tolist() == [0]
    assert routing.complete_cumsum(np.array([3, 0, 2])).tolist() == [0, 3, 3, 5]


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("T,E,K", [(50, 8, 2), (200, 64, 8), (31, 128, 8), (9, 4, 4)])
def test_select_top_k_against_torch(dtype, T, E, K):
    g = torch.Generator().manual_seed(E * K)
    tdt = torch.float32 if dtype == "fp32" else torch.bfloat16
    scores = F.softmax(torch.randn(T, E, generator=g) * 2, dim=1).to(tdt)
    idx, gates = routing.select_top_k(scores.float().numpy(), K, dtype)
    # selected set: equal to torch.topk's wherever the K-th and (K+1)-th scores differ
    tv, ti = scores.float().topk(min(K + 1, E), dim=1)
    distinct = (tv[:, K - 1] != tv[:, K]).numpy() if K < E else np.ones(T, bool)
    ref_sets = np.sort(scores.topk(K, dim=1).indices.numpy(), axis=1)
    assert np.array_equal(np.sort(idx, axis=1)[distinct], ref_sets[distinct])
    # slot order: descending score, ties by ascending expert id
    v = np.take_along_axis(scores.float().numpy(), idx, 1)
    assert np.all(np.diff(v, axis=1) <= 0)
    tie = np.diff(v, axis=1) == 0
    assert np.all(np.diff(idx, axis=1)[tie] > 0)
    # gates: F.normalize of the masked scores, gathered (fast_moe_module.py:100-103,129)
    mask = torch.zeros_like(scores).scatter_(1, torch.from_numpy(idx), 1)
    ref = F.normalize(scores * mask, p=1, dim=1).gather(1, torch.from_numpy(idx)).float().numpy()
    ulp = 2.0 ** -23 if dtype == "fp32" else 2.0 ** -8
    assert np.all(np.abs(gates - ref) <= 2 * ulp * np.abs(ref))
    assert np.all(gates >= 0)
    assert np.allclose(gates.sum(1), 1.0, atol=K * ulp * 2)


def test_select_top_k_ties_take_lowest_expert():
    scores = np.full((3, 6), 0.25, dtype=np.float32)
    idx, gates = routing.select_top_k(scores, 2, "fp32")
    assert idx.tolist() == [[0, 1]] * 3
    assert np.allclose(gates, 0.5)
    scores = np.array([[0.1, 0.4, 0.4, 0.1]], dtype=np.float32)
    idx, _ = routing.select_top_k(scores, 3, "fp32")
    assert idx.tolist() == [[1, 2, 0]]


def test_select_top_k_brute_force_tiny():
    rng = np.random.default_rng(0)
    scores = rng.random((20, 7)).astype(np.float32)
    idx, _ = routing.select_top_k(scores, 3, "fp32", renorm=False)
    for t in range(20):
        order = sorted(range(7), key=lambda e: (-scores[t, e], e))[:3]
        assert idx[t].tolist() == order


def test_round_to_bf16_matches_torch():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(100000, generator=g) * torch.exp(torch.randn(100000, generator=g) * 10)
    ref = x.to(torch.bfloat16).float().numpy()
    assert np.array_equal(routing.round_to_bf16(x.numpy()), ref)


def test_top_k_total_order_with_nan_inf_and_ties():
    """torch.topk ranks NaN above +inf; ties go to the lower expert id (canonical).  Every row
    yields k distinct ids in range whatever it holds."""
    s = special_scores()
    T, E = s.shape
    for k in (1, 2, 5, 16):
        idx, _ = routing.select_top_k(s.numpy(), k, renorm=False)
        assert idx.min() >= 0 and idx.max() < E
        assert all(len(set(row)) == k for row in idx.tolist())
        ref = s.topk(k, dim=1).indices
        for t in range(T):
            if t in (1, 5, 6):          # ties at the cut: the canonical rule decides, checked below
                continue
            if t == 2 and k == 1:       # two NaN tie for one slot
                continue
            assert set(idx[t].tolist()) == set(ref[t].tolist()), (t, k)
    idx, _ = routing.select_top_k(s.numpy(), 5, renorm=False)
    assert idx[1].tolist() == [0, 1, 2, 3, 4] and idx[5].tolist() == [0, 1, 2, 3, 4]
    assert idx[2].tolist()[:2] == [3, 9]                    # the NaN first, in id order
    assert idx[7].tolist()[:2] == [2, 11]                   # NaN above +inf
    assert idx[3].tolist()[0] == 5
    assert 7 not in routing.select_top_k(s.numpy(), E - 1, renorm=False)[0][4].tolist()   # -inf last
    key = routing.order_key(np.array([-0.0, 0.0, -1.0, 1.0, np.inf, -np.inf, np.nan, -np.nan], dtype=np.float32))
    assert key[0] == key[1] and key[6] == key[7] and key[5] < key[2] < key[0] < key[3] < key[4] < key[6]
    # gates of a row with a NaN among the selected: F.normalize propagates NaN to the whole row
    _, gates = routing.select_top_k(s.numpy(), 4)
    ref = F.normalize(torch.gather(s, 1, torch.from_numpy(routing.select_top_k(s.numpy(), 4)[0])), p=1, dim=1)
    assert np.array_equal(np.isnan(gates), torch.isnan(ref).numpy())
    ok = ~np.isnan(gates)
    assert np.allclose(gates[ok], ref.numpy()[ok], rtol=1e-6, atol=0)
