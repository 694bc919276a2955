"""GPU parity: routing tensors bit-exact against the oracle (through the C ABI)."""
import numpy as np
import pytest
import torch
from torch.nn import functional as F

from oracle import routing as o_routing

pytestmark = pytest.mark.gpu

INT_KEYS = ("topk_idx", "lengths", "offsets", "gate_index", "token_index", "reverse_index")


def softmax_scores(T, E, seed, dtype, temp=2.0):
    g = torch.Generator().manual_seed(seed)
    return F.softmax(torch.randn(T, E, generator=g) * temp, dim=1).to(dtype)


def check_route(scores, K, renorm=True):
    from fast_moe_amd.kernels.hip import ops
    name = "bf16" if scores.dtype == torch.bfloat16 else "fp32"
    ref = o_routing.route(scores.float().numpy(), K, dtype=name, renorm=renorm)
    got = ops.route_topk(scores.cuda(), K, renorm=renorm)
    torch.cuda.synchronize()
    for key in INT_KEYS:
        g = got[key].cpu().numpy().reshape(ref[key].shape)
        assert np.array_equal(g, ref[key]), f"{key} differs (T={scores.shape[0]} E={scores.shape[1]} K={K})"
    gates = got["gates"].float().cpu().numpy()
    assert np.array_equal(gates, ref["gates"]), "gates differ from the oracle bit pattern"
    return got, ref


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,E,K", [
    (1, 4, 1), (5, 4, 2), (64, 8, 2), (33, 16, 4), (17, 5, 5), (300, 64, 8), (1000, 128, 8),
    (129, 24, 3), (7, 300, 6), (50, 512, 8), (2048, 8, 2), (100, 64, 33), (40, 200, 64)])
def test_route_topk_matches_oracle(dtype, T, E, K):
    print(f"route_topk T={T} E={E} K={K} {dtype}", flush=True)
    check_route(softmax_scores(T, E, T * 7 + E + K, dtype), K)


def test_route_topk_ties_and_no_renorm():
    # bf16 softmax over many experts: plenty of exactly equal scores
    scores = softmax_scores(512, 64, 3, torch.bfloat16, temp=0.3)
    check_route(scores, 8)
    check_route(scores, 8, renorm=False)
    flat = torch.full((37, 16), 1.0 / 16)
    got, _ = check_route(flat, 4)
    assert got["topk_idx"].cpu().tolist() == [[0, 1, 2, 3]] * 37


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E", [16, 64, 128])
def test_route_topk_nan_inf_and_equal_rows(E, dtype):
    """Scores after a divergence (rows of NaN, single NaN, +-inf, +-0, all-equal rows): NaN ranks
    above +inf as in torch.topk, every token still fills K distinct slots with ids in [0, E), the
    integer outputs equal the oracle's, lengths sum to T*K, and the gates carry the same NaN."""
    from fast_moe_amd.kernels.hip import ops
    from tests.helpers import special_scores
    scores = special_scores(T=64, E=E, seed=E).to(dtype)
    name = "bf16" if dtype == torch.bfloat16 else "fp32"
    for K in (1, 4, 8):
        for renorm in (True, False):
            ref = o_routing.route(scores.float().numpy(), K, dtype=name, renorm=renorm)
            got = ops.route_topk(scores.cuda(), K, renorm=renorm)
            idx = got["topk_idx"].cpu()
            assert int(idx.min()) >= 0 and int(idx.max()) < E
            assert all(len(set(row)) == K for row in idx.tolist())
            assert int(got["lengths"].sum()) == 64 * K
            for key in INT_KEYS:
                assert np.array_equal(got[key].cpu().numpy().reshape(ref[key].shape), ref[key]), (key, K, renorm)
            assert np.array_equal(got["gates"].float().cpu().numpy(), ref["gates"], equal_nan=True), (K, renorm)


@pytest.mark.parametrize("T,E,K,dtype", [(16384, 64, 8, torch.float32), (8192, 8, 2, torch.bfloat16),
                                         (32768, 128, 8, torch.float32)])
def test_route_topk_full_size(T, E, K, dtype):
    """The benchmark sizes: exact against the oracle and the permutation invariants."""
    got, ref = check_route(softmax_scores(T, E, 11, dtype), K)
    gi = got["gate_index"].cpu().numpy()
    assert np.array_equal(np.sort(gi), np.arange(T * K))
    off = got["offsets"].cpu().numpy()
    assert off[0] == 0 and off[-1] == T * K
    ti = got["token_index"].cpu().numpy()
    ri = got["reverse_index"].cpu().numpy()
    assert np.all(ti[ri] == np.arange(T)[:, None])


@pytest.mark.parametrize("T,E,K", [(16, 4, 2), (100, 16, 4), (500, 8, 2), (1000, 128, 8), (3, 1000, 2),
                                   (20000, 64, 8)])
def test_route_from_topk_matches_oracle(T, E, K):
    from fast_moe_amd.kernels.hip import ops
    g = torch.Generator().manual_seed(T + E)
    topk = torch.randn(T, E, generator=g).topk(K, dim=1).indices
    ref = o_routing.routing_metadata(topk.numpy(), E)
    got = ops.route_from_topk(topk.cuda(), E)
    torch.cuda.synchronize()
    for key in ("lengths", "offsets", "gate_index", "token_index", "reverse_index"):
        assert np.array_equal(got[key].cpu().numpy().reshape(ref[key].shape), ref[key]), key
    assert got["bad_count"].item() == 0


def test_route_from_topk_duplicates_and_big_shape():
    """Repeated expert ids inside a token row keep slot order (stable); the row count of
    kernels/tests/moe_test.py:132-161 scaled to fit a quick run still crosses 2^20 positions."""
    from fast_moe_amd.kernels.hip import ops
    g = torch.Generator().manual_seed(5)
    topk = torch.randint(0, 4, (2000, 4), generator=g)
    ref = o_routing.routing_metadata(topk.numpy(), 4)
    got = ops.route_from_topk(topk.cuda(), 4)
    for key in ("lengths", "offsets", "gate_index", "token_index", "reverse_index"):
        assert np.array_equal(got[key].cpu().numpy().reshape(ref[key].shape), ref[key]), key
    topk = torch.randint(0, 4, (700000, 2), generator=g)
    ref = o_routing.routing_metadata(topk.numpy(), 4)
    got = ops.route_from_topk(topk.cuda(), 4)
    for key in ("lengths", "offsets", "gate_index", "token_index", "reverse_index"):
        assert np.array_equal(got[key].cpu().numpy().reshape(ref[key].shape), ref[key]), key


def test_route_from_topk_flags_bad_ids_and_empty_input():
    from fast_moe_amd.kernels.hip import ops
    topk = torch.tensor([[0, 9], [1, 2], [-1, 3]])
    got = ops.route_from_topk(topk.cuda(), 4)
    assert got["bad_count"].item() == 2
    assert got["lengths"].cpu().tolist() == [1, 1, 1, 1]
    got = ops.route_from_topk(torch.zeros((0, 2), dtype=torch.int64).cuda(), 4)
    assert got["offsets"].cpu().tolist() == [0] * 5
    got = ops.route_topk(torch.zeros((0, 8)).cuda(), 2)
    assert got["lengths"].cpu().tolist() == [0] * 8
