"""Pins of oracle/mrn.py (CPU): the router's gates, the dispatcher's order and the whole layer
against independent formulations."""
import numpy as np
import torch
import torch.nn.functional as F

from oracle import moe as o_moe
from oracle import mrn as o_mrn
from oracle import routing as o_routing


def params(D, H, O, E, seed=0, noisy=False):
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g)
    p = {"_w_gate": rn(D, E) * D ** -0.5, "_experts_hidden_w": rn(E, H, D) * D ** -0.5,
         "_experts_hidden_bias": rn(E, H) * 0.1, "_experts_w": rn(E, O, H) * H ** -0.5,
         "_experts_bias": rn(E, O) * 0.1, "_output_weight": rn(D, O) * D ** -0.5,
         "_norm_w": 1 + 0.1 * rn(D), "_norm_bias": 0.1 * rn(D)}
    if noisy:
        p["_w_noise"] = rn(D, E) * D ** -0.5
    return p


def test_gates_are_softmax_of_normalised_logits_at_the_top_k():
    p = params(32, 16, 8, 8)
    x = torch.randn(50, 32, generator=torch.Generator().manual_seed(1))
    for post in (False, True):
        gates, loss = o_mrn.noisy_gating(p, x, 3, train=False, noisy=False, post_softmax=post)
        n = F.normalize(x @ p["_w_gate"], dim=1)
        top = n.topk(3, dim=1)
        full = F.softmax(n, dim=1)
        expect = F.softmax(top.values, dim=1) if post else full.gather(1, top.indices)
        assert ((gates > 0).sum(1) == 3).all() and loss.item() == 0
        torch.testing.assert_close(gates.gather(1, top.indices), expect)
        if post:
            torch.testing.assert_close(gates.sum(1), torch.ones(50))


def test_dispatch_groups_rows_by_expert():
    """mrn.py:56 sorts without stable=True: inside an expert the row order is whatever torch's
    sort leaves, so the pin is per expert segment as a set, with every gate staying with its row."""
    p = params(16, 8, 8, 6)
    x = torch.randn(40, 16, generator=torch.Generator().manual_seed(2))
    gates, _ = o_mrn.noisy_gating(p, x, 2, train=False, noisy=False)
    batch_index, nz_gates, sizes = o_mrn.dispatch_order(gates)
    topk = torch.nonzero(gates)[:, 1].view(40, 2)              # ascending expert id per token
    meta = o_routing.routing_metadata(topk.numpy(), 6)
    assert sizes == meta["lengths"].tolist()
    off = meta["offsets"]
    for e in range(6):
        seg = batch_index[off[e]:off[e + 1]]
        assert np.array_equal(np.sort(seg.numpy()), meta["token_index"][off[e]:off[e + 1]])
        torch.testing.assert_close(nz_gates[off[e]:off[e + 1], 0], gates[seg, e])


def test_router_matches_the_operator_level_oracle():
    """The comparison of kernels/tests/mrn_test.py: dense dispatch against the jagged operators."""
    D, H, O, E, k, T = 32, 48, 24, 8, 2, 96
    p = params(D, H, O, E, seed=3)
    x = torch.randn(T, D, generator=torch.Generator().manual_seed(4))
    y, loss, load = o_mrn.router_forward(p, x, k, train=True)
    n = F.normalize(x @ p["_w_gate"], dim=1)
    order = n.sort(descending=True, dim=1, stable=True)
    topk, gates = order.indices[:, :k].contiguous(), F.softmax(order.values, dim=1)[:, :k].contiguous()
    meta = o_routing.routing_metadata(topk.numpy(), E)
    t = lambda name: torch.from_numpy(np.ascontiguousarray(meta[name]))
    hidden = o_moe.index_select_jagged_bmm(t("offsets"), t("gate_index").view(-1, k), x,
                                           p["_experts_hidden_w"].permute(0, 2, 1), p["_experts_hidden_bias"])
    y2 = o_moe.silu_jagged_bmm_combine(t("offsets"), hidden, p["_experts_w"].permute(0, 2, 1), p["_experts_bias"],
                                       t("token_index"), k, gates, t("gate_index"))
    torch.testing.assert_close(y, y2, rtol=1e-5, atol=1e-5)
    dense = torch.zeros(T, E).scatter(1, topk, gates)
    expect_loss = (o_mrn.cv_squared(dense.sum(0)) + o_mrn.cv_squared((dense > 0).sum(0))) * 1e-2
    torch.testing.assert_close(loss, expect_loss)
    torch.testing.assert_close(load.sum(), torch.tensor(1.0))


def test_noisy_load_is_a_probability_and_matches_the_closed_form():
    D, E, k, T = 16, 6, 2, 30
    p = params(D, 8, 8, E, seed=5, noisy=True)
    g = torch.Generator().manual_seed(6)
    x, noise = torch.randn(T, D, generator=g), torch.randn(T, E, generator=g)
    gates, loss = o_mrn.noisy_gating(p, x, k, train=True, noisy=True, noise=noise)
    clean = x @ p["_w_gate"]
    std = F.softplus(x @ p["_w_noise"]) + 1e-2
    noisy = clean + noise * std
    top = F.normalize(noisy, dim=1).sort(descending=True, dim=1, stable=True).values[:, :k + 1]
    prob = o_mrn.prob_in_top_k(clean, noisy, std, top, k)
    assert ((prob >= 0) & (prob <= 1)).all() and loss.item() > 0
    # brute force for one entry: Phi((clean - threshold) / std) with the k-th / (k+1)-th normalised logit
    t, e = 3, 1
    thr = top[t, k] if noisy[t, e] > top[t, k] else top[t, k - 1]
    expect = 0.5 * (1 + torch.erf((clean[t, e] - thr) / std[t, e] / 2 ** 0.5))
    torch.testing.assert_close(prob[t, e], expect)
