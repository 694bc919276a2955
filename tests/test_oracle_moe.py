"""Pins oracle.moe / oracle.moe_fp8 / oracle.layer: reductions to a plain matmul,
pure-Python loops on tiny inputs, the dense every-expert MoE."""
import numpy as np
import pytest
import torch
from torch.nn import functional as F

from oracle import layer, moe, moe_fp8, routing


def make_routing(L, E, K, seed=0):
    """The input generator of kernels/tests/moe_test.py:191-197,241."""
    g = torch.Generator().manual_seed(seed)
    gate = torch.randn(L, E, generator=g).topk(K, dim=1).indices
    expert, index = gate.contiguous().view(-1).sort(stable=True)
    lengths = torch.zeros(E, dtype=torch.int64).scatter_add(0, expert, torch.ones_like(expert))
    offsets = torch.from_numpy(routing.complete_cumsum(lengths.numpy()))
    return gate, index.view(-1, K), offsets


def test_gather_gemm_tiny_pure_python():
    L, E, K, Din, Dout = 5, 3, 2, 4, 3
    g = torch.Generator().manual_seed(1)
    gate, index, offsets = make_routing(L, E, K, 1)
    x = torch.randn(L, Din, generator=g)
    w = torch.randn(E, Din, Dout, generator=g)
    b = torch.randn(E, Dout, generator=g)
    out = moe.index_select_jagged_bmm(offsets, index, x, w, b)
    flat = index.reshape(-1).tolist()
    off = offsets.tolist()
    for e in range(E):
        for r in range(off[e], off[e + 1]):
            tok = flat[r] // K
            assert gate.reshape(-1)[flat[r]].item() == e
            for n in range(Dout):
                acc = b[e, n].item()
                for k in range(Din):
                    acc += x[tok, k].item() * w[e, k, n].item()
                assert abs(out[r, n].item() - acc) < 1e-5


def test_gather_gemm_reduces_to_dense_matmul():
    g = torch.Generator().manual_seed(2)
    L, Din, Dout = 9, 6, 5
    x = torch.randn(L, Din, generator=g)
    w = torch.randn(1, Din, Dout, generator=g)
    b = torch.randn(1, Dout, generator=g)
    index = torch.arange(L).view(L, 1)
    offsets = torch.tensor([0, L])
    out = moe.index_select_jagged_bmm(offsets, index, x, w, b)
    torch.testing.assert_close(out, x @ w[0] + b[0])
    # strided [E,K,N] view of [E,N,K] storage gives the same answer
    w_t = w.transpose(1, 2).contiguous().transpose(1, 2)
    torch.testing.assert_close(moe.index_select_jagged_bmm(offsets, index, x, w_t, b), out)
    # raw form of moe_fp8.py:78-95 is the same function
    torch.testing.assert_close(moe_fp8.index_select_jagged_bmm_raw(offsets, index, x, w, b), out)


@pytest.mark.parametrize("L,E,K", [(16, 4, 2), (100, 8, 4), (7, 16, 2)])
def test_swiglu_and_gating_compose_from_plain_op(L, E, K):
    g = torch.Generator().manual_seed(L)
    _, index, offsets = make_routing(L, E, K, L)
    x = torch.randn(L, 12, generator=g)
    x2 = torch.randn(L, 12, generator=g)
    w = torch.randn(E, 12, 8, generator=g)
    wp = torch.randn(E, 12, 8, generator=g)
    b = torch.randn(E, 8, generator=g)
    bp = torch.randn(E, 8, generator=g)
    a = moe.index_select_jagged_bmm(offsets, index, x, w, b)
    c = moe.index_select_jagged_bmm(offsets, index, x, wp, bp)
    torch.testing.assert_close(
        moe.index_select_jagged_bmm_swiglu(offsets, index, x, w, b, wp, bp), F.silu(a) * c)
    c2 = moe.index_select_jagged_bmm(offsets, index, x2, wp, bp)
    torch.testing.assert_close(
        moe.index_select_jagged_gating_bmm(offsets, index, x, x2, w, wp, b, bp), F.silu(a) * c2)
    torch.testing.assert_close(
        moe.index_select_jagged_gating_bmm(offsets, index, x, x, w, wp, b, bp), F.silu(a) * c)


def test_3d_variant_tiny():
    g = torch.Generator().manual_seed(3)
    L, E, K = 6, 3, 2
    _, index, offsets = make_routing(L, E, K, 3)
    x = torch.randn(L, E, 4, generator=g)
    w = torch.randn(E, 4, 5, generator=g)
    out = moe.index_select_jagged_bmm_3D(offsets, index, x, w, None)
    flat = index.reshape(-1)
    for e in range(E):
        for r in range(offsets[e], offsets[e + 1]):
            torch.testing.assert_close(out[r], x[flat[r] // K, e] @ w[e])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mul_merge_k_add_double_loop(dtype):
    """Generator of kernels/tests/moe_test.py:344-367 (non-contiguous weight, permuted weight_index)."""
    N, K, D = 33, 4, 8
    g = torch.Generator().manual_seed(4)
    x = torch.empty(N * K, D).uniform_(-1, 1, generator=g).to(dtype)
    w = torch.empty(N, 2 * K).uniform_(-1, 1, generator=g).to(dtype)[:, :K]
    w_index = torch.randperm(N * K, generator=g)
    perm = torch.randperm(N * K, generator=g)
    o2i = torch.arange(N).repeat(K)[perm]
    out = moe.mul_merge_k_add(o2i, x, K, w, w_index)
    wf = w.contiguous().view(-1)
    ref = torch.zeros(N, D, dtype=torch.float32)
    for r in range(N * K):           # ascending row order: the CPU index_add order
        prod = (x[r] * wf[w_index[r]]).float()     # product rounded to the value dtype
        ref[o2i[r]] = ref[o2i[r]] + prod
    assert torch.equal(out, ref.to(dtype))
    assert out.dtype == dtype
    # no weight: plain segmented sum
    out2 = moe.mul_merge_k_add(o2i, x, K)
    ref2 = torch.zeros(N, D).index_add(0, o2i, x.float()).to(dtype)
    assert torch.equal(out2, ref2)


def test_combine_and_fused_compose():
    g = torch.Generator().manual_seed(5)
    L, E, K, D, H, O = 40, 8, 2, 16, 24, 12
    scores = F.softmax(torch.randn(L, E, generator=g), dim=1)
    r = layer.route_scores(scores, K)
    x = torch.randn(L, D, generator=g)
    wg = torch.randn(E, D, H, generator=g) / 4
    wu = torch.randn(E, D, H, generator=g) / 4
    wd = torch.randn(E, H, O, generator=g) / 4
    bd = torch.randn(E, O, generator=g)
    idx2 = r["gate_index"].view(-1, K)
    hidden = moe.index_select_jagged_bmm_swiglu(r["offsets"], idx2, x, wg, None, wu, None)
    y = moe.silu_jagged_bmm_combine(r["offsets"], hidden, wd, bd, r["token_index"], K,
                                    r["gates"], r["gate_index"], has_silu=False)
    y2 = moe.fused_jagged_bmm_swiglu_combine(r["offsets"], idx2, x, wg, None, wu, None, wd, bd, K,
                                             r["gates"], r["gate_index"])
    torch.testing.assert_close(y, y2)
    # per-token closed form
    topk = r["topk_idx"]
    for t in range(0, L, 7):
        acc = torch.zeros(O)
        for j in range(K):
            e = topk[t, j].item()
            h = F.silu(x[t] @ wg[e]) * (x[t] @ wu[e])
            acc += r["gates"][t, j] * (h @ wd[e] + bd[e])
        torch.testing.assert_close(y[t], acc, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("k,bias", [(1, 0.0), (2, 0.5)])
def test_layer_matches_dense_moe_constant_weights(k, bias):
    """The construction of modules/tests/test_moe_parity.py:72-106."""
    torch.manual_seed(42)
    B, S, D, H, O, E = 4, 8, 10, 16, 10, 8
    x = torch.randn(B, S, D)
    c = lambda *s: torch.full(s, 0.5)
    cb = lambda *s: torch.full(s, bias)
    args = (x, c(E, D), cb(E), c(E, H, D), cb(E, H), c(E, O, H), cb(E, O), k)
    y, _ = layer.moe_layer_forward(*args)
    torch.testing.assert_close(y, layer.dense_moe_forward(*args), atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("k", [1, 2, 3])
def test_layer_matches_dense_moe_random_weights(k):
    g = torch.Generator().manual_seed(7)
    B, S, D, H, O, E = 2, 16, 12, 20, 9, 6
    x = torch.randn(B, S, D, generator=g)
    args = (x, torch.randn(E, D, generator=g), torch.randn(E, generator=g),
            torch.randn(E, H, D, generator=g) / 3, torch.randn(E, H, generator=g),
            torch.randn(E, O, H, generator=g) / 4, torch.randn(E, O, generator=g), k)
    y, r = layer.moe_layer_forward(*args)
    torch.testing.assert_close(y, layer.dense_moe_forward(*args), atol=1e-5, rtol=1e-4)
    assert r["offsets"][-1].item() == B * S * k


def test_fp8_gemm_agrees_with_dequantised_fp32_oracle():
    g = torch.Generator().manual_seed(8)
    L, E, K, Din, Dout = 64, 4, 2, 64, 32
    _, index, offsets = make_routing(L, E, K, 8)
    x = torch.empty(L, Din).uniform_(-1, 1, generator=g).to(torch.bfloat16)
    w = torch.empty(E, Din, Dout).uniform_(-1, 1, generator=g).to(torch.bfloat16)
    b = torch.empty(E, Dout).uniform_(-1, 1, generator=g).to(torch.bfloat16)
    out = moe_fp8.index_select_jagged_bmm_fp8(offsets, index, x, w, b)
    qa, sa = moe_fp8.rowwise_quant_fp8(x)
    qw, sw = moe_fp8.rowwise_quant_fp8(w.permute(0, 2, 1))
    xd = moe_fp8.dequant(qa) / sa[:, None]
    wd = (moe_fp8.dequant(qw) / sw[:, :, None]).permute(0, 2, 1)
    ref = moe.index_select_jagged_bmm(offsets, index, xd, wd, b.float())
    torch.testing.assert_close(out.float(), ref, atol=2e-2, rtol=2e-2)
    # and stays close to the unquantised op (tolerance of kernels/tests/moe_fp8_test.py:302-335)
    raw = moe_fp8.index_select_jagged_bmm_raw(offsets, index, x.float(), w.float(), b.float())
    torch.testing.assert_close(out.float(), raw, atol=4e-1, rtol=1e-1)


@pytest.mark.parametrize("with_bias", [True, False])
def test_fp8_backward_is_exact_where_quantisation_is_lossless(with_bias):
    """Integers up to 7 (three significant bits) times a power of two survive e4m3 with the
    power-of-two scales unchanged, so the fp8 backward must give torch autograd's gradients of
    the unquantised operator exactly: a wrong gather, a transposed operand, a missing scale or
    a wrong axis for a scale would each show."""
    g = torch.Generator().manual_seed(5)
    L, E, K, Din, Dout = 48, 4, 2, 24, 16
    _, index, offsets = make_routing(L, E, K, 5)

    def ints(*shape, step):
        t = torch.randint(-7, 8, shape, generator=g).float() * step
        t.view(-1, shape[-1])[:, 0] = 7 * step          # every row (and column block) reaches the same amax
        return t
    x = ints(L, Din, step=2.0 ** -3)
    x[0, :] = 7 * 2.0 ** -3                              # ... and every column of x
    w = ints(E, Din, Dout, step=2.0 ** -5)
    d_out = ints(L * K, Dout, step=2.0 ** -6)
    d_out[0, :] = 7 * 2.0 ** -6
    b = torch.zeros(E, Dout) if with_bias else None
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    br = b.clone().requires_grad_(True) if with_bias else None
    moe_fp8.index_select_jagged_bmm_raw(offsets, index, xr, wr, br).backward(d_out)
    dx, dw, db = moe_fp8.index_select_jagged_bmm_fp8_backward(offsets, index, x, w, b, d_out)
    assert torch.equal(dx, xr.grad)
    assert torch.equal(dw, wr.grad)
    if with_bias:
        assert torch.equal(db, br.grad)
    else:
        assert db is None


def test_fp8_backward_tracks_the_unquantised_gradients():
    g = torch.Generator().manual_seed(9)
    L, E, K, Din, Dout = 96, 4, 2, 64, 32
    _, index, offsets = make_routing(L, E, K, 9)
    x = torch.empty(L, Din).uniform_(-1, 1, generator=g).to(torch.bfloat16)
    w = torch.empty(E, Din, Dout).uniform_(-1, 1, generator=g).to(torch.bfloat16)
    d_out = torch.empty(L * K, Dout).uniform_(-1, 1, generator=g).to(torch.bfloat16)
    xr, wr = x.float().requires_grad_(True), w.float().requires_grad_(True)
    moe_fp8.index_select_jagged_bmm_raw(offsets, index, xr, wr, None).backward(d_out.float())
    dx, dw, _ = moe_fp8.index_select_jagged_bmm_fp8_backward(offsets, index, x, w, None, d_out)
    assert dx.dtype == torch.bfloat16 and dw.dtype == torch.bfloat16
    for got, ref in ((dx, xr.grad), (dw, wr.grad)):
        err = (got.float() - ref).abs().max() / ref.abs().max()
        assert err < 0.06, err


def test_fp8_swiglu_chain_runs_and_tracks_bf16_chain():
    g = torch.Generator().manual_seed(9)
    L, E, K, D, H = 48, 8, 2, 64, 32
    scores = F.softmax(torch.randn(L, E, generator=g), dim=1)
    r = layer.route_scores(scores, K)
    bf = torch.bfloat16
    x = torch.randn(L, D, generator=g).to(bf)
    wg = (torch.randn(E, D, H, generator=g) / 8).to(bf)
    wu = (torch.randn(E, D, H, generator=g) / 8).to(bf)
    wd = (torch.randn(E, H, D, generator=g) / 6).to(bf)
    idx2 = r["gate_index"].view(-1, K)
    gates = r["gates"].to(bf)
    y8, h8 = moe_fp8.swiglu_moe_fp8(r["offsets"], idx2, x, wg, None, wu, None, wd, None,
                                    r["token_index"], K, gates, r["gate_index"])
    y16 = moe.fused_jagged_bmm_swiglu_combine(r["offsets"], idx2, x, wg, None, wu, None, wd, None, K,
                                              gates, r["gate_index"])
    assert y8.dtype == bf and y8.shape == (L, D)
    err = (y8.float() - y16.float()).abs().max() / y16.float().abs().max()
    assert err < 0.15
