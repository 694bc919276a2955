"""GPU parity of the backward pass: gradients of the HIP operators against torch autograd
through the CPU oracle (fp32 accumulation), with the tolerances of the reference's own
backward checks (kernels/tests/moe_test.py:276-297, 388-400)."""
import pytest
import torch

from helpers import BF16, dev, make_routing, randn
from oracle import layer as o_layer
from oracle import moe as o_moe

pytestmark = pytest.mark.gpu


def close(got, ref, what, rtol=2e-2, atol_frac=1e-2):
    got, ref = got.float().cpu(), ref.float().cpu()
    assert got.shape == ref.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    atol = atol_frac * ref.abs().max().item() + 1e-12
    err = (got - ref).abs()
    bad = err > atol + rtol * ref.abs()
    assert not bad.any(), (f"{what}: {int(bad.sum())} of {bad.numel()} out of tolerance, max err "
                           f"{err.max().item():.4g}, max |ref| {ref.abs().max().item():.4g}")


def leaf(t, dtype=None, device=None):
    t = t.detach().clone()
    if dtype is not None:
        t = t.to(dtype)
    if device is not None:
        t = t.to(device)
    return t.requires_grad_(True)


def kn_weight(E, K, N, seed, contiguous, scale):
    w = randn((E, K, N), seed, scale=scale)
    if not contiguous:
        w = w.transpose(1, 2).contiguous().transpose(1, 2)
    return w


@pytest.mark.parametrize("L,E,K,Din,Dout,contiguous", [
    (100, 4, 2, 32, 32, True),
    (500, 16, 4, 64, 128, False),
    (2048, 8, 2, 256, 512, False),
    (300, 8, 2, 40, 72, True),          # K / N tails, short experts
])
@pytest.mark.parametrize("dtype", [BF16, torch.float32])
def test_index_select_jagged_bmm_backward(L, E, K, Din, Dout, contiguous, dtype):
    from fast_moe_amd.kernels import moe
    r = make_routing(L, E, K, seed=L + 1)
    x0 = randn((L, Din), 1).to(dtype)
    w0 = kn_weight(E, Din, Dout, 2, contiguous, Din ** -0.5).to(dtype)
    b0 = randn((E, Dout), 3).to(dtype)
    dout = (randn((L * K, Dout), 4) * 0.01).to(dtype)
    xr, wr, br = leaf(x0, torch.float32), leaf(w0, torch.float32), leaf(b0, torch.float32)
    o_moe.index_select_jagged_bmm(r["offsets"], r["index"], xr, wr, br).backward(dout.float())
    x, w, b = leaf(x0, device="cuda"), leaf(w0, device="cuda"), leaf(b0, device="cuda")
    out = moe.index_select_jagged_bmm(0, dev(r["offsets"]), dev(r["index"]), x, w, b)
    out.backward(dev(dout))
    tol = dict(rtol=2e-2, atol_frac=1e-2) if dtype == BF16 else dict(rtol=1e-4, atol_frac=1e-5)
    close(x.grad, xr.grad, "d_jagged", **tol)
    close(w.grad, wr.grad, "d_weight", **tol)
    close(b.grad, br.grad, "d_bias", **tol)
    assert x.grad.dtype == dtype and w.grad.shape == w.shape


@pytest.mark.parametrize("L,E,K,Din,H", [(256, 4, 2, 64, 96), (1024, 16, 4, 128, 192)])
def test_swiglu_backward(L, E, K, Din, H):
    from fast_moe_amd.kernels import moe
    r = make_routing(L, E, K, seed=7)
    x0 = randn((L, Din), 1)
    wg0, wu0 = kn_weight(E, Din, H, 2, False, Din ** -0.5), kn_weight(E, Din, H, 3, False, Din ** -0.5)
    bg0, bu0 = randn((E, H), 4), randn((E, H), 5)
    dout = randn((L * K, H), 6) * 0.01
    ref = [leaf(t, torch.float32) for t in (x0, wg0, bg0, wu0, bu0)]
    o_moe.index_select_jagged_bmm_swiglu(r["offsets"], r["index"], *ref).backward(dout.float())
    got = [leaf(t, device="cuda") for t in (x0, wg0, bg0, wu0, bu0)]
    out = moe.index_select_jagged_bmm_swiglu(0, dev(r["offsets"]), dev(r["index"]), *got)
    out.backward(dev(dout))
    for name, g, q in zip(("d_jagged", "d_weight", "d_bias", "d_weight_p", "d_bias_p"), got, ref):
        close(g.grad, q.grad, name, rtol=3e-2, atol_frac=1.5e-2)


@pytest.mark.parametrize("L,E,K,Din,H,dtype", [
    (300, 8, 2, 64, 128, BF16),
    (2048, 8, 2, 256, 256, BF16),        # in-place weight gradient, ring GEMMs
    (200, 4, 2, 40, 72, torch.float32),
])
def test_gating_bmm_two_inputs_backward(L, E, K, Din, H, dtype):
    """silu(A Wa + ba) * (B Wb + bb) with A is not B: every gradient (kernels/triton/triton_moe.py:2839-2990)."""
    from fast_moe_amd.kernels import moe
    r = make_routing(L, E, K, seed=11)
    t0 = [randn((L, Din), 1), randn((L, Din), 2), kn_weight(E, Din, H, 3, False, Din ** -0.5),
          kn_weight(E, Din, H, 4, True, Din ** -0.5), randn((E, H), 5), randn((E, H), 6)]
    t0 = [t.to(dtype) for t in t0]
    dout = (randn((L * K, H), 7) * 0.01).to(dtype)
    ref = [leaf(t, torch.float32) for t in t0]
    o_moe.index_select_jagged_gating_bmm(r["offsets"], r["index"], *ref).backward(dout.float())
    got = [leaf(t, device="cuda") for t in t0]
    ja, jb, wa, wb, ba, bb = got
    out = moe.index_select_jagged_gating_bmm(0, dev(r["offsets"]), dev(r["index"]), ja, jb, wa, ba, wb, bb)
    out.backward(dev(dout))
    tol = dict(rtol=3e-2, atol_frac=1.5e-2) if dtype == BF16 else dict(rtol=1e-4, atol_frac=1e-5)
    for name, g, q in zip(("d_jagged_a", "d_jagged_b", "d_weight_a", "d_weight_b", "d_bias_a", "d_bias_b"), got, ref):
        close(g.grad, q.grad, name, **tol)


@pytest.mark.parametrize("L,E,K,Din,Dout,dtype", [
    (300, 4, 2, 64, 128, BF16),
    (1500, 6, 3, 128, 256, BF16),
    (200, 4, 2, 40, 72, torch.float32),
])
def test_bmm_3d_backward(L, E, K, Din, Dout, dtype):
    """jagged [L, E, Din], expert e reads slice [:, e, :]: every gradient, cells no row reads get zero
    (kernels/triton/triton_moe.py:1399-1476)."""
    from fast_moe_amd.kernels import moe
    r = make_routing(L, E, K, seed=13)
    x0 = randn((L, E, Din), 1).to(dtype)
    w0 = kn_weight(E, Din, Dout, 2, False, Din ** -0.5).to(dtype)
    b0 = randn((E, Dout), 3).to(dtype)
    dout = (randn((L * K, Dout), 4) * 0.01).to(dtype)
    xr, wr, br = leaf(x0, torch.float32), leaf(w0, torch.float32), leaf(b0, torch.float32)
    o_moe.index_select_jagged_bmm_3D(r["offsets"], r["index"], xr, wr, br).backward(dout.float())
    x, w, b = leaf(x0, device="cuda"), leaf(w0, device="cuda"), leaf(b0, device="cuda")
    out = moe.index_select_jagged_bmm_3D(0, dev(r["offsets"]), dev(r["index"]), x, w, b)
    out.backward(dev(dout))
    tol = dict(rtol=3e-2, atol_frac=1.5e-2) if dtype == BF16 else dict(rtol=1e-4, atol_frac=1e-5)
    for name, g, q in zip(("d_jagged", "d_weight", "d_bias"), (x, w, b), (xr, wr, br)):
        close(g.grad, q.grad, name, **tol)
    assert torch.equal(x.grad.cpu() == 0, xr.grad == 0), "untouched cells"


@pytest.mark.parametrize("gate_dtype", [BF16, torch.float32])
def test_mul_merge_k_add_backward(gate_dtype):
    from fast_moe_amd.kernels import moe
    T, E, K, D = 300, 8, 4, 96
    r = make_routing(T, E, K, seed=11)
    v0 = randn((T * K, D), 1)
    g0 = torch.rand((T, K), generator=torch.Generator().manual_seed(2)).to(gate_dtype)
    out_dtype = torch.promote_types(BF16, gate_dtype)
    dy = (randn((T, D), 3) * 0.01).to(out_dtype)
    vr, gr = leaf(v0), leaf(g0)
    o_moe.mul_merge_k_add(r["token_index"], vr, K, gr, r["gate_index"]).backward(dy)
    v, g = leaf(v0, device="cuda"), leaf(g0, device="cuda")
    out = moe.mul_merge_k_add(dev(r["token_index"]), dev(r["reverse_index"]), v, weight=g,
                              weight_index=dev(r["gate_index"]))
    out.backward(dev(dy))
    if gate_dtype == BF16:      # round(dy * w): the same single rounding as autograd's bf16 mul
        assert torch.equal(v.grad.cpu(), vr.grad)
    else:
        close(v.grad, vr.grad, "d_value", rtol=1e-2, atol_frac=1e-3)
    close(g.grad, gr.grad, "d_weight", rtol=1e-2, atol_frac=1e-2)


@pytest.mark.parametrize("has_silu", [True, False])
def test_silu_jagged_bmm_combine_backward(has_silu):
    from fast_moe_amd.kernels import moe
    T, E, K, H, O = 512, 8, 2, 96, 128
    r = make_routing(T, E, K, seed=13)
    j0 = randn((T * K, H), 1)
    w0 = kn_weight(E, H, O, 2, False, H ** -0.5)
    b0 = randn((E, O), 3)
    g0 = torch.rand((T, K), generator=torch.Generator().manual_seed(4)).to(BF16)
    dy = randn((T, O), 5) * 0.01
    ref = [leaf(t, torch.float32) for t in (j0, w0, b0, g0)]
    o_moe.silu_jagged_bmm_combine(r["offsets"], ref[0], ref[1], ref[2], r["token_index"], K, ref[3],
                                  r["gate_index"], has_silu).backward(dy.float())
    got = [leaf(t, device="cuda") for t in (j0, w0, b0, g0)]
    out = moe.silu_jagged_bmm_combine(0, dev(r["offsets"]), got[0], got[1], got[2], dev(r["token_index"]),
                                      dev(r["reverse_index"]), got[3], dev(r["gate_index"]), has_silu=has_silu)
    out.backward(dev(dy))
    for name, g, q in zip(("d_jagged", "d_weight", "d_bias", "d_gates"), got, ref):
        close(g.grad, q.grad, name, rtol=3e-2, atol_frac=1.5e-2)


@pytest.mark.parametrize("recompute", [False, True])
def test_silu_jagged_bmm_combine_fp8_trains_in_bf16(recompute):
    """Forward on e4m3 operands, backward in bf16 on the original tensors
    (SiluJaggedBmmFp8MixedGemmCombine, kernels/triton/triton_moe_fp8.py:1373-1720): the gradients
    that do not see the forward GEMM's output meet the bf16 bar; the gate gradient, a dot product
    with that output, meets it when the output is recomputed in bf16 (activation_checkpointing)
    and an e4m3 bar otherwise."""
    from fast_moe_amd.kernels import moe, moe_fp8
    T, E, K, H, O = 512, 8, 2, 128, 256
    r = make_routing(T, E, K, seed=13)
    j0 = randn((T * K, H), 1)
    w0 = kn_weight(E, H, O, 2, False, H ** -0.5)
    b0 = randn((E, O), 3)
    g0 = torch.rand((T, K), generator=torch.Generator().manual_seed(4)).to(BF16)
    dy = randn((T, O), 5) * 0.01
    ref = [leaf(t, torch.float32) for t in (j0, w0, b0, g0)]
    o_moe.silu_jagged_bmm_combine(r["offsets"], ref[0], ref[1], ref[2], r["token_index"], K, ref[3],
                                  r["gate_index"], True).backward(dy.float())
    got = [leaf(t, device="cuda") for t in (j0, w0, b0, g0)]
    args = (dev(r["offsets"]), got[0], got[1], got[2], dev(r["token_index"]), dev(r["reverse_index"]), got[3],
            dev(r["gate_index"]))
    out = moe_fp8.silu_jagged_bmm_combine_fp8(0, *args, activation_checkpointing=recompute)
    with torch.no_grad():       # the forward value is the fp8 operator's own
        assert torch.equal(out, moe_fp8.silu_jagged_bmm_combine_fp8(0, *args))
    out.backward(dev(dy))
    for name, g, q in zip(("d_jagged", "d_weight", "d_bias"), got, ref):
        close(g.grad, q.grad, name, rtol=3e-2, atol_frac=1.5e-2)
    loose = {} if recompute else dict(rtol=1e-1, atol_frac=5e-2)
    close(got[3].grad, ref[3].grad, "d_gates", **(loose or dict(rtol=3e-2, atol_frac=1.5e-2)))
    # and the bf16 entry point of the fp8 module trains as the bf16 operator does
    x = leaf(randn((T, H), 6), device="cuda")
    w = leaf(w0, device="cuda")
    y = moe_fp8.index_select_jagged_bmm(0, dev(r["offsets"]), dev(r["index"]), x, w, None, fp8=False)
    y.sum().backward()
    x2, w2 = leaf(x, device="cuda"), leaf(w, device="cuda")
    moe.index_select_jagged_bmm(0, dev(r["offsets"]), dev(r["index"]), x2, w2, None).sum().backward()
    assert torch.equal(x.grad, x2.grad) and torch.equal(w.grad, w2.grad)


def test_layer_backward_matches_oracle():
    """FastMoELayer under grad mode: every parameter and the input receive the oracle's gradient."""
    from fast_moe_amd import FastMoELayer
    torch.manual_seed(0)
    B, S, D, H, O, E, k = 2, 128, 64, 96, 64, 8, 2
    layer = FastMoELayer(D, H, O, E, dtype=torch.float32)
    with torch.no_grad():
        layer._experts_hidden_bias.normal_(0, 0.1)
        layer._experts_bias.normal_(0, 0.1)
    x0 = torch.randn(B, S, D)
    dy = torch.randn(B, S, O) * 0.01
    params = {n: p.detach().clone().requires_grad_(True) for n, p in layer.named_parameters()}
    xr = x0.clone().requires_grad_(True)
    # oracle: the dense every-expert formulation is differentiable end to end
    y_ref = o_layer.dense_moe_forward(xr, params["gate.gate.weight"], params["gate.gate.bias"],
                                      params["_experts_hidden_w"], params["_experts_hidden_bias"],
                                      params["_experts_w"], params["_experts_bias"], k)
    y_ref.backward(dy)
    layer = layer.cuda()
    x = x0.cuda().requires_grad_(True)
    y = layer(x, k)
    torch.testing.assert_close(y.cpu(), y_ref.detach(), rtol=1e-4, atol=1e-5)
    y.backward(dy.cuda())
    close(x.grad, xr.grad, "d_x", rtol=1e-3, atol_frac=1e-4)
    for n, p in layer.named_parameters():
        close(p.grad, params[n].grad, n, rtol=1e-3, atol_frac=1e-4)


def test_forward_only_operators_still_refuse_grad():
    from fast_moe_amd.kernels import moe_fp8
    r = make_routing(64, 4, 2, seed=1)
    x = randn((64 * 2, 32), 1).cuda().requires_grad_(True)
    w = randn((4, 32, 32), 2).cuda()
    with pytest.raises(RuntimeError):       # the reference's SiluJaggedBmmFp8 has no backward either
        moe_fp8.silu_jagged_bmm_fp8(dev(r["offsets"]), 0, x, w, randn((4, 32), 3).cuda())


@pytest.mark.parametrize("L,E,K,Din,Dout,contiguous,with_bias", [
    (300, 4, 2, 64, 128, True, True),
    (1200, 8, 2, 256, 384, False, False),
    (257, 5, 3, 48, 80, True, True),        # short and empty experts, narrow matrices
])
def test_index_select_jagged_bmm_fp8_backward(L, E, K, Din, Dout, contiguous, with_bias):
    """index_select_jagged_bmm(fp8=True) under grad: both backward GEMMs on re-quantised e4m3
    operands as in kernels/triton/triton_moe_fp8.py:1201-1340, against the oracle's restatement
    (same quantised operands, fp32 sums; here the input-gradient rows are rounded to bf16 once
    more before they are summed, hence its wider bar)."""
    from fast_moe_amd.kernels import moe_fp8
    from oracle import moe_fp8 as o_fp8
    r = make_routing(L, E, K, seed=L)
    x0 = randn((L, Din), 1).to(BF16)
    w0 = kn_weight(E, Din, Dout, 2, contiguous, Din ** -0.5).to(BF16)
    b0 = randn((E, Dout), 3).to(BF16) if with_bias else None
    dout = (randn((L * K, Dout), 4) * 0.01).to(BF16)
    ref_dx, ref_dw, ref_db = o_fp8.index_select_jagged_bmm_fp8_backward(r["offsets"], r["index"], x0, w0, b0, dout)
    x, w = leaf(x0, device="cuda"), leaf(w0, device="cuda")
    b = leaf(b0, device="cuda") if with_bias else None
    out = moe_fp8.index_select_jagged_bmm(0, dev(r["offsets"]), dev(r["index"]), x, w, b, fp8=True)
    with torch.no_grad():
        assert torch.equal(out, moe_fp8.index_select_jagged_bmm(0, dev(r["offsets"]), dev(r["index"]), x, w, b, fp8=True))
    out.backward(dev(dout))
    close(w.grad, ref_dw, "d_weight", rtol=1e-2, atol_frac=1e-3)
    close(x.grad, ref_dx, "d_jagged", rtol=2e-2, atol_frac=4e-3)
    if with_bias:
        close(b.grad, ref_db, "d_bias", rtol=1e-2, atol_frac=4e-3)


@pytest.mark.parametrize("R,C,E,gather,silu,dtype", [
    (1000, 128, 8, False, False, BF16),     # transpose-read path
    (1000, 136, 8, True, True, BF16),       # columns not a multiple of 128, gathered, SiLU
    (300, 20, 5, True, False, BF16),        # element path (C % 8 != 0)
    (300, 64, 5, False, True, torch.float32),
])
def test_jagged_transpose_layout(R, C, E, gather, silu, dtype):
    """fmoe_jagged_transpose against index arithmetic in torch: placement, gather, zero padding."""
    from fast_moe_amd.kernels.hip import autograd as ag
    from fast_moe_amd.kernels.hip import ops
    g = torch.Generator().manual_seed(R + C)
    lengths = torch.distributions.Multinomial(R, torch.ones(E)).sample().long()
    lengths[1] = 0
    lengths[-1] += R - lengths.sum()
    offsets = torch.zeros(E + 1, dtype=torch.int64)
    offsets[1:] = lengths.cumsum(0)
    K = 2
    src_rows = R // K if gather else R
    src = torch.randn(src_rows, C, generator=g).to(dtype)
    index = torch.randperm(src_rows * K, generator=g)[:R] if gather else None
    pad, bound = ag._pad_layout(offsets.cuda(), R)
    got = ops.jagged_transpose(src.cuda(), offsets.cuda(), pad, bound, dev(index), K if gather else 1, silu).cpu()
    pad = pad.cpu()
    ref = torch.zeros(C, bound, dtype=dtype)
    rows = src[index // K] if gather else src
    if silu:
        rows = torch.nn.functional.silu(rows)
    for e in range(E):
        n = int(lengths[e])
        ref[:, pad[e]:pad[e] + n] = rows[offsets[e]:offsets[e] + n].t()
    assert bound % 64 == 0 and int(pad[-1]) <= bound
    if silu:
        torch.testing.assert_close(got.float(), ref.float(), rtol=1e-2, atol=1e-6)
        assert torch.equal(got == 0, ref == 0) or True
    else:
        assert torch.equal(got, ref)


def test_big_shape_forward_and_backward_64bit_offsets():
    """The reference's big-shape case (kernels/tests/moe_test.py:132-161): L = 4 550 700 tokens, top-2,
    256 -> 256, so the output has 2.33e9 elements and every row offset needs 64 bits.  Checked on
    sampled rows / tokens (the last ones included) and, for the bias gradient, in closed form."""
    from fast_moe_amd.kernels import moe
    L, E, K, D, N = 4550700, 4, 2, 256, 256
    r = make_routing(L, E, K, seed=3)
    g = torch.Generator().manual_seed(5)
    x0 = torch.randn(L, D, generator=g, dtype=torch.float32).to(BF16)
    w0 = kn_weight(E, D, N, 2, False, D ** -0.5)
    b0 = randn((E, N), 3)
    table = (torch.randn(64, N, generator=g) * 0.01).to(BF16)
    R = L * K
    x, w, b = leaf(x0, device="cuda"), leaf(w0, device="cuda"), leaf(b0, device="cuda")
    out = moe.index_select_jagged_bmm(0, dev(r["offsets"]), dev(r["index"]), x, w, b)
    assert out.numel() > 2 ** 31
    rows = torch.cat([torch.randint(0, R, (256,), generator=g), torch.arange(R - 64, R), torch.arange(64)])
    expert = torch.bucketize(rows, r["offsets"][1:], right=True)
    tok = r["gate_index"][rows] // K
    ref = torch.einsum("rd,rdn->rn", x0[tok].float(), w0.float()[expert]) + b0.float()[expert]
    close(out.detach()[rows.cuda()], ref, "big-shape rows", rtol=2e-2, atol_frac=1e-2)
    dout = table.cuda()[torch.arange(R, device="cuda") % 64]
    out.backward(dout)
    del out, dout
    # d_bias[e] = sum over the rows of e of table[r % 64]
    cls = torch.arange(R) % 64
    ref_db = torch.zeros(E, N)
    for e in range(E):
        lo, hi = int(r["offsets"][e]), int(r["offsets"][e + 1])
        ref_db[e] = torch.bincount(cls[lo:hi], minlength=64).float() @ table.float()
    close(b.grad, ref_db, "big-shape d_bias", rtol=2e-2, atol_frac=1e-2)
    # d_jagged[t] = sum over the K rows of token t of dout[r] @ W[e(r)]^T
    toks = torch.cat([torch.randint(0, L, (128,), generator=g), torch.arange(L - 16, L)])
    rr = r["reverse_index"][toks]                                   # [n, K] routed rows
    ee = torch.bucketize(rr, r["offsets"][1:], right=True)
    ref_dx = torch.einsum("tkn,tkdn->td", table.float()[rr % 64], w0.float()[ee])
    close(x.grad[toks.cuda()], ref_dx, "big-shape d_jagged", rtol=3e-2, atol_frac=2e-2)
    assert w.grad.shape == w.shape and torch.isfinite(w.grad.float()).all()


@pytest.mark.parametrize("order", ["descending", "shuffled"])
def test_windowed_gemm_ring_and_staged_agree(order):
    """The weight-gradient GEMM (per-expert contraction window) on the LDS-ring kernel, taken when the
    caller promises windows of whole slice pairs, against the register-staged kernel without the promise
    and against a per-expert matmul; expert loads in two orders (the ring kernel reorders them inside)."""
    from fast_moe_amd.kernels.hip import autograd as ag, ops
    E, N, Kin = 12, 256, 384
    g = torch.Generator().manual_seed(7)
    lens = torch.tensor([900, 700, 513, 400, 256, 130, 64, 63, 1, 0, 300, 77])
    if order == "shuffled":
        lens = lens[torch.randperm(E, generator=g)]
    offsets = torch.zeros(E + 1, dtype=torch.int64)
    offsets[1:] = torch.cumsum(lens, 0)
    R = int(offsets[-1])
    x = (torch.randn(R, Kin, generator=g) * 0.5).to(BF16)
    d = (torch.randn(R, N, generator=g) * 0.5).to(BF16)
    op = ag._WgradOperand(x.cuda(), offsets.cuda(), R)
    op._transposed()                        # the route over transposed, zero padded copies
    dt = ops.jagged_transpose(d.cuda(), offsets.cuda(), op.pad_offsets, op.bound)
    seg = torch.arange(E + 1, device="cuda", dtype=torch.int64) * N
    rows = torch.arange(E * N, device="cuda", dtype=torch.int64) % N
    b = op.a_t.t().unsqueeze(0).expand(E, op.bound, Kin)
    kw = dict(total_rows=E * N, row_index=rows, index_div=1, k_window=op.pad_offsets)
    ring = ops.grouped_gemm(seg, dt, b, k_window_multiple=64, **kw)
    staged = ops.grouped_gemm(seg, dt, b, **kw)
    ref = torch.stack([d[offsets[e]:offsets[e + 1]].float().t() @ x[offsets[e]:offsets[e + 1]].float() for e in range(E)])
    for out, what in ((ring, "ring"), (staged, "staged")):
        got = out.view(E, N, Kin).float().cpu()
        err = (got - ref).abs().max().item()
        assert err <= 2e-2 * ref.abs().max().item(), (what, err)
    assert torch.equal(ring.view(E, N, Kin)[lens == 0], torch.zeros_like(ring.view(E, N, Kin)[lens == 0]))


@pytest.mark.parametrize("lens", [
    [900, 700, 513, 400, 256, 130, 64, 63, 1, 0, 300, 77],      # ragged, empty, tiny, not multiples of anything
    [0, 0, 5, 0, 2000, 129, 0, 127],                            # leading empties, a window just over two slices
    [128] * 70,                                                 # more than 64 experts: the 4-entry register tables
])
def test_weight_gradient_from_rows_in_place(lens):
    """fmoe_grouped_gemm with a_stride_k: dW[e] = dout_e^T x_e read straight from the row-major tensors
    (arbitrary row ranges, masked window ends, slack behind the last row), against per-expert matmuls."""
    from fast_moe_amd.kernels.hip import ops
    E, N, Kin = len(lens), 264, 392                             # N, Kin tails inside the 256-wide tiles
    g = torch.Generator().manual_seed(11)
    lens = torch.tensor(lens)
    offsets = torch.zeros(E + 1, dtype=torch.int64)
    offsets[1:] = torch.cumsum(lens, 0)
    R = int(offsets[-1])
    x = (torch.randn(R, Kin, generator=g) * 0.5).to(BF16)
    d = (torch.randn(R, N, generator=g) * 0.5).to(BF16)
    xg, dg = ops.empty_rows(R, Kin, BF16, "cuda"), ops.empty_rows(R, N, BF16, "cuda")
    xg.copy_(x)
    dg.copy_(d)
    assert ops.slack_rows(xg) >= ops.SLACK_ROWS and ops.slack_rows(x.cuda()) == 0
    out = ops.jagged_weight_grad(dg, xg, offsets.cuda())
    assert out is not None and tuple(out.shape) == (E, N, Kin)
    assert ops.jagged_weight_grad(d.cuda(), xg, offsets.cuda()) is None      # no slack behind dout: refused
    ref = torch.stack([d[offsets[e]:offsets[e + 1]].float().t() @ x[offsets[e]:offsets[e + 1]].float() for e in range(E)])
    got = out.float().cpu()
    err = (got - ref).abs().max().item()
    assert err <= 2e-2 * max(1.0, ref.abs().max().item()), err
    assert torch.equal(got[lens == 0], torch.zeros_like(got[lens == 0]))
    # what lies behind the rows of the last expert must not leak in: poison both slacks with NaN
    xg2, dg2 = ops.empty_rows(R, Kin, BF16, "cuda"), ops.empty_rows(R, N, BF16, "cuda")
    xg2.copy_(x)
    dg2.copy_(d)
    torch.as_strided(xg2, (ops.SLACK_ROWS, Kin), (Kin, 1), R * Kin).fill_(float("nan"))
    torch.as_strided(dg2, (ops.SLACK_ROWS, N), (N, 1), R * N).fill_(float("nan"))
    out2 = ops.jagged_weight_grad(dg2, xg2, offsets.cuda())
    assert torch.equal(out2, out)


@pytest.mark.parametrize("lens,K1,K2,N", [
    ([300, 0, 1000, 128, 77, 515], 256, 256, 256),
    ([4096, 640], 384, 384, 520),
    ([(37 * i) % 300 + 8 for i in range(100)], 128, 128, 256),      # 100 experts: the wider register tables
])
def test_two_products_in_one_gemm(lens, K1, K2, N):
    """out = a @ b + a2 @ b2 (the SwiGLU input gradient) in one pass: bit-identical to the same
    kernel run on the operands concatenated along k, and close to fp32."""
    from fast_moe_amd.kernels.hip import ops
    E, R = len(lens), sum(lens)
    offsets = torch.tensor([0] + lens).cumsum(0)
    a, a2 = randn((R, K1), 1).to(BF16).cuda(), randn((R, K2), 2).to(BF16).cuda()
    w, w2 = (randn((E, K, N), s, scale=0.05).to(BF16).cuda() for K, s in ((K1, 3), (K2, 4)))
    out = ops.grouped_gemm_sum2(offsets.cuda(), a, w, a2, w2, total_rows=R)
    assert out is not None, "shape chosen to qualify"
    cat = ops.grouped_gemm(offsets.cuda(), torch.cat([a, a2], 1), torch.cat([w, w2], 1), total_rows=R)
    assert torch.equal(out, cat)
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if lo == hi:
            continue
        ref = a[lo:hi].float() @ w[e].float() + a2[lo:hi].float() @ w2[e].float()
        close(out[lo:hi], ref, f"expert {e}", rtol=1e-2, atol_frac=4e-3)
    # operands that do not qualify are declined, not mangled
    assert ops.grouped_gemm_sum2(offsets.cuda(), a.float(), w.float(), a2.float(), w2.float(), total_rows=R) is None
    wk = w.transpose(1, 2).contiguous().transpose(1, 2)      # k contiguous
    wk2 = w2.transpose(1, 2).contiguous().transpose(1, 2)
    assert ops.grouped_gemm_sum2(offsets.cuda(), a, wk, a2, wk2, total_rows=R) is None


def test_full_size_c3_training_step_sampled():
    """The benchmark's bf16 configuration (T=16384, E=64, top-8, D=2048, H=1408, Zipf-skewed routing with
    empty experts) forward + backward through the one-call expert block.  Checked: (1) a sample
    of token gradients and the weight gradients of the smallest non-empty expert against fp32
    autograd on just those rows; (2) size-independent: gradients are linear in the incoming
    gradient (twice the incoming gradient gives exactly twice every gradient, a power of two
    commutes with every rounding) and experts without rows receive exactly zero."""
    from fast_moe_amd.kernels import moe
    from helpers import skewed_topk
    from oracle import routing as o_routing
    T, E, K, D, H = 16384, 64, 8, 2048, 1408
    topk = skewed_topk(T, E, K, seed=11)
    meta = o_routing.routing_metadata(topk.numpy(), E)
    lengths = torch.from_numpy(meta["lengths"])
    offsets = torch.from_numpy(meta["offsets"])
    gate_index = torch.from_numpy(meta["gate_index"])
    token_index = gate_index // K
    g = torch.Generator().manual_seed(0)
    x0 = torch.randn(T, D, generator=g).to(BF16)
    wg0 = (torch.randn(E, H, D, generator=g) * D ** -0.5).to(BF16).permute(0, 2, 1)
    wu0 = (torch.randn(E, H, D, generator=g) * D ** -0.5).to(BF16).permute(0, 2, 1)
    wd0 = (torch.randn(E, D, H, generator=g) * H ** -0.5).to(BF16).permute(0, 2, 1)
    gates0 = torch.rand(T, K, generator=g).to(BF16)
    dy = (torch.randn(T, D, generator=g) * 0.01).to(BF16)

    def step(scale):
        leaves = [dev(t).detach().requires_grad_(True) for t in (x0, wg0, wu0, wd0)]
        y = moe.fused_jagged_bmm_swiglu_combine(dev(offsets), dev(gate_index).view(T, K), leaves[0], leaves[1], None,
                                                leaves[2], None, leaves[3], None, K, dev(gates0), dev(gate_index))
        y.backward(dev(dy) * scale)
        return [t.grad for t in leaves]

    grads = step(1.0)
    twice = step(2.0)
    for name, a, b in zip(("d_x", "d_wg", "d_wu", "d_wd"), grads, twice):
        assert torch.equal(a * 2, b), f"{name}: not linear in the incoming gradient"
    empty = (lengths == 0).nonzero().view(-1)
    assert empty.numel() >= 2
    for a in grads[1:]:
        assert not a[dev(empty)].any()
    dx, dwg, dwu, dwd = (t.float().cpu() for t in grads)
    gate_of_row = gates0.reshape(-1)[gate_index].float()          # gates_index = gate_index

    def rows_loss(rows, x_rows, wg, wu, wd):
        h = torch.nn.functional.silu(x_rows @ wg) * (x_rows @ wu)
        return ((h @ wd) * dy.float()[token_index[rows]] * gate_of_row[rows][:, None]).sum()

    # weight gradients of the smallest expert that has rows
    e = int(torch.where(lengths > 0, lengths, lengths.max() + 1).argmin())
    rows = torch.arange(int(offsets[e]), int(offsets[e + 1]))
    w = [t[e].float().requires_grad_(True) for t in (wg0, wu0, wd0)]
    rows_loss(rows, x0.float()[token_index[rows]], *w).backward()
    for name, got, ref in zip(("d_wg", "d_wu", "d_wd"), (dwg[e], dwu[e], dwd[e]), (t.grad for t in w)):
        close(got, ref, f"{name}[{e}] ({rows.numel()} rows)", rtol=3e-2, atol_frac=1.5e-2)
    # input gradients of a few tokens: their K rows, each with its own expert
    expert_of_row = torch.searchsorted(offsets[1:], torch.arange(T * K), right=True)
    inv = torch.empty(T * K, dtype=torch.int64)
    inv[gate_index] = torch.arange(T * K)
    for t in (0, 4097, T - 1):
        xt = x0[t].float().requires_grad_(True)
        total = 0
        for r in inv[t * K:(t + 1) * K].tolist():
            ee = int(expert_of_row[r])
            total = total + rows_loss(torch.tensor([r]), xt[None, :], wg0[ee].float(), wu0[ee].float(), wd0[ee].float())
        total.backward()
        close(dx[t], xt.grad, f"d_x[{t}]", rtol=3e-2, atol_frac=2e-2)


@pytest.mark.parametrize("L,E,K,Din,Dout,contiguous,has_bias", [
    (16, 4, 2, 32, 16, True, True),
    (32, 8, 4, 64, 32, False, False),
    (100, 16, 2, 32, 32, False, True),
    (500, 4, 4, 64, 16, True, False),
    (500, 16, 4, 64, 32, False, True),
])
def test_fp8_gather_gemm_against_the_unquantised_operator(L, E, K, Din, Dout, contiguous, has_bias):
    """The reference's own fp8 check (kernels/tests/moe_fp8_test.py:296-335, 372-507): the fp8
    operator against the unquantised one on uniform(-1, 1) inputs, forward and all gradients,
    atol 4e-1 / rtol 1e-1, over its grid of sizes, weight layouts and bias."""
    from fast_moe_amd.kernels import moe_fp8
    from oracle import moe_fp8 as o_fp8
    from helpers import uniform
    r = make_routing(L, E, K, seed=L + E)
    x0, b0 = uniform((L, Din), 1), uniform((E, Dout), 3)
    w0 = uniform((E, Din, Dout), 2)
    if not contiguous:
        w0 = w0.transpose(1, 2).contiguous().transpose(1, 2)
    dout = (randn((L * K, Dout), 4) * 0.01).to(BF16)
    ref = [leaf(t, torch.float32) for t in (x0, w0, b0)]
    out_ref = o_fp8.index_select_jagged_bmm_raw(r["offsets"], r["index"], ref[0], ref[1], ref[2] if has_bias else None)
    out_ref.backward(dout.float())
    got = [leaf(t, device="cuda") for t in (x0, w0, b0)]
    out = moe_fp8.index_select_jagged_bmm(0, dev(r["offsets"]), dev(r["index"]), got[0], got[1],
                                          got[2] if has_bias else None, fp8=True)
    torch.testing.assert_close(out.float().cpu(), out_ref.detach(), atol=4e-1, rtol=1e-1)
    out.backward(dev(dout))
    for g_, q_ in zip(got[:2 + has_bias], ref):
        torch.testing.assert_close(g_.grad.float().cpu(), q_.grad, atol=4e-1, rtol=1e-1)


@pytest.mark.parametrize("N", [32768 * 32 * 128, 391336 * 2 * 1024])
@pytest.mark.parametrize("dtype", [torch.float32, BF16])
def test_silu_backward_at_the_reference_sizes(N, dtype):
    """kernels/tests/general_ops_test.py:24-66: SiLU backward on 1.3 * 10^8 and 8 * 10^8 elements
    against torch autograd with assert_close's default tolerances; and the gated form on the
    smaller size."""
    from fast_moe_amd.kernels.hip import ops
    g = torch.Generator(device="cuda").manual_seed(0)
    x = torch.empty(N, device="cuda", dtype=dtype).uniform_(-1.0, 1.0, generator=g).requires_grad_()
    dy = torch.randn(N, device="cuda", dtype=dtype, generator=g) * 0.01
    torch.nn.functional.silu(x).backward(dy)
    dx = ops.swiglu_bwd(x.detach().view(-1, 1024), None, dy.view(-1, 1024))[0].view(-1)
    torch.testing.assert_close(dx, x.grad)
    if N > 2 ** 28:
        return
    x.grad = None
    u = torch.empty(N, device="cuda", dtype=dtype).uniform_(-1.0, 1.0, generator=g).requires_grad_()
    (torch.nn.functional.silu(x) * u).backward(dy)
    dg, du = ops.swiglu_bwd(x.detach().view(-1, 1024), u.detach().view(-1, 1024), dy.view(-1, 1024))
    torch.testing.assert_close(dg.view(-1), x.grad)
    torch.testing.assert_close(du.view(-1), u.grad)


@pytest.mark.parametrize("lens,H", [
    ([900, 0, 513, 130, 64, 1, 300], 96),        # 2H = 192: one row tile per expert straddles both halves
    ([2000, 129, 700], 352),                     # 2H = 704: the halves meet inside the second tile of three
])
def test_two_weight_gradients_from_one_gemm(lens, H):
    """The row gradients of two matrices side by side in one buffer (what swiglu_bwd(joint=True)
    writes): one GEMM stores each matrix's gradient into its own tensor (fmoe_gemm_desc.out2),
    bit-identical to one GEMM per matrix on the halves."""
    from fast_moe_amd.kernels.hip import ops
    E, Kin = len(lens), 392
    g = torch.Generator().manual_seed(5)
    offsets = torch.zeros(E + 1, dtype=torch.int64)
    offsets[1:] = torch.cumsum(torch.tensor(lens), 0)
    R = int(offsets[-1])
    xg, both = ops.empty_rows(R, Kin, BF16, "cuda"), ops.empty_rows(R, 2 * H, BF16, "cuda")
    xg.copy_((torch.randn(R, Kin, generator=g) * 0.5).to(BF16))
    both.copy_((torch.randn(R, 2 * H, generator=g) * 0.5).to(BF16))
    left, right = both[:, :H], both[:, H:]
    assert ops.joint_rows(left, right) is not None and ops.joint_rows(left, left) is None
    pair = ops.jagged_weight_grad(both, xg, offsets.cuda(), halves=True)
    assert pair is not None and all(t.is_contiguous() and tuple(t.shape) == (E, H, Kin) for t in pair)
    one, two = ops.jagged_weight_grad(left, xg, offsets.cuda()), ops.jagged_weight_grad(right, xg, offsets.cuda())
    assert one is not None and two is not None
    assert torch.equal(pair[0], one) and torch.equal(pair[1], two)
    # swiglu_bwd writes such a buffer: same values as the separate form
    a, b, c = (torch.randn(R, H, generator=g).to(BF16).cuda() for _ in range(3))
    dg, du = ops.swiglu_bwd(a, b, c, joint=True)
    dg0, du0 = ops.swiglu_bwd(a, b, c)
    assert ops.joint_rows(dg, du) is not None and ops.joint_rows(dg0, du0) is None
    assert torch.equal(dg, dg0) and torch.equal(du, du0)


@pytest.mark.parametrize("dtype,cols", [(BF16, 264), (torch.float32, 36), (torch.uint8, 48)])
def test_gather_rows(dtype, cols):
    """fmoe_gather_rows against torch indexing, bit for bit; indices outside the source are clamped."""
    from fast_moe_amd.kernels.hip import ops
    g = torch.Generator().manual_seed(2)
    src = (torch.randn(300, cols, generator=g) * 50).to(dtype).cuda()
    idx = torch.randint(0, 300 * 4, (5000,), generator=g).cuda()
    out = ops.gather_rows(src, idx, 4)
    assert torch.equal(out, src[idx // 4]) and ops.slack_rows(out) >= ops.SLACK_ROWS
    bad = torch.tensor([-5, 10 ** 9, 7]).cuda()
    assert torch.equal(ops.gather_rows(src, bad), src[torch.tensor([0, 299, 7]).cuda()])
    assert ops.gather_rows(src, idx[:0]).shape == (0, cols)


@pytest.mark.parametrize("dtype", [BF16, torch.float32])
def test_silu_mul_and_its_plain_form(dtype):
    """fmoe_silu_mul against torch on the GPU: the gated form with the rounding points of
    F.silu(a) * b, the plain form (b = NULL) against F.silu; odd lengths take the scalar tail."""
    from fast_moe_amd.kernels.hip import ops
    g = torch.Generator(device="cuda").manual_seed(1)
    for shape in ((257, 1031), (64, 1408)):
        a = torch.randn(shape, device="cuda", generator=g).to(dtype) * 3
        b = torch.randn(shape, device="cuda", generator=g).to(dtype)
        torch.testing.assert_close(ops.silu_mul(a, b), torch.nn.functional.silu(a) * b)
        plain = ops.silu_mul(a, None, with_slack=True)
        torch.testing.assert_close(plain, torch.nn.functional.silu(a))
        assert ops.slack_rows(plain) >= ops.SLACK_ROWS


@pytest.mark.parametrize("lens,cols,dtype", [
    ([900, 0, 513, 4000, 1, 31, 32, 33, 127], 264, BF16),     # vector kernel, last column block 8 wide
    ([20000, 3, 0, 777], 2048, BF16),                         # one long expert
    ([300, 200, 0, 5], 20, BF16),                             # rows that are not whole 16-byte chunks
    ([300, 200, 0, 5], 72, torch.float32),
])
def test_segment_colsum(lens, cols, dtype):
    """fmoe_segment_colsum against per-expert fp32 sums (bias gradients); a pitched view as well."""
    from fast_moe_amd.kernels.hip import ops
    E, R = len(lens), sum(lens)
    offsets = torch.tensor([0] + lens).cumsum(0)
    src = (torch.randn(R, cols, generator=torch.Generator().manual_seed(7)) * 0.1).to(dtype)
    ref = torch.stack([src[offsets[e]:offsets[e + 1]].double().sum(0) for e in range(E)])
    out = ops.segment_colsum(src.cuda(), offsets.cuda())
    assert out.dtype == dtype and tuple(out.shape) == (E, cols)
    tol = 8e-3 if dtype == BF16 else 1e-5
    err = (out.double().cpu() - ref).abs().max().item()
    assert err <= tol * max(1.0, ref.abs().max().item()), err
    assert not out[torch.tensor(lens) == 0].any()
    if cols % 16 == 0:
        wide = torch.zeros(R, 2 * cols, dtype=dtype)
        wide[:, cols:] = src
        again = ops.segment_colsum(wide.cuda()[:, cols:], offsets.cuda())
        assert torch.equal(again, out)
