"""GPU parity: jagged GEMM operators (bf16 and fp8) against the oracle, through the
operator API (and therefore the C ABI)."""
import itertools

import numpy as np
import pytest
import torch

from oracle import moe as o_moe
from oracle import moe_fp8 as o_fp8
from tests.helpers import BF16, assert_bf16_close, dev, make_routing, randn, skewed_topk, uniform
from oracle import routing as o_routing

pytestmark = pytest.mark.gpu

# kernels/tests/moe_test.py:35-84: default assert_close for bf16 is rtol 1.6e-2, atol 1e-5
REF_RTOL, REF_ATOL = 1.6e-2, 1e-5


def weights(E, K, N, seed, contiguous=True, scale=None):
    w = uniform((E, K, N), seed) if scale is None else randn((E, K, N), seed, scale=scale)
    if not contiguous:          # [E, K, N] view of [E, N, K] storage (moe_test.py:223-239)
        w = w.transpose(1, 2).contiguous().transpose(1, 2)
    return w


GRID = [(L, E, K, Din, Dout) for L, E, K, Din, Dout in itertools.product(
    [16, 100, 500], [4, 16], [2, 4], [12, 32, 64], [32, 128])]


@pytest.mark.parametrize("L,E,K,Din,Dout", GRID[::3])
@pytest.mark.parametrize("contiguous", [True, False])
@pytest.mark.parametrize("has_bias", [True, False])
def test_index_select_jagged_bmm_reference_grid(L, E, K, Din, Dout, contiguous, has_bias):
    from fast_moe_amd.kernels import moe
    print(f"bmm L={L} E={E} K={K} Din={Din} Dout={Dout} contiguous={contiguous} bias={has_bias}", flush=True)
    r = make_routing(L, E, K, seed=L + E)
    x = uniform((L, Din), 1)
    w = weights(E, Din, Dout, 2, contiguous)
    b = uniform((E, Dout), 3) if has_bias else None
    ref = o_moe.index_select_jagged_bmm(r["offsets"], r["index"], x.float(), w.float(),
                                        None if b is None else b.float())
    with torch.no_grad():
        out = moe.index_select_jagged_bmm(int(r["lengths"].max()), dev(r["offsets"]), dev(r["index"]), dev(x),
                                          dev(w), dev(b))
    assert out.dtype == BF16 and tuple(out.shape) == (L * K, Dout)
    torch.testing.assert_close(out.cpu(), ref.to(BF16), rtol=REF_RTOL, atol=REF_ATOL)


@pytest.mark.parametrize("L,E,K,Din,Dout,contiguous", [
    (2048, 8, 2, 256, 512, False),      # tall tiles, K-contiguous weights (the layer's layout)
    (2048, 8, 2, 256, 512, True),       # tall tiles, N-contiguous weights
    (1500, 4, 2, 200, 136, False),      # ragged rows, K tail, N tail
    (4096, 64, 8, 128, 96, False),
    (300, 128, 8, 64, 256, False),      # short tiles
])
def test_index_select_jagged_bmm_larger(L, E, K, Din, Dout, contiguous):
    from fast_moe_amd.kernels import moe
    r = make_routing(L, E, K, seed=L)
    x = randn((L, Din), 1)
    w = weights(E, Din, Dout, 2, contiguous, scale=Din ** -0.5)
    b = randn((E, Dout), 3)
    ref = o_moe.index_select_jagged_bmm(r["offsets"], r["index"], x.float(), w.float(), b.float())
    with torch.no_grad():
        out = moe.index_select_jagged_bmm(0, dev(r["offsets"]), dev(r["index"]), dev(x), dev(w), dev(b))
    assert_bf16_close(out, ref, rtol=1e-2, atol=1e-2, what="index_select_jagged_bmm")


def test_skewed_and_empty_experts():
    from fast_moe_amd.kernels import moe
    T, E, K, D, H = 4096, 64, 8, 128, 192
    topk = skewed_topk(T, E, K, seed=3)
    meta = o_routing.routing_metadata(topk.numpy(), E)
    assert (meta["lengths"] == 0).sum() >= 2 and meta["lengths"].max() > 8 * meta["lengths"][meta["lengths"] > 0].min()
    offsets = torch.from_numpy(meta["offsets"])
    index = torch.from_numpy(meta["gate_index"]).view(-1, K)
    x = randn((T, D), 1)
    wg = weights(E, D, H, 2, False, scale=D ** -0.5)
    wu = weights(E, D, H, 3, False, scale=D ** -0.5)
    ref = o_moe.index_select_jagged_bmm_swiglu(offsets, index, x.float(), wg.float(), None, wu.float(), None)
    with torch.no_grad():
        out = moe.index_select_jagged_bmm_swiglu(0, dev(offsets), dev(index), dev(x), dev(wg), None, dev(wu), None)
    # product of two bf16-rounded GEMM results: the reference's own bf16 rtol (1.6e-2)
    assert_bf16_close(out, ref, rtol=1.6e-2, atol=1e-2, what="swiglu, skewed")


@pytest.mark.parametrize("L,E,K,Din,Dout,bias,contiguous", [
    (100, 8, 2, 32, 64, True, True), (500, 4, 4, 64, 64, False, False), (2048, 8, 2, 128, 256, True, False),
    (64, 16, 2, 24, 40, True, True)])
def test_swiglu_and_gating(L, E, K, Din, Dout, bias, contiguous):
    from fast_moe_amd.kernels import moe
    r = make_routing(L, E, K, seed=L + 1)
    x, x2 = uniform((L, Din), 1), uniform((L, Din), 4)
    w, wp = weights(E, Din, Dout, 2, contiguous), weights(E, Din, Dout, 5, contiguous)
    b = uniform((E, Dout), 3) if bias else None
    bp = uniform((E, Dout), 6) if bias else None
    f = lambda t: None if t is None else t.float()
    ref = o_moe.index_select_jagged_bmm_swiglu(r["offsets"], r["index"], f(x), f(w), f(b), f(wp), f(bp))
    with torch.no_grad():
        out = moe.index_select_jagged_bmm_swiglu(0, dev(r["offsets"]), dev(r["index"]), dev(x), dev(w), dev(b),
                                                 dev(wp), dev(bp))
        xa = dev(x)
        out_same = moe.index_select_jagged_gating_bmm(0, dev(r["offsets"]), dev(r["index"]), xa, xa, dev(w),
                                                      dev(b), dev(wp), dev(bp))
        out_two = moe.index_select_jagged_gating_bmm(0, dev(r["offsets"]), dev(r["index"]), dev(x), dev(x2),
                                                     dev(w), dev(b), dev(wp), dev(bp))
    # tolerance of kernels/tests/moe_test.py:729-949 for bf16 products of two GEMMs
    assert_bf16_close(out, ref, rtol=1.6e-2, atol=2e-2, what="swiglu")
    assert torch.equal(out, out_same)
    ref2 = o_moe.index_select_jagged_gating_bmm(r["offsets"], r["index"], f(x), f(x2), f(w), f(wp), f(b), f(bp))
    assert_bf16_close(out_two, ref2, rtol=1.6e-2, atol=2e-2, what="gating")


@pytest.mark.parametrize("L,E,K,Din,Dout,bias,contiguous", [
    (8192, 8, 2, 512, 384, True, False),       # LDS-ring kernel
    (8192, 8, 2, 512, 384, False, True),       # the same with [E, K, N]-contiguous weights read in place
    (4096, 16, 4, 256, 200, True, False),      # ring, N tail: 200 columns of a 256-column tile
    (600, 4, 2, 128, 136, True, False),        # register-staged kernel, tall tile
    (64, 16, 2, 128, 64, False, False),        # register-staged kernel, 64-row tile
    (100, 8, 2, 24, 40, True, True),           # element loads and element stores
    (300, 4, 2, 64, 36, True, False),          # gate rows that start off 8-byte boundaries (N = 36)
])
def test_two_input_gating_multiplies_in_the_second_gemm(L, E, K, Din, Dout, bias, contiguous):
    """index_select_jagged_gating_bmm with two different inputs: the second GEMM's epilogue multiplies
    by the SiLU of the first one's result (no element-wise pass, no second [rows, N] round trip).
    Against the oracle, and against the three-launch composition (which differs by the SiLU's last
    fp32 bits before its bf16 rounding: the element-wise kernel divides, the epilogue uses the
    hardware reciprocal)."""
    from fast_moe_amd.kernels import moe
    from fast_moe_amd.kernels.hip import ops
    r = make_routing(L, E, K, seed=L + 3)
    x, x2 = randn((L, Din), 1), randn((L, Din), 4)
    w, wp = (weights(E, Din, Dout, s, contiguous, scale=Din ** -0.5) for s in (2, 5))
    b = randn((E, Dout), 3) if bias else None
    bp = randn((E, Dout), 6) if bias else None
    f = lambda t: None if t is None else t.float()
    ref = o_moe.index_select_jagged_gating_bmm(r["offsets"], r["index"], f(x), f(x2), f(w), f(wp), f(b), f(bp))
    off, idx = dev(r["offsets"]), dev(r["index"])
    calls = []
    real = ops.silu_mul
    ops.silu_mul = lambda *a, **k: calls.append(1) or real(*a, **k)
    try:
        with torch.no_grad():
            out = moe.index_select_jagged_gating_bmm(0, off, idx, dev(x), dev(x2), dev(w), dev(b), dev(wp), dev(bp))
    finally:
        ops.silu_mul = real
    assert not calls, "the element-wise pass ran"
    assert_bf16_close(out, ref, rtol=1.6e-2, atol=2e-2, what="gating, two inputs")
    kw = dict(total_rows=L * K, row_index=idx, index_div=K)
    alpha = ops.grouped_gemm(off, dev(x), dev(w), bias=dev(b), **kw)
    beta = ops.grouped_gemm(off, dev(x2), dev(wp), bias=dev(bp), **kw)
    three = ops.silu_mul(alpha, beta)
    diff = (out.view(torch.int16).int() - three.view(torch.int16).int()).abs()
    # (one bf16 step of the rounded SiLU is up to two steps of the rounded product)
    assert int(diff.max()) <= 2 and float((diff != 0).float().mean()) < 2e-3, (int(diff.max()), float((diff != 0).float().mean()))
    # a gate tensor that is a column slice of a wider one (row stride > N)
    wide = torch.zeros((L * K, Dout + 12), dtype=BF16, device="cuda")
    wide[:, 4:4 + Dout] = alpha
    sliced = ops.grouped_gemm(off, dev(x2), dev(wp), bias=dev(bp), epilogue=3, gate=wide[:, 4:4 + Dout], **kw)
    assert torch.equal(sliced, out)


def test_3d_variant():
    from fast_moe_amd.kernels import moe
    L, E, K, Din, Dout = 200, 4, 2, 8, 4
    r = make_routing(L, E, K, seed=9)
    x = uniform((L, E, Din), 1)
    w = weights(E, Din, Dout, 2)
    b = uniform((E, Dout), 3)
    ref = o_moe.index_select_jagged_bmm_3D(r["offsets"], r["index"], x.float(), w.float(), b.float())
    with torch.no_grad():
        out = moe.index_select_jagged_bmm_3D(0, dev(r["offsets"]), dev(r["index"]), dev(x), dev(w), dev(b))
    torch.testing.assert_close(out.cpu(), ref.to(BF16), rtol=REF_RTOL, atol=REF_ATOL)
    L, Din, Dout = 600, 64, 64
    r = make_routing(L, E, K, seed=10)
    x = uniform((L, E, Din), 1)
    w = weights(E, Din, Dout, 2, contiguous=False)
    ref = o_moe.index_select_jagged_bmm_3D(r["offsets"], r["index"], x.float(), w.float(), None)
    with torch.no_grad():
        out = moe.index_select_jagged_bmm_3D(0, dev(r["offsets"]), dev(r["index"]), dev(x), dev(w), None)
    torch.testing.assert_close(out.cpu(), ref.to(BF16), rtol=REF_RTOL, atol=1e-4)


@pytest.mark.parametrize("E,K,Din,Dout,has_silu,has_bias,max_len", [
    (4, 1, 128, 128, True, True, 64), (8, 2, 256, 128, False, True, 200), (8, 2, 128, 256, True, False, 200),
    (4, 2, 256, 256, False, False, 32), (8, 2, 1024, 512, True, True, 700)])
def test_silu_jagged_bmm_combine(E, K, Din, Dout, has_silu, has_bias, max_len):
    """Generator of kernels/tests/moe_test.py:1017-1032; tolerance far inside its atol 5e-1 / rtol 1.5e-1."""
    from fast_moe_amd.kernels import moe
    g = torch.Generator().manual_seed(E + K + Din)
    seq_len = torch.randint(32, max_len + 1, (E,), generator=g)
    N = int(seq_len.sum())
    logits = (torch.rand(N, E, generator=g) + 1e-2).to(BF16)
    topk_gates, topk_idx = logits.topk(K, dim=1)
    meta = o_routing.routing_metadata(topk_idx.numpy(), E)
    t = lambda k: torch.from_numpy(meta[k])
    jagged = uniform((N * K, Din), 1)
    w = weights(E, Din, Dout, 2)
    b = uniform((E, Dout), 3) if has_bias else None
    ref = o_moe.silu_jagged_bmm_combine(t("offsets"), jagged, w, b, t("token_index"), K, topk_gates,
                                        t("gate_index"), has_silu)
    ref32 = o_moe.silu_jagged_bmm_combine(
        t("offsets"), (torch.nn.functional.silu(jagged) if has_silu else jagged).float(), w.float(),
        None if b is None else b.float(), t("token_index"), K, topk_gates.float(), t("gate_index"), False)
    with torch.no_grad():
        out = moe.silu_jagged_bmm_combine(0, dev(t("offsets")), dev(jagged), dev(w), dev(b), dev(t("token_index")),
                                          dev(t("reverse_index")), dev(topk_gates), dev(t("gate_index")),
                                          has_silu=has_silu)
    assert out.dtype == BF16 and tuple(out.shape) == (N, Dout)
    assert_bf16_close(out, ref32, rtol=2e-2, atol=5e-2 * (Din / 128) ** 0.5, what="combine vs fp32")
    torch.testing.assert_close(out.cpu().float(), ref.float(), atol=5e-1, rtol=1.5e-1)


@pytest.mark.parametrize("N,K,D,dtype,wdtype", [
    (2, 4, 128, torch.float32, torch.float32), (33, 16, 256, BF16, BF16), (100, 32, 128, BF16, BF16),
    (1000, 4, 256, torch.float32, torch.float32), (512, 8, 2048, BF16, BF16), (64, 3, 100, BF16, BF16),
    (40, 5, 37, torch.float32, torch.float32), (128, 8, 512, BF16, torch.float32)])
def test_mul_merge_k_add_bit_exact(N, K, D, dtype, wdtype):
    """Generator of kernels/tests/moe_test.py:344-367: non-contiguous weight, permuted weight_index,
    arbitrary row -> output map.  The fp32 adds follow the CPU index_add order, so the result is
    bit-identical to the oracle."""
    from fast_moe_amd.kernels import moe
    g = torch.Generator().manual_seed(N + K)
    x = uniform((N * K, D), 1, dtype)
    w = uniform((N, 2 * K), 2, wdtype)[:, :K]
    w_index = torch.randperm(N * K, generator=g)
    perm = torch.randperm(N * K, generator=g)
    o2i = torch.arange(N).repeat(K)[perm]
    i2o = o2i.sort(stable=True)[1].view(-1, K)
    ref = o_moe.mul_merge_k_add(o2i, x, K, w, w_index)
    with torch.no_grad():
        out = moe.mul_merge_k_add(dev(o2i), dev(i2o), dev(x), weight=dev(w), weight_index=dev(w_index))
        out_nw = moe.mul_merge_k_add(dev(o2i), dev(i2o), dev(x))
    assert out.dtype == ref.dtype
    assert torch.equal(out.cpu(), ref), f"max diff {(out.cpu().float() - ref.float()).abs().max()}"
    assert torch.equal(out_nw.cpu(), o_moe.mul_merge_k_add(o2i, x, K))


# ------------------------------------------------------------------------ fp8
@pytest.mark.parametrize("L,E,K,Din,Dout,bias,contiguous", [
    (16, 4, 2, 32, 16, True, True), (100, 8, 4, 64, 32, False, True), (500, 16, 2, 64, 16, True, False),
    (2048, 8, 2, 256, 512, True, False), (300, 4, 2, 48, 24, True, True), (4096, 64, 8, 256, 128, False, False)])
def test_fp8_gather_gemm(L, E, K, Din, Dout, bias, contiguous):
    """kernels/tests/moe_fp8_test.py:337-370: fp8 kernel vs the PyTorch fp8 emulation, 1e-2 / 1e-2."""
    from fast_moe_amd.kernels import moe_fp8
    r = make_routing(L, E, K, seed=L + 2)
    x = uniform((L, Din), 1)
    w = weights(E, Din, Dout, 2, contiguous)
    b = uniform((E, Dout), 3) if bias else None
    ref = o_fp8.index_select_jagged_bmm_fp8(r["offsets"], r["index"], x, w, b)
    with torch.no_grad():
        out = moe_fp8.index_select_jagged_bmm(0, dev(r["offsets"]), dev(r["index"]), dev(x), dev(w), dev(b),
                                              fp8=True)
        raw = moe_fp8.index_select_jagged_bmm(0, dev(r["offsets"]), dev(r["index"]), dev(x), dev(w), dev(b),
                                              fp8=False)
    if Din <= 64:       # the reference's shapes and its tolerance
        torch.testing.assert_close(out.cpu().float(), ref.float(), atol=1e-2, rtol=1e-2)
    else:               # longer sums: one-ulp bf16 flips next to bias cancellation; 3e-2 relative
        assert_bf16_close(out, ref, rtol=3e-2, atol=3e-2, what="fp8 vs fp8 oracle")
    # vs the unquantised op: tolerance of moe_fp8_test.py:302-335, quantisation noise grows with Din
    torch.testing.assert_close(out.cpu().float(), raw.cpu().float(), atol=4e-1 * max(1.0, Din / 64),
                               rtol=1e-1)


def test_fp8_outlier_rows_and_zero_rows():
    from fast_moe_amd.kernels import moe_fp8
    L, E, K, Din, Dout = 512, 8, 2, 128, 64
    r = make_routing(L, E, K, seed=4)
    x = randn((L, Din), 1)
    x[::50] *= 100
    x[7] = 0
    w = weights(E, Din, Dout, 2, False, scale=Din ** -0.5)
    w[3, :, 5] = 0
    ref = o_fp8.index_select_jagged_bmm_fp8(r["offsets"], r["index"], x, w, None)
    with torch.no_grad():
        out = moe_fp8.index_select_jagged_bmm(0, dev(r["offsets"]), dev(r["index"]), dev(x), dev(w), None, fp8=True)
    assert bool(torch.isfinite(out).all())
    err = (out.cpu().float() - ref.float()).abs()
    assert bool((err <= 3e-2 * ref.float().abs() + 3e-2).all())


@pytest.mark.parametrize("E,K,Din,Dout,has_silu", [(4, 2, 128, 128, True), (8, 2, 256, 64, False)])
def test_fp8_combine(E, K, Din, Dout, has_silu):
    from fast_moe_amd.kernels import moe_fp8
    g = torch.Generator().manual_seed(E)
    N = 300
    logits = (torch.rand(N, E, generator=g) + 1e-2).to(BF16)
    gates, topk_idx = logits.topk(K, dim=1)
    meta = o_routing.routing_metadata(topk_idx.numpy(), E)
    t = lambda k: torch.from_numpy(meta[k])
    jagged = uniform((N * K, Din), 1)
    w = weights(E, Din, Dout, 2)
    b = uniform((E, Dout), 3)
    # oracle: the same fp8 emulation for the GEMM, then the merge
    h = torch.nn.functional.silu(jagged) if has_silu else jagged
    qa, sa = o_fp8.rowwise_quant_fp8(h)
    qw, sw = o_fp8.rowwise_quant_fp8(w.permute(0, 2, 1))
    sizes = (t("offsets")[1:] - t("offsets")[:-1]).tolist()
    rows = o_fp8.fp8_linear_per_expert(list(o_fp8.dequant(qa).split(sizes)), list(sa.split(sizes)),
                                       o_fp8.dequant(qw), sw, b, BF16)
    ref = o_moe.mul_merge_k_add(t("token_index"), torch.cat(rows), K, gates, t("gate_index"))
    with torch.no_grad():
        out = moe_fp8.silu_jagged_bmm_combine_fp8(0, dev(t("offsets")), dev(jagged), dev(w), dev(b),
                                                  dev(t("token_index")), dev(t("reverse_index")), dev(gates),
                                                  dev(t("gate_index")), has_silu=has_silu)
    err = (out.cpu().float() - ref.float()).abs()
    assert bool((err <= 3e-2 * ref.float().abs() + 3e-2).all()), err.max()


def test_fp8_weight_pair_of_other_origin_is_not_taken_for_powers_of_two():
    """A caller may hand the fp8 operators its own (bytes, scales) pair.  Only scale tensors that
    the package's quantiser returned (and nobody wrote to since) are taken for exact powers of
    two and given to the MFMAs as block scales; any other pair has its scales divided out in the
    epilogue, which is right for every positive scale."""
    from fast_moe_amd.kernels import moe_fp8
    from fast_moe_amd.kernels.hip import ops
    L, E, K, Din, Dout = 4096, 8, 2, 256, 512
    r = make_routing(L, E, K, seed=3)
    x = dev(randn((L, Din), 1))
    w = dev(weights(E, Din, Dout, 2, False, scale=Din ** -0.5))
    offsets, index = dev(r["offsets"]), dev(r["index"])
    qw, sw = moe_fp8.quantize_expert_weights(w)
    assert ops.scales_are_pow2(sw)
    other = sw * 1.5                         # a legitimate pair of other origin: same bytes, weights 1.5 times smaller
    assert not ops.scales_are_pow2(other) and not ops.scales_are_pow2(sw.clone())
    qa, sa = ops.quant_rows_fp8(x)
    kw = dict(total_rows=L * K, row_index=index.reshape(-1), index_div=K, a_scale=sa)
    want = ops.grouped_gemm(offsets, qa, qw, b_scale=other, scales_pow2=False, **kw)
    got = moe_fp8.index_select_jagged_bmm(0, offsets, index, x, w, None, fp8=True, fp8_weight=(qw, other))
    assert torch.equal(got, want)
    base = moe_fp8.index_select_jagged_bmm(0, offsets, index, x, w, None, fp8=True, fp8_weight=(qw, sw))
    assert_bf16_close(got.float() * 1.5, base.float(), rtol=1.6e-2, atol=1e-2, what="scales 1.5 times larger")
    sw.mul_(1.0)                              # written to: no longer vouched for
    assert not ops.scales_are_pow2(sw)


def test_forward_only_and_dtype_errors():
    from fast_moe_amd.kernels import moe, moe_fp8
    r = make_routing(16, 4, 2)
    x = uniform((16, 32), 1).cuda().requires_grad_()
    w = weights(4, 32, 32, 2).cuda()
    x2 = uniform((32, 32), 1).cuda().requires_grad_()
    with pytest.raises(RuntimeError, match="forward-only"):       # no backward for this one, as in the reference
        moe_fp8.silu_jagged_bmm_fp8(dev(r["offsets"]), 0, x2, w, uniform((4, 32), 3).cuda())
    with pytest.raises(NotImplementedError):
        with torch.no_grad():
            moe.index_select_jagged_bmm(0, dev(r["offsets"]), dev(r["index"]), x.half(), w.half(), None)


# ------------------------------------------------------------- ring-kernel specifics
@pytest.mark.parametrize("L,E,K,Din,Dout,epi", [
    (4096, 8, 2, 96, 256, "plain"),        # three K-slices only: the ring never fills
    (4096, 8, 2, 1024, 264, "plain"),      # N = 264: last column tile 8 wide
    (9000, 3, 1, 512, 512, "plain"),       # fewer tiles than CUs, K_top = 1 (index_shift 0)
    (6144, 24, 3, 256, 384, "swiglu"),     # top-3: index division, not a shift
    (20000, 200, 2, 128, 128, "swiglu"),   # many experts, about 200 rows each (register tables, 4 entries)
    (30000, 300, 2, 128, 128, "swiglu"),   # more than 256 experts: 4-slot ring with its tables in LDS
    (3000, 2, 2, 2048, 128, "swiglu"),     # long K, one column tile
])
def test_ring_kernel_shapes(L, E, K, Din, Dout, epi):
    from fast_moe_amd.kernels import moe
    r = make_routing(L, E, K, seed=L + E)
    x = randn((L, Din), 1)
    w = weights(E, Din, Dout, 2, False, scale=Din ** -0.5)
    b = randn((E, Dout), 3)
    if epi == "plain":
        ref = o_moe.index_select_jagged_bmm(r["offsets"], r["index"], x.float(), w.float(), b.float())
        with torch.no_grad():
            out = moe.index_select_jagged_bmm(0, dev(r["offsets"]), dev(r["index"]), dev(x), dev(w), dev(b))
        assert_bf16_close(out, ref, rtol=1e-2, atol=1e-2, what=f"ring plain {L},{E},{K},{Din},{Dout}")
    else:
        wp = weights(E, Din, Dout, 5, False, scale=Din ** -0.5)
        ref = o_moe.index_select_jagged_bmm_swiglu(r["offsets"], r["index"], x.float(), w.float(), b.float(),
                                                   wp.float(), None)
        with torch.no_grad():
            out = moe.index_select_jagged_bmm_swiglu(0, dev(r["offsets"]), dev(r["index"]), dev(x), dev(w), dev(b),
                                                     dev(wp), None)
        assert_bf16_close(out, ref, rtol=1.6e-2, atol=1e-2, what=f"ring swiglu {L},{E},{K},{Din},{Dout}")


@pytest.mark.parametrize("epi,fp8", [("plain", False), ("swiglu", False), ("plain", True)])
def test_ring_kernel_tiles_with_few_valid_rows(epi, fp8):
    """Experts whose last (or only) 256-row tile ends at, just before and just after every 32-row
    block boundary: tiles that end in their first half run the ring kernel's shortened main loop,
    and the two wave rows share a tile's row blocks alternately.  Against the oracle, and the plan
    must say RING."""
    from fast_moe_amd.kernels import moe, moe_fp8
    from fast_moe_amd.kernels.hip import _lib, ops
    lens = [1, 31, 32, 33, 63, 64, 65, 96, 127, 128, 129, 160, 191, 193, 255, 256, 257, 288, 320, 383, 384, 385,
            511, 513, 640, 0, 769, 2048 + 17, 3000]
    E, Din, Dout = len(lens), 192, 320
    g = torch.Generator().manual_seed(7)
    experts = torch.repeat_interleave(torch.arange(E), torch.tensor(lens))
    topk = experts[torch.randperm(experts.numel(), generator=g)].view(-1, 1)
    L = topk.shape[0]
    meta = o_routing.routing_metadata(topk.numpy(), E)
    offsets = torch.from_numpy(meta["offsets"])
    index = torch.from_numpy(meta["gate_index"]).view(-1, 1)
    assert (offsets[1:] - offsets[:-1]).tolist() == lens
    x = randn((L, Din), 1)
    w = weights(E, Din, Dout, 2, False, scale=Din ** -0.5)
    b = randn((E, Dout), 3)
    # (the plan of the bf16 descriptor of this shape; the e4m3 one differs in the operand type only)
    assert ops.grouped_gemm(dev(offsets), dev(x), dev(w), total_rows=L, row_index=dev(index).view(-1), index_div=1,
                            plan_only=True) == _lib.PLAN_RING
    with torch.no_grad():
        if fp8:
            ref = o_fp8.index_select_jagged_bmm_fp8(offsets, index, x, w, b)
            out = moe_fp8.index_select_jagged_bmm(0, dev(offsets), dev(index), dev(x), dev(w), dev(b), fp8=True)
        elif epi == "plain":
            ref = o_moe.index_select_jagged_bmm(offsets, index, x.float(), w.float(), b.float())
            out = moe.index_select_jagged_bmm(0, dev(offsets), dev(index), dev(x), dev(w), dev(b))
        else:
            wp = weights(E, Din, Dout, 5, False, scale=Din ** -0.5)
            ref = o_moe.index_select_jagged_bmm_swiglu(offsets, index, x.float(), w.float(), b.float(),
                                                       wp.float(), None)
            out = moe.index_select_jagged_bmm_swiglu(0, dev(offsets), dev(index), dev(x), dev(w), dev(b),
                                                     dev(wp), None)
    # every expert on its own, so that a failure names the row count it happens at
    for e, n in enumerate(lens):
        lo = int(offsets[e])
        if n:
            assert_bf16_close(out[lo:lo + n], ref[lo:lo + n], rtol=3e-2 if fp8 else 1.6e-2, atol=3e-2 if fp8 else 1e-2,
                              what=f"expert {e} with {n} rows ({epi}, fp8={fp8})")


def test_ring_kernel_is_deterministic_and_ignores_garbage_offsets():
    """Two launches give identical bits; offsets outside [0, R] are clamped instead of followed."""
    from fast_moe_amd.kernels.hip import ops
    L, E, K, D, N = 8192, 16, 2, 256, 256
    r = make_routing(L, E, K, seed=5)
    x, w = dev(randn((L, D), 1)), dev(weights(E, D, N, 2, False, scale=D ** -0.5))
    a = ops.grouped_gemm(dev(r["offsets"]), x, w, total_rows=L * K, row_index=dev(r["gate_index"]), index_div=K)
    b = ops.grouped_gemm(dev(r["offsets"]), x, w, total_rows=L * K, row_index=dev(r["gate_index"]), index_div=K)
    assert torch.equal(a, b)
    bad = r["offsets"].clone()
    bad[-1] = 10 ** 12
    bad[3] = -7
    out = ops.grouped_gemm(dev(bad), x, w, total_rows=L * K, row_index=dev(r["gate_index"]), index_div=K)
    torch.cuda.synchronize()
    assert out.shape == a.shape


@pytest.mark.parametrize("fp8", [False, True], ids=["bf16", "fp8"])
def test_ring_kernel_repeats_bit_identically_while_another_stream_loads_the_memory_system(fp8):
    """The ring kernel keeps its own count of the LDS-DMA in flight; a wait that is one operation
    short would read a slot before its data has landed, and whether that shows depends on timing.
    Both GEMMs of the benchmark sizes (SwiGLU with gather, plain), 24 launches each, while a second
    stream copies 1 GiB back and forth: every launch must reproduce the first bit for bit."""
    from fast_moe_amd.kernels.hip import _lib, ops
    T, E, K, D, H = 16384, 64, 8, 2048, 1408
    topk = skewed_topk(T, E, K, seed=11)
    meta = o_routing.routing_metadata(topk.numpy(), E)
    offsets, gate_index = dev(torch.from_numpy(meta["offsets"])), dev(torch.from_numpy(meta["gate_index"]))
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn(T, D, generator=g, device="cuda").to(BF16)
    wg = (torch.randn(E, H, D, generator=g, device="cuda") * D ** -0.5).to(BF16).permute(0, 2, 1)
    wu = (torch.randn(E, H, D, generator=g, device="cuda") * D ** -0.5).to(BF16).permute(0, 2, 1)
    wd = (torch.randn(E, D, H, generator=g, device="cuda") * H ** -0.5).to(BF16).permute(0, 2, 1)
    if fp8:
        (qx, sx), (qg, sg), (qu, su), (qd, sd) = (ops.quant_rows_fp8(x), ops.quant_rows_fp8(wg.permute(0, 2, 1)),
                                                    ops.quant_rows_fp8(wu.permute(0, 2, 1)),
                                                    ops.quant_rows_fp8(wd.permute(0, 2, 1)))
        gemm1 = lambda: ops.grouped_gemm(offsets, qx, qg.permute(0, 2, 1), total_rows=T * K, row_index=gate_index,
                                         index_div=K, b2=qu.permute(0, 2, 1), epilogue=_lib.EPI_SWIGLU, a_scale=sx,
                                         b_scale=sg, b2_scale=su, scales_pow2=True)
    else:
        gemm1 = lambda: ops.grouped_gemm(offsets, x, wg, total_rows=T * K, row_index=gate_index, index_div=K, b2=wu,
                                         epilogue=_lib.EPI_SWIGLU)
    hidden = gemm1()
    if fp8:
        qh, sh = ops.quant_rows_fp8(hidden)
        gemm2 = lambda: ops.grouped_gemm(offsets, qh, qd.permute(0, 2, 1), total_rows=T * K, a_scale=sh, b_scale=sd,
                                         scales_pow2=True)
    else:
        gemm2 = lambda: ops.grouped_gemm(offsets, hidden, wd, total_rows=T * K)
    first2 = gemm2()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    a, b = torch.empty(1 << 28, dtype=torch.int32, device="cuda"), torch.empty(1 << 28, dtype=torch.int32, device="cuda")
    for i in range(24):
        with torch.cuda.stream(side):               # (default priority) a copy that competes for HBM and L2
            (b if i % 2 else a).copy_(a if i % 2 else b, non_blocking=True)
        h, o = gemm1(), gemm2()
        assert torch.equal(h, hidden), f"gemm1, launch {i}"
        assert torch.equal(o, first2), f"gemm2, launch {i}"
    torch.cuda.synchronize()


@pytest.mark.parametrize("fp8", [False, True])
def test_full_size_c3_c4_sampled_rows(fp8):
    """The benchmark sizes (T=16384, E=64, top-8, D=2048, H=1408, Zipf-skewed, empty experts): the
    whole SwiGLU GEMM runs on the GPU, a sample of its rows is checked against the oracle, and
    size-independent properties hold (rows of empty experts absent, duplicate tokens give equal rows)."""
    from fast_moe_amd.kernels import moe_fp8
    from fast_moe_amd.kernels.hip import ops
    T, E, K, D, H = 16384, 64, 8, 2048, 1408
    topk = skewed_topk(T, E, K, seed=11)
    meta = o_routing.routing_metadata(topk.numpy(), E)
    assert (meta["lengths"] == 0).sum() >= 2
    offsets = torch.from_numpy(meta["offsets"])
    gate_index = torch.from_numpy(meta["gate_index"])
    g = torch.Generator().manual_seed(0)
    x = torch.randn(T, D, generator=g).to(BF16)
    x[5] = x[4]                                            # two identical tokens
    if fp8:
        x[::100] *= 100
    wg = (torch.randn(E, H, D, generator=g) * D ** -0.5).to(BF16).permute(0, 2, 1)
    wu = (torch.randn(E, H, D, generator=g) * D ** -0.5).to(BF16).permute(0, 2, 1)
    with torch.no_grad():
        if fp8:
            qg, sg = moe_fp8.quantize_expert_weights(dev(wg))
            qu, su = moe_fp8.quantize_expert_weights(dev(wu))
            qx, sx = ops.quant_rows_fp8(dev(x))
            out = ops.grouped_gemm(dev(offsets), qx, qg, total_rows=T * K, row_index=dev(gate_index), index_div=K,
                                   b2=qu, epilogue=2, a_scale=sx, b_scale=sg, b2_scale=su)
        else:
            out = ops.grouped_gemm(dev(offsets), dev(x), dev(wg), total_rows=T * K, row_index=dev(gate_index),
                                   index_div=K, b2=dev(wu), epilogue=2)
    out = out.cpu()
    assert bool(torch.isfinite(out).all())
    rows = torch.randperm(T * K, generator=g)[:192]
    experts = torch.searchsorted(offsets[1:], rows, right=True)
    tok = gate_index[rows] // K
    for i in range(rows.numel()):
        e, t = int(experts[i]), int(tok[i])
        if fp8:
            one = torch.tensor([0, 1])
            eo = torch.zeros(2, dtype=torch.int64)
            eo[1] = 1
            # the oracle's fp8 path on a single row / single expert
            from oracle import moe_fp8 as o8
            qa, sa = o8.rowwise_quant_fp8(x[t:t + 1])
            qwg, swg = o8.rowwise_quant_fp8(wg[e:e + 1].permute(0, 2, 1))
            qwu, swu = o8.rowwise_quant_fp8(wu[e:e + 1].permute(0, 2, 1))
            gg = o8.fp8_linear_per_expert([o8.dequant(qa)], [sa], o8.dequant(qwg), swg, None, BF16)[0]
            uu = o8.fp8_linear_per_expert([o8.dequant(qa)], [sa], o8.dequant(qwu), swu, None, BF16)[0]
            ref = (torch.nn.functional.silu(gg) * uu)[0]
            tol = 3e-2
        else:
            xr = x[t].float()
            ref = torch.nn.functional.silu(xr @ wg[e].float()) * (xr @ wu[e].float())
            tol = 1.6e-2
        err = (out[rows[i]].float() - ref.float()).abs()
        scale = ref.float().abs().max().item()
        assert bool((err <= tol * ref.float().abs() + tol * scale * 0.5 + 1e-3).all()), (int(rows[i]), err.max())
    # identical tokens routed to the same expert give identical rows
    pos = {}
    for tkn in (4, 5):
        for j in range(K):
            pos[(tkn, int(topk[tkn, j]))] = int(torch.from_numpy(meta["reverse_index"])[tkn][
                sorted(range(K), key=lambda q: int(topk[tkn, q])).index(j)])
    common = set(int(e) for e in topk[4]) & set(int(e) for e in topk[5])
    for e in common:
        assert torch.equal(out[pos[(4, e)]], out[pos[(5, e)]])


def test_n_contiguous_weights_and_the_transposing_copy():
    """[E, K, N]-contiguous weights (the layout of kernels/tests/moe_test.py:205-209) of a useful
    size are transposed once on the device and then streamed; the result equals the in-place
    element-load kernel's and the oracle's."""
    from fast_moe_amd.kernels import moe
    from fast_moe_amd.kernels.hip import ops
    L, E, K, Din, Dout = 8192, 8, 2, 512, 384
    r = make_routing(L, E, K, seed=21)
    x = randn((L, Din), 1)
    w = weights(E, Din, Dout, 2, True, scale=Din ** -0.5)
    assert w.is_contiguous()
    wt = ops.to_k_contiguous(dev(w))
    assert wt.stride(1) == 1 and torch.equal(wt.cpu(), w)
    odd = weights(3, 70, 130, 4, True)           # extents that are not multiples of the 64 x 64 tile
    assert torch.equal(ops.to_k_contiguous(dev(odd)).cpu(), odd)
    q = (torch.arange(5 * 33 * 65) % 251).to(torch.uint8).view(5, 33, 65).view(torch.float8_e4m3fn)
    assert torch.equal(ops.to_k_contiguous(dev(q)).cpu().view(torch.uint8), q.view(torch.uint8))
    ref = o_moe.index_select_jagged_bmm(r["offsets"], r["index"], x.float(), w.float(), None)
    with torch.no_grad():
        out = moe.index_select_jagged_bmm(0, dev(r["offsets"]), dev(r["index"]), dev(x), dev(w), None)
        out_k = moe.index_select_jagged_bmm(0, dev(r["offsets"]), dev(r["index"]), dev(x), wt, None)
    assert torch.equal(out, out_k)
    assert_bf16_close(out, ref, rtol=1e-2, atol=1e-2, what="N-contiguous weights")


# ------------------------------------------------------------------------ fp32
@pytest.mark.parametrize("L,E,K,Din,Dout", GRID[1::4])
@pytest.mark.parametrize("contiguous", [True, False])
@pytest.mark.parametrize("has_bias", [True, False])
def test_index_select_jagged_bmm_fp32_reference_grid(L, E, K, Din, Dout, contiguous, has_bias):
    """fp32 half of kernels/tests/moe_test.py:35-84 (allow_tf32 off): default fp32 assert_close."""
    from fast_moe_amd.kernels import moe
    r = make_routing(L, E, K, seed=L + E + 1)
    x = uniform((L, Din), 1, torch.float32)
    w = uniform((E, Din, Dout), 2, torch.float32)
    if not contiguous:
        w = w.transpose(1, 2).contiguous().transpose(1, 2)
    b = uniform((E, Dout), 3, torch.float32) if has_bias else None
    ref = o_moe.index_select_jagged_bmm(r["offsets"], r["index"], x, w, b)
    with torch.no_grad():
        out = moe.index_select_jagged_bmm(0, dev(r["offsets"]), dev(r["index"]), dev(x), dev(w), dev(b))
    assert out.dtype == torch.float32
    torch.testing.assert_close(out.cpu(), ref)


def test_fp32_swiglu_gating_3d_and_combine():
    from fast_moe_amd.kernels import moe
    L, E, K, Din, Dout = 700, 8, 2, 64, 96
    f32 = torch.float32
    r = make_routing(L, E, K, seed=31)
    x, x2 = uniform((L, Din), 1, f32), uniform((L, Din), 4, f32)
    w, wp = uniform((E, Din, Dout), 2, f32), uniform((E, Din, Dout), 5, f32)
    b, bp = uniform((E, Dout), 3, f32), uniform((E, Dout), 6, f32)
    a = [dev(r["offsets"]), dev(r["index"])]
    with torch.no_grad():
        sw = moe.index_select_jagged_bmm_swiglu(0, *a, dev(x), dev(w), dev(b), dev(wp), dev(bp))
        gt = moe.index_select_jagged_gating_bmm(0, *a, dev(x), dev(x2), dev(w), dev(b), dev(wp), dev(bp))
    torch.testing.assert_close(sw.cpu(), o_moe.index_select_jagged_bmm_swiglu(r["offsets"], r["index"], x, w, b, wp, bp),
                               rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(gt.cpu(), o_moe.index_select_jagged_gating_bmm(r["offsets"], r["index"], x, x2, w, wp, b, bp),
                               rtol=1e-5, atol=1e-5)
    x3 = uniform((L, E, Din), 7, f32)
    with torch.no_grad():
        o3 = moe.index_select_jagged_bmm_3D(0, *a, dev(x3), dev(w), dev(b))
    torch.testing.assert_close(o3.cpu(), o_moe.index_select_jagged_bmm_3D(r["offsets"], r["index"], x3, w, b))
    # SiLU-on-load GEMM + merge
    g = torch.Generator().manual_seed(3)
    gates = torch.rand(L, K, generator=g)
    jag = uniform((L * K, Din), 8, f32)
    ref = o_moe.silu_jagged_bmm_combine(r["offsets"], jag, w, b, r["token_index"], K, gates, r["gate_index"], True)
    with torch.no_grad():
        out = moe.silu_jagged_bmm_combine(0, dev(r["offsets"]), dev(jag), dev(w), dev(b), dev(r["token_index"]),
                                          dev(r["reverse_index"]), dev(gates), dev(r["gate_index"]), has_silu=True)
    torch.testing.assert_close(out.cpu(), ref, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("L,E,K,Din,Dout,dtype,bias", [
    (4096, 8, 2, 256, 384, "bf16", True),     # ring kernel
    (4096, 8, 2, 256, 384, "bf16", False),
    (300, 4, 2, 72, 40, "bf16", True),        # element kernel, scalar stores
    (1000, 4, 2, 64, 128, "f32", True),
    (4096, 8, 2, 256, 384, "fp8", True),
])
def test_swiglu_pre_activation_outputs(L, E, K, Din, Dout, dtype, bias):
    """aux / aux2 of the SWIGLU epilogue are bit for bit the outputs of the two plain GEMMs, and the
    main output does not change when they are requested."""
    from fast_moe_amd.kernels.hip import ops
    from fast_moe_amd.kernels.hip._lib import EPI_SWIGLU
    r = make_routing(L, E, K, seed=L)
    td = torch.float32 if dtype == "f32" else BF16
    x = randn((L, Din), 1).to(td).cuda()
    w = weights(E, Din, Dout, 2, False, Din ** -0.5).to(td).cuda()
    wp = weights(E, Din, Dout, 3, False, Din ** -0.5).to(td).cuda()
    b = randn((E, Dout), 4).to(td).cuda() if bias else None
    bp = randn((E, Dout), 5).to(td).cuda() if bias else None
    kw = dict(total_rows=L * K, row_index=dev(r["index"]), index_div=K)
    sc = [{}, {}, {}]
    if dtype == "fp8":
        xq, xs = ops.quant_rows_fp8(x)
        wq, ws = ops.quant_rows_fp8(w.permute(0, 2, 1))
        wpq, wps = ops.quant_rows_fp8(wp.permute(0, 2, 1))
        x, w, wp = xq, wq.permute(0, 2, 1), wpq.permute(0, 2, 1)
        sc = [dict(a_scale=xs, b_scale=ws), dict(a_scale=xs, b_scale=wps), dict(a_scale=xs, b_scale=ws, b2_scale=wps)]
    off = dev(r["offsets"])
    g = ops.grouped_gemm(off, x, w, bias=b, **kw, **sc[0])
    u = ops.grouped_gemm(off, x, wp, bias=bp, **kw, **sc[1])
    plain = ops.grouped_gemm(off, x, w, bias=b, b2=wp, bias2=bp, epilogue=EPI_SWIGLU, **kw, **sc[2])
    aux = (torch.full_like(g, 7.0), torch.full_like(g, 7.0))
    out = ops.grouped_gemm(off, x, w, bias=b, b2=wp, bias2=bp, epilogue=EPI_SWIGLU, aux=aux, **kw, **sc[2])
    assert torch.equal(out, plain)
    assert torch.equal(aux[0], g) and torch.equal(aux[1], u)
    with pytest.raises(ValueError, match="SWIGLU"):
        ops.grouped_gemm(off, x, w, bias=b, aux=aux, **kw, **sc[0])


@pytest.mark.parametrize("L,E,K,Din,Dout,epi", [
    (8192, 8, 2, 512, 384, "none"),
    (8192, 8, 2, 512, 384, "swiglu"),
    (4096, 16, 4, 256, 200, "none"),       # N tail: 200 columns of a 256-column tile
    (4096, 16, 4, 256, 72, "swiglu"),      # N tail inside the gate / up halves
    (20000, 200, 2, 128, 128, "swiglu"),   # register tables with 4 entries
    (3000, 4, 2, 1408, 2048, "none"),      # the input-gradient shape of the layer
])
def test_ring_kernel_reads_n_contiguous_weights_in_place(L, E, K, Din, Dout, epi):
    """[E, K, N]-contiguous weights (the reference tests' default layout, and what the input-gradient
    GEMM multiplies by): the plan says RING, and the result is bit for bit the one from the same
    weights stored K-contiguous."""
    from fast_moe_amd.kernels.hip import _lib, ops
    r = make_routing(L, E, K, seed=L + 1)
    x = dev(randn((L, Din), 1))
    w, wp = (dev(weights(E, Din, Dout, s, True, scale=Din ** -0.5)) for s in (2, 3))
    b, bp = dev(randn((E, Dout), 4)), dev(randn((E, Dout), 5))
    assert w.is_contiguous()
    wk, wpk = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (w, wp))
    kw = dict(total_rows=L * K, row_index=dev(r["index"]), index_div=K, bias=b)
    if epi == "swiglu":
        kw.update(bias2=bp, epilogue=_lib.EPI_SWIGLU)
    off = dev(r["offsets"])
    seen = []
    real_plan = ops.gemm_plan
    ops.gemm_plan = lambda d: seen.append(real_plan(d)) or seen[-1]
    try:
        out = ops.grouped_gemm(off, x, w, b2=wp if epi == "swiglu" else None, **kw)
    finally:
        ops.gemm_plan = real_plan
    assert seen == [_lib.PLAN_RING]
    ref = ops.grouped_gemm(off, x, wk, b2=wpk if epi == "swiglu" else None, **kw)
    assert torch.equal(out, ref)
    # a view with a larger row pitch (columns of a wider tensor) is read in place as well
    wide = torch.zeros((E, Din, Dout + 24), dtype=BF16, device="cuda")
    wide[:, :, 8:8 + Dout] = w
    if epi == "none":
        assert torch.equal(ops.grouped_gemm(off, x, wide[:, :, 8:8 + Dout], **kw), ref)


@pytest.mark.parametrize("G", [1, 4, 16])
@pytest.mark.parametrize("M", [0, 64, 512, 1000000])
@pytest.mark.parametrize("K,fp8", [(29, False), (256, False), (256, True)])
def test_reference_grouped_gemm_grid(G, M, K, fp8):
    """The grid of kernels/tests/grouped_gemm_test.py:28-199: M rows cut at G - 1 random points
    (empty groups included), N = 256, weights [G * N, K]; bf16 against the fp32 product (atol
    1e-5, rtol 1.6e-2 there; the absolute term here is scaled to sqrt(K)-sized sums), e4m3
    against the product of the dequantised operands (2e-2 / 5e-2 and 1.6e-2).  The million-row
    case is checked on the GPU in fp32, expert by expert."""
    from fast_moe_amd.kernels.hip import ops
    N = 256
    g = torch.Generator().manual_seed(G * 1000 + M % 997 + K)
    a = torch.randn(M, K, generator=g).to(BF16).cuda()
    b = torch.randn(G * N, K, generator=g).to(BF16).cuda()
    cuts = torch.sort(torch.randint(0, max(M, 1), (G - 1,), generator=g)).values if M > 0 else torch.zeros(G - 1, dtype=torch.int64)
    offsets = torch.cat([torch.zeros(1, dtype=torch.int64), cuts.to(torch.int64), torch.tensor([M])])
    w = b.view(G, N, K).permute(0, 2, 1)                      # [G, K, N], K contiguous
    if fp8:
        qa, sa = ops.quant_rows_fp8(a) if M else (torch.empty((0, K), dtype=ops.FP8_DTYPE, device="cuda"), torch.empty(0, device="cuda"))
        qb, sb = ops.quant_rows_fp8(b)
        out = ops.grouped_gemm(offsets.cuda(), qa, qb.view(G, N, K).permute(0, 2, 1), total_rows=M,
                               a_scale=sa, b_scale=sb.view(G, N))
    else:
        out = ops.grouped_gemm(offsets.cuda(), a, w, total_rows=M)
    assert tuple(out.shape) == (M, N) and out.dtype == BF16
    if M == 0:
        return
    for e in range(G):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if lo == hi:
            continue
        if fp8:
            ref = (qa[lo:hi].float() @ qb.view(G, N, K)[e].float().T) / (sa[lo:hi, None] * sb.view(G, N)[e][None, :])
            atol = 5e-2 if M > 16384 else 2e-2
        else:
            ref = a[lo:hi].float() @ w[e].float()
            atol = 1e-5 + 4e-3 * K ** 0.5
        torch.testing.assert_close(out[lo:hi].float(), ref.to(BF16).float(), atol=atol, rtol=1.6e-2)


@pytest.mark.parametrize("seed", range(24))
def test_seeded_random_shapes_all_operators(seed):
    """A seeded draw of sizes in the spirit of the reference's hypothesis grids
    (kernels/tests/moe_test.py:27-57, 401-423, 729-751): token counts, expert counts, top-k, widths
    (multiples of 8 and not), weight layouts and bias, for the plain, SwiGLU and merge operators,
    forward against the oracle and, on every third draw, backward as well."""
    import random
    from fast_moe_amd.kernels import moe
    rnd = random.Random(1000 + seed)
    E = rnd.choice([1, 2, 3, 8, 17, 40, 70])
    K = rnd.randint(1, min(E, 4))
    L = rnd.choice([1, 7, 64, 333, 1500, 5000])
    Din = rnd.choice([8, 24, 40, 72, 128, 200, 256, 520]) + rnd.choice([0, 0, 0, 3])
    Dout = rnd.choice([8, 16, 56, 128, 136, 256, 264]) + rnd.choice([0, 0, 0, 5])
    contiguous, has_bias = rnd.random() < 0.5, rnd.random() < 0.5
    r = make_routing(L, E, K, seed=seed)
    x = randn((L, Din), seed + 1)
    w = weights(E, Din, Dout, seed + 2, contiguous, scale=Din ** -0.5)
    wp = weights(E, Din, Dout, seed + 3, contiguous, scale=Din ** -0.5)
    b = randn((E, Dout), seed + 4) if has_bias else None
    gates = torch.rand((L, K), generator=torch.Generator().manual_seed(seed)).to(BF16)
    tag = f"seed {seed}: L={L} E={E} K={K} Din={Din} Dout={Dout} contiguous={contiguous} bias={has_bias}"
    f32 = lambda t: None if t is None else t.float()
    ref_plain = o_moe.index_select_jagged_bmm(r["offsets"], r["index"], f32(x), f32(w), f32(b))
    ref_glu = o_moe.index_select_jagged_bmm_swiglu(r["offsets"], r["index"], f32(x), f32(w), f32(b), f32(wp), f32(b))
    ref_merge = o_moe.mul_merge_k_add(r["token_index"], ref_plain.to(BF16), K, gates, r["gate_index"])
    d = lambda t: None if t is None else dev(t)
    with torch.no_grad():
        plain = moe.index_select_jagged_bmm(0, d(r["offsets"]), d(r["index"]), d(x), d(w), d(b))
        glu = moe.index_select_jagged_bmm_swiglu(0, d(r["offsets"]), d(r["index"]), d(x), d(w), d(b), d(wp), d(b))
        merged = moe.mul_merge_k_add(d(r["token_index"]), d(r["reverse_index"]), d(ref_plain.to(BF16)),
                                     weight=d(gates), weight_index=d(r["gate_index"]))
    assert_bf16_close(plain, ref_plain, rtol=1.6e-2, atol=2e-2, what="plain " + tag)
    assert_bf16_close(glu, ref_glu, rtol=1.6e-2, atol=2e-2, what="swiglu " + tag)
    assert torch.equal(merged.cpu(), ref_merge), "merge " + tag
    if seed % 3:
        return
    leaves_ref = [t.float().requires_grad_(True) for t in (x, w, wp)]
    dout = randn((L * K, Dout), seed + 5) * 0.01
    o_moe.index_select_jagged_bmm_swiglu(r["offsets"], r["index"], leaves_ref[0], leaves_ref[1], f32(b), leaves_ref[2],
                                         f32(b)).backward(dout.float())
    leaves = [dev(t).requires_grad_(True) for t in (x, w, wp)]
    moe.index_select_jagged_bmm_swiglu(0, d(r["offsets"]), d(r["index"]), leaves[0], leaves[1], d(b), leaves[2],
                                       d(b)).backward(dev(dout))
    for name, got, ref in zip(("d_x", "d_w", "d_wp"), leaves, leaves_ref):
        err = (got.grad.float().cpu() - ref.grad).abs().max().item()
        assert err <= 3e-2 * ref.grad.abs().max().item() + 1e-6, (name, tag, err, ref.grad.abs().max().item())


def test_silu_on_load_at_ring_size_takes_the_silu_pass():
    """silu_jagged_bmm_combine(has_silu=True) large enough for the LDS-ring kernel: SiLU is applied by
    an element-wise pass (the ring kernel has no SiLU on load) with the rounding of the staged
    kernel's SiLU on load, so the GEMM input is bit-identical and the result meets the same bar."""
    from fast_moe_amd.kernels import moe
    from fast_moe_amd.kernels.hip import ops
    T, E, K, H, O = 4096, 8, 2, 256, 512
    r = make_routing(T, E, K, seed=21)
    j = randn((T * K, H), 1)
    w = weights(E, H, O, 2, False, scale=H ** -0.5)
    b = randn((E, O), 3)
    gates = torch.rand((T, K), generator=torch.Generator().manual_seed(4)).to(BF16)
    ref = o_moe.silu_jagged_bmm_combine(r["offsets"], j.float(), w.float(), b.float(), r["token_index"], K,
                                        gates.float(), r["gate_index"], True)
    with torch.no_grad():
        out = moe.silu_jagged_bmm_combine(0, dev(r["offsets"]), dev(j), dev(w), dev(b), dev(r["token_index"]),
                                          dev(r["reverse_index"]), dev(gates), dev(r["gate_index"]), has_silu=True)
        # the pass is what the caller could have done by hand
        rows = ops.grouped_gemm(dev(r["offsets"]), dev(j), dev(w), total_rows=T * K, bias=dev(b), a_silu=True)
        rows2 = ops.grouped_gemm(dev(r["offsets"]), ops.silu_mul(dev(j), None), dev(w), total_rows=T * K, bias=dev(b))
        # ... and a slice small enough for the staged kernel's SiLU on load sees the same input bits
        n_small = int(r["offsets"][1])
        small = ops.grouped_gemm(dev(r["offsets"][:2]), dev(j[:n_small]), dev(w[:1]), total_rows=n_small,
                                 bias=dev(b[:1]), a_silu=True)
    assert torch.equal(rows, rows2)
    assert_bf16_close(small, rows[:n_small].float(), rtol=1e-2, atol=1e-2, what="staged SiLU on load vs pass + ring")
    scale = ref.abs().max().item()
    assert_bf16_close(out, ref, rtol=1.6e-2, atol=1e-2 * scale, what="silu combine at ring size")


@pytest.mark.parametrize("lens,Din,Dout", [([300, 0, 77, 1000], 64, 32), ([2048, 4096], 256, 512)])
def test_silu_jagged_bmm_fp8(lens, Din, Dout):
    """moe_fp8.silu_jagged_bmm_fp8 (weight [E, D_out, D_in]): SiLU + row quantisation of the rows,
    row quantisation of the weight, fp8 GEMM + bias, against the same composition of the oracle's
    pieces (kernels/pytorch/moe_fp8.py:17-33, 127-137) and, loosely, the unquantised result the
    reference's PyTorch path returns (:46-75); the second call hits the weight cache."""
    from fast_moe_amd.kernels import moe_fp8
    from oracle import fp8 as o_q
    E, R = len(lens), sum(lens)
    offsets = torch.tensor([0] + lens).cumsum(0)
    j = randn((R, Din), 1)
    w = randn((E, Dout, Din), 2, scale=Din ** -0.5)
    b = randn((E, Dout), 3)
    qa, sa = o_q.silu_rowwise_quant_fp8(j.float().numpy(), "bf16")
    qw, sw = o_q.rowwise_quant_fp8(w.float().numpy(), "bf16")
    qa_f, qw_f = torch.from_numpy(o_q.e4m3fn_decode(qa)), torch.from_numpy(o_q.e4m3fn_decode(qw))
    rows = [qa_f[offsets[e]:offsets[e + 1]] for e in range(E)]
    srow = [torch.from_numpy(sa)[offsets[e]:offsets[e + 1]] for e in range(E)]
    ref = torch.cat(o_fp8.fp8_linear_per_expert(rows, srow, qw_f, torch.from_numpy(sw), b, BF16), dim=0)
    with torch.no_grad():
        out = moe_fp8.silu_jagged_bmm_fp8(dev(offsets), 0, dev(j), dev(w), dev(b))
        again = moe_fp8.silu_jagged_bmm_fp8(dev(offsets), 0, dev(j), dev(w), dev(b))
    assert torch.equal(out, again)
    scale = ref.float().abs().max().item()
    assert_bf16_close(out, ref.float(), rtol=1e-2, atol=1e-2 * scale, what="silu_jagged_bmm_fp8")
    raw = torch.cat([torch.nn.functional.silu(j[offsets[e]:offsets[e + 1]].float()) @ w[e].float().T + b[e].float()
                     for e in range(E)])
    assert (out.float().cpu() - raw).abs().max().item() <= 0.1 * scale


@pytest.mark.parametrize("swiglu", [False, True])
@pytest.mark.parametrize("M", [96, 8192])
def test_fp8_weight_scales_at_any_alignment(M, swiglu):
    """The e4m3 epilogue loads a register quad's 4 weight scales at once when the scale tensors sit
    on 16-byte boundaries and one by one otherwise: both give the same bits."""
    from fast_moe_amd.kernels.hip import ops
    E, K, N = 8, 512, 512
    g = torch.Generator().manual_seed(77 + M)
    a = torch.randn(M, K, generator=g).to(BF16).cuda()
    w = [torch.randn(E * N, K, generator=g).to(BF16).cuda() for _ in range(2)]
    offsets = (torch.arange(E + 1, dtype=torch.int64) * (M // E)).cuda()
    qa, sa = ops.quant_rows_fp8(a)
    (qb, sb), (qb2, sb2) = ops.quant_rows_fp8(w[0]), ops.quant_rows_fp8(w[1])
    # make the scales differ from column to column by more than the quantiser's choice does
    sb = sb * torch.tensor([1.0, 2.0, 0.5, 4.0], device="cuda").repeat(E * N // 4)
    sb2 = sb2 * torch.tensor([0.25, 1.0, 8.0, 2.0], device="cuda").repeat(E * N // 4)

    def run(shift):
        def place(s):
            buf = torch.zeros(E * N + 4, device="cuda")
            buf[shift:shift + E * N] = s
            return buf[shift:shift + E * N].view(E, N)
        kw = dict(total_rows=M, a_scale=sa, b_scale=place(sb))
        if swiglu:
            kw.update(b2=qb2.view(E, N, K).permute(0, 2, 1), b2_scale=place(sb2), epilogue=ops.EPI_SWIGLU)
        return ops.grouped_gemm(offsets, qa, qb.view(E, N, K).permute(0, 2, 1), **kw)

    aligned = run(0)
    assert aligned.float().abs().max() > 0
    for shift in (1, 2, 3):
        assert torch.equal(run(shift), aligned)


@pytest.mark.parametrize("epi", ["none", "silu", "swiglu"])
@pytest.mark.parametrize("M", [96, 8192])
def test_bias_at_any_alignment(M, epi):
    """Bias tensors at any 2-byte alignment and with any expert pitch give the same bits."""
    from fast_moe_amd.kernels.hip import ops
    E, K, N = 8, 256, 512
    g = torch.Generator().manual_seed(5 + M)
    a = torch.randn(M, K, generator=g).to(BF16).cuda()
    w = [(torch.randn(E, K, N, generator=g) / 16).to(BF16).cuda() for _ in range(2)]
    bias = [torch.randn(E, N, generator=g).to(BF16).cuda() for _ in range(2)]
    offsets = (torch.arange(E + 1, dtype=torch.int64) * (M // E)).cuda()

    def run(shift, pitch):
        def place(b):
            buf = torch.zeros(E * pitch + 8, dtype=BF16, device="cuda")
            v = buf[shift:shift + E * pitch].view(E, pitch)[:, :N]
            v.copy_(b)
            return v
        kw = dict(total_rows=M, bias=place(bias[0]))
        if epi == "swiglu":
            kw.update(b2=w[1], bias2=place(bias[1]), epilogue=ops.EPI_SWIGLU)
        elif epi == "silu":
            kw.update(epilogue=ops.EPI_SILU)
        return ops.grouped_gemm(offsets, a, w[0], **kw)

    aligned = run(0, N)
    ref = a[:M // E].float() @ w[0][0].float() + bias[0][0].float()
    if epi == "none":
        torch.testing.assert_close(aligned[:M // E].float(), ref.to(BF16).float(), atol=3e-2, rtol=1.6e-2)
    for shift, pitch in ((1, N), (2, N), (3, N), (0, N + 2), (4, N + 4)):
        assert torch.equal(run(shift, pitch), aligned), (shift, pitch)


@pytest.mark.parametrize("rows", [256, 64])
def test_accumulation_error_stays_under_the_floors_the_stage_checks_use(rows):
    """The absolute-error floors of tests/chain.py (BF16_FLOOR = 2^-18, FP8_FLOOR = 2^-14 of
    S = sum |a||b|) rest on a measurement: on outputs that are small by cancellation, where the final
    bf16 rounding is out of the way, the GEMMs' error against float64 is a fraction of S that
    depends on how the MFMA adds (e4m3: 64 products per instruction in a block-aligned adder that
    keeps fewer bits than an fp32 sum).  One expert, 1536-term sums, operands that are exactly
    representable in both types; rows = 256 runs the ring kernel, 64 the short streaming tile.
    Asserted: both stay a factor 4 under their floor, and e4m3 does accumulate less exactly than bf16."""
    from fast_moe_amd.kernels.hip import ops
    from tests.chain import BF16_FLOOR, FP8_FLOOR
    torch.manual_seed(0)
    K, N = 1536, 4096
    a = torch.randn(rows, K, device="cuda").to(BF16)
    w = (torch.randn(1, N, K, device="cuda") * K ** -0.5).to(BF16)
    qa, sa = ops.quant_rows_fp8(a)
    qw, sw = ops.quant_rows_fp8(w)
    off = torch.tensor([0, rows], device="cuda")
    out8 = ops.grouped_gemm(off, qa, qw.permute(0, 2, 1), total_rows=rows, a_scale=sa, b_scale=sw.reshape(1, N))
    da, dw = qa.float(), qw.float()
    scale = sa.double()[:, None] * sw[0].double()[None, :]
    exact = (da.double() @ dw[0].double().T) / scale
    S = (da.double().abs() @ dw[0].double().abs().T) / scale
    # the same values through the bf16 kernel: exact products, fp32 accumulation
    out16 = ops.grouped_gemm(off, da.to(BF16), dw.to(BF16).permute(0, 2, 1), total_rows=rows)
    exact16 = da.double() @ dw[0].double().T
    S16 = da.double().abs() @ dw[0].double().abs().T
    small8, small16 = exact.abs() < 2.0 ** -12 * S, exact16.abs() < 2.0 ** -12 * S16
    assert int(small8.sum()) > 100 and int(small16.sum()) > 100
    worst8 = ((out8.double() - exact).abs()[small8] / S[small8]).max().item()
    worst16 = ((out16.double() - exact16).abs()[small16] / S16[small16]).max().item()
    # (each such output also carries half a bf16 ulp of itself: below 2^-21 of S by the selection)
    assert worst16 <= BF16_FLOOR / 4, f"bf16 accumulation error {worst16:.3g} of S"
    assert worst8 <= FP8_FLOOR / 4, f"e4m3 accumulation error {worst8:.3g} of S"
    assert worst8 > worst16


@pytest.mark.parametrize("E,rows,K,N,epi,bias,gather", [
    (8, 4096, 2048, 1408, 2, False, True),        # SwiGLU, gathered rows, last column tile partial
    (8, 4096, 1408, 2048, 0, False, False),       # plain epilogue, rows in place
    (8, 3000, 512, 512, 1, True, True),           # SiLU with bias
    (128, 40000, 1024, 768, 2, True, True),       # the register-table variant for up to 256 experts
    (6, 700, 256, 256, 0, True, False),           # short experts: tiles that run the shortened loop
])
def test_scales_applied_by_the_mfma_equal_scales_divided_out_in_the_epilogue(E, rows, K, N, epi, bias, gather):
    """fmoe_gemm_desc.scale_pow2: with power-of-two scales the ring kernel lets the MFMA apply them
    (E8M0 block scales) instead of dividing them out in its epilogue.  A power-of-two factor on
    every product of an output element commutes with the fp32 accumulation, so the two paths must
    agree bit for bit, also with rows and columns whose scales differ by 2^20 and with the scale of
    an all-zero row (2^127)."""
    from fast_moe_amd.kernels.hip import _lib, ops
    g = torch.Generator().manual_seed(E * 7 + rows)
    T = rows // 2 if gather else rows
    x = torch.randn(T, K, generator=g)
    x[::7] *= 300.0                     # other row scales
    x[5] = 0.0                          # scale 2^127
    x[::11] *= 2.0 ** -12
    w = torch.randn(E, N, K, generator=g) * K ** -0.5
    w[:, ::5] *= 64.0                   # other column scales
    w[:, 3] = 0.0
    w2 = torch.randn(E, N, K, generator=g) * K ** -0.5
    qx, sx = ops.quant_rows_fp8(x.to(BF16).cuda())
    qw, sw = ops.quant_rows_fp8(w.to(BF16).cuda())
    qw2, sw2 = ops.quant_rows_fp8(w2.to(BF16).cuda())
    cuts = torch.sort(torch.randint(0, rows, (E - 1,), generator=g)).values
    if E == 6:
        cuts = torch.tensor([100, 228, 357, 390, 650])          # 100, 128, 129, 33, 260, 50 rows
    offsets = torch.cat([torch.zeros(1, dtype=torch.int64), cuts.to(torch.int64), torch.tensor([rows])]).cuda()
    kw = dict(total_rows=rows, a_scale=sx, b_scale=sw, epilogue=epi)
    if gather:
        kw.update(row_index=torch.randint(0, T * 2, (rows,), generator=g).cuda(), index_div=2)
    if epi == 2:
        kw.update(b2=qw2.permute(0, 2, 1), b2_scale=sw2)
    if bias:
        kw.update(bias=torch.randn(E, N, generator=g).to(BF16).cuda())
        if epi == 2:
            kw.update(bias2=torch.randn(E, N, generator=g).to(BF16).cuda())
    assert ops.grouped_gemm(offsets, qx, qw.permute(0, 2, 1), plan_only=True, scales_pow2=True, **kw) == _lib.PLAN_RING
    plain = ops.grouped_gemm(offsets, qx, qw.permute(0, 2, 1), scales_pow2=False, **kw)
    folded = ops.grouped_gemm(offsets, qx, qw.permute(0, 2, 1), scales_pow2=True, **kw)
    again = ops.grouped_gemm(offsets, qx, qw.permute(0, 2, 1), scales_pow2=True, **kw)
    assert torch.isfinite(plain.float()).all()
    assert torch.equal(folded.view(torch.int16), plain.view(torch.int16))
    assert torch.equal(again.view(torch.int16), folded.view(torch.int16))
