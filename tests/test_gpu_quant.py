"""GPU parity: FP8 row-wise scales and quantised bytes bit-exact against the oracle."""
import numpy as np
import pytest
import torch

from oracle import fp8 as o_fp8

pytestmark = pytest.mark.gpu

NAME = {torch.bfloat16: "bf16", torch.float32: "fp32"}


def check_quant(a, transpose=False, both_nan_ok=False):
    from fast_moe_amd.kernels import moe_fp8
    src = a.transpose(-2, -1) if transpose else a
    q_ref, s_ref = o_fp8.rowwise_quant_fp8(src.float().numpy(), NAME[a.dtype])
    fn = moe_fp8.transpose_rowwise_quant_fp8 if transpose else moe_fp8.rowwise_quant_fp8
    q, s = fn(a.cuda())
    torch.cuda.synchronize()
    assert q.dtype == torch.float8_e4m3fn and q.is_contiguous() and s.is_contiguous()
    assert tuple(q.shape) == q_ref.shape and tuple(s.shape) == s_ref.shape
    assert np.array_equal(s.cpu().numpy(), s_ref), "scales differ"
    got = q.view(torch.uint8).cpu().numpy()
    if both_nan_ok:   # the sign of a NaN code is not defined by the arithmetic (inf * 0)
        nan = (q_ref & 0x7F) == 0x7F
        assert np.array_equal((got & 0x7F) == 0x7F, nan)
        assert np.array_equal(got[~nan], q_ref[~nan])
    else:
        assert np.array_equal(got, q_ref), f"{np.sum(got != q_ref)} bytes differ"
    return q, s


@pytest.mark.parametrize("shape", [(32, 16), (32, 8, 16), (7, 9, 13), (51, 5)])
@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("contiguous", [True, False])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_reference_shapes(shape, transpose, contiguous, dtype):
    """The grid of kernels/tests/quant_fp8_test.py:25-33."""
    print(f"quant {shape} T={transpose} contiguous={contiguous} {dtype}", flush=True)
    g = torch.Generator().manual_seed(sum(shape) + transpose)
    a = torch.randn(shape, generator=g).to(dtype)
    if not contiguous:
        a = a.transpose(-2, -1).contiguous().transpose(-2, -1)
    check_quant(a, transpose)


@pytest.mark.parametrize("rows,cols", [(64, 8), (100, 512), (257, 1408), (300, 2048), (64, 4096), (33, 6000),
                                       (16, 8192), (5, 8200), (9, 20000), (7, 140032), (3, 9001)])
def test_wave_per_row_path_and_beyond(rows, cols):
    g = torch.Generator().manual_seed(rows + cols)
    a = (torch.randn(rows, cols, generator=g) * torch.exp(torch.randn(rows, 1, generator=g) * 4)).to(torch.bfloat16)
    a[:: 17] *= 100                       # outlier rows
    check_quant(a)


def test_full_size_tokens_and_outliers():
    """Config C4: 16384 x 2048 bf16 tokens, 1 % of the rows scaled x100."""
    g = torch.Generator().manual_seed(0)
    a = torch.randn(16384, 2048, generator=g)
    rows = torch.randperm(16384, generator=g)[:164]
    a[rows] *= 100
    a = a.to(torch.bfloat16)
    q, s = check_quant(a)
    # size-independent properties: power-of-two scales, amax lands in (224, 448], round trip bound
    sc = s.cpu().double()
    m, _ = np.frexp(sc.numpy())
    assert np.all(m == 0.5)
    amax = a.float().abs().amax(dim=1).double()
    prod = amax * sc
    assert bool(((prod > 224) & (prod <= 448)).all())
    deq = q.cpu().float() / s.cpu()[:, None]
    assert bool(((deq - a.float()).abs() <= a.float().abs() * 2.0 ** -4 + 2.0 ** -10 / s.cpu()[:, None]).all())


def test_special_rows():
    a = torch.zeros(8, 64)
    a[1, 3] = float("inf")
    a[2, 5] = float("nan")
    a[3] = 1e-40
    a[4, 7] = -3.0e38
    a[5] = torch.linspace(-1, 1, 64) * 1e-30
    a[6, 0] = 2.0 ** -126
    a[7] = torch.linspace(-448, 448, 64)
    check_quant(a, both_nan_ok=True)
    check_quant(a.to(torch.bfloat16), both_nan_ok=True)
    wide = torch.zeros(4, 512)
    wide[1, 100] = float("inf")
    wide[2, 7] = float("nan")
    wide[3] = torch.linspace(-5, 5, 512)
    check_quant(wide.to(torch.bfloat16), both_nan_ok=True)


def test_long_rows_special_values_and_silu():
    """Rows longer than a wave keeps in registers (one block per row, two passes)."""
    g = torch.Generator().manual_seed(3)
    a = torch.randn(6, 16384, generator=g)
    a[1, 9000] = float("inf")
    a[2, 16383] = float("nan")
    a[3] = 0
    a[4, 5] = -3.0e38
    check_quant(a.to(torch.bfloat16), both_nan_ok=True)
    from fast_moe_amd.kernels.hip import ops
    from oracle import fp8 as o_fp8
    x = torch.randn(5, 12288, generator=g).to(torch.bfloat16)
    q, sc = ops.quant_rows_fp8(x.cuda(), apply_silu=True)
    ref_q, ref_s = o_fp8.silu_rowwise_quant_fp8(x.float().numpy(), "bf16")
    assert np.array_equal(q.cpu().view(torch.uint8).numpy(), ref_q)
    assert np.array_equal(sc.cpu().numpy(), ref_s)


def test_fp32_scale_near_power_of_two_follows_reference_formula():
    """448/amax just below 2^n: the fp32 log2 of the formula rounds up to n."""
    n = np.arange(-20, 21)
    q = np.nextafter((2.0 ** n).astype(np.float32), np.float32(0))
    amax = (np.float32(448.0) / q).astype(np.float32)
    a = torch.zeros(len(n) * 3, 8)
    for i, v in enumerate(np.concatenate([amax, np.nextafter(amax, np.float32(0)),
                                          np.nextafter(amax, np.float32(1e30))])):
        a[i, i % 8] = float(v)
    check_quant(a)


def test_exhaustive_bf16_amax_scales():
    """Every positive finite bf16 value as the row maximum."""
    bits = (torch.arange(1, 0x7F80, dtype=torch.int32) << 16)
    amax = bits.view(torch.float32).to(torch.bfloat16)
    a = torch.zeros(amax.numel(), 8, dtype=torch.bfloat16)
    a[:, 3] = amax
    a[:, 5] = -amax / 3
    check_quant(a)


def test_bf16_silu_is_bit_exact_on_every_input():
    """All 65536 bf16 inputs through the element-wise SiLU kernel (the device function the SiLU
    quantiser shares) against the oracle, NaN payloads aside; then the quantiser itself on rows
    that hold every input."""
    from fast_moe_amd.kernels import moe_fp8
    from fast_moe_amd.kernels.hip import ops
    bits = (torch.arange(65536, dtype=torch.int32) << 16)
    x = bits.view(torch.float32).to(torch.bfloat16)
    want = o_fp8.silu_bf16(x.float().numpy())
    got = ops.silu_mul(x.cuda(), None).float().cpu().numpy()
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))
    assert np.all(np.isnan(got[~ok]))
    # the finite inputs as 62 rows of 1024 columns (sorted by magnitude, so that rows of small
    # values keep their resolution): bytes and nothing else come back from silu_jagged_fp8
    fin = x[torch.isfinite(x.float())]
    fin = fin[torch.argsort(fin.float().abs(), stable=True)]
    rows = fin[: fin.numel() // 1024 * 1024].reshape(-1, 1024)
    q_ref, _ = o_fp8.silu_rowwise_quant_fp8(rows.float().numpy(), "bf16")
    dummy = torch.empty(0)
    n = rows.shape[0]
    q = moe_fp8.silu_jagged_fp8(torch.tensor([0, n]).cuda(), rows.cuda(), n, 1024, dummy, dummy, dummy)
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), q_ref)


def test_silu_quant_and_weight_quant():
    from fast_moe_amd.kernels import moe_fp8
    g = torch.Generator().manual_seed(2)
    j = (torch.randn(200, 1408, generator=g) * 3).to(torch.bfloat16)
    q_ref, s_ref = o_fp8.silu_rowwise_quant_fp8(j.float().numpy(), "bf16")
    dummy = torch.empty(0)
    q = moe_fp8.silu_jagged_fp8(torch.tensor([0, 200]).cuda(), j.cuda(), 200, 1408, dummy, dummy, dummy)
    got = q.view(torch.uint8).cpu().numpy()
    assert np.array_equal(got, q_ref)       # SiLU is rounded to bf16 identically on both sides

    w = torch.randn(4, 48, 40, generator=g).to(torch.bfloat16)
    qw_ref, _ = o_fp8.bmm_weight_rowwise_quant_fp8(w.float().numpy(), "bf16")
    qw = moe_fp8.bmm_weight_rowwise_quant_fp8(w.cuda())
    assert tuple(qw.shape) == (4, 48, 40)
    assert np.array_equal(qw.view(torch.uint8).cpu().numpy(), qw_ref)
    # strided [E, K, N] view of [E, N, K] storage
    wt = w.transpose(1, 2).contiguous().transpose(1, 2)
    qw2 = moe_fp8.bmm_weight_rowwise_quant_fp8(wt.cuda())
    assert np.array_equal(qw2.view(torch.uint8).cpu().numpy(), qw_ref)
    q3, s3 = moe_fp8.quantize_expert_weights(w.cuda())
    q3_ref, s3_ref = o_fp8.rowwise_quant_fp8(w.permute(0, 2, 1).float().numpy(), "bf16")
    assert np.array_equal(q3.permute(0, 2, 1).contiguous().view(torch.uint8).cpu().numpy(), q3_ref)
    assert np.array_equal(s3.cpu().numpy(), s3_ref)


def test_fp8_operators_requantise_every_call_and_take_a_kept_pair():
    """The fp8 operators quantise their weight on every call, as the reference does
    (kernels/pytorch/moe_fp8.py:111): updates the version counter cannot see -- writes through
    ``.data``, an optimizer step -- are picked up.  The kept pair is opt-in (``fp8_weight=``)."""
    from fast_moe_amd.kernels import moe_fp8
    from helpers import make_routing, randn
    r = make_routing(512, 8, 2, seed=5)
    x = randn((512, 128), 1).cuda()
    w = torch.nn.Parameter((randn((8, 128, 96), 2) * 128 ** -0.5).cuda())
    off, idx = r["offsets"].cuda(), r["index"].cuda()
    cache = moe_fp8.weight_quant_cache
    cache.clear()
    h0, m0 = cache.hits, cache.misses
    with torch.no_grad():
        y1 = moe_fp8.index_select_jagged_bmm(0, off, idx, x, w, None, fp8=True)
        w.data.mul_(2.0)                                  # invisible to w._version
        y2 = moe_fp8.index_select_jagged_bmm(0, off, idx, x, w, None, fp8=True)
        torch.testing.assert_close(y2.float(), 2 * y1.float(), rtol=0, atol=0)   # a power of two: exact
        assert (cache.hits - h0, cache.misses - m0) == (0, 0)                    # the operator does not cache
        # the kept pair: same bits as the default path, until the weight moves
        pair = moe_fp8.cached_quantize_expert_weights(w)
        assert moe_fp8.cached_quantize_expert_weights(w)[0] is pair[0]
        y3 = moe_fp8.index_select_jagged_bmm(0, off, idx, x, w, None, fp8=True, fp8_weight=pair)
        assert torch.equal(y3, y2)
    opt = torch.optim.SGD([w], lr=0.5)
    w.grad = torch.ones_like(w) * 0.01
    opt.step()                                            # an in-place update: the version counter moves
    with torch.no_grad():
        pair2 = moe_fp8.cached_quantize_expert_weights(w)
        assert pair2[0] is not pair[0]
        y4 = moe_fp8.index_select_jagged_bmm(0, off, idx, x, w, None, fp8=True)
        y5 = moe_fp8.index_select_jagged_bmm(0, off, idx, x, w, None, fp8=True, fp8_weight=pair2)
        assert torch.equal(y4, y5) and not torch.equal(y4, y2)
        fresh = moe_fp8.quantize_expert_weights(w)
        assert torch.equal(fresh[0].view(torch.uint8), pair2[0].view(torch.uint8)) and torch.equal(fresh[1], pair2[1])
        # a write through .data leaves the cache stale until it is invalidated
        w.data.mul_(2.0)
        assert moe_fp8.cached_quantize_expert_weights(w)[0] is pair2[0]
        cache.invalidate(w)
        assert torch.equal(moe_fp8.cached_quantize_expert_weights(w)[1], pair2[1] * 0.5)
    with pytest.raises(ValueError):
        moe_fp8.index_select_jagged_bmm(0, off, idx, x, w, None, fp8=True, fp8_weight=(pair[0][:4], pair[1]))
