"""Pins oracle.fp8 against the torch library routines the reference calls and
against what the format fixes mathematically."""
import numpy as np
import pytest
import torch

from oracle import fp8
from oracle.routing import round_to_bf16


def torch_calculate_scale(a_max: torch.Tensor) -> torch.Tensor:
    """The formula of kernels/pytorch/quant_fp8.py:13-24 in plain torch ops."""
    s = torch.div(448.0, a_max).to(torch.float32)
    s = torch.exp2(torch.floor(torch.log2(s)))
    bad = (s != s) | (s == float("inf")) | (s == float("-inf"))
    return torch.where(bad, 2.0 ** 127, s)


def all_positive_bf16():
    bits = np.arange(1, 0x7F80, dtype=np.uint32) << 16     # every positive finite bf16
    return bits.view(np.float32)


def test_decode_table_matches_torch():
    codes = torch.arange(256, dtype=torch.uint8)
    ref = codes.view(torch.float8_e4m3fn).float().numpy()
    mine = fp8.e4m3fn_decode_table()
    assert np.array_equal(np.isnan(ref), np.isnan(mine))
    ok = ~np.isnan(ref)
    assert np.array_equal(ref[ok], mine[ok])
    assert np.nanmax(mine) == 448.0


def test_encode_round_trips_every_code():
    table = fp8.e4m3fn_decode_table()
    codes = np.arange(256, dtype=np.uint8)
    finite = ~np.isnan(table)
    assert np.array_equal(fp8.e4m3fn_encode(table[finite]), codes[finite])


def test_encode_matches_torch_cast_dense_sweep():
    g = torch.Generator().manual_seed(0)
    x = torch.cat([
        torch.randn(400000, generator=g) * 200,
        torch.randn(200000, generator=g) * 2.0 ** -7,
        torch.linspace(-500, 500, 200001),
        torch.tensor([0.0, -0.0, 448.0, 464.0, 464.0001, 479.9, 480.0, 1e9, -1e9,
                      float("inf"), float("-inf"), float("nan"), 2.0 ** -10, 2.0 ** -9,
                      1.5 * 2.0 ** -10, 2.5 * 2.0 ** -10, 0.9999 * 2.0 ** -6]),
    ])
    # midpoints between neighbouring codes: the ties-to-even cases
    t = fp8.e4m3fn_decode_table()[:0x7F].astype(np.float64)
    mids = torch.tensor(((t[:-1] + t[1:]) / 2).astype(np.float32))
    x = torch.cat([x, mids, -mids])
    ref = x.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    mine = fp8.e4m3fn_encode(x.numpy())
    assert np.array_equal(ref, mine)


def test_scale_exhaustive_over_bf16_amax():
    amax = all_positive_bf16()
    ref_bf16 = torch_calculate_scale(torch.from_numpy(amax).to(torch.bfloat16)).numpy()
    ref_fp32 = torch_calculate_scale(torch.from_numpy(amax)).numpy()
    assert np.array_equal(fp8.calculate_scale(amax, "bf16"), ref_bf16)
    assert np.array_equal(fp8.calculate_scale(amax, "fp32"), ref_fp32)
    # dividing in bf16 or in fp32 gives the same power of two for bf16 inputs
    assert np.array_equal(ref_bf16, ref_fp32)
    s = ref_fp32.astype(np.float64)
    m, _ = np.frexp(s)
    assert np.all(m == 0.5)                                  # powers of two
    unclamped = s < 2.0 ** 127
    prod = amax.astype(np.float64) * s
    assert np.all((prod[unclamped] > 224) & (prod[unclamped] <= 448))
    assert np.all(prod[~unclamped] <= 448)


def test_scale_fp32_dense_sample_and_specials():
    g = torch.Generator().manual_seed(3)
    amax = (torch.randn(300000, generator=g).abs() * torch.exp(torch.randn(300000, generator=g) * 20))
    amax = amax[amax > 0]
    assert np.array_equal(fp8.calculate_scale(amax.numpy(), "fp32"),
                          torch_calculate_scale(amax).numpy())
    sp = torch.tensor([0.0, float("inf"), float("nan"), 1e-45, 3.4e38, 448.0, 1.0])
    got = fp8.calculate_scale(sp.numpy(), "fp32")
    assert np.array_equal(got, torch_calculate_scale(sp).numpy())
    assert got[0] == 2.0 ** 127 and got[1] == 0.0 and got[2] == 2.0 ** 127 and got[5] == 1.0


@pytest.mark.parametrize("shape", [(32, 16), (32, 8, 16), (7, 9, 13), (51, 5), (4, 2048)])
@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
def test_rowwise_quant_against_torch_ops(shape, dtype):
    """kernels/pytorch/quant_fp8.py:27-34 spelled with torch ops (shapes of
    kernels/tests/quant_fp8_test.py:25)."""
    tdt = torch.bfloat16 if dtype == "bf16" else torch.float32
    g = torch.Generator().manual_seed(sum(shape))
    a = torch.randn(shape, generator=g).to(tdt)
    a.view(-1)[:: 97] *= 100
    a_max, _ = torch.max(torch.abs(a), dim=-1)
    s_ref = torch_calculate_scale(a_max)
    q_ref = (a * s_ref.unsqueeze(-1)).to(torch.float8_e4m3fn).view(torch.uint8)
    q, s = fp8.rowwise_quant_fp8(a.float().numpy(), dtype)
    assert np.array_equal(s, s_ref.numpy())
    assert np.array_equal(q, q_ref.numpy())
    # round trip: dequantised value within half a quantum of the input
    deq = fp8.e4m3fn_decode(q) / s[..., None]
    err = np.abs(deq - a.float().numpy())
    assert np.all(err <= np.abs(a.float().numpy()) * 2.0 ** -4 + 2.0 ** -10 / s[..., None])
    # transpose variant (quant_fp8.py:37-40)
    if len(shape) >= 2:
        qt, st = fp8.transpose_rowwise_quant_fp8(a.float().numpy(), dtype)
        at = a.transpose(-2, -1).contiguous()
        amt, _ = torch.max(torch.abs(at), dim=-1)
        assert np.array_equal(st, torch_calculate_scale(amt).numpy())
        assert qt.shape == tuple(at.shape)


def test_rowwise_quant_zero_and_nonfinite_rows():
    a = np.zeros((4, 8), dtype=np.float32)
    a[1, 3] = np.inf
    a[2, 5] = np.nan
    a[3] = 1e-40
    ta = torch.from_numpy(a)
    a_max, _ = torch.max(torch.abs(ta), dim=-1)
    s_ref = torch_calculate_scale(a_max)
    q_ref = (ta * s_ref.unsqueeze(-1)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    q, s = fp8.rowwise_quant_fp8(a, "fp32")
    assert np.array_equal(s, s_ref.numpy())
    assert np.array_equal(q, q_ref)


def test_bmm_weight_quant_against_torch_ops():
    """kernels/pytorch/moe_fp8.py:36-43."""
    g = torch.Generator().manual_seed(5)
    w = torch.randn(4, 16, 32, generator=g).to(torch.bfloat16)
    wm, _ = torch.max(torch.abs(w), dim=1)
    s_ref = torch_calculate_scale(wm)
    q_ref = (w * s_ref[:, None, :]).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    q, s = fp8.bmm_weight_rowwise_quant_fp8(w.float().numpy(), "bf16")
    assert np.array_equal(s, s_ref.numpy()) and np.array_equal(q, q_ref)


def test_silu_quant_against_torch_ops():
    """kernels/pytorch/moe_fp8.py:17-33 (bf16 SiLU, fp32 scale path)."""
    g = torch.Generator().manual_seed(6)
    j = (torch.randn(64, 48, generator=g) * 3).to(torch.bfloat16)
    sj = torch.nn.functional.silu(j).to(torch.float32)
    m, _ = torch.max(torch.abs(sj), dim=1)
    s_ref = torch_calculate_scale(m)
    q_ref = (sj * s_ref[:, None]).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    q, s = fp8.silu_rowwise_quant_fp8(j.float().numpy(), "bf16")
    assert np.array_equal(s, s_ref.numpy())
    # exp() of two libraries may differ in the last fp32 bit before the bf16 rounding
    assert np.mean(q != q_ref) < 1e-3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_library_cast_path_equals_bit_level_path(dtype):
    """oracle.moe_fp8.rowwise_quant_fp8 has two casts: the bit-level encoder and, for operands of
    10^9 elements, Tensor.to(float8_e4m3fn).  Same codes and scales on random rows, outlier rows,
    zero rows, rows whose scaled values land in the subnormal range, and inf / NaN rows."""
    from oracle import moe_fp8 as o8
    g = torch.Generator().manual_seed(17)
    a = torch.randn(3, 40, 256, generator=g)
    a[0, ::7] *= 100
    a[1, 3] = 0
    a[1, 4, 1:] *= 2.0 ** -12            # one large entry, the rest rounds into subnormals / zero
    a[2, 5, 9] = float("inf")
    a[2, 6, 11] = float("nan")
    a = a.to(dtype)
    qb, sb = o8.rowwise_quant_fp8(a, cast="bits")
    qt, st = o8.rowwise_quant_fp8(a, cast="torch")
    assert torch.equal(sb, st)
    assert torch.equal(qb, qt)
    big = torch.randn(1 << 11, 1 << 11, generator=g).to(dtype)      # above the size switch
    q_auto, s_auto = o8.rowwise_quant_fp8(big)
    q_bits, s_bits = o8.rowwise_quant_fp8(big[:64], cast="bits")
    assert torch.equal(q_auto[:64], q_bits) and torch.equal(s_auto[:64], s_bits)


def test_silu_bf16_is_torch_silu_on_every_bf16_input():
    """All 65536 bf16 bit patterns: the oracle's bf16 SiLU against torch's CPU kernel (the library
    routine the reference calls) and against the fp32 formula with numpy's exp, NaN patterns aside."""
    import torch
    from oracle.routing import round_to_bf16
    bits = (np.arange(65536, dtype=np.uint32) << 16)
    x = bits.view(np.float32)
    got = fp8.silu_bf16(x)
    want = torch.nn.functional.silu(torch.from_numpy(x.copy()).to(torch.bfloat16)).float().numpy()
    ok = ~np.isnan(want)
    assert ok.sum() == 65536 - 2 * 127 - 1 and np.all(np.isnan(got[~ok]))      # NaN inputs and -inf
    assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))
    with np.errstate(all="ignore"):
        f32 = round_to_bf16(fp8.silu_f32(x))
    assert np.array_equal(got[ok].view(np.uint32), f32[ok].view(np.uint32))
    # closed-form anchors: silu(0) = 0, silu(x) = x beyond 2^5 (x e^-x below half a bf16 step), odd part x / 2
    assert got[0] == 0 and got[np.uint32(0x4200)] == 32.0            # 0x4200 = 32.0
    pos, neg = fp8.silu_bf16(np.float32([0.5, 1.0, 3.0])), fp8.silu_bf16(np.float32([-0.5, -1.0, -3.0]))
    assert np.all(np.abs((pos - neg) - np.float32([0.5, 1.0, 3.0])) <= 2.0 ** -7 * np.float32([0.5, 1.0, 3.0]))
