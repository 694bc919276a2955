"""GPU parity of the SGMoE / MRN front-end: the softmax gate modes of fmoe_route_topk against
torch on the CPU, and the SGMoE layer against oracle/mrn.py (the original dense-dispatch layer)."""
import pytest
import torch
import torch.nn.functional as F

from oracle import mrn as o_mrn

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("T,E,K", [(300, 8, 2), (257, 64, 8), (100, 130, 5), (64, 16, 16)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("post", [False, True])
def test_softmax_gate_modes(T, E, K, dtype, post):
    from fast_moe_amd.kernels.hip import ops
    g = torch.Generator().manual_seed(T + E)
    logits = torch.randn(T, E, generator=g).to(dtype)
    logits[0] = 0                                   # zero row: norm clamps to eps, all ties
    logits[1, : E // 2] = logits[1, 0]              # ties: lower expert id first
    n = F.normalize(logits, dim=1)
    order = n.sort(descending=True, dim=1, stable=True)
    idx = order.indices[:, :K]
    if post and K > 1:
        ref = F.softmax(order.values[:, :K], dim=1)
    else:
        ref = F.softmax(order.values, dim=1)[:, :K]
    mode = ops.GATE_SOFTMAX_TOPK if (post and K > 1) else ops.GATE_SOFTMAX_ALL
    r = ops.route_topk(logits.cuda(), K, renorm=mode)
    assert torch.equal(r["topk_idx"].cpu(), idx), "selection order differs"
    assert r["gates"].dtype == dtype
    tol = dict(rtol=2e-6, atol=1e-7) if dtype == torch.float32 else dict(rtol=8e-3, atol=1e-6)
    torch.testing.assert_close(r["gates"].cpu().float(), ref.float(), **tol)


def make_layer(D, H, O, E, k, noisy, dtype):
    from fast_moe_amd.modules.sgmoe import SGConfig, SGMoE
    torch.manual_seed(0)
    layer = SGMoE(D, O, False, 1, SGConfig(model_d=H, num_experts=E, num_activated_experts=k,
                                           enable_noisy_gating=noisy))
    with torch.no_grad():
        for name, prm in layer.named_parameters():
            if name in ("_w_gate", "_w_noise"):
                prm.normal_(0, D ** -0.5)
            elif "bias" in name:
                prm.normal_(0, 0.1)
    return layer.to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_sgmoe_inference_matches_oracle(dtype):
    D, H, O, E, k, T = 64, 96, 48, 8, 2, 512
    layer = make_layer(D, H, O, E, k, False, dtype).eval()
    x = torch.randn(T, D, generator=torch.Generator().manual_seed(1)).to(dtype)
    p = {n: t.detach().clone() for n, t in layer.named_parameters()}
    y_ref, loss_ref, load_ref = o_mrn.sgmoe_forward(p, x, k, train=False)
    with torch.no_grad():
        out = layer.cuda()(x.cuda())
    if dtype == torch.float32:
        torch.testing.assert_close(out.x.cpu(), y_ref, rtol=1e-4, atol=1e-5)
    else:
        torch.testing.assert_close(out.x.cpu().float(), y_ref.float(), rtol=3e-2, atol=3e-2)
    assert out.loss.item() == 0
    torch.testing.assert_close(out.load.cpu(), load_ref)


@pytest.mark.parametrize("noisy", [False, True])
def test_sgmoe_training_loss_and_gradients(noisy):
    D, H, O, E, k, T = 32, 64, 32, 8, 2, 256
    layer = make_layer(D, H, O, E, k, noisy, torch.float32).train()
    g = torch.Generator().manual_seed(2)
    x0 = torch.randn(T, D, generator=g)
    noise = torch.randn(T, E, generator=g) if noisy else None
    dy = torch.randn(T, O, generator=g) * 0.01
    p = {n: t.detach().clone().requires_grad_(True) for n, t in layer.named_parameters()}
    xr = x0.clone().requires_grad_(True)
    y_ref, loss_ref, _ = o_mrn.sgmoe_forward(p, xr, k, train=True, noisy=noisy, noise=noise)
    ((y_ref * dy).sum() + loss_ref).backward()
    layer = layer.cuda()
    x = x0.cuda().requires_grad_(True)
    out = layer(x, None if noise is None else noise.cuda())
    torch.testing.assert_close(out.x.detach().cpu(), y_ref.detach(), rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(out.loss.detach().cpu(), loss_ref.detach(), rtol=1e-4, atol=1e-7)
    ((out.x * dy.cuda()).sum() + out.loss).backward()
    torch.testing.assert_close(x.grad.cpu(), xr.grad, rtol=2e-3, atol=1e-5)
    for n, prm in layer.named_parameters():
        ref = p[n].grad if p[n].grad is not None else torch.zeros_like(p[n])
        got = prm.grad if prm.grad is not None else torch.zeros_like(prm)
        torch.testing.assert_close(got.cpu(), ref, rtol=2e-3, atol=1e-5, msg=lambda m, n=n: f"{n}: {m}")
