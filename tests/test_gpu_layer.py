"""GPU parity: FastMoELayer and the composed SwiGLU / fp8 forward against the oracle."""
import numpy as np
import pytest
import torch
from torch.nn import functional as F

from oracle import layer as o_layer
from oracle import moe as o_moe
from oracle import moe_fp8 as o_fp8
from tests.helpers import BF16, assert_bf16_close, dev, randn

pytestmark = pytest.mark.gpu


def build_layer(D, H, O, E, seed=0):
    from fast_moe_amd import FastMoELayer
    torch.manual_seed(seed)
    layer = FastMoELayer(D, H, O, E).to(BF16)
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        layer._experts_hidden_w.copy_(torch.randn(E, H, D, generator=g) * D ** -0.5)
        layer._experts_w.copy_(torch.randn(E, O, H, generator=g) * H ** -0.5)
        layer._experts_hidden_bias.copy_(torch.randn(E, H, generator=g) * 0.1)
        layer._experts_bias.copy_(torch.randn(E, O, generator=g) * 0.1)
        layer.gate.gate.weight.copy_(torch.randn(E, D, generator=g) * D ** -0.5)
        layer.gate.gate.bias.zero_()
    return layer


@pytest.mark.parametrize("B,S,D,H,O,E,k", [(4, 8, 16, 32, 16, 4, 1), (8, 16, 32, 16, 32, 8, 2),
                                           (2, 512, 256, 512, 256, 8, 2), (4, 512, 1024, 4096, 1024, 8, 2),
                                           (8, 1024, 1024, 4096, 1024, 8, 2)])    # the last: 8192 tokens
def test_layer_matches_oracle(B, S, D, H, O, E, k):
    """Shapes of modules/tests/test_kernel_parity.py:29-90 plus the plumbing configuration."""
    print(f"layer B={B} S={S} D={D} H={H} O={O} E={E} k={k}", flush=True)
    layer = build_layer(D, H, O, E)
    x = randn((B, S, D), 1)
    sd = {k_: v.detach().clone() for k_, v in layer.state_dict().items()}
    gpu = layer.cuda()
    with torch.no_grad():
        y = gpu(x.cuda(), k)
        scores = gpu.gate(x.cuda()).reshape(-1, E).cpu()
    # the gate GEMM + softmax stay torch calls; feed the oracle the same probabilities so that
    # the comparison covers exactly what the library computes
    r = o_layer.route_scores(scores, k)
    xf = x.reshape(-1, D)
    hidden = o_moe.index_select_jagged_bmm(r["offsets"], r["gate_index"].view(-1, k), xf,
                                           sd["_experts_hidden_w"].permute(0, 2, 1), sd["_experts_hidden_bias"])
    ref = o_moe.silu_jagged_bmm_combine(r["offsets"], hidden, sd["_experts_w"].permute(0, 2, 1),
                                        sd["_experts_bias"], r["token_index"], k, r["gates"], r["gate_index"])
    assert y.dtype == BF16 and tuple(y.shape) == (B, S, O)
    assert_bf16_close(y.reshape(-1, O), ref, rtol=1e-2, atol=1e-2, what="FastMoELayer")
    # and against an fp32-accumulated evaluation of the same routed computation
    h32 = o_moe.index_select_jagged_bmm(r["offsets"], r["gate_index"].view(-1, k), xf.float(),
                                        sd["_experts_hidden_w"].permute(0, 2, 1).float(),
                                        sd["_experts_hidden_bias"].float())
    ref32 = o_moe.silu_jagged_bmm_combine(r["offsets"], h32, sd["_experts_w"].permute(0, 2, 1).float(),
                                          sd["_experts_bias"].float(), r["token_index"], k, r["gates"].float(),
                                          r["gate_index"])
    assert_bf16_close(y.reshape(-1, O), ref32, rtol=2e-2, atol=2e-2, what="FastMoELayer vs fp32")


def test_layer_constant_weights_equals_dense_moe():
    """modules/tests/test_moe_parity.py:72-106: identical experts -> output independent of routing."""
    from fast_moe_amd import FastMoELayer
    torch.manual_seed(42)
    B, S, D, H, O, E, k = 4, 16, 16, 16, 16, 8, 2
    layer = FastMoELayer(D, H, O, E).to(BF16)
    with torch.no_grad():
        for p in layer.parameters():
            p.fill_(0.0625)
    x = randn((B, S, D), 2)
    with torch.no_grad():
        y = layer.cuda()(x.cuda(), k)
    c = lambda *s: torch.full(s, 0.0625)
    ref = o_layer.dense_moe_forward(x.float(), c(E, D), c(E), c(E, H, D), c(E, H), c(E, O, H), c(E, O), k)
    assert_bf16_close(y, ref, rtol=2e-2, atol=1e-2, what="dense parity")


def swiglu_inputs(T, E, K, D, H, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, D, generator=g).to(BF16)
    wg = (torch.randn(E, H, D, generator=g) * D ** -0.5).to(BF16)
    wu = (torch.randn(E, H, D, generator=g) * D ** -0.5).to(BF16)
    wd = (torch.randn(E, D, H, generator=g) * H ** -0.5).to(BF16)
    zipf = torch.log((torch.arange(E, dtype=torch.float32) + 1) ** -1.1)
    logits = torch.randn(T, E, generator=g) + 2.0 * zipf
    scores = F.softmax(logits, dim=1)
    return x, wg, wu, wd, scores


@pytest.mark.parametrize("T,E,K,D,H", [(512, 16, 4, 128, 192), (2048, 64, 8, 256, 352)])
def test_swiglu_moe_bf16_and_fp8_composition(T, E, K, D, H):
    """Configs C3 / C4 at reduced size: routing from skewed scores, SwiGLU GEMM, down GEMM, merge."""
    from fast_moe_amd.kernels import moe, moe_fp8
    from fast_moe_amd.kernels.hip import ops
    x, wg, wu, wd, scores = swiglu_inputs(T, E, K, D, H)
    x[::100] *= 100                     # outlier rows (C4)
    r = o_layer.route_scores(scores, K)
    idx2 = r["gate_index"].view(-1, K)
    gates = r["gates"].to(BF16)
    wg_v, wu_v, wd_v = wg.permute(0, 2, 1), wu.permute(0, 2, 1), wd.permute(0, 2, 1)
    ref16 = o_moe.fused_jagged_bmm_swiglu_combine(r["offsets"], idx2, x, wg_v, None, wu_v, None, wd_v, None, K,
                                                  gates, r["gate_index"])
    ref8, _ = o_fp8.swiglu_moe_fp8(r["offsets"], idx2, x, wg_v, None, wu_v, None, wd_v, None,
                                   r["token_index"], K, gates, r["gate_index"])
    with torch.no_grad():
        rg = ops.route_topk(scores.cuda(), K)
        for key in ("offsets", "gate_index", "token_index", "reverse_index"):
            assert torch.equal(rg[key].cpu().view(-1), r[key].view(-1)), key
        hidden = moe.index_select_jagged_bmm_swiglu(0, rg["offsets"], rg["gate_index"].view(-1, K), dev(x),
                                                    dev(wg_v), None, dev(wu_v), None)
        y16 = moe.silu_jagged_bmm_combine(0, rg["offsets"], hidden, dev(wd_v), None, rg["token_index"],
                                          rg["reverse_index"], dev(gates), rg["gate_index"], has_silu=False)
        # the one-call form of the same chain (kernels/pytorch/moe.py:306-391)
        fused = moe.fused_jagged_bmm_swiglu_combine(rg["offsets"], rg["gate_index"].view(-1, K), dev(x), dev(wg_v), None,
                                                    dev(wu_v), None, dev(wd_v), None, K, dev(gates), rg["gate_index"])
        assert torch.equal(fused, y16)
        # fp8: weights quantised once, activations per call
        qg, sg = moe_fp8.quantize_expert_weights(dev(wg_v))
        qu, su = moe_fp8.quantize_expert_weights(dev(wu_v))
        qd, sd = moe_fp8.quantize_expert_weights(dev(wd_v))
        qx, sx = ops.quant_rows_fp8(dev(x))
        h8 = ops.grouped_gemm(rg["offsets"], qx, qg, total_rows=T * K, row_index=rg["gate_index"], index_div=K,
                              b2=qu, epilogue=2, scales_pow2=True, a_scale=sx, b_scale=sg, b2_scale=su)
        qh, sh = ops.quant_rows_fp8(h8)
        o8 = ops.grouped_gemm(rg["offsets"], qh, qd, total_rows=T * K, scales_pow2=True, a_scale=sh, b_scale=sd)
        y8 = ops.combine(o8, rg["reverse_index"], dev(gates), rg["gate_index"])
    scale16 = ref16.float().abs().max().item()
    assert_bf16_close(y16, ref16, rtol=1e-2, atol=1e-2 * scale16, what="swiglu bf16")
    # ... which trains: gradients of the one-call form against autograd through the oracle
    leaves = [t.detach().float().requires_grad_(True) for t in (x, wg_v, wu_v, wd_v)]
    dy = torch.randn(T, D, generator=torch.Generator().manual_seed(3)) * 0.01
    o_moe.fused_jagged_bmm_swiglu_combine(r["offsets"], idx2, leaves[0], leaves[1], None, leaves[2], None, leaves[3],
                                          None, K, gates.float(), r["gate_index"]).backward(dy)
    got = [dev(t).detach().requires_grad_(True) for t in (x, wg_v, wu_v, wd_v)]
    moe.fused_jagged_bmm_swiglu_combine(rg["offsets"], rg["gate_index"].view(-1, K), got[0], got[1], None, got[2], None,
                                        got[3], None, K, dev(gates), rg["gate_index"]).backward(dev(dy.to(BF16)))
    for name, g_, q_ in zip(("d_x", "d_w", "d_wp", "d_w_out"), got, leaves):
        ref_g = q_.grad
        err = (g_.grad.float().cpu() - ref_g).abs().max().item()
        assert err <= 3e-2 * ref_g.abs().max().item(), (name, err, ref_g.abs().max().item())
    # fp8 against the oracle's own fp8 path: 3e-2 relative (of the output scale for small entries)
    scale8 = ref8.float().abs().max().item()
    assert_bf16_close(y8, ref8, rtol=3e-2, atol=3e-2 * scale8, what="swiglu fp8")


@pytest.mark.parametrize("B,S,D,H,O,E,k", [(4, 4, 16, 16, 16, 4, 1), (8, 16, 32, 32, 16, 8, 2), (4, 512, 1024, 4096, 1024, 8, 2)])
def test_layer_fp32_matches_oracle(B, S, D, H, O, E, k):
    """modules/tests/test_kernel_parity.py:29-90 (fp32, atol 1e-4) and configuration C1 of the
    baseline (fp32, 8 experts, top-2, [4, 512, 1024] tokens, hidden 4096) against the oracle's
    PyTorch-kernel path on the CPU."""
    from fast_moe_amd import FastMoELayer
    torch.manual_seed(0)
    layer = FastMoELayer(D, H, O, E, dtype=torch.float32)
    g = torch.Generator().manual_seed(0)
    with torch.no_grad():
        layer._experts_hidden_w.copy_(torch.randn(E, H, D, generator=g) * D ** -0.5)
        layer._experts_w.copy_(torch.randn(E, O, H, generator=g) * H ** -0.5)
        layer.gate.gate.weight.copy_(torch.randn(E, D, generator=g) * D ** -0.5)
        layer.gate.gate.bias.zero_()
    x = torch.randn(B, S, D, generator=g)
    sd = {n: v.detach().clone() for n, v in layer.state_dict().items()}
    gpu = layer.cuda()
    with torch.no_grad():
        y = gpu(x.cuda(), k)
        scores = gpu.gate(x.cuda()).reshape(-1, E).cpu()
    ref, r = o_layer.moe_layer_forward(x, sd["gate.gate.weight"], sd["gate.gate.bias"], sd["_experts_hidden_w"],
                                       sd["_experts_hidden_bias"], sd["_experts_w"], sd["_experts_bias"], k)
    # routing from the GPU's own gate probabilities (a last-bit softmax difference may flip a near-tie)
    r2 = o_layer.route_scores(scores, k)
    if not torch.equal(r2["topk_idx"], r["topk_idx"]):
        xf = x.reshape(-1, D)
        hidden = o_moe.index_select_jagged_bmm(r2["offsets"], r2["gate_index"].view(-1, k), xf,
                                               sd["_experts_hidden_w"].permute(0, 2, 1), sd["_experts_hidden_bias"])
        ref = o_moe.silu_jagged_bmm_combine(r2["offsets"], hidden, sd["_experts_w"].permute(0, 2, 1),
                                            sd["_experts_bias"], r2["token_index"], k, r2["gates"],
                                            r2["gate_index"]).view(B, S, O)
    assert y.dtype == torch.float32
    torch.testing.assert_close(y.cpu(), ref, atol=1e-4, rtol=1e-4)


def test_layer_forward_replays_from_a_captured_graph():
    """Serving loops replay the forward from a HIP graph: the library neither allocates nor
    synchronises nor clears memory with memset nodes, so the whole layer (gate, routing, both
    GEMMs, merge) captures.  Every replay, with eager work and synchronisations in between, must
    give the eager result of its input bit for bit, routing included (decode-sized and larger)."""
    from fast_moe_amd.modules.fast_moe_module import FastMoELayer
    torch.manual_seed(0)
    D, H, O, E, k = 256, 512, 256, 16, 4
    layer = FastMoELayer(D, H, O, E).to(BF16).cuda()
    for B, S in ((1, 8), (4, 300)):
        static_x = torch.zeros(B, S, D, dtype=BF16, device="cuda")
        with torch.no_grad():
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):                 # warm-up outside the capture
                layer(static_x, k)
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                static_y = layer(static_x, k)
            for seed in range(4):
                x = randn((B, S, D), 100 + seed).cuda()
                eager = layer(x, k)                       # eager work between the replays
                torch.cuda.synchronize()
                static_x.copy_(x)
                graph.replay()
                torch.cuda.synchronize()
                assert torch.equal(static_y, eager), (B, S, seed)
        del graph


@pytest.mark.parametrize("fp8", [False, True])
def test_forward_replays_from_a_hip_graph(fp8):
    """Every entry point enqueues on the caller's stream and neither allocates nor synchronises, so the
    whole forward (routing, [quantisers,] two GEMMs, merge) can be captured once and replayed.  The
    replays alternate with eager calls and host synchronisations, and each one is compared with the
    eager result bit for bit."""
    from fast_moe_amd.kernels import moe_fp8
    from fast_moe_amd.kernels.hip import ops
    T, E, K, D, H = 2048, 16, 2, 256, 384
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(T, D, generator=g)).to(BF16).cuda()
    v = lambda t: t.permute(0, 2, 1)
    wg, wu = (v((torch.randn(E, H, D, generator=g) * D ** -0.5).to(BF16).cuda()) for _ in range(2))
    wd = v((torch.randn(E, D, H, generator=g) * H ** -0.5).to(BF16).cuda())
    scores = torch.softmax(torch.randn(T, E, generator=g), dim=1).cuda()
    if fp8:
        (qg, sg), (qu, su), (qd, sd) = (moe_fp8.quantize_expert_weights(w) for w in (wg, wu, wd))

    def forward():
        r = ops.route_topk(scores, K)
        kw = dict(total_rows=T * K)
        if fp8:
            qx, sx = ops.quant_rows_fp8(x)
            hid = ops.grouped_gemm(r["offsets"], qx, qg, row_index=r["gate_index"], index_div=K, b2=qu, epilogue=2,
                                   scales_pow2=True, a_scale=sx, b_scale=sg, b2_scale=su, **kw)
            qh, sh = ops.quant_rows_fp8(hid)
            rows = ops.grouped_gemm(r["offsets"], qh, qd, scales_pow2=True, a_scale=sh, b_scale=sd, **kw)
        else:
            hid = ops.grouped_gemm(r["offsets"], x, wg, row_index=r["gate_index"], index_div=K, b2=wu, epilogue=2, **kw)
            rows = ops.grouped_gemm(r["offsets"], hid, wd, **kw)
        return ops.combine(rows, r["reverse_index"], r["gates"].to(BF16), r["gate_index"])

    with torch.no_grad():
        ref = forward().clone()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y = forward()
        torch.cuda.synchronize()
        for i in range(4):
            y.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y, ref), f"replay {i}"
            assert torch.equal(forward(), ref)      # eager work between the replays
            torch.cuda.synchronize()
