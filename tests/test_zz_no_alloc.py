"""fmoe_route_topk_static (routing whose scratch is built into the library, for callers that cannot
allocate) against fmoe_route_topk, bit for bit, through the C ABI: two calls in a row, the second
smaller than the first, so that what the first left in the shared buffer must not leak into it."""
import ctypes

import pytest
import torch
from torch.nn import functional as F

pytestmark = pytest.mark.gpu

KEYS = ("topk_idx", "gates", "lengths", "offsets", "gate_index", "token_index", "reverse_index")


def scores_of(T, E, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    return F.softmax(torch.randn(T, E, generator=g) * 2.0, dim=1).to(dtype).cuda()


def outputs(T, E, K, dtype):
    i64 = dict(dtype=torch.int64, device="cuda")
    return {"topk_idx": torch.full((T, K), -1, **i64), "gates": torch.full((T, K), -1.0, dtype=dtype, device="cuda"),
            "lengths": torch.full((E,), -1, **i64), "offsets": torch.full((E + 1,), -1, **i64),
            "gate_index": torch.full((T * K,), -1, **i64), "token_index": torch.full((T * K,), -1, **i64),
            "reverse_index": torch.full((T, K), -1, **i64)}


def call_static(lib, scores, K, renorm, out):
    from fast_moe_amd.kernels.hip import _lib
    T, E = scores.shape
    code = _lib.FMOE_F32 if scores.dtype == torch.float32 else _lib.FMOE_BF16
    rc = lib.fmoe_route_topk_static(scores.data_ptr(), code, T, E, K, renorm, *(out[k].data_ptr() for k in KEYS),
                                    torch.cuda.current_stream().cuda_stream)
    return rc


def call_workspace(lib, scores, K, renorm, out):
    from fast_moe_amd.kernels.hip import _lib
    T, E = scores.shape
    code = _lib.FMOE_F32 if scores.dtype == torch.float32 else _lib.FMOE_BF16
    ws_bytes = lib.fmoe_route_workspace_bytes(T, E, K)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device="cuda")
    rc = lib.fmoe_route_topk(scores.data_ptr(), code, T, E, K, renorm, *(out[k].data_ptr() for k in KEYS),
                             ws.data_ptr(), ws_bytes, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return rc


def test_static_scratch_routing_equals_workspace_routing_on_consecutive_calls():
    from fast_moe_amd.kernels.hip import _lib
    lib = _lib.load()
    # large first (fills 256 chunks x 64 experts of histograms and 2^17 ids), then smaller calls with other
    # E / K / dtype / gate mode, then the large one again
    cases = [(16384, 64, 8, torch.float32, 1), (100, 16, 4, torch.bfloat16, 1), (3000, 128, 8, torch.float32, 0),
             (1, 8, 2, torch.float32, 1), (777, 300, 6, torch.bfloat16, 3), (16384, 64, 8, torch.float32, 1),
             (131072, 8, 8, torch.bfloat16, 1)]                  # the last: exactly 2^20 routed positions
    for n, (T, E, K, dtype, renorm) in enumerate(cases):
        print(f"static routing T={T} E={E} K={K} {dtype} mode={renorm}", flush=True)
        scores = scores_of(T, E, 40 + n, dtype)
        want, got = outputs(T, E, K, dtype), outputs(T, E, K, dtype)
        assert call_workspace(lib, scores, K, renorm, want) == 0, lib.fmoe_last_error()
        torch.cuda.synchronize()
        before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
        assert call_static(lib, scores, K, renorm, got) == 0, lib.fmoe_last_error()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before          # torch's allocator saw nothing ...
        if n > 0:       # ... and the device's free memory did not move either (hipMemGetInfo sees a
            assert torch.cuda.mem_get_info()[0] == free_before  # hipMalloc inside the library; call 0 loads code objects)
        for key in KEYS:
            a, b = got[key], want[key]
            if a.dtype != torch.int64:
                a, b = a.view(torch.int16 if dtype == torch.bfloat16 else torch.int32), b.view(
                    torch.int16 if dtype == torch.bfloat16 else torch.int32)
            assert torch.equal(a, b), (key, T, E, K)
        assert int(got["offsets"][-1]) == T * K


def test_static_scratch_routing_through_the_wrapper_and_empty_input():
    from fast_moe_amd.kernels.hip import ops
    scores = scores_of(4096, 64, 7, torch.float32)
    want = ops.route_topk(scores, 8)
    got = ops.route_topk(scores, 8, static_scratch=True)
    again = ops.route_topk(scores_of(64, 64, 8, torch.float32), 8, static_scratch=True)
    want2 = ops.route_topk(scores_of(64, 64, 8, torch.float32), 8)
    for key in KEYS:
        assert torch.equal(got[key], want[key]) and torch.equal(again[key], want2[key]), key
    # written in place into a dict of a previous call: nothing is allocated at all
    ops.route_topk(scores, 8, static_scratch=True, out=got)
    empty = ops.route_topk(torch.zeros((0, 8), device="cuda"), 2, static_scratch=True)
    assert empty["offsets"].cpu().tolist() == [0] * 9


def test_static_scratch_routing_replays_from_a_captured_graph():
    """The use the entry point is for: captured into a HIP graph (after one call outside the capture,
    which looks the scratch address up), replayed with new scores in the same buffers, every replay
    bit-identical to the eager workspace routing of those scores."""
    from fast_moe_amd.kernels.hip import ops
    T, E, K = 2048, 64, 8
    scores = scores_of(T, E, 11, torch.float32)
    out = ops.route_topk(scores, K, static_scratch=True)             # outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            ops.route_topk(scores, K, static_scratch=True, out=out)
    torch.cuda.current_stream().wait_stream(side)
    for seed in (12, 13, 14):
        scores.copy_(scores_of(T, E, seed, torch.float32))
        want = ops.route_topk(scores, K)                                 # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for key in KEYS:
            assert torch.equal(out[key], want[key]), (key, seed)


def test_route_topk_checks_every_tensor_of_out():
    from fast_moe_amd.kernels.hip import ops
    scores = scores_of(128, 16, 3, torch.float32)
    good = ops.route_topk(scores, 4)
    for name, bad in (("offsets", good["offsets"][:-1]), ("gate_index", good["gate_index"].to(torch.int32)),
                      ("token_index", good["token_index"][: 128 * 4 - 1]),
                      ("reverse_index", good["reverse_index"].t().contiguous().t()),
                      ("gates", good["gates"].to(torch.bfloat16)), ("lengths", good["lengths"].cpu())):
        out = dict(good)
        out[name] = bad
        with pytest.raises(ValueError, match=name):
            ops.route_topk(scores, 4, out=out)
    with pytest.raises(ValueError, match="topk_idx"):
        ops.route_topk(scores, 4, out={k: v for k, v in good.items() if k != "topk_idx"})


def test_static_scratch_routing_turns_away_what_does_not_fit():
    from fast_moe_amd.kernels.hip import _lib
    lib = _lib.load()
    T, E, K = 131073, 8, 8                                        # 2^20 + 8 positions
    scores = scores_of(T, E, 1, torch.float32)
    out = outputs(T, E, K, torch.float32)
    assert call_static(lib, scores, K, 1, out) == 1
    assert b"exceed" in lib.fmoe_last_error()
    assert int(out["offsets"][0]) == -1                           # nothing was launched
    scores = scores_of(4, 600, 1, torch.float32)
    out = outputs(4, 600, 2, torch.float32)
    assert call_static(lib, scores, 2, 1, out) == 1 and b"experts" in lib.fmoe_last_error()
    # K beyond E or 64 and an unknown gate mode are refused by the entry point's own checks
    scores = scores_of(16, 8, 1, torch.float32)
    out = outputs(16, 8, 9, torch.float32)
    assert call_static(lib, scores, 9, 1, out) == 1 and b"K=9" in lib.fmoe_last_error()
    out = outputs(16, 8, 2, torch.float32)
    assert call_static(lib, scores, 2, 7, out) == 1 and b"gate mode" in lib.fmoe_last_error()
    assert int(out["offsets"][0]) == -1
