"""CPU-side checks of the C ABI: the library loads, exports every symbol that
include/fast_moe_amd.h declares, and rejects bad arguments before touching a GPU."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "fast_moe_amd.h")


@pytest.fixture(scope="module")
def lib():
    from fast_moe_amd.kernels.hip import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from fast_moe_amd import build
        build.build(verbose=False)
    return _lib.load()


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fmoe_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported(lib):
    from fast_moe_amd.kernels.hip import _lib
    names = declared_functions()
    assert len(names) >= 9
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in the header but not exported"
    assert sorted(_lib.EXPORTED_SYMBOLS) == names


def test_static_routing_rejects_oversize_calls_without_a_gpu(lib):
    """fmoe_route_topk_static checks its limits before it touches a device."""
    bad = ctypes.c_void_p(16)
    args = [bad] * 7 + [None]
    assert lib.fmoe_route_topk_static(bad, 0, (1 << 20) // 8 + 1, 8, 8, 1, *args) == 1
    assert b"routed positions exceed" in lib.fmoe_last_error()
    assert lib.fmoe_route_topk_static(bad, 0, 4, 513, 2, 1, *args) == 1
    assert b"experts" in lib.fmoe_last_error()


def test_gemm_desc_layout_matches_header():
    from fast_moe_amd.kernels.hip._lib import GemmDesc
    text = open(HEADER).read()
    body = text[text.index("typedef struct fmoe_gemm_desc {"):text.index("} fmoe_gemm_desc;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = []
    for stmt in body.split("{", 1)[1].split(";"):
        stmt = stmt.strip()
        if not stmt:
            continue
        for part in stmt.split(","):
            name = re.findall(r"([A-Za-z_][A-Za-z0-9_]*)\s*$", part.strip())
            fields.append(name[0])
    assert [f[0] for f in GemmDesc._fields_] == fields
    # sizes and offsets as the C compiler lays them out
    import subprocess
    import tempfile
    prog = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{HEADER}"', 'int main(void) {',
            '  printf("%zu\\n", sizeof(fmoe_gemm_desc));']
    prog += [f'  printf("%zu\\n", offsetof(fmoe_gemm_desc, {f}));' for f in fields]
    prog += ['  return 0;', '}']
    with tempfile.TemporaryDirectory() as tmp:
        src = os.path.join(tmp, "layout.c")
        open(src, "w").write("\n".join(prog))
        exe = os.path.join(tmp, "layout")
        subprocess.run(["gcc", src, "-o", exe], check=True)
        out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout.split()
    assert int(out[0]) == ctypes.sizeof(GemmDesc)
    assert [int(v) for v in out[1:]] == [getattr(GemmDesc, f).offset for f in fields]


def test_enum_values_match_the_header():
    """The Python constants are the header's enumerators."""
    from fast_moe_amd.kernels.hip import _lib
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    enums = dict((name, int(value)) for name, value in re.findall(r"\b(FMOE_[A-Z0-9_]+)\s*=\s*(-?\d+)", text))
    assert (enums["FMOE_EPI_NONE"], enums["FMOE_EPI_SILU"], enums["FMOE_EPI_SWIGLU"], enums["FMOE_EPI_GATED"]) == \
        (_lib.EPI_NONE, _lib.EPI_SILU, _lib.EPI_SWIGLU, _lib.EPI_GATED)
    assert (enums["FMOE_F32"], enums["FMOE_BF16"], enums["FMOE_E4M3"]) == (_lib.FMOE_F32, _lib.FMOE_BF16, _lib.FMOE_E4M3)


def test_version_and_workspace(lib):
    assert lib.fmoe_version() >= 100
    assert lib.fmoe_route_workspace_bytes(0, 8, 2) > 0
    small = lib.fmoe_route_workspace_bytes(64, 8, 2)
    big = lib.fmoe_route_workspace_bytes(16384, 64, 8)
    assert big > small >= 64 * 2 * 2
    assert lib.fmoe_route_workspace_bytes(-1, 8, 2) == 0


def test_argument_errors_are_reported_without_a_gpu(lib):
    from fast_moe_amd.kernels.hip._lib import GemmDesc
    assert lib.fmoe_grouped_gemm(None, None) == 1
    assert b"desc is NULL" in lib.fmoe_last_error()
    d = GemmDesc()
    d.num_experts, d.n, d.k = 4, 0, 8
    assert lib.fmoe_grouped_gemm(ctypes.byref(d), None) == 1
    assert b"n, k >= 1" in lib.fmoe_last_error()
    d.n, d.total_rows, d.a_dtype, d.out_dtype = 8, 16, 7, 1
    assert lib.fmoe_grouped_gemm(ctypes.byref(d), None) == 1
    assert b"bf16, e4m3 or fp32" in lib.fmoe_last_error()
    d.a_dtype = 0                                    # fp32 operands need an fp32 output
    assert lib.fmoe_grouped_gemm(ctypes.byref(d), None) == 1
    assert b"fp32 for fp32 operands" in lib.fmoe_last_error()
    # pre-activation outputs come in pairs and belong to the SWIGLU epilogue; the plan query runs the same checks
    d.a_dtype, d.out_dtype = 1, 1
    d.offsets = d.a = d.b = d.out = 64
    d.a_rows, d.index_div, d.a_stride_row, d.out_stride_row = 16, 1, 8, 8
    d.aux = 64
    assert lib.fmoe_grouped_gemm(ctypes.byref(d), None) == 1
    assert b"aux and aux2 come together" in lib.fmoe_last_error()
    d.aux2 = 64
    assert lib.fmoe_grouped_gemm(ctypes.byref(d), None) == 1
    assert b"SWIGLU pre-activations" in lib.fmoe_last_error()
    plan = ctypes.c_int(7)
    assert lib.fmoe_grouped_gemm_plan(ctypes.byref(d), ctypes.byref(plan)) == 1 and plan.value == 7
    assert lib.fmoe_grouped_gemm_plan(ctypes.byref(d), None) == 1
    assert b"plan is NULL" in lib.fmoe_last_error()
    d.aux = d.aux2 = None
    # the gated epilogue reads its gate from aux, takes bf16 operands only and no second product
    d.epilogue = 3
    assert lib.fmoe_grouped_gemm_plan(ctypes.byref(d), ctypes.byref(plan)) == 1
    assert b"GATED reads its gate from aux" in lib.fmoe_last_error()
    d.aux, d.aux2 = 64, 64
    assert lib.fmoe_grouped_gemm_plan(ctypes.byref(d), ctypes.byref(plan)) == 1
    assert b"aux2 stays NULL" in lib.fmoe_last_error()
    d.aux2 = None
    d.aux_stride_row = 4                      # narrower than n
    assert lib.fmoe_grouped_gemm_plan(ctypes.byref(d), ctypes.byref(plan)) == 1
    assert b"aux row stride" in lib.fmoe_last_error()
    d.aux_stride_row = 8
    d.a_dtype, d.out_dtype = 0, 0
    assert lib.fmoe_grouped_gemm_plan(ctypes.byref(d), ctypes.byref(plan)) == 2       # unsupported, not malformed
    assert b"built for bf16" in lib.fmoe_last_error()
    d.a_dtype, d.out_dtype = 1, 1
    d.epilogue = 4
    assert lib.fmoe_grouped_gemm_plan(ctypes.byref(d), ctypes.byref(plan)) == 1
    assert b"unknown epilogue" in lib.fmoe_last_error()
    d.epilogue, d.aux, d.aux_stride_row = 0, None, 0
    d.a2, d.k2 = 64, 128                     # a second product needs b2 and goes with no epilogue
    assert lib.fmoe_grouped_gemm_plan(ctypes.byref(d), ctypes.byref(plan)) == 1
    assert b"a2 needs b2" in lib.fmoe_last_error()
    d.a2, d.k2 = None, 0
    d.out2 = 64                              # a second output belongs to the row-indexed weight-gradient form
    assert lib.fmoe_grouped_gemm_plan(ctypes.byref(d), ctypes.byref(plan)) == 1
    assert b"out2 goes with a_stride_k" in lib.fmoe_last_error()
    d.out2 = None
    d.total_rows = 0
    assert lib.fmoe_grouped_gemm_plan(ctypes.byref(d), ctypes.byref(plan)) == 0 and plan.value == -1
    # routing: K > E, K > 64, workspace too small
    args = [None] * 7
    assert lib.fmoe_route_topk(None, 0, 4, 8, 80, 1, *args, None, 0, None) == 1
    assert b"K=80" in lib.fmoe_last_error()
    assert lib.fmoe_route_topk(None, 0, 4, 8, 2, 1, *args, ctypes.c_void_p(64), 1, None) == 3
    assert b"workspace" in lib.fmoe_last_error()
    # quant: zero columns
    assert lib.fmoe_quant_rows_e4m3(None, 1, 1, 4, 0, 0, 0, 1, 0, None, 0, 0, 1, None, 0, None) == 1
    # combine: out dtype must be the promoted dtype
    assert lib.fmoe_combine(ctypes.c_void_p(64), 1, 4, 2, 8, 8, ctypes.c_void_p(64), ctypes.c_void_p(64), 0, 2,
                            2, 1, None, ctypes.c_void_p(64), 1, None) == 1
    assert b"promoted" in lib.fmoe_last_error()
    # backward helpers: dtype and stride checks come before any launch
    P = ctypes.c_void_p(64)
    assert lib.fmoe_jagged_transpose(P, 2, 8, 8, 8, None, 1, P, P, 2, P, 16, 16, 0, None) == 1
    assert b"bf16 or fp32" in lib.fmoe_last_error()
    assert lib.fmoe_jagged_transpose(P, 1, 8, 8, 4, None, 1, P, P, 2, P, 16, 16, 0, None) == 1
    assert b"row stride" in lib.fmoe_last_error()
    assert lib.fmoe_gather_rows(P, 4, 24, 24, P, 1, 4, P, 24, None) == 1      # rows of whole 16-byte chunks
    assert b"16-byte aligned chunks" in lib.fmoe_last_error()
    assert lib.fmoe_segment_colsum(P, 1, 8, 8, 4, P, 2, P, None) == 1
    assert lib.fmoe_swiglu_bwd(P, P, P, P, None, 1, 8, 8, 0, None) == 1    # gated form needs du
    assert lib.fmoe_swiglu_bwd(P, P, P, P, P, 0, 64, 8, 16, None) == 1     # pitched outputs: bf16 only
    assert b"row pitch" in lib.fmoe_last_error()
    assert lib.fmoe_combine_bwd(P, None, 1, 4, 2, 8, 8, P, None, 0, 1, 1, 1, None, P,
                                ctypes.cast(P, ctypes.POINTER(ctypes.c_float)), None) == 1
    assert b"d_gates needs value" in lib.fmoe_last_error()


def test_pytorch_kernel_is_refused():
    import torch
    from fast_moe_amd import FastMoELayer, KernelType
    from fast_moe_amd.kernels import moe
    with pytest.raises(NotImplementedError):
        moe.index_select_jagged_bmm(1, torch.zeros(2, dtype=torch.int64), torch.zeros(1, 1, dtype=torch.int64),
                                    torch.zeros(1, 8), torch.zeros(1, 8, 8), None, kernel=KernelType.PYTORCH)
    layer = FastMoELayer(8, 16, 8, 4, kernel=KernelType.PYTORCH)
    with pytest.raises(NotImplementedError):
        layer(torch.zeros(1, 2, 8, dtype=torch.bfloat16), 2)


def test_cpu_tensors_are_refused():
    import torch
    from fast_moe_amd.kernels import moe
    with pytest.raises(ValueError, match="no CPU path"):
        moe.mul_merge_k_add(torch.zeros(4, dtype=torch.int64), torch.zeros(2, 2, dtype=torch.int64),
                            torch.zeros(4, 8))


def test_state_dict_layout_matches_reference_names():
    from fast_moe_amd import FastMoELayer
    layer = FastMoELayer(16, 32, 8, 4)
    sd = layer.state_dict()
    assert set(sd) == {"gate.gate.weight", "gate.gate.bias", "_experts_hidden_w", "_experts_hidden_bias",
                       "_experts_w", "_experts_bias"}
    assert tuple(sd["_experts_hidden_w"].shape) == (4, 32, 16)
    assert tuple(sd["_experts_w"].shape) == (4, 8, 32)


def test_weight_quant_cache_hits_and_invalidation():
    """The cache logic of moe_fp8 on CPU tensors with a stand-in quantiser (no GPU work)."""
    import torch
    from fast_moe_amd.kernels.moe_fp8 import _WeightQuantCache
    cache = _WeightQuantCache(max_entries=4)
    calls = []

    def quantize(w):
        calls.append(w.data_ptr())
        return (w.detach().clone(), w.abs().amax(1))

    param = torch.nn.Parameter(torch.randn(3, 8, 4))
    view = lambda: param.permute(0, 2, 1)
    a = cache.get(view(), quantize)
    b = cache.get(view(), quantize)                       # a fresh view object of the same owner
    assert len(calls) == 1 and a[0] is b[0] and (cache.hits, cache.misses) == (1, 1)
    with torch.no_grad():
        param.mul_(2.0)                                   # in-place update: version counter moves
    c = cache.get(view(), quantize)
    assert len(calls) == 2 and torch.equal(c[0], view())
    d = cache.get(param[:2].permute(0, 2, 1), quantize)   # another geometry of the same owner
    assert len(calls) == 3 and d[0].shape[0] == 2
    other = torch.randn(3, 4, 8)
    cache.get(other, quantize)
    del other
    for _ in range(6):                                    # dead owners are evicted, the table stays bounded
        cache.get(torch.randn(3, 4, 8), quantize)
    assert len(cache._entries) <= 4


def test_reference_helper_names_import_without_a_gpu():
    """Names a caller of the reference imports beside the operators (kernels/utils.py:28-53,
    utils/configs.py:13-36)."""
    import torch
    from fast_moe_amd.kernels.utils import KernelType, fx_infer_max_len, fx_torch_zeros_like, to_fp32_if_pytorch_kernel
    from fast_moe.utils.configs import MRNOutput, SGConfig
    assert fx_infer_max_len(torch.tensor([3, 9, 2])) == 9
    assert fx_torch_zeros_like(torch.ones(2, 3), torch.bfloat16).dtype == torch.bfloat16
    assert to_fp32_if_pytorch_kernel(torch.ones(1, dtype=torch.bfloat16), KernelType.HIP).dtype == torch.bfloat16
    cfg = SGConfig(model_d=8, num_experts=4, num_activated_experts=2)
    assert cfg.loss_coef == 1e-2 and not cfg.enable_noisy_gating
    assert MRNOutput._fields == ("x", "loss", "load")


def test_reference_import_paths_resolve():
    """The import statements of code written against the reference's operator path."""
    from fast_moe import FastMoELayer, KernelType
    from fast_moe.kernels import moe as m1
    from fast_moe.kernels.moe import index_select_jagged_bmm, mul_merge_k_add, silu_jagged_bmm_combine
    from fast_moe.kernels.moe_fp8 import index_select_jagged_bmm as bmm_fp8
    from fast_moe.kernels.utils import KernelType as K2
    from fast_moe.modules.fast_moe_module import FastMoELayer as L2
    from fast_moe.utils.utils import _compute_top_logits, _dispatch
    import fast_moe_amd.kernels.moe as real
    assert m1 is real and index_select_jagged_bmm is real.index_select_jagged_bmm
    assert K2 is KernelType and L2 is FastMoELayer and callable(bmm_fp8) and callable(_dispatch)


def test_imports_of_the_reference_test_files_resolve():
    """The import block of kernels/tests/moe_test.py:17-28 (and of moe_fp8_test.py, quant_fp8_test.py,
    test_kernel_parity.py) through the fast_moe.* root."""
    from fast_moe.dev_settings import get_verbose_level, is_dev_mode, set_dev_mode, set_verbose_level
    from fast_moe.kernels.triton.triton_moe import IndexSelectJaggedBmmOption, SiluJaggedBmmCombineOption
    from fast_moe.kernels.utils import (fx_infer_max_len, fx_torch_zeros_like, gpu_unavailable, KernelType,
                                        to_fp32_if_pytorch_kernel)
    from fast_moe.modules.fast_moe_module import FastMoELayer
    from fast_moe.utils.configs import MRNOutput, SGConfig
    import fast_moe_amd.kernels.moe as real
    assert IndexSelectJaggedBmmOption is real.IndexSelectJaggedBmmOption
    assert SiluJaggedBmmCombineOption().activation_checkpointing is False
    # (skip?, reason), the argument pair of unittest.skipIf
    skip, reason = gpu_unavailable
    assert isinstance(reason, str) and reason
    import torch
    assert bool(skip) == (not torch.cuda.is_available())
    import os
    if "FASTMOE_DEV_MODE" not in os.environ:
        before = is_dev_mode()
        set_dev_mode(True)
        assert is_dev_mode() is True
        set_dev_mode(before)
    set_verbose_level(2)
    assert get_verbose_level() == 2
    set_verbose_level(0)
    assert callable(fx_infer_max_len) and callable(fx_torch_zeros_like) and callable(to_fp32_if_pytorch_kernel)
    assert FastMoELayer and MRNOutput and SGConfig and KernelType.HIP
    # kernels/tests/mrn_test.py:24 (utils/enums.py:10-26: member names and values)
    from fast_moe.utils.enums import ExpertType, LossType, RouterChoice
    from fast_moe import ExpertType as root_expert_type
    assert root_expert_type is ExpertType
    assert [(m.name, m.value) for m in ExpertType] == [("MLP", "MLP"), ("FFN", "FFN"), ("FFNBIAS", "FFN_WITH_BIAS")]
    assert [(m.name, m.value) for m in RouterChoice] == [("TopK", "TOP_K"), ("Vanilla", "VANILLA")]
    assert [(m.name, m.value) for m in LossType] == [("LB", "LOAD_BALANCE"), ("MI", "MUTAL_INFORMATION")]


def test_combine_helper_opens_the_reference_profiler_range():
    """utils/utils.py:55: the merge runs inside record_function("## combine ##")."""
    import inspect
    from fast_moe.utils import utils as u
    assert '"## combine ##"' in inspect.getsource(u._combine)
