"""CPU oracle for the MoE-forward hot path: TEST INFRASTRUCTURE, not product code.

Everything in this package is a clean-room CPU restatement (numpy for the
integer / byte arithmetic, torch-on-CPU for the floating-point contractions)
of the reference's PyTorch-kernel path.  Each function cites the reference
file:line whose behaviour it restates.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import it, and only as the checker / the reported CPU
baseline.  The product package ``fast_moe_amd`` never imports it.

How each function is pinned (no function here is "parity unpinned"):

* ``routing.complete_cumsum``            closed form ``[0, cumsum]`` + invariants
* ``routing.select_top_k``               ``torch.topk`` set equality on distinct
                                         scores, ``F.normalize`` on the gates,
                                         brute-force selection on tiny inputs
* ``routing.routing_metadata``           ``torch.sort(stable=True)`` (the library
                                         routine the reference calls), brute-force
                                         counting sort on tiny inputs, invariants
* ``fp8.e4m3fn_encode/decode``           exhaustive over all 256 codes and a dense
                                         float sweep against ``Tensor.to(float8_e4m3fn)``
* ``fp8.calculate_scale``                exhaustive over every positive bf16 amax
                                         against the torch formula; power-of-two and
                                         ``amax*scale in (224, 448]`` invariants
* ``fp8.rowwise_quant_fp8``              dequantise round trip + the two above
* ``moe.*`` (GEMM-type ops)              E=1 / K=1 reductions to a plain ``x @ W + b``,
                                         pure-Python triple loop on tiny inputs, dense
                                         run-every-expert einsum as an end-to-end check
* ``moe.mul_merge_k_add``                pure-Python double loop on tiny inputs
* ``moe_fp8.index_select_jagged_bmm_fp8``  dequantise-then-fp32-oracle agreement
* ``moe_fp8.index_select_jagged_bmm_fp8_backward``  inputs whose quantisation is
                                         lossless (small integers times powers of two):
                                         must equal torch autograd through the
                                         unquantised operator exactly
* ``layer.moe_layer_forward``            dense every-expert MoE (the construction of
                                         modules/tests/test_moe_parity.py:72-106)
* ``mrn.*`` (SGMoE layer)                the dense-dispatch layer against the
                                         operator-level oracle on the same routing, the
                                         comparison kernels/tests/mrn_test.py makes
"""
