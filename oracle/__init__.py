"""CPU oracle for the quantized-linear hot path.  TEST INFRASTRUCTURE ONLY.

A plain torch/numpy restatement of the reference's algorithms (each function cites the
reference file:line it follows).  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import this package, and only as the checker or
as the reported CPU baseline -- never as a code path of the product.  ``sglang_amd``
itself never imports it and has no CPU fallback: without the HIP library it raises.

Pinning status (what, besides this file's own formulas, fixes each function's results):
  fp8.e4m3fn_encode / decode   closed form checked against torch's CPU float8_e4m3fn cast
                               on every bf16 value in range and on rounding-boundary
                               floats (tests/test_oracle_cpu.py).
  quant.group_quant (divide)   invariants of the closed form (arg-max -> +-448, error
                               bounds, all-zero group, exactly-representable round trip
                               per test/registered/quant/test_fp8_kernel.py:34-116) and
                               equality with a line-by-line torch evaluation of
                               test/manual/quant/test_block_fp8.py:41-66.
  quant.group_quant (reciprocal, UE8M0)
                               <=1 code / <=1 ulp from the divide form; UE8M0 exponent
                               bytes brute-forced over all exponents and mantissa edges.
  quant.silu_mul_group_quant_masked
                               equals moe.silu_and_mul -> group_quant(reciprocal, UE8M0) on each
                               expert's first masked_m[e] tokens, empty elsewhere (the mask is all
                               it adds).
  quant.fused_rms_group_quant  the torch model of the reference's own test evaluated line by line on fp32
                               inputs; constant-row and all-zero closed forms.  (The fused op itself is
                               AITER's, which is not in the reference tree: the test's model is the anchor.)
  quant.per_token_quant_fp8/int8  closed forms + round-trip/extreme-value invariants.
  quant.static_quant_fp8       torch's CPU evaluation of the reference's own expression for the same step
                               ((x * scale.reciprocal()).clamp(-448, 448).to(float8_e4m3fn),
                               fp8_utils.py:1497-1501) on every bf16 value in range and on outlier rows.
  quant.dynamic_per_tensor_quant_fp8
                               the reference test's own statement of the arithmetic evaluated in torch on the CPU
                               (test/manual/quant/test_custom_ops.py:22-30: (x.float() * scale.reciprocal())
                               .clamp(-448, 448).to(float8_e4m3fn) with scale = max|x| / 448), incl. its 11 x 11 case.
  gemm.*                       special cases (unit scales -> plain fp32 matmul of the fp8
                               values; one-hot rows read back scaled weight rows; int8 is
                               exact integer arithmetic checked against int64 matmul; the block
                               forms also against dequantise-then-matmul in float64, ragged
                               last tiles included).
  moe.moe_align_block_size     brute force on tiny inputs + the invariants the reference's
                               own test checks (sgl-kernel/tests/test_moe_align.py:233-255).
  moe.topk_softmax             brute force in float64 python loops on tiny rows (incl. soft-capping
                               and bias), unit sum after renormalisation, lower index wins ties.
  moe.fused_moe                top-1/weight-1 equals a dense two-layer MLP; token
                               permutation equivariance (fp8 and int8 forms).
  moe.fused_moe (block shapes [64,64], [64,128], [128,64])
                               the reference test's torch model (test/manual/quant/test_block_fp8.py:518-547)
                               evaluated line by line with that block_shape.
  moe.fused_moe_row_scaled     torch_w8a8_per_column_moe (test/registered/quant/test_int8_kernel.py:39-79) evaluated
                               line by line, int8 and its FP8 twin; top-1/weight-1 equals the dense two-layer
                               MLP bit for bit; zero weights leave the bias; constant per-channel scales equal
                               per-tensor ones.
  moe.topk_sigmoid             brute force in float64 python loops on tiny rows (bias, renormalisation, ties) and
                               torch.topk(torch.sigmoid(x)), the model of the reference's own test.
  moe.prepare_moe_input        brute force with python sets on small inputs (span membership, order,
                               inverse permutation, 128-rounded offsets, dropped ids).
  moe.fp8_blockwise_scaled_grouped_mm / apply_shuffle_mul_sum / shuffle_rows
                               per-expert dequantise-then-matmul in float64; the torch expression
                               of the reference's doc comment in float64; plain indexing.
  moe.cutlass_fused_experts_fp8  identical to moe.fused_moe for top-1/weight-1, within 1e-2 otherwise
                               (the two formulations apply the routing weight at different points).
No function here is "parity unpinned".
"""
