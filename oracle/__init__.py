"""CPU oracle for the quantized mixture-of-experts hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package (`triton_amd`,
`triton_kernels`) may import this package; only `tests/`, the smoke check and
the `cpu_baseline` leg of `bench.py` use it, and only as the checker.

Every function restates, on the CPU with numpy / torch-CPU, the algorithm of
one of the reference's `*_torch` twins under
`python/triton_kernels/triton_kernels/` and cites the lines it follows.  The
reference's Python files are never imported or executed.

Pin status (what fixes each function independently of its own formula):

  mxfp.downcast_to_mxfp / upcast_from_mxfp
      golden vectors of `tests/test_mxfp.py:92-205` (rounding cases, the
      ROUND_DOWN scale, extreme values, the exact round-trip set), the
      power-of-two closed form of the scale, a nearest-candidate brute force of
      the e2m1 rounding over every bf16 bit pattern.
  routing.topk
      textbook stable descending argsort; the all-equal payload case of
      `tests/test_topk.py:39-51`; brute force.
  routing.make_bitmatrix_metadata
      the worked example in the `BitmatrixMetadata` docstring
      (`tensor_details/bitmatrix.py:11-19`); inverse-permutation and bincount
      invariants.
  routing.make_ragged_tensor_metadata
      the `block_offs` rows of the `RaggedTensorMetadata` docstring
      (`tensor_details/ragged_tensor.py:16-29`); the layout shape
      `[1, 4, 24, 2, 256]` asserted in `tests/test_tensor.py:121-125` is not
      used because that layout is out of scope; closed forms.
  moe.matmul / swiglu / reduce
      reduce to `torch.matmul` in fp32 plus closed-form element-wise maths;
      permutation-equivariance and single-expert reductions to a dense GEMM.
  moe.quantize_fp8_rowwise / the per-token x per-channel fp8 layer (config 5)
      PARITY UNPINNED by the reference: `apply_precision`
      (`matmul.py:772-813`) ignores row/column tensor scales unless an MX scale
      is present and no reference test passes them with plain fp8.  The oracle
      dequantises and calls the pinned GEMM oracle.
  moe.moe_layer gate-weighted combine
      PARITY UNPINNED by the reference as a whole (its tests never derive
      `gammas` from the router's values); each step it is composed of is pinned
      above.
"""
