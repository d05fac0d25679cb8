"""CPU oracle for the quantized-MoE hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg
do, and only as the checker.  Every function restates, on the CPU with
numpy / torch-CPU, the algorithm of the reference's torch implementation for
one op of the path and cites the reference lines it follows (paths relative to
python/triton_kernels/triton_kernels/ of the reference tree).

Pinning status (what independent evidence each function is checked against in
tests/test_oracle_*.py):

  mxfp_ref.downcast_to_mxfp_ref   pinned: literals of tests/test_mxfp.py:92-151,
                                  round-to-nearest-even brute force over every
                                  bf16 input, closed-form scale exponents
  mxfp_ref.upcast_from_mxfp_ref   pinned: value table mxfp.py:373, exact
                                  round trip of tests/test_mxfp.py:171-205
  routing_ref.topk_ref            pinned: torch.topk on tie-free inputs, crafted
                                  ties, brute-force selection
  routing_ref.bitmatrix_metadata_ref   pinned: docstring example
                                  tensor_details/bitmatrix.py:11-19, permutation
                                  invariants, python-loop brute force
  routing_ref.ragged_metadata_ref pinned: docstring example
                                  tensor_details/ragged_tensor.py:15-29,
                                  python-loop brute force, n_blocks closed form
  matmul_ref.matmul_ref           pinned: float64 GEMM on small shapes, one-hot
                                  rows reproduce dequantised weight rows, zero
                                  weights give bias*beta*gamma
  matmul_ref.swiglu_ref           pinned: float64 evaluation of the formula,
                                  limits g -> -inf and large g
  matmul_ref.reduce_ref           pinned: direct python-loop sum
"""
