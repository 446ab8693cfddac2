"""CPU oracle for the SVDQuant W4A4 + low-rank linear layer.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this directory: it is the
checker that the parity tests, the smoke run and the bench's CPU-baseline leg compare the HIP
kernels against.  Every function restates, in plain torch/numpy on the CPU, what one piece of the
reference computes and cites the reference file:line it follows.

What pins each part (parity status):

* INT4 / NVFP4 activation quantizers (``quant.py``): IEEE fp32 restatement of the reference
  arithmetic; pinned by closed-form checks (ties, saturation, zero groups, |dequant error| <=
  scale/2, exhaustive sweep over every bf16 value in a one-element group).  The reference uses
  NVIDIA approximate reciprocal/divide instructions; the oracle uses correctly rounded IEEE
  operations instead, so "bit exact" in this repository means bit exact against this restatement.
* Reference checkpoint layouts (``layouts.py``): two independent derivations (packer reshapes vs
  closed-form lane formulas read from the kernel loaders) must agree, the lane tables printed in
  the reference comments are transcribed as known-answer tests, and golden vectors written by the
  reference's own packer are committed under ``tests/golden``.
* GEMM + epilogue (``linear.py``): dequantize then ``torch.matmul`` in fp32/fp64 (library routine),
  GELU by ``torch.nn.functional.gelu(approximate="tanh")``.
* The reference's own tests hold no op-level golden vectors for this path (only end-to-end image
  metrics that need NVIDIA GPUs and downloads), so beyond the checks above parity is unpinned by
  reference fixtures.
"""
