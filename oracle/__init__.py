"""CPU oracle for the mask-routed linear / SwiGLU-FFN path.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package (ffn_kernel_amd) imports this; only
tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg do, and only as the checker or
the timed CPU baseline — never as a compute path.

Contents
  modules.py     restatement of the reference's PyTorch modules (test_linear.py:41-49,
                 test_ffn.py:32-47; README.md:49-57, 83-98) in "blend" form, plus row-select
                 fp32 / fp64 forms of the same maths and the stable row partition.
  masked_ref.c   the same maths as plain C loops in double precision on raw bf16 bits —
                 independent of torch's matmul; built by oracle/build.py into oracle/_build/.

How each function is pinned (tests/test_oracle*.py):
  routing            brute force over all 2^M masks for M <= 10 against a sort-based definition
  linear forward     identity / scaled-identity weights (exact), W_v == W_t -> torch.matmul,
                     all-True / all-False masks -> F.linear, C triple loop vs torch fp64,
                     row-permutation equivariance
  SwiGLU / FFN       silu closed forms (0, large +/-), W3 = 0 or W1 = 0 -> 0, the C loops vs torch
  linear backward    autograd of the blend form, dW_v + dW_t == x^T g, empty modality -> exact
                     zeros, W_v == W_t -> dx == g W^T, fp64 finite differences
  FFN backward       (the op the reference leaves at NotImplementedError, ops.py:34-38) chain rule
                     written out vs autograd of the blend form vs the C loops, fp64 finite
                     differences on x and on entries of all six weights, constant-gate reduction
                     to plain matrix products, empty modality -> exact zeros
The reference itself ships no golden vectors, asserts or tolerances for this path
(test_linear.py:92-124 and test_ffn.py:111-115 only print); the bf16 tolerances used here are
max-abs <= 2e-2 and rel-L2 <= 5e-3 against an fp32-accumulated result.
No reference file is imported or executed: the reference is Python + Triton (needs a CUDA GPU,
and its test scripts import un-vendored `profiler` / `IPython`), so there is no oracle/_ref build.
"""
