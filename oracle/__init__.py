"""CPU oracle of the fused non-GEMM transformer ops.  TEST INFRASTRUCTURE ONLY.

Nothing under ``oslo_amd/`` may import this package: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do, and
only as the checker, never as the thing measured or shipped.

Contents
  ``closed_form``  numpy restatement (float64 by default) of every forward and
                   backward formula on the path, with the rounding points of
                   the fused kernels made explicit.
  ``torch_path``   the reference's own unfused chain of torch ops, written from
                   its model / module sources, run on CPU tensors.  This is the
                   "reference CPU path" that parity and the CPU baseline refer
                   to.
  ``philox``       Philox4x32-10 and the dropout keep-mask, integer-exact.

How each function is pinned (tests/test_oracle_*.py, no GPU needed)
  softmax fwd       against torch.softmax on the explicitly masked scores, row
                    sums, exact zeros, shift invariance, non-zero counts.
  softmax bwd       torch.autograd.gradcheck-style finite differences in fp64
                    and torch autograd of the unfused chain.
  LayerNorm fwd/bwd torch.nn.functional.layer_norm + autograd in fp64, and the
                    identities sum(dx)=0, sum(dx*xhat)=0, dbeta=sum(dy).
  RMSNorm fwd/bwd   autograd of the 6-line reference formula in fp64; the
                    rounding order against manual_rms_norm in bf16.
  bias-GeLU         torch.nn.functional.gelu(approximate="tanh") + autograd in
                    fp64; gelu(0)=0, gelu'(0)=0.5, gelu(u)-gelu(-u)=u.
  softmax with an additive term
                    torch.softmax(scale * x + M) + autograd in fp64 for key
                    masks, per-query masks and shared biases, with the diagonal;
                    the rows without a visible key for each fill value;
                    committed torch-float64 vectors (tests/golden).
  bias-dropout-add  p=0 identity; mask scale; autograd with an explicit mask.
  softmax + dropout, bias-dropout-add + norm
                    torch autograd in fp64 through the unfused chain with an
                    explicit keep mask.
  optimizer steps   Adam / AdamW, SGD, Adagrad against torch.optim over five
                    steps; NovoGrad as torch.optim.SGD with momentum on the
                    normalised gradient; LAMB as torch.optim.Adam's direction
                    under the trust ratio with torch's vector norms.  The
                    mixed-precision LAMB's overflow flag and master copies are
                    behaviours of the optimizer class: parity unpinned beyond
                    the reduction to the plain LAMB step.
  Philox            the three Random123 known-answer vectors; an independent
                    pure-Python big-integer implementation; the C++ engine of
                    ATen (PhiloxRNGEngine.h) where torch exposes it.
The reference holds no numeric fixture for any of these ops (its tests draw
unseeded random data), so no function is pinned by a reference-held vector;
softmax, bias-GeLU and bias-dropout have no reference test at all and rest on
the closed forms and library routines above.
"""
