"""CPU oracle for the FP8 grouped-expert path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``pith_train_amd/`` imports this
package; it is used by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker / reported CPU baseline.

Every function restates, in plain PyTorch-CPU / numpy, the semantics of one
reference operator and cites the reference file:line it follows.  The
reference's Triton kernels and its third-party DeepGEMM calls cannot run on a
CPU, so the restatement is pinned by known answers and by independent
formulations (see ``tests/test_oracle_*.py``):

* ``fp8.compute_fp8_scale``  - exhaustive over every bf16 amax against the
  published DeepGEMM rule ``2**ceil(log2(amax/448))`` evaluated in float64.
* ``fp8.cast_e4m3``          - an integer-only numpy encoder checked against
  ``torch.Tensor.to(float8_e4m3fn)`` over every bf16 value times every scale
  exponent that can occur.
* quant layouts              - brute-force per-element Python loops on small
  shapes, ``scale_t == scale.T`` symmetry, rowwise half identical across
  entry points.
* GEMMs                      - definition ``bf16(sum_k a*sa*b*sb)`` with float64
  accumulation vs per-group ``torch.matmul`` on dequantised operands.  The
  reference's GEMM arithmetic lives in DeepGEMM (git ``main``, unpinned), so
  GEMM parity is pinned to tolerance only.
* permute / dedup            - ``argsort(stable=True)`` / ``nonzero`` brute
  force, and the invariants the reference's own tests assert.
* epilogues                  - closed forms vs ``torch.autograd`` of the
  textbook expression.
* combine (both branches)    - bit for bit against the reference's tensor
  expression where the sum has one order, a scalar loop in row order, known
  answers that separate the rounding rules, autograd for the backward.
* router gate                - ``torch.topk`` where no values tie, closed
  forms, a scalar loop over ``math.exp``, a hand-worked group limit.
* cross-entropy              - ``F.cross_entropy`` in float64 (loss, per-row
  loss, autograd gradient), the closed form for uniform logits, the
  two-rounding rule at the target, the ignore rules.
"""
