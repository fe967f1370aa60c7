"""CPU oracle for the actor logprob + GRPO/DAPO policy-loss path.

TEST INFRASTRUCTURE ONLY.  This package restates, in plain torch/numpy on the CPU, the
algorithms of the reference's Python hot path (and of the Megatron-LM cross-entropy the
reference calls into).  It is the checker the HIP kernels are compared with and the CPU
baseline that the benchmark times; nothing in the shipped package imports it.

Every function cites the reference file:line it follows.  Pinning status:

* ``vocab.megatron_vocab_parallel_cross_entropy`` restates megatron-core ``core_v0.12.1``
  (``megatron/core/tensor_parallel/cross_entropy.py``), a dependency that is not vendored
  in the reference tree; the reference's tests mock it.  It is pinned here against
  ``torch.log_softmax``/``F.cross_entropy``, fp64 brute force, shift invariance and
  ``gradcheck`` - but no reference-held vector exists for it, so that boundary is
  **parity unpinned** with respect to the real Megatron/MindSpeed code.
* everything else is pinned by the reference's own unit-test vectors (see
  ``tests/golden/reference_vectors.json``) plus closed forms and brute force.
"""
from . import vocab, packing, loss, advantage  # noqa: F401
