"""CPU oracle for the GRPO/GSPO policy-loss path.  TEST INFRASTRUCTURE ONLY.

This package restates, with torch/numpy on the CPU, what the reference's
``chatlearn/algorithm/grpo_utils`` functions compute.  It exists so that the
HIP kernels can be checked against it; nothing under ``chatlearn_amd/`` may
import it.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` use it, and there only as the checker or
as the timed CPU baseline.

How each function is pinned (the reference's own tests hold no vector for any
of them, so none is pinned by a reference fixture):

* softmax statistics (logprob, entropy) and their gradients: closed forms
  (uniform logits, one dominant logit, shift invariance, zero-sum gradient),
  a pure-Python row loop on tiny shapes, and torch's library routines.
* GRPO / GSPO surrogate losses: closed forms for every clip branch
  (``tests/test_oracle_cpu.py``) and torch autograd for the tie gradients.
* k3 KL estimator: ``kl >= 0``, zero iff equal, derivative ``1 - exp(ref-lp)``.
* bin packing: hand-worked cases stored in ``tests/golden/packing_cases.json``
  that exercise the strict-fit rule, first-on-ties and stable descending
  order, plus invariants on random inputs.
* masks / unpad / pad: brute-force nested loops on tiny shapes and the
  round-trip ``pad(unpad(x)) == x * mask``.
* group advantages: ``numpy.mean`` / ``numpy.std`` and the Bernoulli closed
  form ``(1-k/G)/(sqrt(k/G(1-k/G))+1e-5)``.
* the Megatron trainer's packed batch (sequence padding to tp*cp*2, unpad,
  label roll, rolled loss mask): hand-worked cases in
  ``tests/golden/thd_pack_cases.json``; the context-parallel index split it
  calls from TransformerEngine is restated from the published chunk scheme and
  is PARITY UNPINNED for more than one rank (identity for one rank).
* the FSDP trainer's micro-batch loops (``policy_loop.py``: preprocess_data_list, train_step,
  forward_step): a three-sample case worked by hand from the reference lines with literal expected
  tables (``tests/test_policy_loop_cpu.py``): micro-batch order with a tie on the bin totals, packed
  row, indices, position ids, labels rolling across sequence boundaries, shifted training mask,
  record lengths and values, train_stats and a row of the parameter gradient.
* vocabulary-parallel logprob / entropy (the reference's three all-reduces
  over tensor-parallel ranks): equality with the unsharded log_softmax gather
  and entropy for every way of cutting the vocabulary, and the uniform-logits
  closed form.
"""
