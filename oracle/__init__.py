"""CPU oracle for the per-token log-prob / entropy / policy-loss / advantage path.

TEST INFRASTRUCTURE ONLY.  Nothing in ``relax_amd`` (the product) may import
this package: only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` use it, and only as the checker / timed
CPU baseline.  Every function is a from-scratch PyTorch-CPU restatement of the
arithmetic the reference performs, written against the reference source read
as text, and cites the reference ``file:line`` it follows (paths relative to
the reference checkout).

Pinning status (what independently fixes each function's output; the tests
live in ``tests/test_oracle_*.py``):

* ``logprob``            literal vectors of the reference's own tests
                         (tests/utils/training/test_ppo_logprob_entropy.py:174-337),
                         ``torch.log_softmax`` / ``Categorical.entropy`` library
                         routines, fp64 ``gradcheck``, shift invariance, row-sum
                         of gradient == 0.
* ``losses.policy_clip`` literals tests/backends/megatron/test_reinforce_plus_plus_loss.py:24-59,
                         tests/utils/training/test_rloo_advantages.py:263-290.
* ``losses.approx_kl``   literals tests/utils/training/test_ppo_utils_grpo.py:26-83.
* ``reducers``           literals test_reinforce_plus_plus_loss.py:62-69,
                         test_rloo_policy_loss_dispatch.py:98-187,
                         test_cp_loss_mask_alignment.py:95-139,
                         test_opd_loss_aggregation.py:36-49, brute force.
* ``advantages``         literals test_rloo_advantages.py:70-225,
                         tests/utils/replay/helpers.py:40-55,
                         test_reinforce_reward_processing.py:43-49, brute-force LOO,
                         numpy ``std(ddof=1)``.
* ``policy`` composition hand-derived end-to-end fixture tests/utils/replay/helpers.py:40-55
                         (loss = -0.02; lp=0.5 case 0.877443).
* ``lmhead``             ``F.linear`` + ``log_softmax`` (library routine),
                         test_entropy_grad_wiring.py:68-114 shape/temperature.
* ``losses.gspo_seq_kl``, ``losses.cispo``, ``opd.full_vocab_reverse_kl``
  (tail-bin modes), ``advantages.masked_whiten``: no reference test or fixture
  exists; pinned only by closed forms and brute force written independently of
  the oracle code (explicit python loops / fp64 autograd / ``scipy``-style
  textbook formulas).  The exact edge conventions the closed forms do not fix
  (CISPO ``A == 0`` branch, whiten Bessel switch at n < 2) are taken from
  reading the reference source; each docstring says which.
* ``advantages.reinforce_pp_returns`` / ``reinforce_pp_baseline_advantages``: the input cases of
  tests/utils/training/test_reinforce_plus_plus.py:45-167 with expectations worked out by hand
  (gamma = 1 reverse cumulative sums; the gamma = 0.5 case [0.20625, 0, 1.025]; masked NaN/inf).
  ``advantages.gae``: the textbook sum A_t = sum_l (gamma*lambda)^l delta_{t+l} in fp64 and the shapes case
  of tests/backends/megatron/test_ppo_gae_parity.py:41-60.  ``advantages.masked_normalize``: numpy
  population moments.  ``opd.opd_kl`` union mask / ``log_probs_on_topk_ids``: closed forms (row-prefix
  equivalence, textbook JSD, ``log_softmax`` gather).
* ``opd.reduce_token_mean``: the literal of tests/backends/megatron/test_opd_loss_aggregation.py:36-49 (12 / 3), a
  case where the token mean differs from a mean of sample means, the clamp on the whole count, the gradient
  mask / count.  ``opd.policy_opd_loss`` (opd_utils.py:1368-1455): per-token Python loops for the sampled-token and
  the three top-K selections (row loops over the K entries for reverse / forward KL and JSD in the ``tail`` / ``norm``
  / ``trunc`` modes, the union path's per-row lengths); the clip order (per-token clip, then the truncated importance
  ratio as a constant), both clip fractions as means over every token (masked ones included), the ``None`` returns,
  the detached teacher.  ``opd.apply_to_advantages`` (opd_utils.py:1275-1351): the same row loops; the clip acts on
  the top-K branch only, the term is detached, list entries are replaced.  All in ``tests/test_oracle_opd.py``.
* ``policy.sft_loss_function`` (loss.py:1247-1293): ``F.cross_entropy`` on the shifted targets (row t scores token
  t + 1, pad id 0 for the last row) with the masked reduction written as a loop, both reducer modes.
  ``policy.loss_function`` tail (loss.py:1515-1620): a three-token case with every log-prob = log 1/2 worked by hand
  for the micro-batch scale, ``dynamic_global_batch_size``, ``__loss_scale__``, the per-token mode and dummy
  micro-batches in both modes (zero loss still attached to the graph, zeroed ``values``, normaliser 0 / 1); the
  ``loss_type`` dispatch and an explicit callable.
* ``policy.value_loss_function`` / ``policy.get_values``: a three-token case worked by hand (clipped and unclipped
  branches of the maximum, the clip fraction, the response-row slicing).
* ``losses.opsm_mask`` (ppo_utils.py:142-180): scalar per-sequence / per-token Python loops on a hand-worked case
  (sequence KL exactly at delta is kept, ``A == 0`` kept, a fully masked sequence divides by one, the dropped-token
  count includes masked tokens) and on random ragged batches.  ``losses.icepop`` (loss.py:772-801): brute force per
  token with ratios exactly on either closed bound and one ulp outside, every metric, gradient = weight.
  ``losses.sapo`` (ppo_utils.py:212-270): scalar loops over random ratios with both advantage signs and ``A == 0``
  (takes ``tau_neg``), the gradient ``4 s (1 - s) r A`` against fp64 autograd, the clip-fraction threshold from the
  closed form ``4 s (1 - s) = sech^2(x / 2) < 0.9  <=>  |x| > 2 atanh(sqrt 0.1)``.
* ``reducers.seq_mean_token_sum``: the reference has no implementation of this aggregation (only the reducer plug-in
  point, loss.py:1062-1072; the example file its help text names is not in the tree), so there is nothing of the
  reference's to be at parity with; the definition used here, sum_i sum_t x*m / B, is pinned by a token loop, a
  hand-sized case and its gradient m_t / B.
"""
