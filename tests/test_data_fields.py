"""Host logic of the wire formats either side of the path (CPU).

Field lists: the assertions of the reference's tests/backends/megatron/test_sft_train_data_fields.py:27-74, re-typed,
plus the PPO consumer branches and the distillation schema read off relax/utils/training/data_fields.py:25-82 and
relax/utils/opd/opd_main_worker.py:84-104, 272-278.  Jagged packing: against torch's own list-based constructor, which
is what the reference calls (relax/backends/megatron/actor.py:2356-2360).
"""

from argparse import Namespace

import pytest
import torch

from relax_amd import data_fields as DF


def _args(loss_type="policy_loss", **kw):
    base = dict(loss_type=loss_type, use_rollout_routing_replay=False, multimodal_keys=None, use_opd=False,
                opd_type=None, opd_log_prob_top_k=0)
    base.update(kw)
    return Namespace(**base)


BASE = ["tokens", "total_lengths", "response_lengths", "loss_masks", "rollout_log_probs", "rewards", "sample_indices",
        "sample_index_mask_sums", "raw_reward", "group_index"]


def test_sft_fields_exclude_rl_only_keys():
    fields = DF.build_data_fields(_args("sft"))
    assert fields == ["tokens", "total_lengths", "response_lengths", "loss_masks"]
    for forbidden in ("rollout_log_probs", "rewards", "raw_reward", "teacher_log_probs"):
        assert forbidden not in fields


def test_sequence_classification_sft_requests_labels():
    fields = DF.build_data_fields(_args("sft", task_type="seq_cls"))
    assert "classification_labels" in fields and "sample_weights" not in fields
    assert DF.build_data_fields(_args("sft", multimodal_keys={"image": "images"}))[-1] == "multimodal_train_inputs"


def test_rl_fields_include_replay_metadata_in_reference_order():
    assert DF.build_data_fields(_args()) == BASE
    assert DF.build_data_fields(_args(use_rollout_routing_replay=True, multimodal_keys={"a": "b"})) == \
        BASE + ["rollout_routed_experts", "multimodal_train_inputs"]


def test_ppo_consumers():
    ppo = dict(advantage_estimator="ppo")
    assert DF.build_data_fields(_args(**ppo), consumer="critic") == BASE
    assert DF.build_data_fields(_args(**ppo), consumer="advantages") == BASE + ["values"]
    assert DF.build_data_fields(_args(kl_coef=0.1, **ppo), consumer="advantages") == \
        BASE + ["values", "log_probs", "ref_log_probs"]
    assert DF.build_data_fields(_args(kl_coef=0.1, use_rollout_logprobs=True, **ppo), consumer="advantages") == \
        BASE + ["values", "ref_log_probs"]
    assert DF.build_data_fields(_args(kl_coef=0.1, true_on_policy_mode=True, **ppo), consumer="advantages") == \
        BASE + ["values", "ref_log_probs"]
    # actor: colocated PPO consumes the critic's values; fully asynchronous PPO pulls finished advantages
    assert DF.build_data_fields(_args(**ppo)) == BASE + ["values"]
    assert DF.build_data_fields(_args(kl_coef=0.1, **ppo)) == BASE + ["values", "ref_log_probs"]
    assert DF.build_data_fields(_args(use_kl_loss=True, **ppo)) == BASE + ["values", "ref_log_probs"]
    assert DF.build_data_fields(_args(fully_async=True, **ppo)) == BASE + ["advantages", "returns"]
    assert DF.build_data_fields(_args(fully_async=True, hybrid=True, **ppo)) == BASE + ["values"]
    assert DF.build_data_fields(_args(fully_async=True, use_kl_loss=True, **ppo)) == \
        BASE + ["advantages", "returns", "ref_log_probs"]
    # the consumer is only meaningful for PPO
    assert DF.build_data_fields(_args(advantage_estimator="grpo"), consumer="critic") == BASE


def test_opd_schema():
    sampled = _args(use_opd=True, opd_type="sglang", opd_token_selection="student_sampled")
    assert DF.build_data_fields(sampled) == BASE + ["teacher_log_probs", "rollout_log_probs"]
    topk = _args(use_opd=True, opd_type="sglang", opd_token_selection="teacher_topk", opd_kl_coef=0.0)
    assert DF.build_data_fields(topk) == BASE + ["opd_topk_token_ids", "opd_topk_teacher_log_probs"]
    union_adv = _args(use_opd=True, opd_type="sglang", opd_token_selection="union", opd_kl_coef=0.5)
    assert DF.build_data_fields(union_adv) == BASE + ["opd_topk_token_ids", "opd_topk_teacher_log_probs",
                                                      "opd_topk_student_log_probs", "opd_topk_ksz"]
    # a Megatron teacher computes its side inside the training job: nothing extra is transferred
    assert DF.build_data_fields(_args(use_opd=True, opd_type="megatron", opd_token_selection="union")) == BASE
    extra = []
    DF.consume_opd_advantage_data(extra, _args(use_opd=True, opd_type="megatron", opd_token_selection="student_topk"))
    assert extra == ["opd_topk_token_ids", "opd_topk_teacher_log_probs"]
    with pytest.raises(KeyError):
        DF.opd_transfer_schema(_args(opd_token_selection="everything"))


def test_restore_topk_fields_fixed_k_and_union():
    args = _args(opd_token_selection="student_topk", opd_log_prob_top_k=3)
    data = {"response_lengths": [2, 0, 1],
            "opd_topk_token_ids": [[5, 6, 7, 1, 2, 3], [], [9, 8, 7]],
            "opd_topk_teacher_log_probs": [[-1.0, -2.0, -3.0, -0.5, -1.5, -2.5], [], None]}
    DF.restore_opd_topk_rollout_fields(data, args, "cpu")
    ids = data["opd_topk_token_ids"]
    assert ids[0].dtype == torch.long and ids[0].tolist() == [[5, 6, 7], [1, 2, 3]]
    assert ids[1].shape == (0, 3) and ids[2].tolist() == [[9, 8, 7]]
    assert data["opd_topk_teacher_log_probs"][0].dtype == torch.float32
    assert data["opd_topk_teacher_log_probs"][2] is None

    uargs = _args(opd_token_selection="union", opd_log_prob_top_k=2)
    udata = {"response_lengths": [2, 3, 0],
             "opd_topk_token_ids": [[4, 5, 6, 7, -1, -1], [1, 2, 3], []],
             "opd_topk_ksz": [[3, 1], [1, 1, 1], None]}
    DF.restore_opd_topk_rollout_fields(udata, uargs, "cpu")
    assert udata["opd_topk_token_ids"][0].tolist() == [[4, 5, 6], [7, -1, -1]]  # width = numel / response length
    assert udata["opd_topk_token_ids"][1].shape == (3, 1) and udata["opd_topk_token_ids"][2].shape == (0, 1)
    assert udata["opd_topk_ksz"][0].tolist() == [3, 1] and udata["opd_topk_ksz"][2] is None
    # not a top-K selection, or K = 0: untouched
    keep = {"opd_topk_token_ids": [[1, 2]]}
    DF.restore_opd_topk_rollout_fields(keep, _args(opd_token_selection="student_sampled", opd_log_prob_top_k=2), "cpu")
    DF.restore_opd_topk_rollout_fields(keep, _args(opd_token_selection="union", opd_log_prob_top_k=0), "cpu")
    assert keep == {"opd_topk_token_ids": [[1, 2]]}


def _same_jagged(got, items):
    want = torch.nested.as_nested_tensor([t.cpu() for t in items], layout=torch.jagged)
    assert got.is_nested and got.layout == torch.jagged and got.device.type == "cpu"
    a, b = got.unbind(), want.unbind()
    assert len(a) == len(b)
    for x, y in zip(a, b):
        assert x.dtype == y.dtype and torch.equal(x, y)


def test_jagged_to_host_packed_views_and_loose_tensors():
    packed = torch.arange(17, dtype=torch.float32)
    views = list(packed[2:16].split([3, 0, 7, 4]))  # consecutive views, one of them empty, not starting at 0
    assert DF._packed_parent(views) is not None
    _same_jagged(DF.jagged_to_host(views), views)
    loose = [torch.randn(3), torch.randn(0), torch.randn(5)]
    assert DF._packed_parent(loose) is None
    _same_jagged(DF.jagged_to_host(loose), loose)
    gappy = [packed[0:3], packed[5:9]]  # views of one tensor, but not consecutive
    assert DF._packed_parent(gappy) is None
    _same_jagged(DF.jagged_to_host(gappy), gappy)
    two_d = [torch.randn(2, 4), torch.randn(5, 4)]  # e.g. gathered top-K log-probs
    _same_jagged(DF.jagged_to_host(two_d), two_d)
    with pytest.raises(ValueError):
        DF.jagged_to_host([])


def test_transfer_payload_and_advantages_payload():
    lp = torch.randn(9)
    out = DF.to_transfer_payload({"log_probs": list(lp.split([4, 5])), "entropy_mean": torch.tensor(1.5)})
    _same_jagged(out["log_probs"], list(lp.split([4, 5])))
    assert out["entropy_mean"].item() == 1.5
    adv = [torch.randn(3), torch.randn(6)]
    pay = DF.advantages_payload(adv, adv)
    assert pay["advantages"].is_nested and [t.shape for t in pay["returns"].unbind()] == [t.shape for t in adv]
    assert all(torch.equal(x, y) for x, y in zip(pay["advantages"].unbind(), adv))


def test_ppl_metrics_literals():
    """tests/engine/sft/eval/test_ppl.py:14-33: totals 10.0 over 6 tokens; an empty evaluation gives zeros."""
    import math

    from relax_amd.sft_eval import compute_ppl_metrics

    m = compute_ppl_metrics(total_neg_log_prob=10.0, total_tokens=6)
    assert math.isclose(m["eval/loss"], 10.0 / 6.0, rel_tol=1e-6)
    assert math.isclose(m["eval/ppl"], math.exp(10.0 / 6.0), rel_tol=1e-5) and m["eval/num_tokens"] == 6
    assert compute_ppl_metrics(0.0, 0) == {"eval/loss": 0.0, "eval/ppl": 0.0, "eval/num_tokens": 0}


def test_custom_reward_post_process_hook():
    """``--custom-reward-post-process-path`` (relax/utils/utils.py:186-192): the named function replaces the built-in
    processing; a 2-tuple is taken as (raw, processed), anything else as the processed rewards next to the raw ones."""
    from types import SimpleNamespace

    from relax_amd.utils import post_process_rewards

    class S:
        def __init__(self, r):
            self.r, self.group_index = r, 0

        def get_reward_value(self, args):
            return self.r

    samples = [S(1.0), S(2.0), S(6.0)]
    args = SimpleNamespace(custom_reward_post_process_path="tests.custom_hooks.halved_rewards",
                           advantage_estimator="grpo", rewards_normalization=True)
    assert post_process_rewards(args, samples) == ([1.0, 2.0, 6.0], [0.5, 1.0, 3.0])
    args.custom_reward_post_process_path = "tests.custom_hooks.raw_and_centred_rewards"
    assert post_process_rewards(args, samples) == ([1.0, 2.0, 6.0], [-2.0, -1.0, 3.0])
