"""Host logic of the packed prefill: which prompts share a chunk (no GPU)."""
import random

from climbing_gym_amd.engine import plan_packed_bins, plan_packed_chunks, plan_prefill_chunks


def test_contiguous_packed_chunks_follow_the_reference_rule_on_real_tokens():
    """lfm25_engine.py:646-665 with the budget spent on real tokens: contiguous groups, the first prompt always taken."""
    assert plan_packed_chunks([3, 3, 3, 3], 6) == [(0, 2), (2, 4)]
    assert plan_packed_chunks([9, 1, 1], 4) == [(0, 1), (1, 3)]          # a prompt above the budget goes alone
    assert plan_packed_chunks([2, 2, 2], 100) == [(0, 3)]
    assert plan_prefill_chunks([2, 2, 5, 3, 4], 24) == [(0, 4, 5), (4, 5, 4)]   # the padded rule counts the widest prompt


def test_bins_hold_every_prompt_once_within_the_budget_and_are_never_more_than_the_contiguous_chunks():
    rng = random.Random(7)
    for trial in range(200):
        budget = rng.choice((16, 100, 4096))
        lengths = [rng.randint(1, max(2, budget // rng.choice((1, 2, 5)))) for _ in range(rng.randint(1, 60))]
        if trial % 10 == 0:
            lengths[rng.randrange(len(lengths))] = budget + rng.randint(1, 50)        # one prompt above the budget
        bins = plan_packed_bins(lengths, budget)
        assert sorted(i for group in bins for i in group) == list(range(len(lengths)))
        for group in bins:
            assert group == sorted(group)
            assert sum(lengths[i] for i in group) <= budget or len(group) == 1
        assert len(bins) <= len(plan_packed_chunks(lengths, budget))


def test_bins_of_the_benchmark_prompts_are_nearly_full():
    rng = random.Random(0)
    lengths = [rng.randint(256, 2048) for _ in range(256)]
    bins, chunks = plan_packed_bins(lengths, 4096), plan_packed_chunks(lengths, 4096)
    assert sum(lengths) / (len(bins) * 4096) > 0.95 > sum(lengths) / (len(chunks) * 4096)
