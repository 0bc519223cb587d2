"""Pins the rounding points of the oracle's fused-kernel restatements (`k_rms_norm`, `k_swiglu`, `k_conv_update`,
`k_prepare_qkv`) with inputs on which each single rounding decides the bf16 result.

The fixtures come from tests/golden/make_rounding_cases.py (scalar float32 arithmetic, nothing from the oracle); each
holds the result with every rounding of lfm25_cuda_kernels.py:32-140 in place (`expected`) and the result a
restatement would give if it left that one rounding out (`without`).  Two cases are worked by hand below."""
import json
import os

import pytest
import torch

from oracle import lfm2_oracle as O

CASES = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "rounding_cases.json")))
BF = torch.bfloat16


def _bf(values):
    t = torch.tensor(values, dtype=torch.float32)
    assert torch.equal(t.to(BF).float(), t), "fixture inputs are exact in bf16"
    return t.to(BF)


def test_every_case_discriminates():
    assert sorted(CASES) == ["conv_bx", "conv_p0", "conv_p1", "conv_p2", "conv_sum", "qk_left", "qk_norm", "qk_right",
                             "qk_table", "qk_weight", "rms_add", "rms_norm", "swiglu_act"]
    for name, case in CASES.items():
        assert case["expected"] != case["without"], name


@pytest.mark.parametrize("name", ["rms_add", "rms_norm"])
def test_rms_norm_rounds_the_sum_and_the_normalised_value(name):
    """lfm25_cuda_kernels.py:38-42: x + residual is rounded to bf16 before the statistics, x * rsqrt is rounded before
    the weight multiply."""
    case = CASES[name]
    out, summed = O.k_rms_norm(_bf([case["x"]]), _bf(case["weight"]), case["eps"], _bf([case["residual"]]))
    assert out.float()[0].tolist() == case["expected"] and summed.float()[0].tolist() == case["summed"]


def test_swiglu_rounds_the_activation_before_the_product():
    """lfm25_cuda_kernels.py:64.  By hand: silu(1) = 0.7310586; bf16 numbers near it are 2^-8 apart, 0.73046875 is the
    nearest.  0.73046875 * 1.0078125 = 0.736175..., between 0.734375 and 0.73828125 and nearer the former (0.0018
    against 0.0021): 0.734375.  Without the first rounding: 0.7310586 * 1.0078125 = 0.73677, nearer 0.73828125."""
    case = CASES["swiglu_act"]
    assert (case["gate"], case["up"], case["expected"], case["without"]) == (1.0, 1.0078125, 0.734375, 0.73828125)
    assert O.k_swiglu(_bf([[case["gate"], case["up"]]])).float().item() == case["expected"]


@pytest.mark.parametrize("name", ["conv_bx", "conv_p0", "conv_p1", "conv_p2", "conv_sum"])
def test_conv_update_rounds_each_product_and_the_sum(name):
    """lfm25_cuda_kernels.py:85-96: b*x, the three tap products and their fp32 sum are each rounded to bf16.
    `conv_p2` by hand (b 5, c 0.8984375, x 1, taps in the state 7 and 0.7109375, weights 1, 5, 2.703125): bx = 5;
    p0 = 7; p1 = 3.5546875, a tie between 3.546875 and 3.5625 -> even mantissa 3.5625; p2 = 13.515625 -> 13.5 (bf16
    numbers are 0.0625 apart there); sum 24.0625 -> tie at spacing 0.125 -> 24.0; times c = 21.5625 -> tie -> 21.5.
    With p2 left at 13.515625 the sum is 24.078125 -> 24.125, times c = 21.6748 -> 21.625."""
    case = CASES[name]
    if name == "conv_p2":
        assert (case["expected"], case["without"]) == (21.5, 21.625)
    state = _bf([[case["state"]]])
    out = O.k_conv_update(_bf([[case["b"], case["c"], case["x"]]]), _bf([case["weight"]]), state)
    assert out.float().item() == case["expected"]
    assert state.float()[0, 0].tolist() == case["new_state"]


@pytest.mark.parametrize("name", ["qk_norm", "qk_weight", "qk_table", "qk_left", "qk_right"])
def test_prepare_qkv_rounds_norm_weight_table_and_both_rope_products(name):
    """lfm25_cuda_kernels.py:126-137: the normalised head, its product with the norm weight, the cos/sin table entries
    and the two rotation products are each rounded to bf16; the same head run as a query and as a key."""
    case = CASES[name]
    head, weight = _bf(case["x"]), _bf(case["weight"])
    cos, sin = torch.tensor([case["cos"]], dtype=torch.float32), torch.tensor([case["sin"]], dtype=torch.float32)
    x = torch.cat((head, head, torch.zeros(64, dtype=BF)))[None]
    q, k, v = O.k_prepare_qkv(x, weight, weight, cos, sin, torch.zeros(1, dtype=torch.int32), 1, 1, 64, case["eps"])
    assert q.float().flatten().tolist() == case["expected"] and k.float().flatten().tolist() == case["expected"]
    assert torch.count_nonzero(v) == 0


def test_repetition_penalty_by_brute_force():
    """lfm25_engine.py:1777-1790 with plain loops: a seen token's logit is multiplied by the penalty when negative and
    divided by it otherwise; unseen tokens and penalty 1 leave the row alone; then greedy and raw log-probability of
    lfm25_engine.py:1590-1597 on the penalised row."""
    torch.manual_seed(3)
    logits = torch.randn(5, 11) * 3
    logits[0, 4] = 0.0
    seen = torch.rand(5, 11) < 0.4
    seen[0, 4] = True
    for penalty in (1.0, 1.3, 0.5):
        got = O.repetition_penalty(logits, seen, penalty)
        for r in range(5):
            for c in range(11):
                x = logits[r, c].item()
                want = x if not seen[r, c] or penalty == 1.0 else (x * penalty if x < 0 else x / penalty)
                assert got[r, c].item() == pytest.approx(want, rel=1e-6, abs=0)
        cfg = O.OracleConfig(vocab_size=11, hidden_size=8, mlp_hidden_size=8, num_hidden_layers=0, num_attention_heads=1,
                             num_key_value_heads=1, layer_types=())
        tokens, logprobs = O.OracleEngine.sample(None, logits, temperature=0.0, seen=seen, penalty=penalty)
        for r in range(5):
            row = [got[r, c].item() for c in range(11)]
            best = max(range(11), key=lambda c: (row[c], -c))
            assert tokens[r].item() == best
            import math
            assert logprobs[r].item() == pytest.approx(row[best] - math.log(sum(math.exp(v) for v in row)), abs=1e-5)
    assert O.repetition_penalty(logits, None, 2.0) is logits
