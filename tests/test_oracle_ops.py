"""Pins the oracle's per-operator restatements with checks that do not retype them:
brute force on small inputs, closed forms, and known answers from the
reference's own tests."""
import itertools
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import lfm2_oracle as O


def _all_e4m3_values():
    """Every finite e4m3fn code decoded from its bit fields (OCP FP8 spec: bias 7,
    no infinities, S.1111.111 is NaN)."""
    vals = []
    for code in range(256):
        s, e, m = code >> 7, (code >> 3) & 15, code & 7
        if e == 15 and m == 7:
            continue
        mag = (m / 8) * 2.0 ** -6 if e == 0 else (1 + m / 8) * 2.0 ** (e - 7)
        vals.append((-mag if s else mag, code))
    return vals


def test_e4m3_rounding_is_nearest_even_over_all_codes():
    vals = sorted({v for v, _ in _all_e4m3_values()})
    assert max(vals) == 448.0 and len(vals) == 253  # +-0 collapse
    mant_even = {v: (c & 1) == 0 for v, c in _all_e4m3_values()}
    torch.manual_seed(0)
    x = torch.cat([torch.randn(4000) * 100, torch.randn(2000) * 0.01, torch.tensor(vals),
                   torch.tensor([(a + b) / 2 for a, b in zip(vals[:-1], vals[1:])])]).clamp(-448, 448)
    got = x.to(torch.float8_e4m3fn).float().tolist()
    for xi, gi in zip(x.tolist(), got):
        best = min(abs(v - xi) for v in vals)
        cands = [v for v in vals if abs(v - xi) == best]
        want = cands[0] if len(cands) == 1 else next(v for v in cands if mant_even[v])
        assert gi == want, (xi, gi, want)


def test_quantize_rows_scale_rule_and_error_bound():
    torch.manual_seed(1)
    x = (torch.randn(9, 300) * torch.logspace(-3, 2, 9)[:, None]).bfloat16()
    x[3].zero_()
    q, s = O.k_quantize_rows(x)
    assert s[3].item() == pytest.approx(1e-12)
    assert torch.count_nonzero(q[3].float()) == 0
    for r in (0, 5, 8):
        assert s[r].item() == pytest.approx(x[r].float().abs().max().item() / 448, rel=1e-6)
        # the row maximum maps onto +-448 exactly and relative error stays within half an e4m3 ulp
        assert q[r].float().abs().max().item() == 448.0
        deq = q[r].float() * s[r]
        big = x[r].float().abs() > s[r] * 2 ** -6
        assert ((deq - x[r].float()).abs()[big] <= x[r].float().abs()[big] * (2 ** -4) * 1.0001).all()


def test_fused_quantising_forms_equal_their_two_step_forms():
    torch.manual_seed(2)
    x = torch.randn(7, 256).bfloat16()
    r = torch.randn(7, 256).bfloat16()
    w = torch.randn(256).bfloat16()
    out, summed = O.k_rms_norm(x, w, 1e-5, r)
    q, s, summed2 = O.k_rms_norm_fp8(x, w, 1e-5, r)
    assert torch.equal(summed, summed2) and torch.equal(summed, (x.float() + r.float()).bfloat16())
    q2, s2 = O.k_quantize_rows(out)
    assert torch.equal(q.view(torch.uint8), q2.view(torch.uint8)) and torch.equal(s, s2)


@pytest.mark.parametrize("dt,atol", [(torch.float32, 2e-5), (torch.bfloat16, 0.04)])
def test_rounded_kernels_agree_with_plain_formulas(dt, atol):
    # tolerances of tests/test_lfm25_cuda.py:31-32
    torch.manual_seed(17)
    x, r, w = torch.randn(3, 512).to(dt), torch.randn(3, 512).to(dt), torch.randn(512).to(dt)
    out, summed = O.k_rms_norm(x, w, 1e-5, r)
    torch.testing.assert_close(out, O.rms_norm(x + r, w, 1e-5), atol=atol, rtol=0.01)
    p = torch.randn(3, 2 * 640).to(dt)
    g, u = p.chunk(2, -1)
    torch.testing.assert_close(O.k_swiglu(p), F.silu(g) * u, atol=atol, rtol=0.01)
    # prepare_qkv against eager rms_norm + rotary
    QH, KH, D = 8, 2, 64
    qkv = torch.randn(3, (QH + 2 * KH) * D).to(dt)
    qw, kw = torch.randn(D).to(dt), torch.randn(D).to(dt)
    pos = torch.tensor([3, 27, 101], dtype=torch.int32)
    cos, sin = O.rope_tables(D, 1e7, 128)
    q, k, v = O.k_prepare_qkv(qkv, qw, kw, cos, sin, pos, QH, KH, D, 1e-5)
    eq = O.apply_rotary(O.rms_norm(qkv[:, :QH * D].reshape(3, QH, D), qw, 1e-5), cos[pos.long(), None], sin[pos.long(), None])
    ek = O.apply_rotary(O.rms_norm(qkv[:, QH * D:(QH + KH) * D].reshape(3, KH, D), kw, 1e-5), cos[pos.long(), None], sin[pos.long(), None])
    torch.testing.assert_close(q[:, 0], eq, atol=atol, rtol=0.01)
    torch.testing.assert_close(k[:, 0], ek, atol=atol, rtol=0.01)
    assert torch.equal(v[:, 0], qkv[:, (QH + KH) * D:].reshape(3, KH, D))


def test_conv_update_is_a_causal_depthwise_conv_by_brute_force():
    torch.manual_seed(4)
    H, T = 16, 9
    w = torch.randn(H, 3)
    b, c, x = torch.randn(T, H), torch.randn(T, H), torch.randn(T, H)
    state = torch.zeros(1, H, 3)
    got = torch.stack([O.k_conv_update(torch.cat((b[t], c[t], x[t]))[None], w, state)[0] for t in range(T)])
    bx = b * x
    for t, ch in itertools.product(range(T), range(H)):
        acc = sum(w[ch, j].item() * bx[t - 2 + j, ch].item() for j in range(3) if t - 2 + j >= 0)
        assert got[t, ch].item() == pytest.approx(c[t, ch].item() * acc, rel=1e-4, abs=1e-5)
    torch.testing.assert_close(state[0], bx[-3:].T)  # index 2 = newest tap
    # masked rows and slot indirection: state of an inactive row is untouched, slot -1 clamps to 0
    state = torch.randn(4, H, 3)
    keep = state.clone()
    bcx = torch.randn(3, 3 * H)
    O.k_conv_update(bcx, w, state, active=torch.tensor([True, False, True]), slot_ids=torch.tensor([2, 1, -1], dtype=torch.int32))
    assert torch.equal(state[1], keep[1]) and torch.equal(state[3], keep[3])
    assert not torch.equal(state[2], keep[2]) and not torch.equal(state[0], keep[0])


def test_prefill_conv_state_and_output_match_stepwise_decode():
    torch.manual_seed(5)
    from climbing_gym_amd.synthetic import random_state_dict
    shape = dict(hidden=32, mlp_hidden=64, layer_types=("conv", "conv"), q_heads=4, kv_heads=2, vocab=50)
    cfg = O.OracleConfig(vocab_size=50, hidden_size=32, mlp_hidden_size=64, num_hidden_layers=2,
                         num_attention_heads=4, num_key_value_heads=2, max_position_embeddings=64,
                         layer_types=shape["layer_types"])
    eng = O.OracleEngine(cfg, random_state_dict(**shape, seed=5, std=0.2), torch.float32, 64)
    prompt = [3, 9, 4, 17, 8]
    cache_a, logits_a = eng.prefill([prompt], cap=8)
    cache_b, _ = eng.prefill([prompt[:1]], cap=8)
    for t in prompt[1:]:
        logits_b = eng.append_tokens(cache_b, torch.tensor([0]), torch.tensor([t]))
    torch.testing.assert_close(logits_a, logits_b, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(cache_a.conv, cache_b.conv, atol=1e-6, rtol=1e-5)


def _filter_brute(row, top_k, top_p):
    """Definition by loops: the k-th largest value is the threshold (ties kept); sort
    descending, accumulate softmax mass, drop a rank when the running mass exceeds
    top_p, never rank 0."""
    vals = list(row)
    if 0 < top_k < len(vals):
        kth = sorted(vals, reverse=True)[top_k - 1]
        vals = [v if v >= kth else -math.inf for v in vals]
    if top_p < 1.0:
        order = sorted(range(len(vals)), key=lambda i: -vals[i])
        m = max(vals)
        z = sum(math.exp(v - m) for v in vals)
        run, out = 0.0, [-math.inf] * len(vals)
        for rank, i in enumerate(order):
            run += math.exp(vals[i] - m) / z
            if rank == 0 or run <= top_p:
                out[i] = vals[i]
        vals = out
    return vals


@pytest.mark.parametrize("top_k,top_p", [(0, 0.5), (3, 1.0), (4, 0.8), (1, 0.1), (50, 0.95), (0, 0.999)])
def test_top_k_top_p_filter_by_brute_force(top_k, top_p):
    g = torch.Generator().manual_seed(6)
    logits = torch.randn(6, 11, generator=g, dtype=torch.float64) * 2
    got = O.top_k_top_p_filter(logits, top_k, top_p)
    for r in range(6):
        want = _filter_brute(logits[r].tolist(), top_k, top_p)
        assert [math.isinf(a) for a in got[r].tolist()] == [math.isinf(b) for b in want]
    # ties at the k-th value are all kept
    tie = torch.tensor([[1.0, 3.0, 3.0, 3.0, 0.0]])
    assert torch.isfinite(O.top_k_top_p_filter(tie, 2, 1.0)).sum() == 3
    # the head of the distribution survives even when it alone exceeds top_p
    assert torch.isfinite(O.top_k_top_p_filter(torch.tensor([[9.0, 0.0, 0.0]]), 0, 0.01)).sum() == 1


@pytest.mark.parametrize("temperature,top_k,top_p", [(1.0, 0, 1.0), (0.7, 0, 1.0), (0.7, 3, 1.0), (1.3, 0, 0.6), (0.5, 4, 0.8), (0.0, 0, 1.0)])
def test_sampling_logprobs_by_brute_force(temperature, top_k, top_p):
    """The third value of the reference's `_sample`: the pick's probability among the survivors of the tempered
    logits, worked out term by term in Python floats.  A missing temperature, a normaliser over the whole row instead
    of the survivors, or the raw logit in the numerator each fail one of the cases."""
    g = torch.Generator().manual_seed(16)
    logits = torch.randn(5, 9, generator=g) * 2
    for r in range(5):
        row = logits[r].tolist()
        if temperature == 0.0:
            kept, scaled = row, row
        else:
            scaled = [v / temperature for v in row]
            kept = _filter_brute(scaled, top_k, top_p)
        m = max(kept)
        log_z = m + math.log(sum(math.exp(v - m) for v in kept if not math.isinf(v)))
        for tok in range(9):
            got = O.sampling_logprobs(logits[r:r + 1], torch.tensor([tok]), temperature, top_k, top_p).item()
            if math.isinf(kept[tok]):
                assert got == -math.inf
            else:
                assert abs(got - (scaled[tok] - log_z)) < 2e-6
        # the survivors' probabilities sum to one
        alive = [t for t in range(9) if not math.isinf(kept[t])]
        total = sum(math.exp(O.sampling_logprobs(logits[r:r + 1], torch.tensor([t]), temperature, top_k, top_p).item()) for t in alive)
        assert abs(total - 1.0) < 1e-5


def test_sample_returns_raw_and_sampling_logprobs():
    logits = torch.randn(6, 40, generator=torch.Generator().manual_seed(17))
    gen = torch.Generator().manual_seed(0)
    tok, raw, tempered = O.OracleEngine.sample_with_sampling_logprobs(None, logits, temperature=0.8, top_k=5, top_p=0.9, generator=gen)
    torch.testing.assert_close(raw, logits.log_softmax(-1).gather(1, tok[:, None])[:, 0])
    assert torch.isfinite(tempered).all()   # drawn tokens are survivors
    torch.testing.assert_close(tempered, O.sampling_logprobs(logits, tok, 0.8, 5, 0.9))
    tok0, raw0, tempered0 = O.OracleEngine.sample_with_sampling_logprobs(None, logits, temperature=0.0)
    assert torch.equal(tok0, logits.argmax(-1)) and torch.equal(raw0, tempered0)


def test_greedy_picks_first_maximum_and_true_log_softmax():
    logits = torch.randn(4, 1000, generator=torch.Generator().manual_seed(7)).bfloat16()
    logits[1, 12] = logits[1, 900] = 20
    tok, lp = O.greedy_with_logprob(logits)
    assert tok[1].item() == 12
    torch.testing.assert_close(lp, logits.double().log_softmax(-1).gather(1, tok[:, None])[:, 0].float(), atol=3e-6, rtol=2e-6)


def test_stop_table_known_answer_from_reference_test():
    # tests/test_text_stops.py:7-19,68-78: pieces '<', '/', 'summary', '>', 'x', padded ids decode to ''
    pieces = ['<', '/', 'summary', '>', 'x'] + [''] * 11
    table = O.build_stop_table(pieces, ('</summary>',))
    state, hits = 0, []
    for tok in [15, 0, 1, 9, 2, 15, 3]:
        value = int(table[state, tok])
        state = value & 65535
        hits.append(value >= 65536)
    assert hits == [False] * 6 + [True]
    # a wrong continuation falls back to the longest matching prefix
    s = int(table[0, 0]) & 65535
    assert int(table[s, 0]) & 65535 == s  # '<<' still ends with '<'
    assert int(table[s, 4]) & 65535 == 0  # '<x' matches nothing


def test_finish_codes_and_rng_key():
    assert O.record_sample_row(7, 0, 10, 0, 0, eos=7, ignore_eos=False) == 1
    assert O.record_sample_row(7, 0, 10, 0, 0, eos=7, ignore_eos=True) == 0
    assert O.record_sample_row(5, 0, 10, 0, 65536 + 3, eos=7, ignore_eos=False) == 2
    assert O.record_sample_row(5, 9, 10, 0, 0, eos=7, ignore_eos=False) == 3
    assert O.record_sample_row(7, 9, 10, 0, 65536, eos=7, ignore_eos=False) == 1  # EOS wins
    assert O.session_rng_key(-1, 0) == 0x7FFFFFFFFFFFFFFF
    assert O.session_rng_key(5, 2) == (5 + 2 * 0x9E3779B97F4A7C15) & 0x7FFFFFFFFFFFFFFF


def test_decode_attention_row_matches_causal_attention_last_row():
    torch.manual_seed(8)
    T, QH, KH, D = 37, 8, 2, 32
    q, k, v = torch.randn(T, QH, D), torch.randn(T, KH, D), torch.randn(T, KH, D)
    full = O.causal_attention(q, k, v, D ** -0.5)
    for t in (0, 5, 36):
        torch.testing.assert_close(O.k_attend(q[t], k, v, t + 1, D ** -0.5), full[t], atol=1e-5, rtol=1e-5)
    kq, ks, vq, vs = O.k_store_kv(k, v)
    deq = O.k_attend(q[36], kq, vq, 37, D ** -0.5, ks, vs)
    torch.testing.assert_close(deq, full[36], atol=0.05, rtol=0.05)


def test_w8a8_emulation_is_exact_on_grid_inputs_and_bounded_otherwise():
    """Inputs that already sit on the e4m3 grid of their row (maximum mapped to 448) survive quantisation unchanged,
    so the emulated projection equals the exact one; for arbitrary inputs the deviation obeys the half-ulp bound
    |dy| <= sum |x||w| * ((1 + 2^-4)^2 - 1) of two relative roundings of at most 2^-4 each."""
    from climbing_gym_amd.synthetic import random_state_dict
    codes = torch.tensor([v for v, _ in _all_e4m3_values() if abs(v) >= 2 ** -6 or v == 0])
    g = torch.Generator().manual_seed(9)
    pick = lambda r, c: codes[torch.randint(0, len(codes), (r, c), generator=g)]
    x, w = pick(6, 96) * 0.37, pick(10, 96) * 0.011
    x[:, 0], w[:, 0] = 448 * 0.37, 448 * 0.011
    cfg = O.OracleConfig(vocab_size=16, hidden_size=8, mlp_hidden_size=8, num_hidden_layers=1, num_attention_heads=2,
                         num_key_value_heads=1, max_position_embeddings=8, layer_types=("conv",))
    state = random_state_dict(hidden=8, mlp_hidden=8, layer_types=("conv",), q_heads=2, kv_heads=1, vocab=16)
    eng = O.OracleEngine(cfg, state, torch.float32, 8, fp8=("mlp",))
    torch.testing.assert_close(eng._lin(x, w, "mlp"), (x.double() @ w.double().T).float(), atol=1e-3, rtol=1e-5)
    assert torch.equal(eng._lin(x, w, "head"), torch.nn.functional.linear(x, w))  # other parts stay exact
    x, w = torch.randn(7, 200, generator=g), torch.randn(9, 200, generator=g) * 0.02
    dy = (eng._lin(x, w, "mlp") - x @ w.T).abs()
    bound = (x.abs() @ w.abs().T) * ((1 + 2 ** -4) ** 2 - 1) + 2 ** -6 * 448 ** -1 * (x.abs().amax(1)[:, None] * w.abs().sum(1)[None] + w.abs().amax(1)[None] * x.abs().sum(1)[:, None])
    assert (dy <= bound).all() and dy.max() > 0
    k, v = torch.randn(5, 2, 16, generator=g), torch.randn(5, 2, 16, generator=g)
    kv = O.OracleEngine(cfg, state, torch.float32, 8, fp8=("kv",))
    kq, vq = kv._kv(k, v)
    assert ((kq - k).abs() <= k.abs() * 2 ** -4 + k.abs().amax(-1, keepdim=True) / 448 * 2 ** -7).all()
    assert kv._kv(kq, vq)[0].sub(kq).abs().max() < 1e-6  # the round trip is idempotent
