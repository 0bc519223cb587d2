"""GPU parity tests: every HIP kernel, called through the C ABI, against the CPU oracle on the same
seeded inputs.  The cases follow the reference's own kernel tests (tests/test_lfm25_cuda.py:19-63,
316-347, tests/test_lfm25_fp8.py:14-56, tests/test_lfm25_fp8_kv.py:27-88).

Bars: integer/index outputs exact; e4m3 codes and model-dtype roundings bit-exact except where a
differently ordered fp32 reduction moves a value across a rounding boundary (bounded below as a
fraction of elements and by one unit in the last place); fp32 within the stated tolerances.
"""
import math

import pytest
import torch

from oracle import lfm2_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def ops():
    from climbing_gym_amd import ops as module
    return module


TOL = {torch.float32: (2e-5, 1e-5), torch.bfloat16: (0.04, 0.01), torch.float16: (0.004, 0.01)}


def _close_mostly_exact(actual, expected, dtype, max_fraction=2e-3):
    """Within the reference's kernel-test tolerances (tests/test_lfm25_cuda.py:31-32) everywhere and, for
    the 16-bit dtypes, bit-exact except for rare flips caused by the order of an fp32 reduction."""
    a, e = actual.float().cpu(), expected.float().cpu()
    atol, rtol = TOL[dtype]
    torch.testing.assert_close(a, e, atol=atol, rtol=rtol)
    if dtype != torch.float32:
        frac = (a != e).float().mean().item()
        assert frac <= max_fraction, f"{frac:.2e} of elements differ from the oracle"


@pytest.mark.parametrize("dtype", (torch.float32, torch.bfloat16, torch.float16))
@torch.inference_mode()
def test_fused_decode_kernels_match_oracle(ops, dtype):
    torch.manual_seed(17)
    batch, width = 3, 2048
    x, residual = torch.randn(batch, width, dtype=dtype), torch.randn(batch, width, dtype=dtype)
    weight = torch.randn(width, dtype=dtype)
    out, summed = ops.rms_norm(x.to(DEV), weight.to(DEV), 1e-5, residual.to(DEV))
    eo, es = O.k_rms_norm(x, weight, 1e-5, residual)
    assert torch.equal(summed.cpu(), es)
    _close_mostly_exact(out, eo, dtype)
    out2, same = ops.rms_norm(x.to(DEV), weight.to(DEV), 1e-5)
    assert same.data_ptr() != out2.data_ptr()
    _close_mostly_exact(out2, O.k_rms_norm(x, weight, 1e-5)[0], dtype)

    projected = torch.randn(batch, 2 * 10752, dtype=dtype)
    _close_mostly_exact(ops.swiglu(projected.to(DEV)), O.k_swiglu(projected), dtype, 5e-3)

    bcx = torch.randn(batch, width * 3, dtype=dtype)
    state = torch.randn(batch, width, 3, dtype=dtype)
    conv_w = torch.randn(width, 3, dtype=dtype)
    dstate = state.to(DEV)
    got = ops.conv_update(bcx.to(DEV), conv_w.to(DEV), dstate)
    want = O.k_conv_update(bcx, conv_w, state)
    assert torch.equal(dstate.cpu(), state)
    assert torch.equal(got.cpu(), want)

    QH, KH, D = 32, 8, 64
    qkv = torch.randn(batch, (QH + 2 * KH) * D, dtype=dtype)
    qw, kw = torch.randn(D, dtype=dtype), torch.randn(D, dtype=dtype)
    pos = torch.tensor([3, 27, 101], dtype=torch.int32)
    cos, sin = O.rope_tables(D, 1e7, 128)
    q, k, v = ops.prepare_qkv(qkv.to(DEV), qw.to(DEV), kw.to(DEV), cos.to(DEV), sin.to(DEV), pos.to(DEV), QH, KH, D, 1e-5)
    eq, ek, ev = O.k_prepare_qkv(qkv, qw, kw, cos, sin, pos, QH, KH, D, 1e-5)
    assert q.shape == (batch, 1, QH, D) and k.shape == (batch, 1, KH, D)
    assert torch.equal(v.cpu(), ev)
    _close_mostly_exact(q, eq, dtype, 5e-3)
    _close_mostly_exact(k, ek, dtype, 5e-3)


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float16))
@torch.inference_mode()
def test_prepare_qkv_on_a_prefill_sized_batch_matches_oracle(ops, dtype):
    """From 512 rows on, head_dim 64 runs the 16-bytes-per-lane form (eight lanes per head); the rows' count is not a
    multiple of what a workgroup takes, positions are spread over the rotary table."""
    torch.manual_seed(19)
    rows, QH, KH, D = 777, 32, 8, 64
    qkv = torch.randn(rows, (QH + 2 * KH) * D, dtype=dtype)
    qw, kw = torch.randn(D, dtype=dtype), torch.randn(D, dtype=dtype)
    pos = torch.randint(0, 4096, (rows,), dtype=torch.int32)
    cos, sin = O.rope_tables(D, 1e6, 4096)
    q, k, v = ops.prepare_qkv(qkv.to(DEV), qw.to(DEV), kw.to(DEV), cos.to(DEV), sin.to(DEV), pos.to(DEV), QH, KH, D, 1e-5)
    eq, ek, ev = O.k_prepare_qkv(qkv, qw, kw, cos, sin, pos, QH, KH, D, 1e-5)
    assert torch.equal(v.cpu(), ev)
    _close_mostly_exact(q, eq, dtype, 5e-3)
    _close_mostly_exact(k, ek, dtype, 5e-3)
    few = ops.prepare_qkv(qkv[:40].to(DEV), qw.to(DEV), kw.to(DEV), cos.to(DEV), sin.to(DEV), pos[:40].to(DEV), QH, KH, D, 1e-5)
    _close_mostly_exact(q[:40], few[0].cpu(), dtype, 5e-3)      # the wave-per-head form on the same rows


@torch.inference_mode()
def test_conv_update_masks_rows_and_follows_slot_ids(ops):
    torch.manual_seed(3)
    H = 256
    state = torch.randn(5, H, 3).bfloat16()
    bcx = torch.randn(3, 3 * H).bfloat16()
    w = torch.randn(H, 3).bfloat16()
    active = torch.tensor([True, False, True])
    slots = torch.tensor([4, 2, -1], dtype=torch.int32)
    active[2] = False  # padding rows are inactive and read slot 0
    dstate = state.to(DEV)
    got = ops.conv_update(bcx.to(DEV), w.to(DEV), dstate, active.to(DEV), slots.to(DEV))
    want = O.k_conv_update(bcx, w, state, active, slots)
    assert torch.equal(dstate.cpu(), state) and torch.equal(got.cpu(), want)


@pytest.mark.parametrize("width", (129, 2048, 16384))
@torch.inference_mode()
def test_fused_activation_quantization_matches_separate_kernels_and_oracle(ops, width):
    # tests/test_lfm25_fp8.py:14-33: the fused forms are bitwise the two-step forms
    torch.manual_seed(10)
    x, residual = torch.randn(17, width).bfloat16(), torch.randn(17, width).bfloat16()
    weight = torch.randn(width).bfloat16()
    dx, dr, dw = x.to(DEV), residual.to(DEV), weight.to(DEV)
    normalized, expected_sum = ops.rms_norm(dx, dw, 1e-5, dr)
    if width % 8 == 0:
        expected, scales = ops.quantize_rows(normalized)
    else:
        expected, scales = ops.quantize_rows(normalized.contiguous())
    actual, actual_scales, summed = ops.rms_norm_fp8(dx, dw, 1e-5, dr)
    assert torch.equal(summed, expected_sum) and torch.equal(actual_scales, scales)
    assert torch.equal(actual.view(torch.uint8), expected.view(torch.uint8))
    # the quantising half is bit-exact: the oracle's row quantisation of the very values the norm kernel produced
    oq, oscale = O.k_quantize_rows(normalized.cpu())
    assert torch.equal(actual_scales.cpu(), oscale) and torch.equal(actual.cpu().view(torch.uint8), oq.view(torch.uint8))
    # end to end against the oracle the only freedom is the order of the norm's fp32 sum of squares, which moves a
    # normalised value across a bf16 boundary in well under 1 % of the elements; a row's scale differs only when that
    # happens to the row's largest element, and then by one bf16 step
    oq, oscale, _ = O.k_rms_norm_fp8(x, weight, 1e-5, residual)
    torch.testing.assert_close(actual_scales.cpu(), oscale, rtol=2 ** -7, atol=0)
    same_scale = actual_scales.cpu() == oscale
    mismatch = (actual.cpu().view(torch.uint8) != oq.view(torch.uint8))[same_scale].float().mean().item()
    print(f"width {width}: rows with the oracle's scale {int(same_scale.sum())}/17, differing e4m3 codes in those rows {mismatch:.2e}")
    assert same_scale.sum() >= 16 and mismatch < 1e-3
    projected = torch.randn(17, 2 * width).bfloat16()
    expected, scales = ops.quantize_rows(ops.swiglu(projected.to(DEV)))
    actual, actual_scales = ops.swiglu_fp8(projected.to(DEV))
    assert torch.equal(actual_scales, scales) and torch.equal(actual.view(torch.uint8), expected.view(torch.uint8))


@torch.inference_mode()
def test_quantize_rows_is_bit_exact_with_oracle_and_rejects_bad_input(ops):
    torch.manual_seed(5)
    x = (torch.randn(33, 1000) * torch.logspace(-4, 3, 33)[:, None]).bfloat16()
    x[4].zero_()
    x.view(-1)[::97] *= 20
    q, s = ops.quantize_rows(x.to(DEV))
    oq, os_ = O.k_quantize_rows(x)
    assert torch.equal(s.cpu(), os_)
    assert torch.equal(q.cpu().view(torch.uint8), oq.view(torch.uint8))
    with pytest.raises(ValueError):
        ops.quantize_rows(x)  # CPU tensor
    with pytest.raises(ValueError):
        ops.quantize_rows(x.to(DEV).float())
    with pytest.raises(ValueError):
        ops.quantize_rows(torch.zeros(2, 40000, device=DEV, dtype=torch.bfloat16))


@pytest.mark.parametrize("batch,width,outputs", [(3, 129, 193), (128, 2048, 512), (32, 8192, 128), (1, 2048, 3072),
                                                 (257, 5632, 2048), (64, 2048, 1040), (16, 5632, 2048), (48, 5632, 2048)])
@torch.inference_mode()
def test_fp8_projection_matches_independently_dequantized_operands(ops, batch, width, outputs):
    torch.manual_seed(42)
    x = torch.randn(batch, width).bfloat16()
    x.view(-1)[::101] *= 20  # outliers as in the GEMM benchmark inputs
    weight = (torch.randn(outputs, width) * 0.025).bfloat16()
    if batch > 1:
        x[0].zero_()
    weight[0].zero_()
    packed = ops.PackedFP8Weight.from_weight(weight.to(DEV))
    q, scale = ops.quantize_rows(x.to(DEV))
    expected = O.k_fp8_linear(q.cpu(), scale.cpu(), packed.values.cpu(), packed.scales.cpu(), torch.float32)
    actual = packed.linear(x.to(DEV))
    assert actual.dtype == torch.bfloat16
    err = (actual.float().cpu() - expected).norm() / expected.norm()
    assert err < 1e-2  # relative error bar of the FP8 GEMM against the dequantised matmul
    torch.testing.assert_close(actual.float().cpu(), expected, atol=0.02, rtol=0.015)
    assert torch.isfinite(actual).all()
    assert actual[:, 0].count_nonzero() == 0 and (batch == 1 or actual[0].count_nonzero() == 0)
    reference = (x.float() @ weight.float().T)
    assert (actual.float().cpu() - reference).norm() / reference.norm() < 0.065
    if width % 16 == 0:
        for tile in range(23):
            for split in (1, 2, 4):
                got = packed.linear_quantized(q, scale, config=(tile, split))
                torch.testing.assert_close(got.float().cpu(), expected, atol=0.02, rtol=0.015)
        f32 = packed.linear_quantized(q, scale, dtype=torch.float32)
        assert (f32.cpu() - expected).norm() / expected.norm() < 5e-4, (f32.cpu() - expected).norm() / expected.norm()
        torch.testing.assert_close(f32.cpu(), expected, atol=3e-3, rtol=2e-3)


@torch.inference_mode()
def test_fp8_weight_refresh_reuses_buffers(ops):
    # tests/test_lfm25_fp8.py:82-90: policy sync re-quantises in place
    torch.manual_seed(1)
    w = (torch.randn(64, 256, device=DEV) * 0.02).bfloat16()
    packed = ops.PackedFP8Weight.from_weight(w)
    ptrs = (packed.values.data_ptr(), packed.scales.data_ptr())
    before = packed.values.clone()
    w.normal_(std=0.05)
    packed.refresh()
    assert ptrs == (packed.values.data_ptr(), packed.scales.data_ptr())
    assert not torch.equal(before.view(torch.uint8), packed.values.view(torch.uint8))
    oq, os_ = O.k_quantize_rows(w.cpu())
    assert torch.equal(packed.values.cpu().view(torch.uint8), oq.view(torch.uint8)) and torch.equal(packed.scales.cpu(), os_)


@pytest.mark.parametrize("m,k,n", [(1, 2048, 6144), (5, 2048, 512), (256, 2048, 3072), (300, 5632, 2048), (64, 104, 72)])
@torch.inference_mode()
def test_bf16_linear_matches_fp32_matmul_of_the_same_operands(ops, m, k, n):
    torch.manual_seed(7)
    x, w = torch.randn(m, k).bfloat16(), (torch.randn(n, k) * 0.02).bfloat16()
    expected = x.float() @ w.float().T
    for tile, split in [(-1, 0), (0, 1), (2, 2), (4, 1), (5, 4), (6, 1), (7, 2), (8, 1)]:
        got = ops.linear(x.to(DEV), w.to(DEV), tile=tile, split_k=split)
        torch.testing.assert_close(got.float().cpu(), expected, atol=2e-3, rtol=2 ** -7)


@pytest.mark.parametrize("m,k,n,parts", [(16, 2048, 8192, 1), (16, 2048, 2048, 1), (24, 5632, 2048, 2), (300, 2048, 2048, 1),
                                         (300, 5632, 2048, 4)])
@torch.inference_mode()
def test_fp8_partial_sums_through_the_c_abi_add_up_to_the_product(ops, m, k, n, parts):
    """`lfm2_fp8_gemm_partials` asked for a given number of parts of K, one included (a single fp32 plane: on few rows of
    a wide output the few-row kernel, which then keeps one column tile per workgroup): the planes, summed in order and
    scaled, round to the product `lfm2_fp8_gemm` stores."""
    g = torch.Generator().manual_seed(m + n + parts)
    packed = ops.PackedFP8Weight.from_weight((torch.randn(n, k, generator=g) * 0.03).bfloat16().to(DEV))
    xq, xs = ops.quantize_rows(torch.randn(m, k, generator=g).bfloat16().to(DEV))
    partials = torch.full((parts, m, n), float("nan"), device=DEV, dtype=torch.float32)
    ops.call("lfm2_fp8_gemm_partials", partials, xq, packed.values, m, n, k, -1, parts)
    total = partials[0].clone()
    for part in partials[1:]:
        total += part
    got = ((total * xs[:, None]) * packed.scales[None, :]).bfloat16()
    want = packed.linear_quantized(xq, xs)
    # the product itself may sum its K steps in another order than the parts do (other tile, other split): one bf16 step
    exact = packed.linear_quantized(xq, xs, config=(-1, parts)) if parts > 1 else want
    assert bool(torch.isfinite(partials).all())
    torch.testing.assert_close(got.float(), exact.float(), atol=2e-3, rtol=2 ** -7)
    torch.testing.assert_close(got.float(), want.float(), atol=2e-3, rtol=2 ** -7)


@pytest.mark.parametrize("fp8", [True, False])
@pytest.mark.parametrize("m,k,n", [(48, 512, 1000), (200, 2048, 4096), (7, 100, 72), (40, 512, 1024), (9, 1024, 2048)])
@torch.inference_mode()
def test_placed_rows_equal_the_product_followed_by_scatter_logits(ops, fp8, m, k, n):
    """The placing GEMMs against the plain product + `scatter_logits` (lfm25_batching.py:25-32): bit-identical live
    rows, untouched rows elsewhere; padding slots (-1), inactive rows and out-of-range slots are skipped.  K = 100 takes the
    any-shape kernel."""
    torch.manual_seed(m + n)
    x, w = torch.randn(m, k, device=DEV).bfloat16(), (torch.randn(n, k, device=DEV) * 0.05).bfloat16()
    capacity = m + 9
    slots = torch.randperm(capacity, device=DEV)[:m].to(torch.int32)
    slots[1] = -1
    slots[m - 1] = capacity + 3                      # beyond the destination: dropped, never written
    active = torch.rand(m, device=DEV) > 0.3
    active[0] = True
    packed = ops.PackedFP8Weight.from_weight(w) if fp8 else None
    q, scales = ops.quantize_rows(x) if fp8 else (None, None)

    def product(place=None, tile=-1):
        if fp8:
            return packed.linear_quantized(q, scales, dtype=torch.bfloat16, config=(tile, 0), place=place)
        return ops.linear(x, w, tile=tile, place=place)

    for tile in (-1, 0, 2, 6, 12, 14, 15, 17):
        if not fp8 and tile >= 9:
            continue
        plain = product(tile=tile)
        for use_slots, use_mask in [(True, True), (True, False), (False, True), (False, False)]:
            saved = torch.full((capacity, n), 7.0, device=DEV, dtype=torch.bfloat16)
            expected = saved.clone()
            rows = torch.arange(m, device=DEV)
            target = slots.long() if use_slots else rows
            keep = (target >= 0) & (target < capacity)
            if use_mask:
                keep &= active
            expected[target[keep]] = plain[keep]
            out = product(ops.RowPlacement(saved, slots if use_slots else None, active if use_mask else None), tile)
            assert out is saved
            assert torch.equal(saved.view(torch.int16), expected.view(torch.int16)), (tile, use_slots, use_mask)
    with pytest.raises(ValueError):
        product(ops.RowPlacement(torch.zeros(m - 1, n, device=DEV, dtype=torch.bfloat16)))
    with pytest.raises(ValueError):
        product(ops.RowPlacement(torch.zeros(capacity, n, device=DEV, dtype=torch.float16), slots))


def _cache_tensors(batch, capacity, heads, dim, layout):
    if layout == "HND":
        k = torch.zeros(batch, heads, capacity, dim, device=DEV, dtype=torch.float8_e4m3fn).transpose(1, 2)
        s = torch.zeros(batch, heads, capacity, device=DEV, dtype=torch.float32).transpose(1, 2)
    else:
        k = torch.zeros(batch, capacity, heads, dim, device=DEV, dtype=torch.float8_e4m3fn)
        s = torch.zeros(batch, capacity, heads, device=DEV, dtype=torch.float32)
    return k, torch.zeros_like(k), s, torch.zeros_like(s)


@pytest.mark.parametrize("layout", ["NHD", "HND"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@torch.inference_mode()
def test_scaled_storage_handles_strided_prefill_views_zeros_and_outliers(ops, layout, dtype):
    torch.manual_seed(18)
    kc, vc, ks, vs = _cache_tensors(5, 79, 3, 64, layout)
    k = torch.randn(2, 37, 3, 64, dtype=dtype)
    v = torch.randn_like(k)
    k[0, 0].zero_(), v[0, 0].zero_()
    k[1, :, 1] *= 100
    v[1, :, 2] *= 0.0001
    ops.store_kv(k.to(DEV), v.to(DEV), kc[2:4, :37], vc[2:4, :37], ks[2:4, :37], vs[2:4, :37])
    ekq, eks, evq, evs = O.k_store_kv(k, v)
    for values, scales, eq, es in ((kc, ks, ekq, eks), (vc, vs, evq, evs)):
        assert torch.equal(scales[2:4, :37].cpu(), es)
        assert torch.equal(values[2:4, :37].cpu().view(torch.uint8), eq.view(torch.uint8))
        assert torch.count_nonzero(values[:2].float()) == 0
        assert torch.count_nonzero(values[2:4, 37:].float()) == 0
        assert torch.count_nonzero(values[4:].float()) == 0


@torch.inference_mode()
def test_append_preserves_inactive_histories_and_uses_independent_positions(ops):
    kc, vc, ks, vs = _cache_tensors(3, 19, 2, 64, "HND")
    k = torch.randn(3, 1, 2, 64, device=DEV, dtype=torch.bfloat16)
    v = torch.randn_like(k)
    positions = torch.tensor([3, 18, 7], device=DEV, dtype=torch.int32)
    active = torch.tensor([True, False, True], device=DEV)
    ops.store_kv(k, v, kc, vc, ks, vs, positions=positions, active=active)
    assert torch.count_nonzero(kc[1].float()) == 0 and torch.count_nonzero(ks[1]) == 0
    for row, pos in [(0, 3), (2, 7)]:
        assert ks[row, pos].min() > 0
        torch.testing.assert_close(kc[row, pos].float() * ks[row, pos, :, None], k[row, 0].float(), atol=.12, rtol=.05)
        assert torch.count_nonzero(ks[row, :pos]) == 0 and torch.count_nonzero(ks[row, pos + 1:]) == 0
    # slot indirection
    slots = torch.tensor([2, 0, 1], device=DEV, dtype=torch.int32)
    kc2, vc2, ks2, vs2 = _cache_tensors(3, 19, 2, 64, "NHD")
    ops.store_kv(k, v, kc2, vc2, ks2, vs2, positions=positions, slot_ids=slots)
    assert torch.equal(kc2[2, 3].view(torch.uint8), kc[0, 3].view(torch.uint8))
    assert torch.count_nonzero(ks2[0, 18]) == 2


@pytest.mark.parametrize("dim,groups", [(32, 1), (64, 4), (128, 2), (256, 1), (64, 8)])
@pytest.mark.parametrize("fp8", [True, False])
@torch.inference_mode()
def test_decode_matches_independent_fp32_softmax_with_ragged_lengths_and_inactive_rows(ops, dim, groups, fp8):
    torch.manual_seed(92)
    batch, capacity, heads = 5, 1300, 2
    k = torch.randn(batch, capacity, heads, dim).bfloat16()
    v = torch.randn_like(k)
    q = torch.randn(batch, 1, heads * groups, dim).bfloat16()
    positions = torch.tensor([0, 36, 250, 250, 1299], dtype=torch.int32)
    active = torch.tensor([True, True, True, False, True])
    if fp8:
        kc, vc, ks, vs = _cache_tensors(batch, capacity, heads, dim, "HND")
        ops.store_kv(k.to(DEV), v.to(DEV), kc, vc, ks, vs)
        hist = (kc.cpu(), vc.cpu(), ks.cpu(), vs.cpu())
    else:
        kc, vc, ks, vs = k.to(DEV), v.to(DEV), None, None
        hist = (k, v, None, None)
    actual = ops.attend(q.to(DEV), kc, vc, ks, vs, positions.to(DEV), active=active.to(DEV))
    for row in (0, 1, 2, 4):
        expected = O.k_attend(q[row, 0], hist[0][row], hist[1][row], int(positions[row]) + 1, dim ** -0.5,
                              None if hist[2] is None else hist[2][row], None if hist[3] is None else hist[3][row])
        torch.testing.assert_close(actual[row, 0].float().cpu(), expected, atol=0.012, rtol=0.025)
    assert torch.count_nonzero(actual[3]) == 0
    # slot indirection: rows read other slots, a negative slot is padding
    slots = torch.tensor([4, 2, 1, -1, 0], dtype=torch.int32)
    pos2 = positions[slots.clamp_min(0).long()]
    moved = ops.attend(q.to(DEV), kc, vc, ks, vs, pos2.to(DEV), active=torch.tensor([True, True, True, False, True]).to(DEV),
                       slot_ids=slots.to(DEV))
    expected = O.k_attend(q[0, 0], hist[0][4], hist[1][4], 1300, dim ** -0.5,
                          None if hist[2] is None else hist[2][4], None if hist[3] is None else hist[3][4])
    torch.testing.assert_close(moved[0, 0].float().cpu(), expected, atol=0.012, rtol=0.025)
    assert torch.count_nonzero(moved[3]) == 0


@pytest.mark.parametrize("rows,longest", [(1500, 3000), (300, 1200)])
@torch.inference_mode()
def test_work_list_lists_every_chunk_once_longest_first(ops, rows, longest):
    """Layout of the decode-attention work list: pair count and chunk size (512 tokens when the rows would make at
    least 3072 chunks of 256, else 256); a record per row (first full pair, partial pair, length or 0 for rows that
    sit out); a record per pair (row, chunk, length, slot), full chunks first, then partial chunks by decreasing
    number of 64-token tiles.  1500 rows: more than one block of the device scan."""
    torch.manual_seed(3)
    lengths = torch.randint(1, longest, (rows,))
    lengths[:8] = torch.tensor([1, 64, 65, 256, 257, 512, longest - 1, 255])
    active = torch.rand(rows) > 0.1
    slots = torch.randperm(rows).to(torch.int32)
    slots[torch.rand(rows) < 0.05] = -1
    schedule = ops.decode_schedule((lengths - 1).to(torch.int32).to(DEV), active.to(DEV), slots.to(DEV), capacity=3072).cpu()
    live = active & (slots >= 0)
    eff = torch.where(live, lengths, torch.zeros_like(lengths))
    short_pairs = int((eff + 255).div(256, rounding_mode="floor").sum())
    chunk = 512 if short_pairs >= 3072 else 256
    assert int(schedule[1]) == chunk and chunk == (512 if rows == 1500 else 256)
    pairs = int((eff + chunk - 1).div(chunk, rounding_mode="floor").sum())
    assert int(schedule[0]) == pairs
    row_rec = schedule[4:4 + 4 * rows].view(rows, 4)
    pair_rec = schedule[4 + 4 * rows:4 + 4 * rows + 4 * pairs].view(pairs, 4)
    assert torch.equal(row_rec[:, 2].long(), eff)
    # every (row, chunk) exactly once, with the row's length and slot
    seen = set()
    for r, c, n, slot in pair_rec.tolist():
        assert live[r] and n == int(lengths[r]) and slot == int(slots[r]) and 0 <= c * chunk < n
        assert (r, c) not in seen
        seen.add((r, c))
    assert len(seen) == pairs
    # order: tiles per item never increase
    tiles = [min(chunk, n - c * chunk + 0) for r, c, n, s in pair_rec.tolist()]
    tiles = [(t + 63) // 64 for t in tiles]
    assert tiles == sorted(tiles, reverse=True)
    # the rows' records point at their pairs
    for r in torch.nonzero(live).flatten().tolist()[:200]:
        n = int(lengths[r])
        for c in range(n // chunk):
            assert pair_rec[int(row_rec[r, 0]) + c].tolist()[:2] == [r, c]
        if n % chunk:
            assert pair_rec[int(row_rec[r, 1])].tolist()[:2] == [r, n // chunk]


@pytest.mark.parametrize("quantized", [False, True])
@pytest.mark.parametrize("fp8", [True, False])
@torch.inference_mode()
def test_decode_over_more_rows_than_one_scan_block(ops, quantized, fp8):
    """1100 rows (the device scan of the work list handles 1024 per block) with lengths across the chunk and tile
    boundaries, inactive rows and slot indirection, against the oracle on sampled rows; e4m3 history (64-token
    tiles) and bf16 history stored head-major (32-token tiles)."""
    torch.manual_seed(17)
    rows, capacity, heads, groups, dim = 1100, 600, 8, 4, 64
    k = torch.randn(rows, capacity, heads, dim).bfloat16()
    v = torch.randn_like(k)
    q = torch.randn(rows, 1, heads * groups, dim).bfloat16()
    lengths = torch.randint(1, capacity + 1, (rows,))
    lengths[:10] = torch.tensor([1, 64, 256, 257, 512, 600, 31, 32, 33, 289])
    active = torch.rand(rows) > 0.1
    slots = torch.randperm(rows).to(torch.int32)
    picked = [int(torch.nonzero(slots == i)[0]) for i in range(10)]     # the rows that read the hand-picked lengths
    active[picked] = True
    if fp8:
        kc, vc, ks, vs = _cache_tensors(rows, capacity, heads, dim, "HND")
        ops.store_kv(k.to(DEV), v.to(DEV), kc, vc, ks, vs)
        hist = (kc.cpu(), vc.cpu(), ks.cpu(), vs.cpu())
    else:
        head_major = lambda t: t.to(DEV).permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
        kc, vc, ks, vs = head_major(k), head_major(v), None, None
        hist = (k, v, [None] * rows, [None] * rows)
    positions = (lengths[slots.long()] - 1).to(torch.int32)     # row i reads slot slots[i]
    out = ops.attend(q.to(DEV), kc, vc, ks, vs, positions.to(DEV), active=active.to(DEV), slot_ids=slots.to(DEV),
                     quantized=quantized)
    if quantized:
        codes, scales = out
        result = (codes.float() * scales[:, None]).view(rows, heads * groups, dim).cpu()
    else:
        result = out[:, 0].float().cpu()
    for row in picked + [0, 1, 2, 3, 4, 5, 511, 1023, 1024, 1025, 1099]:
        if not active[row]:
            assert torch.count_nonzero(result[row]) == 0
            continue
        slot = int(slots[row])
        expected = O.k_attend(q[row, 0], hist[0][slot], hist[1][slot], int(lengths[slot]), dim ** -0.5, hist[2][slot], hist[3][slot])
        tolerance = dict(atol=0.05, rtol=0.07) if quantized else dict(atol=0.012, rtol=0.025)   # e4m3 rows: 1/16 relative steps
        torch.testing.assert_close(result[row], expected, **tolerance)
    assert torch.count_nonzero(result[~active]) == 0


@pytest.mark.parametrize("groups,rows,capacity", [(1, 37, 700), (2, 37, 700), (4, 37, 700), (4, 1001, 300)])
@pytest.mark.parametrize("quantized", [False, True])
@pytest.mark.parametrize("fp8", [True, False])
@torch.inference_mode()
def test_decode_with_a_workgroup_per_row_and_kv_head_matches_the_oracle(ops, groups, rows, capacity, quantized, fp8):
    """37 rows of 8 KV heads: from 64 (row, KV head) pairs on, a workgroup's four waves share one pair's tiles and merge
    through LDS.  Lengths sit on both sides of the 32- and 64-token tile and of the four-tile round; a row count that is
    no multiple of 8 leaves empty places in the last round of the XCD mapping; inactive rows and padding slots give
    zeros; every live row is checked against the oracle (of 1001 rows, near the 1024 the rows are ranked for, a sample)."""
    torch.manual_seed(41)
    heads, dim = 8, 64
    k = torch.randn(rows, capacity, heads, dim).bfloat16()
    v = torch.randn_like(k)
    q = torch.randn(rows, 1, heads * groups, dim).bfloat16()
    lengths = torch.randint(1, capacity + 1, (rows,))
    fixed = [n for n in (1, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 512, 513, 700) if n <= capacity]
    lengths[:len(fixed)] = torch.tensor(fixed)
    active = torch.rand(rows) > 0.15
    slots = torch.randperm(rows).to(torch.int32)
    padding = [5, 20]
    slots[padding] = -1
    if fp8:
        kc, vc, ks, vs = _cache_tensors(rows, capacity, heads, dim, "HND")
        ops.store_kv(k.to(DEV), v.to(DEV), kc, vc, ks, vs)
        hist = (kc.cpu(), vc.cpu(), ks.cpu(), vs.cpu())
    else:
        head_major = lambda t: t.to(DEV).permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
        kc, vc, ks, vs = head_major(k), head_major(v), None, None
        hist = (k, v, [None] * rows, [None] * rows)
    positions = (lengths[slots.clamp_min(0).long()] - 1).to(torch.int32)     # row i reads slot slots[i]
    out = ops.attend(q.to(DEV), kc, vc, ks, vs, positions.to(DEV), active=active.to(DEV), slot_ids=slots.to(DEV),
                     quantized=quantized)
    if quantized:
        codes, scales = out
        result = (codes.float() * scales[:, None]).view(rows, heads * groups, dim).cpu()
        # the bits of the row quantiser on the plain result, also through a schedule shared by two calls
        plain = ops.attend(q.to(DEV), kc, vc, ks, vs, positions.to(DEV), active=active.to(DEV), slot_ids=slots.to(DEV))
        want_codes, want_scales = ops.quantize_rows(plain.view(rows, -1))
        shared = ops.decode_schedule(positions.to(DEV), active.to(DEV), slots.to(DEV), capacity=capacity)
        again = [ops.attend(q.to(DEV), kc, vc, ks, vs, positions.to(DEV), active=active.to(DEV), slot_ids=slots.to(DEV),
                            quantized=True, schedule=shared) for _ in range(2)]
        for got_codes, got_scales in (out, *again):
            assert torch.equal(got_codes.view(torch.uint8), want_codes.view(torch.uint8))
            assert torch.equal(got_scales, want_scales)
    else:
        result = out[:, 0].float().cpu()
    checked = 0
    dead = ~active | (slots < 0)
    assert torch.count_nonzero(result[dead]) == 0
    for row in (range(rows) if rows < 100 else [*range(0, rows, 17), rows - 2, rows - 1]):
        slot = int(slots[row])
        if dead[row]:
            continue
        expected = O.k_attend(q[row, 0], hist[0][slot], hist[1][slot], int(lengths[slot]), dim ** -0.5, hist[2][slot], hist[3][slot])
        tolerance = dict(atol=0.05, rtol=0.07) if quantized else dict(atol=0.012, rtol=0.025)   # e4m3 rows: 1/16 relative steps
        torch.testing.assert_close(result[row], expected, **tolerance)
        checked += 1
    assert checked >= 24


@pytest.mark.parametrize("batch", [6, 11])    # 48 and 88 (row, KV head) pairs: the item list, a workgroup per pair
@pytest.mark.parametrize("fp8", [True, False])
@torch.inference_mode()
def test_paged_slot_mapped_history_equals_dense_history(ops, fp8, batch):
    """Block-16 paged layout: the same tokens reached through a shuffled block table give the same output."""
    torch.manual_seed(4)
    heads, groups, dim, page = 8, 4, 64, 16
    lengths = torch.tensor([1, 16, 17, 300, 1000, 777, 64, 65, 1008, 513, 48][:batch])
    cap = 1008
    k = torch.randn(batch, cap, heads, dim).bfloat16()
    v = torch.randn_like(k)
    q = torch.randn(batch, 1, heads * groups, dim).bfloat16().to(DEV)
    positions = (lengths - 1).to(torch.int32).to(DEV)
    blocks_per_row = cap // page
    perm = torch.randperm(batch * blocks_per_row)
    table = perm.view(batch, blocks_per_row).to(torch.int32)
    if fp8:
        kc, vc, ks, vs = _cache_tensors(batch, cap, heads, dim, "NHD")
        ops.store_kv(k.to(DEV), v.to(DEV), kc, vc, ks, vs)
    else:
        kc, vc, ks, vs = k.to(DEV), v.to(DEV), None, None
    dense = ops.attend(q, kc, vc, ks, vs, positions)

    def to_pages(t):  # [batch, cap, ...] -> pool [pages, page, ...] under the block table
        pool = torch.empty((batch * blocks_per_row, page, *t.shape[2:]), device=DEV, dtype=t.dtype)
        src = t.reshape(batch * blocks_per_row, page, *t.shape[2:])
        if t.dtype == torch.float8_e4m3fn:
            pool.view(torch.uint8)[table.view(-1).long().to(DEV)] = src.view(torch.uint8)
        else:
            pool[table.view(-1).long().to(DEV)] = src
        return pool
    pools = [to_pages(kc), to_pages(vc), None if ks is None else to_pages(ks), None if vs is None else to_pages(vs)]
    paged = ops.attend(q, *pools, positions, block_table=table.to(DEV), page=page)
    assert torch.equal(paged, dense)
    # the same pages stored head-major ([pages, heads, page, ...] behind the [pages, page, heads, ...] view): the
    # strides of a page are arguments, and a head's tokens are then contiguous inside a page
    def head_major(t):
        if t is None:
            return None
        rest = range(3, t.ndim)
        return t.permute(0, 2, 1, *rest).contiguous().permute(0, 2, 1, *rest)
    paged = ops.attend(q, *[head_major(t) for t in pools], positions, block_table=table.to(DEV), page=page)
    assert torch.equal(paged, dense)


@pytest.mark.parametrize("lengths", [[1, 7, 64, 65, 130, 33], [300, 1, 129, 513, 64, 128, 257]])   # up to 3 and up to 9 query blocks per sequence
@pytest.mark.parametrize("dim,qh,kh", [(64, 32, 8), (64, 4, 2), (32, 4, 4), (128, 4, 1)])
@torch.inference_mode()
def test_varlen_prefill_attention_matches_causal_sdpa(ops, dim, qh, kh, lengths):
    torch.manual_seed(11)
    total = sum(lengths)
    q = torch.randn(total, qh, dim).bfloat16()
    k = torch.randn(total, kh, dim).bfloat16()
    v = torch.randn(total, kh, dim).bfloat16()
    cu = torch.tensor([0, *torch.tensor(lengths).cumsum(0).tolist()], dtype=torch.int32)
    got = ops.prefill_attention(q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV), max(lengths)).float().cpu()
    for i, n in enumerate(lengths):
        a, b = int(cu[i]), int(cu[i + 1])
        want = O.causal_attention(q[a:b], k[a:b], v[a:b], dim ** -0.5)
        torch.testing.assert_close(got[a:b], want, atol=0.02, rtol=0.02)


@pytest.mark.parametrize("H,dtype", [(2048, torch.bfloat16), (136, torch.bfloat16), (512, torch.float16), (2056, torch.bfloat16),
                                     (100, torch.bfloat16)])
@torch.inference_mode()
def test_packed_prefill_conv_with_quantised_rows_equals_the_two_launches(ops, H, dtype):
    """`conv_prefill_fp8` against `quantize_rows(conv_prefill(...))`, bit for bit: codes, per-token scales and every
    slot's conv state, on a ragged packed batch whose token count is not a multiple of the four tokens a workgroup
    takes, with a width below a workgroup's 2048 channels (threads that own no channel still take part in the row
    maximum) and widths the one-launch form does not cover (the wrapper then runs the two launches itself)."""
    torch.manual_seed(H)
    lengths, slots = [1, 2, 7, 3, 41, 9], [4, 0, 2, 5, 1, 6]
    total = sum(lengths)
    cu = torch.tensor([0, *torch.tensor(lengths).cumsum(0).tolist()], dtype=torch.int32, device=DEV)
    bcx = torch.randn(total, 3 * H, device=DEV).to(dtype)
    bcx[5] = 0                                         # a row of zeros: its scale is the floor, its codes zero
    w = torch.randn(H, 3, device=DEV).to(dtype)
    seq, _ = ops.build_token_map(cu, total)
    dslots = torch.tensor(slots, dtype=torch.int32, device=DEV)
    state_a = torch.ones(7, H, 3, device=DEV, dtype=dtype)
    state_b = state_a.clone()
    want_q, want_s = ops.quantize_rows(ops.conv_prefill(bcx, w, state_a, cu, seq, dslots))
    got_q, got_s = ops.conv_prefill_fp8(bcx, w, state_b, cu, seq, dslots)
    assert got_q.shape == (total, H) and got_s.shape == (total,)
    assert torch.equal(got_s.view(torch.int32), want_s.view(torch.int32))
    assert torch.equal(got_q.view(torch.uint8), want_q.view(torch.uint8))
    assert torch.equal(state_b.view(torch.int16), state_a.view(torch.int16))
    assert float(got_s[5]) == pytest.approx(1.0e-12) and int((got_q[5].view(torch.uint8) & 0x7F).max()) == 0   # +0 or -0


@pytest.mark.parametrize("H", [128, 100])     # 16-byte accesses, 8 channels x 4 tokens per thread; scalar form
@torch.inference_mode()
def test_packed_prefill_conv_and_kv_store_match_per_sequence_oracle(ops, H):
    torch.manual_seed(12)
    lengths, slots = [1, 2, 5, 3, 40], [4, 0, 2, 5, 1]
    total = sum(lengths)
    cu = torch.tensor([0, *torch.tensor(lengths).cumsum(0).tolist()], dtype=torch.int32)
    bcx = torch.randn(total, 3 * H).bfloat16()
    w = torch.randn(H, 3).bfloat16()
    state = torch.ones(6, H, 3, device=DEV, dtype=torch.bfloat16)  # dirty state must be replaced
    seq, pos = ops.build_token_map(cu.to(DEV), total)
    assert seq.cpu().tolist() == [i for i, n in enumerate(lengths) for _ in range(n)]
    assert pos.cpu().tolist() == [p for n in lengths for p in range(n)]
    got = ops.conv_prefill(bcx.to(DEV), w.to(DEV), state, cu.to(DEV), seq, torch.tensor(slots, dtype=torch.int32, device=DEV))
    b, c, x = bcx.float().chunk(3, -1)
    bx = (b * x).bfloat16().float()
    for i, n in enumerate(lengths):
        a = int(cu[i])
        padded = torch.cat((torch.zeros(2, H), bx[a:a + n]))
        conv = sum(padded[j:j + n] * w.float()[:, j] for j in range(3))
        want = (c[a:a + n] * conv.bfloat16().float()).bfloat16()
        torch.testing.assert_close(got[a:a + n].cpu().float(), want.float(), atol=2e-2, rtol=2 ** -6)
        assert torch.equal(state[slots[i]].cpu().float(), padded[-3:].T.contiguous())
    assert torch.equal(state[3].cpu(), torch.ones(H, 3).bfloat16())
    # KV store of the same packed batch into fp8 and bf16 caches
    KH, D = 2, 64
    k, v = torch.randn(total, KH, D).bfloat16(), torch.randn(total, KH, D).bfloat16()
    kc, vc, ks, vs = _cache_tensors(6, 48, KH, D, "HND")
    dslots = torch.tensor(slots, dtype=torch.int32, device=DEV)
    ops.store_kv_packed(k.to(DEV), v.to(DEV), kc, vc, ks, vs, cu.to(DEV), seq, dslots)
    kb = torch.zeros(6, 48, KH, D, device=DEV, dtype=torch.bfloat16)
    vb = torch.zeros_like(kb)
    ops.store_kv_packed(k.to(DEV), v.to(DEV), kb, vb, None, None, cu.to(DEV), seq, dslots)
    ekq, eks, evq, evs = O.k_store_kv(k, v)
    for i, n in enumerate(lengths):
        a = int(cu[i])
        assert torch.equal(kc[slots[i], :n].cpu().view(torch.uint8), ekq[a:a + n].view(torch.uint8))
        assert torch.equal(vs[slots[i], :n].cpu(), evs[a:a + n])
        assert torch.equal(kb[slots[i], :n].cpu(), k[a:a + n]) and torch.equal(vb[slots[i], :n].cpu(), v[a:a + n])
        assert torch.count_nonzero(kb[slots[i], n:]) == 0


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float16, torch.float32))
@torch.inference_mode()
def test_fused_sampling_greedy_and_raw_logprobs(ops, dtype):
    torch.manual_seed(45)
    logits = torch.randn(9, 128003, dtype=dtype)
    logits[0, :8192] = -torch.inf  # fully masked tiles must not spoil the normaliser
    logits[1, 12] = logits[1, 125000] = 20  # ties choose the first token
    tokens, logprobs = ops.sample_logits(logits.to(DEV), temperature=0, seed=0, step=0, return_logprobs=True)
    et, elp = O.greedy_with_logprob(logits)
    assert torch.equal(tokens.cpu(), et)
    torch.testing.assert_close(logprobs.cpu(), elp, atol=3e-6, rtol=2e-6)
    sampled, raw = ops.sample_logits(logits.to(DEV), temperature=0.7, seed=31, step=4095, return_logprobs=True)
    expected = logits.double().log_softmax(-1).gather(1, sampled.cpu()[:, None]).squeeze(1).float()
    torch.testing.assert_close(raw.cpu(), expected, atol=3e-6, rtol=2e-6)
    assert (sampled.cpu() >= 8192)[0]


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float32))
@torch.inference_mode()
def test_full_support_sampling_reports_the_tempered_logprob(ops, dtype):
    """Third value of lfm25_engine.py:1574-1609 for the full-support draw: log softmax(logits / T) of the pick; the
    raw log-probability at temperature 0 (:1594-1596) and at temperature 1."""
    torch.manual_seed(46)
    logits = (torch.randn(7, 9001) * 2).to(dtype)
    logits[2, :4096] = -torch.inf
    for temperature in (0.6, 1.0, 1.7, 0.0):
        tempered = torch.empty(7, device=DEV, dtype=torch.float32)
        tok, raw = ops.sample_logits(logits.to(DEV), temperature=temperature, seed=3, step=9, return_logprobs=True,
                                     sampling_logprobs=tempered)
        plain = ops.sample_logits(logits.to(DEV), temperature=temperature, seed=3, step=9, return_logprobs=True)
        assert torch.equal(tok, plain[0]) and torch.equal(raw, plain[1])
        want = O.sampling_logprobs(logits.double(), tok.cpu(), temperature, 0, 1.0).float()
        torch.testing.assert_close(tempered.cpu(), want, atol=5e-6, rtol=2e-6)
        if temperature in (0.0, 1.0):
            torch.testing.assert_close(tempered, raw, atol=5e-6, rtol=2e-6)
    with pytest.raises(ValueError, match="sampling_logprobs"):
        ops.sample_logits(logits.to(DEV), temperature=1.0, seed=0, step=0, return_logprobs=True,
                          sampling_logprobs=torch.empty(3, device=DEV))


@torch.inference_mode()
def test_fused_categorical_sampling_distribution_and_seed(ops):
    probabilities = torch.tensor([0.05, 0.15, 0.3, 0.5], device=DEV)
    logits = (probabilities.log() * 0.7).expand(20000, -1).contiguous()
    kwargs = dict(temperature=0.7, seed=17, step=0, return_logprobs=False)
    tokens, logprobs = ops.sample_logits(logits, **kwargs)
    assert logprobs is None
    torch.testing.assert_close(tokens.bincount(minlength=4) / tokens.numel(), probabilities, atol=0.012, rtol=0)
    assert torch.equal(tokens, ops.sample_logits(logits, **kwargs)[0])
    for seed, step in ((18, 0), (17, 64), (17, 4095)):
        assert not torch.equal(tokens, ops.sample_logits(logits, **{**kwargs, "seed": seed, "step": step})[0])
    # per-row streams: a row's draw depends only on its own (seed, step, temperature)
    sampler = ops.RowSampler(logits[:64])
    seeds = torch.arange(64, device=DEV)
    steps = torch.arange(64, device=DEV) * 3
    temps = torch.full((64,), 0.7, device=DEV)
    temps[5] = 0.0
    first = sampler.sample(logits[:64], seeds, steps, temps)[0].clone()
    perm = torch.randperm(64, device=DEV)
    second = sampler.sample(logits[:64], seeds[perm], steps[perm], temps[perm])[0]
    assert torch.equal(second, first[perm]) and first[5].item() == 3


@pytest.mark.parametrize("top_k,top_p", [(50, 0.95), (0, 0.9), (5, 1.0), (1, 0.5), (0, 0.3)])
@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float32))
@torch.inference_mode()
def test_filtered_sampling_keeps_exactly_the_oracle_support(ops, top_k, top_p, dtype):
    torch.manual_seed(8)
    rows, vocab, temperature = 48, 5000, 0.8
    logits = (torch.randn(rows, vocab) * 2.5).to(dtype)
    scaled = logits.float() / temperature
    filtered = O.top_k_top_p_filter(scaled, top_k, top_p)
    allowed = torch.isfinite(filtered)
    # equal logits may be ordered either way by the oracle's sort, so support is compared by value:
    # a draw must be at least as large as the smallest logit the oracle kept
    floor = torch.where(allowed, scaled, torch.full_like(scaled, math.inf)).amin(1)
    draws = []
    for step in range(40):
        tok, lp, kept = ops.sample_filtered(logits.to(DEV), temperature=temperature, top_k=top_k, top_p=top_p, seed=5,
                                            step=step, return_kept=True)
        draws.append(tok.cpu())
        assert (scaled.gather(1, tok.cpu()[:, None])[:, 0] >= floor).all(), "a draw fell outside the oracle's support"
    assert len({tuple(d.tolist()) for d in draws}) > 1 or top_k == 1
    # survivors: the count the filter gives in float64 (the fp32 cumulative sum of the reference's filter is itself only
    # good to about 1e-6 of the row's mass; the kernel sums 2^-40 fixed-point masses).  A row may differ only where
    # one rank's cumulative mass lies within 2e-6 of top_p, and then by that one rank.
    exact = O.top_k_top_p_filter(logits.double() / temperature, top_k, top_p)
    count = torch.isfinite(exact).sum(1)
    if top_p < 1.0:
        ranked = torch.sort(O.top_k_top_p_filter(logits.double() / temperature, top_k, 1.0), descending=True, dim=-1).values
        margin = (torch.softmax(ranked, -1).cumsum(-1) - top_p).abs().amin(1)
    else:
        margin = torch.ones(rows, dtype=torch.float64)
    diff = (kept.cpu() - count).abs()
    assert (diff[margin > 2e-6] == 0).all() and (diff <= 1).all(), (diff, margin)
    expected = logits.double().log_softmax(-1).gather(1, tok.cpu()[:, None])[:, 0].float()
    torch.testing.assert_close(lp.cpu(), expected, atol=5e-6, rtol=2e-6)
    # the draw's log-probability under the tempered, filtered distribution it came from (third value of
    # lfm25_engine.py:1574-1609), on the rows whose support is the float64 filter's
    tempered = torch.empty(rows, device=DEV, dtype=torch.float32)
    tok2, lp2 = ops.sample_filtered(logits.to(DEV), temperature=temperature, top_k=top_k, top_p=top_p, seed=5, step=39,
                                    sampling_logprobs=tempered)
    assert torch.equal(tok2, tok) and torch.equal(lp2, lp)
    # equal logits are interchangeable (which of two tied values the oracle's sort ranks first is arbitrary): the pick's
    # own tempered logit over the oracle's normaliser
    want = ((logits.double() / temperature).gather(1, tok.cpu()[:, None])[:, 0] - torch.logsumexp(exact, -1)).float()
    same = diff == 0
    torch.testing.assert_close(tempered.cpu()[same], want[same], atol=1e-5, rtol=0)
    assert (tempered.cpu() <= 1e-6).all()
    again = ops.sample_filtered(logits.to(DEV), temperature=temperature, top_k=top_k, top_p=top_p, seed=5, step=39)[0]
    assert torch.equal(again.cpu(), draws[-1])
    if top_k == 1:
        assert torch.equal(draws[0], logits.float().argmax(-1))


@pytest.mark.parametrize("top_k,top_p", [(50, 0.95), (0, 0.9), (7, 1.0), (0, 0.3)])
@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float32))
@torch.inference_mode()
def test_filtered_sampling_in_registers_and_streamed_make_the_same_draws(ops, top_k, top_p, dtype):
    """Rows of up to 65536 logits are sampled from registers, longer ones by re-reading the row in every pass.  A row
    padded with -inf columns beyond 65536 has the same survivors and the same per-column random numbers as the
    unpadded row, so both forms must return the same tokens, survivor counts and log-probabilities; bf16 rows with
    many equal values put ties on the top-k and nucleus boundaries."""
    torch.manual_seed(21)
    rows, vocab, wide = 24, 6000, 70000
    logits = (torch.randn(rows, vocab) * 2.0).to(dtype)
    logits[:8] = (torch.randn(8, vocab) * 0.5).to(torch.bfloat16).to(dtype)       # coarse values: many ties
    padded = torch.full((rows, wide), -math.inf, dtype=dtype)
    padded[:, :vocab] = logits
    for step in range(6):
        a = ops.sample_filtered(logits.to(DEV), temperature=0.7, top_k=top_k, top_p=top_p, seed=11, step=step, return_kept=True)
        b = ops.sample_filtered(padded.to(DEV), temperature=0.7, top_k=top_k, top_p=top_p, seed=11, step=step, return_kept=True)
        assert torch.equal(a[0], b[0]) and torch.equal(a[2], b[2])
        torch.testing.assert_close(a[1], b[1], atol=2e-6, rtol=1e-6)


@torch.inference_mode()
def test_filtered_sampling_distribution_follows_renormalised_survivors(ops):
    probs = torch.tensor([0.4, 0.3, 0.15, 0.1, 0.05])
    logits = probs.log().expand(30000, -1).contiguous().to(DEV)
    tok, _ = ops.sample_filtered(logits, temperature=1.0, top_k=0, top_p=0.75, seed=3, step=1)
    freq = tok.bincount(minlength=5).float().cpu() / tok.numel()
    torch.testing.assert_close(freq, torch.tensor([0.4, 0.3, 0, 0, 0]) / 0.7, atol=0.012, rtol=0)
    tok, _ = ops.sample_filtered(logits, temperature=1.0, top_k=3, top_p=1.0, seed=3, step=2)
    freq = tok.bincount(minlength=5).float().cpu() / tok.numel()
    torch.testing.assert_close(freq, torch.tensor([0.4, 0.3, 0.15, 0, 0]) / 0.85, atol=0.012, rtol=0)


@torch.inference_mode()
def test_record_sample_and_slot_bookkeeping_follow_the_integer_oracle(ops):
    V, cap, B, eos = 16, 6, 5, 7
    pieces = ['<', '/', 'summary', '>', 'x'] + [''] * 11
    table = torch.cat((torch.zeros(V, dtype=torch.int32), O.build_stop_table(pieces, ('</summary>',)).reshape(-1)))
    dev = lambda t: t.to(DEV)
    tokens = dev(torch.zeros(B, cap, dtype=torch.long)); logprobs = dev(torch.zeros(B, cap))
    lengths = dev(torch.tensor([0, 5, 2, 0, 3], dtype=torch.int32)); limits = dev(torch.full((B,), 6, dtype=torch.int32))
    reasons = dev(torch.zeros(B, dtype=torch.int8)); alive = dev(torch.tensor([True, True, True, False, True]))
    pending = dev(torch.zeros(B, dtype=torch.bool)); inp = dev(torch.full((B,), -1, dtype=torch.long))
    states = dev(torch.tensor([0, 0, 9, 0, 0])); offsets = dev(torch.tensor([0, 0, V, 0, 0]))
    ignore = dev(torch.tensor([False, False, False, False, True])); rng = dev(torch.tensor([0, 10, 20, 30, 40]))
    sampled = dev(torch.tensor([7, 4, 3, 9, 7])); logp = dev(torch.tensor([-1., -2., -3., -4., -5.]))
    # row 2 sits in the automaton state reached after '</summary' so that '>' completes the stop
    st = 0
    for t in [0, 1, 2]:
        st = int(table[V + st * V + t]) & 65535
    states[2] = st
    ops.record_sample(sampled, logp, tokens, logprobs, lengths, limits, reasons, alive, pending, inp, states, offsets,
                      dev(table), ignore, rng, eos, V, cap)
    assert reasons.cpu().tolist() == [1, 3, 2, 0, 0]
    assert alive.cpu().tolist() == [False, False, False, False, True] == pending.cpu().tolist()
    assert lengths.cpu().tolist() == [1, 6, 3, 0, 4] and rng.cpu().tolist() == [1, 11, 21, 30, 41]
    assert inp.cpu().tolist() == [7, 4, 3, -1, 7]
    assert tokens[1, 5].item() == 4 and logprobs[2, 2].item() == -3.0 and tokens[3].sum().item() == 0
    # gather / scatter / advance over a compact batch
    slots = dev(torch.tensor([3, -1, 0], dtype=torch.int32))
    seq_lens = dev(torch.tensor([11, 22, 33, 44], dtype=torch.int32))
    input_tokens = dev(torch.tensor([5, 6, 7, 8])); act = dev(torch.tensor([True, True, False, True]))
    t = dev(torch.zeros(3, dtype=torch.long)); p = dev(torch.zeros(3, dtype=torch.int32)); m = dev(torch.zeros(3, dtype=torch.bool))
    ops.gather_inputs(t, p, m, input_tokens, seq_lens, act, slots)
    assert t.cpu().tolist() == [8, 0, 5] and p.cpu().tolist() == [44, 0, 11] and m.cpu().tolist() == [True, False, True]
    logits = dev(torch.randn(3, 100).bfloat16()); saved = dev(torch.zeros(4, 100).bfloat16())
    ops.scatter_logits(saved, logits, slots, m)
    assert torch.equal(saved[3], logits[0]) and torch.equal(saved[0], logits[2]) and saved[1:3].count_nonzero() == 0
    ops.advance_positions(seq_lens, p, slots, m)
    assert seq_lens.cpu().tolist() == [12, 22, 33, 45]
    masked = dev(torch.tensor([True, False, True, True]))
    ops.advance_positions(seq_lens, seq_lens.clone(), None, masked)
    assert seq_lens.cpu().tolist() == [13, 22, 34, 46]


@torch.inference_mode()
def test_behavior_head_reuses_the_sampler_normaliser(ops):
    torch.manual_seed(2)
    logits = torch.randn(4, 3000).bfloat16().to(DEV)
    tok, lp = ops.sample_logits(logits, temperature=1.0, seed=1, step=0, return_logprobs=True)
    ids, probs = ops.behavior_topk(logits, tok, lp, 8)
    want = logits.float().log_softmax(-1).topk(8).values
    torch.testing.assert_close(probs, want, atol=5e-6, rtol=1e-5)
    with pytest.raises(ValueError):
        ops.behavior_topk(logits, tok, lp, 129)


# ------------------------------------------------------------------------------------------------ fused decode launches
@pytest.mark.parametrize("dim,qh,kh", [(64, 32, 8), (32, 4, 4), (128, 4, 2), (256, 2, 1)])
@pytest.mark.parametrize("fp8", [True, False])
@torch.inference_mode()
def test_prepare_qkv_with_cache_append_equals_the_two_separate_launches(ops, dim, qh, kh, fp8):
    """One launch (QK norm + RoPE + KV append) against prepare_qkv followed by store_kv / append_bf16_kv, which the
    tests above pin to the oracle: q, cache bytes and scales must be identical, untouched cache rows stay untouched."""
    torch.manual_seed(5)
    rows, slots, cap = 7, 9, 40
    x = torch.randn(rows, (qh + 2 * kh) * dim, dtype=torch.bfloat16, device=DEV)
    qw, kw = (torch.randn(dim, dtype=torch.bfloat16, device=DEV) for _ in range(2))
    cos, sin = (t.to(DEV) for t in O.rope_tables(dim, 1e6, 64))
    positions = torch.tensor([0, 5, 39, 17, 3, 8, 21], dtype=torch.int32, device=DEV)
    slot_ids = torch.tensor([4, 0, 8, -1, 2, 6, 1], dtype=torch.int32, device=DEV)
    active = torch.tensor([1, 1, 1, 0, 0, 1, 1], dtype=torch.bool, device=DEV)

    def caches():
        torch.manual_seed(6)
        if fp8:
            kc = torch.randint(0, 255, (slots, kh, cap, dim), dtype=torch.uint8, device=DEV).view(torch.float8_e4m3fn)
            vc = torch.randint(0, 255, (slots, kh, cap, dim), dtype=torch.uint8, device=DEV).view(torch.float8_e4m3fn)
            ks, vs = (torch.rand(slots, kh, cap, device=DEV) for _ in range(2))
            return kc.transpose(1, 2), vc.transpose(1, 2), ks.transpose(1, 2), vs.transpose(1, 2)
        kc, vc = (torch.randn(slots, cap, kh, dim, dtype=torch.bfloat16, device=DEV) for _ in range(2))
        return kc, vc, None, None

    kc0, vc0, ks0, vs0 = caches()
    q0, k0, v0 = ops.prepare_qkv(x, qw, kw, cos, sin, positions, qh, kh, dim, 1e-5)
    if fp8:
        ops.store_kv(k0, v0, kc0, vc0, ks0, vs0, positions=positions, active=active, slot_ids=slot_ids)
    else:
        ops.append_bf16_kv(k0, v0, kc0, vc0, positions, slot_ids, active)
    kc1, vc1, ks1, vs1 = caches()
    q1 = ops.prepare_qkv_store(x, qw, kw, cos, sin, positions, qh, kh, dim, 1e-5, kc1, vc1, ks1, vs1, active=active,
                               slot_ids=slot_ids)
    torch.cuda.synchronize()
    assert torch.equal(q0, q1)
    as_bytes = (lambda t: t.contiguous().view(torch.uint8)) if fp8 else (lambda t: t.contiguous().view(torch.int16))
    assert torch.equal(as_bytes(kc0), as_bytes(kc1)) and torch.equal(as_bytes(vc0), as_bytes(vc1))
    if fp8:
        assert torch.equal(ks0, ks1) and torch.equal(vs0, vs1)


@pytest.mark.parametrize("rows", [5, 64, 256, 300])      # a few rows of one ring tile, a full tile, the decode batch, a ragged last tile
@pytest.mark.parametrize("fp8", [True, False])
@torch.inference_mode()
def test_qkv_projection_with_prepare_and_append_as_its_epilogue_equals_the_two_launches(ops, rows, fp8):
    """The W8A8 QKV projection whose epilogue does QK norm + RoPE + KV append, against linear_quantized followed by
    prepare_qkv_store (pinned above): q, cache bytes and scales identical, untouched cache rows untouched."""
    torch.manual_seed(7)
    qh, kh, dim, hidden, slots, cap = 32, 8, 64, 2048, 320, 24
    act = torch.randn(rows, hidden, dtype=torch.bfloat16, device=DEV)
    packed = ops.PackedFP8Weight.from_weight(torch.randn((qh + 2 * kh) * dim, hidden, dtype=torch.bfloat16, device=DEV) * 0.03)
    xq, xs = ops.quantize_rows(act)
    qw, kw = (torch.randn(dim, dtype=torch.bfloat16, device=DEV) for _ in range(2))
    cos, sin = (t.to(DEV) for t in O.rope_tables(dim, 1e6, 64))
    positions = torch.randint(0, cap, (rows,), dtype=torch.int32, device=DEV)
    slot_ids = torch.randperm(slots, device=DEV)[:rows].to(torch.int32)
    slot_ids[1] = -1
    active = torch.rand(rows, device=DEV) > 0.2
    assert ops.qkv_project_store_supported(packed, dim, torch.bfloat16, torch.empty(slots, cap, kh, dim, device=DEV))

    def caches():
        torch.manual_seed(8)
        if fp8:
            kc = torch.randint(0, 255, (slots, kh, cap, dim), dtype=torch.uint8, device=DEV).view(torch.float8_e4m3fn)
            vc = torch.randint(0, 255, (slots, kh, cap, dim), dtype=torch.uint8, device=DEV).view(torch.float8_e4m3fn)
            ks, vs = (torch.rand(slots, kh, cap, device=DEV) for _ in range(2))
            return kc.transpose(1, 2), vc.transpose(1, 2), ks.transpose(1, 2), vs.transpose(1, 2)
        kc, vc = (torch.randn(slots, kh, cap, dim, dtype=torch.bfloat16, device=DEV).transpose(1, 2) for _ in range(2))
        return kc, vc, None, None

    kc0, vc0, ks0, vs0 = caches()
    qkv = packed.linear_quantized(xq, xs)
    q0 = ops.prepare_qkv_store(qkv, qw, kw, cos, sin, positions, qh, kh, dim, 1e-5, kc0, vc0, ks0, vs0, active=active,
                               slot_ids=slot_ids)
    kc1, vc1, ks1, vs1 = caches()
    q1 = ops.qkv_project_store(xq, xs, packed, qw, kw, cos, sin, positions, qh, kh, dim, 1e-5, kc1, vc1, ks1, vs1,
                               active=active, slot_ids=slot_ids)
    torch.cuda.synchronize()
    assert torch.equal(q0, q1)
    as_bytes = (lambda t: t.contiguous().view(torch.uint8)) if fp8 else (lambda t: t.contiguous().view(torch.int16))
    assert torch.equal(as_bytes(kc0), as_bytes(kc1)) and torch.equal(as_bytes(vc0), as_bytes(vc1))
    if fp8:
        assert torch.equal(ks0, ks1) and torch.equal(vs0, vs1)


@pytest.mark.parametrize("width", (256, 2048, 4096))
@torch.inference_mode()
def test_conv_update_with_quantised_output_equals_the_two_separate_launches(ops, width):
    torch.manual_seed(11)
    rows, slots = 6, 8
    bcx = torch.randn(rows, 3 * width, dtype=torch.bfloat16, device=DEV)
    weight = torch.randn(width, 3, dtype=torch.bfloat16, device=DEV)
    state = torch.randn(slots, width, 3, dtype=torch.bfloat16, device=DEV)
    slot_ids = torch.tensor([3, 0, 7, 5, 1, 2], dtype=torch.int32, device=DEV)
    active = torch.tensor([1, 0, 1, 1, 0, 1], dtype=torch.bool, device=DEV)
    s0, s1 = state.clone(), state.clone()
    expected = ops.quantize_rows(ops.conv_update(bcx, weight, s0, active, slot_ids))
    q, scales = ops.conv_update_fp8(bcx, weight, s1, active, slot_ids)
    torch.cuda.synchronize()
    assert torch.equal(q.view(torch.uint8), expected[0].view(torch.uint8))
    assert torch.equal(scales, expected[1])
    assert torch.equal(s0.view(torch.int16), s1.view(torch.int16))


@pytest.mark.parametrize("dim,qh,kh", [(64, 32, 8), (128, 4, 2), (32, 4, 4)])
@pytest.mark.parametrize("fp8", [True, False])
@torch.inference_mode()
def test_decode_attention_with_quantised_rows_equals_quantising_its_output(ops, dim, qh, kh, fp8):
    torch.manual_seed(23)
    rows, cap = 5, 1300
    q = torch.randn(rows, 1, qh, dim, dtype=torch.bfloat16, device=DEV)
    if fp8:
        kc = torch.randint(0, 120, (rows, kh, cap, dim), dtype=torch.uint8, device=DEV).view(torch.float8_e4m3fn).transpose(1, 2)
        vc = torch.randint(0, 120, (rows, kh, cap, dim), dtype=torch.uint8, device=DEV).view(torch.float8_e4m3fn).transpose(1, 2)
        ks, vs = (torch.rand(rows, kh, cap, device=DEV).transpose(1, 2) * 0.05 for _ in range(2))
    else:
        kc, vc = (torch.randn(rows, cap, kh, dim, dtype=torch.bfloat16, device=DEV) for _ in range(2))
        ks = vs = None
    positions = torch.tensor([0, 1299, 511, 1024, 77], dtype=torch.int32, device=DEV)
    active = torch.tensor([1, 1, 0, 1, 1], dtype=torch.bool, device=DEV)
    plain = ops.attend(q, kc, vc, ks, vs, positions, active=active)
    expected = ops.quantize_rows(plain.view(rows, -1))
    got = ops.attend(q, kc, vc, ks, vs, positions, active=active, quantized=True)
    torch.cuda.synchronize()
    assert torch.equal(got[0].view(torch.uint8), expected[0].view(torch.uint8))
    assert torch.equal(got[1], expected[1])


@torch.inference_mode()
def test_split_k_partials_reduce_inside_the_following_norm(ops):
    """A down projection left as split-K partial sums and reduced by the norm that follows it gives the bytes the
    materialised projection followed by rms_norm_fp8 gives (lfm25_cuda.py:166-184 order of roundings)."""
    torch.manual_seed(29)
    rows, width, outputs = 256, 5632, 2048
    act = torch.randn(rows, width, dtype=torch.bfloat16, device=DEV)
    weight = ops.PackedFP8Weight.from_weight(torch.randn(outputs, width, dtype=torch.bfloat16, device=DEV) * 0.02)
    norm_w = torch.randn(outputs, dtype=torch.bfloat16, device=DEV)
    residual = torch.randn(rows, outputs, dtype=torch.bfloat16, device=DEV)
    xq, xs = ops.quantize_rows(act)
    deferred = weight.linear_quantized(xq, xs, config=(2, 4), defer_reduce=True)
    assert isinstance(deferred, ops.SplitProduct) and deferred.partials.size(0) == 4
    whole = weight.linear_quantized(xq, xs, config=(2, 4))
    assert torch.equal(deferred.materialize().view(torch.int16), whole.view(torch.int16))
    expected = ops.rms_norm_fp8(whole, norm_w, 1e-5, residual)
    got = ops.rms_norm_fp8(deferred, norm_w, 1e-5, residual)
    torch.cuda.synchronize()
    assert torch.equal(got[0].view(torch.uint8), expected[0].view(torch.uint8))
    assert torch.equal(got[1], expected[1])
    assert torch.equal(got[2].view(torch.int16), expected[2].view(torch.int16))
    # the default plan for a deferred reduce at this shape: two halves of K; the same bytes after the norm as the split
    # product materialised by the GEMM's own reduce launch
    halves = weight.linear_quantized(xq, xs, defer_reduce=True)
    assert isinstance(halves, ops.SplitProduct) and halves.partials.size(0) == 2
    whole = weight.linear_quantized(xq, xs, config=(16, 2))
    assert torch.equal(halves.materialize().view(torch.int16), whole.view(torch.int16))
    expected, got = ops.rms_norm_fp8(whole, norm_w, 1e-5, residual), ops.rms_norm_fp8(halves, norm_w, 1e-5, residual)
    assert all(torch.equal(a.view(torch.uint8), b.view(torch.uint8)) for a, b in zip(got, expected))
    # nothing to defer when the plan does not split (a K loop of 16 steps)
    narrow = ops.PackedFP8Weight.from_weight(torch.randn(outputs, 2048, dtype=torch.bfloat16, device=DEV) * 0.02)
    aq, a_s = ops.quantize_rows(act[:, :2048].contiguous())
    assert isinstance(narrow.linear_quantized(aq, a_s, defer_reduce=True), torch.Tensor)


@torch.inference_mode()
def test_bf16_split_k_partials_reduce_inside_the_following_norm(ops):
    """The bf16 down projection at decode size is split along K by default; left as partial sums and reduced by the
    norm that follows, it gives the bytes of the materialised projection followed by rms_norm (and by rms_norm_fp8)."""
    torch.manual_seed(31)
    rows, width, outputs = 256, 5632, 2048
    act = torch.randn(rows, width, dtype=torch.bfloat16, device=DEV)
    weight = torch.randn(outputs, width, dtype=torch.bfloat16, device=DEV) * 0.02
    norm_w = torch.randn(outputs, dtype=torch.bfloat16, device=DEV)
    residual = torch.randn(rows, outputs, dtype=torch.bfloat16, device=DEV)
    deferred = ops.linear(act, weight, defer_reduce=True)
    assert isinstance(deferred, ops.SplitProduct) and deferred.partials.size(0) == 4 and deferred.a_scales is None
    whole = ops.linear(act, weight)
    assert torch.equal(deferred.materialize().view(torch.int16), whole.view(torch.int16))
    torch.testing.assert_close(whole.float(), act.float() @ weight.float().T, atol=0.06, rtol=0.02)
    expected, got = ops.rms_norm(whole, norm_w, 1e-5, residual), ops.rms_norm(deferred, norm_w, 1e-5, residual)
    assert torch.equal(got[0].view(torch.int16), expected[0].view(torch.int16))
    assert torch.equal(got[1].view(torch.int16), expected[1].view(torch.int16))
    expected, got = ops.rms_norm_fp8(whole, norm_w, 1e-5, residual), ops.rms_norm_fp8(deferred, norm_w, 1e-5, residual)
    assert torch.equal(got[0].view(torch.uint8), expected[0].view(torch.uint8)) and torch.equal(got[1], expected[1])
    # the out projection's shape (32 K steps): two halves of K when the reduce is left to the norm, the same bytes
    # after it as the split product summed by the GEMM's own reduce launch
    act2, weight2 = act[:, :2048].contiguous(), weight[:, :2048].contiguous()
    halves = ops.linear(act2, weight2, defer_reduce=True)
    assert isinstance(halves, ops.SplitProduct) and halves.partials.size(0) == 2
    whole = ops.linear(act2, weight2, tile=16, split_k=2)
    assert torch.equal(halves.materialize().view(torch.int16), whole.view(torch.int16))
    expected, got = ops.rms_norm(whole, norm_w, 1e-5, residual), ops.rms_norm(halves, norm_w, 1e-5, residual)
    assert torch.equal(got[0].view(torch.int16), expected[0].view(torch.int16))
    assert torch.equal(got[1].view(torch.int16), expected[1].view(torch.int16))
    # nothing to defer when the plan does not split (16 K steps)
    assert isinstance(ops.linear(act[:, :1024].contiguous(), weight[:, :1024].contiguous(), defer_reduce=True), torch.Tensor)


# ------------------------------------------------------------------------------------------------ rounding points
def _rounding_cases():
    import json, os
    return json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "rounding_cases.json")))


@torch.inference_mode()
def test_kernels_round_where_the_reference_kernels_round(ops):
    """The fixtures of tests/golden/rounding_cases.json: inputs on which one rounding point of
    lfm25_cuda_kernels.py:32-140 decides the bf16 result (the sum, the normalised value, the SwiGLU activation, b*x,
    each tap product and their sum, the QK-norm stages, the table entries and both RoPE products).  The HIP kernels
    must give `expected`, never `without`."""
    cases = _rounding_cases()
    bf = lambda values: torch.tensor(values, dtype=torch.float32).to(torch.bfloat16).to(DEV)
    for name in ("rms_add", "rms_norm"):
        case = cases[name]
        out, summed = ops.rms_norm(bf([case["x"]]), bf(case["weight"]), case["eps"], bf([case["residual"]]))
        assert out.float().cpu()[0].tolist() == case["expected"], name
        assert summed.float().cpu()[0].tolist() == case["summed"], name
        q, scales, _ = ops.rms_norm_fp8(bf([case["x"]]), bf(case["weight"]), case["eps"], bf([case["residual"]]))
        oq, oscale = O.k_quantize_rows(torch.tensor([case["expected"]]).bfloat16())
        assert torch.equal(scales.cpu(), oscale) and torch.equal(q.cpu().view(torch.uint8), oq.view(torch.uint8)), name
    case = cases["swiglu_act"]
    row = bf([[case["gate"]] * 8 + [case["up"]] * 8])
    assert ops.swiglu(row).float().cpu()[0].tolist() == [case["expected"]] * 8
    for name in ("conv_bx", "conv_p0", "conv_p1", "conv_p2", "conv_sum"):
        case = cases[name]
        channels = 8
        state = bf([[case["state"]] * channels])
        bcx = bf([[case["b"]] * channels + [case["c"]] * channels + [case["x"]] * channels])
        out = ops.conv_update(bcx, bf([case["weight"]] * channels), state)
        assert out.float().cpu()[0].tolist() == [case["expected"]] * channels, name
        assert state.float().cpu()[0].tolist() == [case["new_state"]] * channels, name
    for name in ("qk_norm", "qk_weight", "qk_table", "qk_left", "qk_right"):
        case = cases[name]
        head, weight = bf(case["x"]), bf(case["weight"])
        cos = torch.tensor([case["cos"]], dtype=torch.float32, device=DEV)
        sin = torch.tensor([case["sin"]], dtype=torch.float32, device=DEV)
        x = torch.cat((head, head, torch.zeros(64, dtype=torch.bfloat16, device=DEV)))[None].contiguous()
        q, k, v = ops.prepare_qkv(x, weight, weight, cos, sin, torch.zeros(1, dtype=torch.int32, device=DEV), 1, 1, 64, case["eps"])
        assert q.float().cpu().flatten().tolist() == case["expected"], name
        assert k.float().cpu().flatten().tolist() == case["expected"], name


# ------------------------------------------------------------------------------------------------ fused launches
@pytest.mark.parametrize("fp8", (False, True))
@torch.inference_mode()
def test_embedding_fused_into_the_first_norm_equals_the_two_launches(ops, fp8):
    torch.manual_seed(21)
    vocab, width = 1000, 2048
    table = torch.randn(vocab, width, device=DEV).bfloat16()
    weight = torch.randn(width, device=DEV).bfloat16()
    tokens = torch.randint(0, vocab, (37,), device=DEV)
    tokens[3], tokens[4] = -5, vocab + 9          # out-of-range ids are clamped into the table, as `embedding` does
    hidden = ops.embedding(tokens, table)
    fused, fused_hidden = ops.embedding_rms_norm(tokens, table, weight, 1e-5, fp8=fp8)
    assert torch.equal(fused_hidden, hidden)
    if fp8:
        q, scales, _ = ops.rms_norm_fp8(hidden, weight, 1e-5)
        assert torch.equal(fused[0].view(torch.uint8), q.view(torch.uint8)) and torch.equal(fused[1], scales)
    else:
        assert torch.equal(fused, ops.rms_norm(hidden, weight, 1e-5)[0])
    narrow = torch.randn(50, 36, device=DEV).bfloat16()     # a width without 16-byte rows takes the scalar form
    out, kept = ops.embedding_rms_norm(tokens[:5] % 50, narrow, weight[:36].contiguous(), 1e-5, fp8=False)
    again = ops.embedding(tokens[:5] % 50, narrow)
    assert torch.equal(kept, again) and torch.equal(out, ops.rms_norm(again, weight[:36].contiguous(), 1e-5)[0])


@torch.inference_mode()
def test_decode_begin_equals_gather_schedule_and_advance(ops):
    """The step's first launch against the three it replaces: the same positions, gathered inputs, work list and
    advanced lengths, for rows that are the cache's slots (with and without a mask) and for a compact batch."""
    torch.manual_seed(23)
    rows, capacity = 300, 8192
    lengths = torch.randint(0, 4000, (rows,), dtype=torch.int32, device=DEV)
    for active in (None, torch.rand(rows, device=DEV) < 0.7):
        want_lengths = lengths.clone()
        want_schedule = ops.decode_schedule(want_lengths, active, None, capacity=capacity)
        ops.advance_positions(want_lengths, want_lengths.clone(), None, active)
        got_lengths = lengths.clone()
        positions, schedule = ops.decode_begin(got_lengths, active, capacity=capacity)
        assert torch.equal(positions, lengths) and torch.equal(got_lengths, want_lengths)
        used = 4 + 4 * rows + 4 * int(schedule[0])     # header (pair count, chunk size, two unused words), rows, pairs
        assert torch.equal(schedule[:2], want_schedule[:2]) and torch.equal(schedule[4:used], want_schedule[4:used])
    compact = 64
    slots = torch.full((compact,), -1, dtype=torch.int32, device=DEV)
    slots[:40] = torch.randperm(rows, device=DEV)[:40].to(torch.int32)
    slot_active = torch.rand(rows, device=DEV) < 0.8
    inputs = torch.randint(0, 65536, (rows,), device=DEV)
    t0, p0, m0 = (torch.zeros(compact, device=DEV, dtype=d) for d in (torch.long, torch.int32, torch.bool))
    want_lengths = lengths.clone()
    ops.gather_inputs(t0, p0, m0, inputs, want_lengths, slot_active, slots)
    want_schedule = ops.decode_schedule(p0, m0, slots, capacity=capacity)
    ops.advance_positions(want_lengths, p0, slots, m0)
    t1, p1, m1 = (torch.full((compact,), 7, device=DEV).to(d) for d in (torch.long, torch.int32, torch.bool))
    got_lengths = lengths.clone()
    positions, schedule = ops.decode_begin(got_lengths, capacity=capacity, gather=(inputs, slot_active, slots, t1, p1, m1))
    assert positions is p1 and torch.equal(t1, t0) and torch.equal(p1, p0) and torch.equal(m1, m0)
    assert torch.equal(got_lengths, want_lengths) and not torch.equal(got_lengths, lengths)
    used = 4 + 4 * compact + 4 * int(schedule[0])
    assert torch.equal(schedule[:2], want_schedule[:2]) and torch.equal(schedule[4:used], want_schedule[4:used])


@torch.inference_mode()
def test_sampler_that_records_its_draw_equals_sample_then_record(ops):
    torch.manual_seed(25)
    rows, vocab, cap, eos = 9, 10000, 5, 7
    logits = (torch.randn(rows, vocab, device=DEV) * 2).bfloat16()
    logits[2, eos] = 50.0                                   # row 2 draws the end-of-sequence token
    stop_table = torch.zeros(2 * vocab, dtype=torch.int32, device=DEV)
    stop_table[vocab + logits[4].float().argmax()] = 65536  # row 4 (greedy, second automaton) hits a stop token

    class Table:
        pass

    def fresh():
        t = Table()
        t.seeds = torch.arange(100, 100 + rows, device=DEV)
        t.rng_positions = torch.arange(rows, device=DEV) * 3
        t.temperatures = torch.tensor([1.0, 0.0, 1.0, 0.7, 0.0, 1.0, 1.3, 0.0, 1.0], device=DEV)
        t.tokens = torch.zeros((rows, cap), dtype=torch.long, device=DEV)
        t.logprobs = torch.zeros((rows, cap), device=DEV)
        t.lengths = torch.tensor([0, 1, 2, 3, 0, 4, 1, 0, 2], dtype=torch.int32, device=DEV)
        t.limits = torch.full((rows,), cap, dtype=torch.int32, device=DEV)
        t.reasons = torch.zeros(rows, dtype=torch.int8, device=DEV)
        t.alive = torch.tensor([1, 1, 1, 1, 1, 1, 0, 1, 1], dtype=torch.bool, device=DEV)
        t.pending = torch.zeros(rows, dtype=torch.bool, device=DEV)
        t.stop_states = torch.zeros(rows, dtype=torch.long, device=DEV)
        t.stop_offsets = torch.tensor([0, 0, 0, 0, vocab, 0, 0, 0, 0], device=DEV)
        t.ignore_eos = torch.zeros(rows, dtype=torch.bool, device=DEV)
        t.input = torch.full((rows,), -1, dtype=torch.long, device=DEV)
        return t

    two, one = fresh(), fresh()
    sampler_a, sampler_b = ops.RowSampler(logits), ops.RowSampler(logits)
    sampled, logp = sampler_a.sample(logits, two.seeds, two.rng_positions, two.temperatures)
    ops.record_sample(sampled, logp, two.tokens, two.logprobs, two.lengths, two.limits, two.reasons, two.alive, two.pending,
                      two.input, two.stop_states, two.stop_offsets, stop_table, two.ignore_eos, two.rng_positions, eos, vocab, cap)
    got_sampled, got_logp = ops.sample_and_record(sampler_b, logits, one, one.input, stop_table, eos, cap)
    assert torch.equal(got_sampled, sampled) and torch.equal(got_logp.view(torch.int32), logp.view(torch.int32))
    for name in ("tokens", "logprobs", "lengths", "reasons", "alive", "pending", "stop_states", "rng_positions", "input"):
        assert torch.equal(getattr(one, name), getattr(two, name)), name
    assert one.reasons.cpu().tolist()[2] == 1 and one.reasons.cpu().tolist()[4] == 2 and one.reasons.cpu().tolist()[5] == 3
    assert one.input.cpu().tolist()[6] == -1     # a row that is not alive records nothing


@pytest.mark.parametrize("fp8", (True, False))
@pytest.mark.parametrize("m,k,inner", [(4096, 256, 512), (2689, 2048, 5632), (2000, 2048, 5632), (1030, 512, 5632), (1000, 384, 5632), (300, 2048, 5632), (256, 2048, 5632), (200, 2048, 5632), (64, 2048, 5632),
                                       (1, 2048, 1024), (13, 2048, 1024), (40, 1024, 2048), (30, 2048, 3072), (33, 2048, 3072), (49, 2048, 1024)])
@torch.inference_mode()
def test_gate_up_projection_with_swiglu_epilogue_equals_the_two_launches(ops, fp8, m, k, inner):
    """The fused gate+up projection (SwiGLU in the product's epilogue, [M, I] written) against the projection followed
    by the SwiGLU launch, bit for bit: both quantised outputs for W8A8, the bf16 rows otherwise.  64 rows of the model's
    width have no fused form and must take the two launches by themselves; ragged row counts end inside a tile; 256 and
    200 rows run the decode batch's 128 x 96 tile (three MFMA tiles per wave: the odd one is finished by half of the
    lanes); the W8A8 products of up to 48 rows on at most 4096 columns (32 rows up to 8192) run the few-row kernel,
    whose SwiGLU form pairs the gate and up columns out of LDS; 2000 and 1030 rows of the model's 11264 columns run the
    256 x 192 tile (three MFMA tiles per wave again, and a last column tile that ends inside the output)."""
    torch.manual_seed(m + inner)
    weight = (torch.randn(2 * inner, k, device=DEV) * 0.05).bfloat16()
    x = torch.randn(m, k, device=DEV).bfloat16()
    fused_exists = bool(ops.query("lfm2_gemm_swiglu_fits", m, 2 * inner, k, 1 if fp8 else 2))
    few_rows = fp8 and m <= (48 if 2 * inner <= 4096 else 32 if 2 * inner <= 8192 else 0)
    assert fused_exists == (m > 64 or few_rows)
    if fp8:
        packed = ops.PackedFP8Weight.from_weight(weight)
        xq, xs = ops.quantize_rows(x)
        want_q, want_s = ops.swiglu_fp8(packed.linear_quantized(xq, xs))
        got_q, got_s = packed.linear_swiglu_quantized(xq, xs)
        assert torch.equal(got_s, want_s)
        assert torch.equal(got_q.view(torch.uint8), want_q.view(torch.uint8))
    else:
        want = ops.swiglu(ops.linear(x, weight))
        got = ops.linear_swiglu(x, weight)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("fp8", (True, False))
@pytest.mark.parametrize("rows,mapped", [(256, False), (200, False), (160, True)])
@torch.inference_mode()
def test_conv_in_projection_with_conv_update_epilogue_equals_the_two_launches(ops, fp8, rows, mapped):
    """The fused conv in-projection (gated short-conv update in the product's epilogue, [M, H] written, state updated)
    against the projection followed by the conv-update launch, bit for bit: outputs and every slot's state, with an
    activity mask (rows that sit out keep their taps but still get an output) and, for the compact form, rows mapped to
    slots through slot ids with padding rows."""
    torch.manual_seed(rows)
    hidden, k, slots = 2048, 2048, 300
    weight = (torch.randn(3 * hidden, k, device=DEV) * 0.05).bfloat16()
    conv_weight = torch.randn(hidden, 3, device=DEV).bfloat16()
    x = torch.randn(rows, k, device=DEV).bfloat16()
    state = torch.randn(slots, hidden, 3, device=DEV).bfloat16()
    active = torch.rand(rows, device=DEV) < 0.8
    slot_ids = None
    if mapped:
        slot_ids = torch.randperm(slots, device=DEV)[:rows].to(torch.int32)
        slot_ids[-7:] = -1
        active[-7:] = False
    assert ops.query("lfm2_gemm_conv_fits", rows, 3 * hidden, k, 1 if fp8 else 2) == 1
    assert ops.query("lfm2_gemm_conv_fits", 64, 3 * hidden, k, 1 if fp8 else 2) == 0
    want_state, got_state = state.clone(), state.clone()
    if fp8:
        packed = ops.PackedFP8Weight.from_weight(weight)
        xq, xs = ops.quantize_rows(x)
        want = ops.conv_update(packed.linear_quantized(xq, xs), conv_weight, want_state, active, slot_ids)
        got = packed.linear_conv_update(xq, xs, conv_weight, got_state, active, slot_ids)
        assert packed.linear_conv_update(xq[:64], xs[:64], conv_weight, got_state.clone(), None, None) is None
    else:
        want = ops.conv_update(ops.linear(x, weight), conv_weight, want_state, active, slot_ids)
        got = ops.linear_conv_update(x, weight, conv_weight, got_state, active, slot_ids)
    live = slice(0, rows - 7) if mapped else slice(0, rows)   # padding rows have no defined output
    assert torch.equal(got[live].view(torch.int16), want[live].view(torch.int16))
    assert torch.equal(got_state.view(torch.int16), want_state.view(torch.int16))
    assert not torch.equal(got_state, state)


# ------------------------------------------------------------------------------------------------ measurement entry points
@pytest.mark.parametrize("layout", (0, 1))
@torch.inference_mode()
def test_streaming_read_folds_every_word_of_its_blocks_exactly_once(ops, layout):
    """`lfm2_hbm_stream_read` on a small buffer of random words: lane t of workgroup w must end with the XOR of the
    words of its 16-byte vector in every 4 KiB block the layout gives that workgroup (a private run of blocks, or
    blocks w, w + grid, ...); the blocks beyond a whole number per workgroup are not read."""
    groups, blocks = 3, 31                                   # 10 blocks per workgroup, one left over
    words = torch.randint(-2 ** 31, 2 ** 31 - 1, (blocks * 1024,), dtype=torch.int64).to(torch.int32)
    sink = torch.full((groups * 256,), 7, device=DEV, dtype=torch.int32)
    read = ops.hbm_stream_read(words.to(DEV), sink, workgroups=groups, layout=layout)
    per = blocks // groups
    assert read == groups * per * 4096
    grid = words.view(blocks, 256, 4)
    for w in range(groups):
        mine = [w + b * groups for b in range(per)] if layout else list(range(w * per, (w + 1) * per))
        want = torch.zeros(256, dtype=torch.int32)
        for b in mine:
            for e in range(4):
                want ^= grid[b, :, e]
        assert torch.equal(sink[w * 256:(w + 1) * 256].cpu(), want), (layout, w)
    with pytest.raises(ValueError, match="fewer than 4096 bytes"):
        ops.hbm_stream_read(words[:1024].to(DEV), sink, workgroups=groups, layout=layout)
    with pytest.raises(ValueError, match="int32 sink"):
        ops.hbm_stream_read(words.to(DEV), sink[:100], workgroups=groups, layout=layout)


@torch.inference_mode()
def test_device_timestamps_follow_stream_order(ops):
    stamps = torch.zeros(3, device=DEV, dtype=torch.int64)
    ops.timestamp(stamps[0:1])
    torch.zeros(1 << 24, device=DEV).add_(1)                 # some work between the stamps
    ops.timestamp(stamps[1:2])
    ops.timestamp(stamps[2:3])
    a, b, c = stamps.cpu().tolist()
    assert 0 < a < b <= c
    rate = ops.timestamp_rate_hz()
    assert 1e6 <= rate <= 1e10 and (b - a) / rate < 1.0      # a plausible clock: the fill took well under a second
    with pytest.raises(ValueError, match="int64"):
        ops.timestamp(torch.zeros(1, device=DEV, dtype=torch.int32))


@pytest.mark.parametrize("waves", (4, 8, 16))
@torch.inference_mode()
def test_mfma_loop_adds_the_same_product_every_round(ops, waves):
    """`lfm2_mfma_fp8_peak`: the accumulators grow by one fixed e4m3 product per round (small dyadic values: exact in
    fp32 for a few hundred rounds), so twice the rounds give exactly twice the folded result in every lane, every
    workgroup computes the same, and the clock output is filled."""
    groups = 3
    once = torch.zeros(groups * waves * 64, device=DEV, dtype=torch.float32)
    twice, clock = torch.zeros_like(once), torch.zeros(2 * groups, device=DEV, dtype=torch.int64)
    flops = ops.mfma_fp8_peak(once, None, workgroups=groups, waves=waves, iterations=100)
    assert flops == groups * waves * 100 * 8 * 65536
    ops.mfma_fp8_peak(twice, clock, workgroups=groups, waves=waves, iterations=200)
    assert bool((once > 0).all()) and torch.equal(twice, 2 * once)
    per_group = once.view(groups, -1)
    assert torch.equal(per_group[0], per_group[1]) and torch.equal(per_group[0], per_group[2])
    assert torch.equal(per_group[0][:64], per_group[0][64:128])          # every wave holds the same operands
    assert bool((clock > 0).all())
    with pytest.raises(ValueError, match="waves per workgroup"):
        ops.mfma_fp8_peak(once, None, workgroups=groups, waves=2, iterations=10)
    with pytest.raises(ValueError, match="float32 GPU sink"):
        ops.mfma_fp8_peak(once[:10], None, workgroups=groups, waves=waves, iterations=10)


@torch.inference_mode()
def test_silu_of_the_swiglu_kernels_stays_within_its_stated_error(ops):
    """The SwiGLU kernels compute g / (1 + e^-g) on the hardware's base-2 exponential and reciprocal
    (lfm25_cuda_kernels.py:58-72 uses the tracing compiler's sigmoid, itself an approximation).  In fp32, against
    float64: relative error at most (3 + max(-g, 0)) 2^-23 with a factor 1.5 of slack, over gates in [-30, 30]; far
    below -88 the result is zero, far above it is the gate; in bf16 the rounded result equals the exactly rounded one
    in all but a few elements in ten thousand."""
    gen = torch.Generator().manual_seed(3)
    gate = torch.cat((torch.linspace(-30, 30, 20001), torch.randn(45535, generator=gen) * 4)).float()
    x = torch.cat((gate, torch.ones_like(gate))).view(1, -1).to(DEV)
    got = ops.swiglu(x).double().cpu()[0]
    g = gate.double()
    want = g / (1 + torch.exp(-g))
    bound = 1.5 * (3 + (-g).clamp_min(0)) * 2.0 ** -23 * want.abs() + 1e-45
    assert bool(((got - want).abs() <= bound).all()), float(((got - want).abs() / bound).max())
    edge = torch.tensor([-200.0, -100.0, 100.0, 0.0, float("nan")])
    out = ops.swiglu(torch.cat((edge, torch.ones(5))).view(1, -1).to(DEV)).cpu()[0]
    assert out[:2].abs().max() == 0 and float(out[2]) == 100.0 and float(out[3]) == 0.0 and bool(torch.isnan(out[4]))
    half = torch.cat((gate, torch.ones_like(gate))).view(1, -1).bfloat16()
    got16 = ops.swiglu(half.to(DEV)).cpu()[0]
    g16 = half[0, :gate.numel()].double()
    exact16 = (g16 / (1 + torch.exp(-g16))).float().bfloat16()
    assert float((got16 != exact16).float().mean()) < 1e-3
