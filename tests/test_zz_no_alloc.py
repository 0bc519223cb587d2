"""The sampler entry point that allocates nothing (`lfm2_sample_static`): its tile statistics live in a fixed device
array inside the library.  Checked through the C ABI against `lfm2_sample` (caller-provided scratch), bit for bit, on
two calls in a row on the same GPU, the second on a smaller input, and with the allocator watched."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _reference(logits, temperature, seed, step):
    from climbing_gym_amd import ops
    return ops.sample_logits(logits, temperature=temperature, seed=seed, step=step, return_logprobs=True)


@pytest.mark.parametrize("temperature", (0.0, 1.0, 0.7))
def test_static_scratch_sampler_equals_the_allocating_one_on_two_calls_in_a_row(temperature):
    from climbing_gym_amd import ops
    gen = torch.Generator(device="cuda").manual_seed(3)
    big = (torch.randn(96, 65536, device="cuda", generator=gen) * 3).bfloat16()
    small = (torch.randn(5, 10000, device="cuda", generator=gen) * 3).bfloat16()     # fewer rows, fewer and ragged tiles
    for number, logits in enumerate((big, small)):
        want_tokens, want_logprobs = _reference(logits, temperature, seed=11, step=number)
        tokens = torch.full((logits.size(0),), -1, device="cuda", dtype=torch.long)
        logprobs = torch.full((logits.size(0),), float("nan"), device="cuda", dtype=torch.float32)
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats()["allocation.all.allocated"]
        free_before = torch.cuda.mem_get_info()[0]
        ops.sample_logits_static(logits, tokens, logprobs, temperature=temperature, seed=11, step=number)
        torch.cuda.synchronize()
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == before    # nothing came from torch's allocator
        # nor from the driver: a hipMalloc inside the library would lower the device's free bytes (the first call of the
        # process looks the array's address up, which allocates nothing either: the array is part of the code object)
        assert torch.cuda.mem_get_info()[0] >= free_before
        assert torch.equal(tokens, want_tokens)
        assert torch.equal(logprobs.view(torch.int32), want_logprobs.view(torch.int32))


def test_static_scratch_sampler_refuses_what_does_not_fit():
    from climbing_gym_amd import _lib, ops
    logits = torch.zeros((2, 8), device="cuda", dtype=torch.bfloat16)
    tokens = torch.zeros(2, device="cuda", dtype=torch.long)
    lib = _lib.load()
    # 5000 rows x 4 tiles = 20000 tile records > 16384: refused before anything is launched
    status = lib.lfm2_sample_static(tokens.data_ptr(), None, logits.data_ptr(), None, None, None, 0, 0, 1.0, 5000, 16384, 0, None)
    assert status == -1 and b"static scratch holds 16384" in lib.lfm2_last_error()
    with pytest.raises(ValueError, match="static scratch"):
        ops.call("lfm2_sample_static", tokens, None, logits, None, None, None, 0, 0, 1.0, 16385, 8, 0)
    # the Python mirror checks the caller's outputs before the raw pointers reach the kernels
    with pytest.raises(ValueError, match="tokens"):
        ops.sample_logits_static(logits, tokens.int(), None, temperature=1.0, seed=0, step=0)
    with pytest.raises(ValueError, match="tokens"):
        ops.sample_logits_static(logits, tokens[:1], None, temperature=1.0, seed=0, step=0)
    with pytest.raises(ValueError, match="logprobs"):
        ops.sample_logits_static(logits, tokens, torch.zeros(2, device="cuda", dtype=torch.float64), temperature=1.0, seed=0, step=0)
    with pytest.raises(ValueError, match="nonnegative temperature"):
        ops.sample_logits_static(logits, tokens, None, temperature=-1.0, seed=0, step=0)
