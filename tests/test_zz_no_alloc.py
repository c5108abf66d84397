"""The greedy sampler's entry point that allocates nothing, called through ``ctypes`` as a
caller without torch's wrappers would: against ``hal_sample_greedy`` (whose partial results
go to a buffer of the caller's) on two calls in a row, the second with a smaller input, so
that what the first call left in the library's own array is still there."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _greedy(lib, logits, static: bool):
    n, vocab = logits.shape
    tokens = torch.full((n,), -7, dtype=torch.int32, device=logits.device)
    logprobs = torch.full((n,), 3.0, dtype=torch.float32, device=logits.device)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731
    if static:
        rc = lib.hal_sample_greedy_static(ptr(logits), vocab, n, vocab, ptr(tokens), ptr(logprobs), stream)
    else:
        parts = torch.empty((n, 32, 4), dtype=torch.float32, device=logits.device)
        rc = lib.hal_sample_greedy(ptr(logits), vocab, n, vocab, ptr(parts), ptr(tokens), ptr(logprobs), stream)
    assert rc == 0, lib.hal_last_error().decode()
    torch.cuda.synchronize()
    return tokens.cpu(), logprobs.cpu()


def test_greedy_without_allocation_matches_on_two_calls_in_a_row():
    from halite_amd.kernels import library

    lib = library.core_library()
    assert lib.hal_sample_greedy_static_max_rows() == 1024
    gen = torch.Generator().manual_seed(11)
    # the second call is smaller in both directions: the array still holds the first call's rows
    for n, vocab in ((37, 5003), (5, 771)):
        logits = (torch.randn((n, vocab), generator=gen) * 3).cuda()
        logits[1, vocab - 1] = 40.0  # a maximum in the last share
        logits[2, 17] = logits[2, 600] = 35.0  # a tie: the first index wins
        want_tok, want_lp = _greedy(lib, logits, static=False)
        got_tok, got_lp = _greedy(lib, logits, static=True)
        assert torch.equal(got_tok, want_tok)
        assert torch.equal(got_lp, want_lp)  # same kernels, same order of sums
        ref = torch.log_softmax(logits.double().cpu(), dim=-1)
        assert torch.equal(got_tok.long(), ref.argmax(-1))
        assert got_tok[1] == vocab - 1 and got_tok[2] == 17
        assert torch.allclose(got_lp.double(), ref.gather(1, got_tok.long()[:, None])[:, 0], atol=1e-4)


def test_greedy_without_allocation_refuses_what_does_not_fit():
    from halite_amd.kernels import library

    lib = library.core_library()
    logits = torch.zeros((1, 64), dtype=torch.float32, device="cuda")
    out = torch.zeros(2, dtype=torch.int32, device="cuda")
    p = ctypes.c_void_p(logits.data_ptr())
    o = ctypes.c_void_p(out.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # 1025 rows are more than the array holds: refused before anything is launched
    assert lib.hal_sample_greedy_static(p, 64, 1025, 64, o, o, stream) != 0
    assert "at most 1024" in lib.hal_last_error().decode()
    assert lib.hal_sample_greedy_static(p, 64, 0, 64, o, o, stream) == 0
