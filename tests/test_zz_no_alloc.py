"""The entry point that allocates nothing (lmsf_greedy_tokens_static, csrc/no_alloc.h) against the
existing greedy search of lmsf_sample with a caller's scratch buffer, called through ctypes: two
calls in a row, the second with a smaller input, so that what the first call left in the library's
own buffer would show."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

MAX_ROWS = 1024     # LMSF_GREEDY_STATIC_MAX_ROWS


@pytest.fixture(scope="module")
def lib():
    from lmsf_amd.ops import library
    return library.load_library()


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _existing(lib, logits):
    R, V = logits.shape
    elems = lib.lmsf_sample_scratch_elems(R, V)
    assert elems > 0
    scratch = torch.empty(2 * elems, dtype=torch.float32, device=logits.device)
    out = torch.full((R,), -1, dtype=torch.int32, device=logits.device)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.lmsf_sample(_p(logits), logits.stride(0), R, V, None, None, None, None, None, None, _p(out), _p(scratch),
                         stream)
    assert rc == 0, lib.lmsf_last_error()
    return out


def _static(lib, logits):
    R, V = logits.shape
    out = torch.full((R,), -1, dtype=torch.int32, device=logits.device)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.lmsf_greedy_tokens_static(_p(logits), logits.stride(0), R, V, _p(out), stream)
    assert rc == 0, lib.lmsf_last_error()
    return out


def test_two_calls_second_smaller(lib):
    g = torch.Generator().manual_seed(11)
    big = torch.randn(200, 50001, generator=g).to("cuda:0")
    big[7, 123] = big[7, 40000] = 9.0          # equal maxima: the first wins
    small = torch.randn(3, 16411, generator=g).to("cuda:0")
    for logits in (big, small):
        got, want = _static(lib, logits), _existing(lib, logits)
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        assert torch.equal(got.long(), logits.argmax(dim=1))
    assert int(_static(lib, big)[7]) == 123


def test_small_vocabulary_and_row_stride(lib):
    # fewer entries than shares of a row, and rows that are a slice of a wider buffer
    wide = torch.randn(5, 40, generator=torch.Generator().manual_seed(3)).to("cuda:0")
    logits = wide[:, :19]
    got = _static(lib, logits)
    torch.cuda.synchronize()
    assert torch.equal(got.long(), logits.argmax(dim=1))


def test_too_many_rows_are_refused(lib):
    logits = torch.zeros(MAX_ROWS + 1, 8, device="cuda:0")
    out = torch.full((MAX_ROWS + 1,), -1, dtype=torch.int32, device="cuda:0")
    rc = lib.lmsf_greedy_tokens_static(_p(logits), logits.stride(0), MAX_ROWS + 1, 8, _p(out), None)
    assert rc != 0
    assert b"1024" in lib.lmsf_last_error()
    torch.cuda.synchronize()
    assert bool((out == -1).all())
    full = torch.randn(MAX_ROWS, 300, generator=torch.Generator().manual_seed(5)).to("cuda:0")
    got = _static(lib, full)
    torch.cuda.synchronize()
    assert torch.equal(got.long(), full.argmax(dim=1))
