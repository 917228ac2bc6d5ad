"""The token-choice entry point that allocates nothing (``jv_sample_noalloc``), called through
ctypes as a caller without an allocator would, against ``jv_sample`` with a workspace."""
import ctypes
from ctypes import c_int, c_longlong, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu


def _lib():
    from jax_vllm_amd.ops import library

    lib = library.core()
    lib.jv_sample_scratch_bytes.restype = c_longlong
    lib.jv_sample_noalloc_last_error.restype = ctypes.c_char_p
    return lib


def _ptr(t):
    return c_void_p(0 if t is None else t.data_ptr())


def _both(lib, logits, temperature, keys):
    """(tokens of jv_sample with a torch workspace, tokens of jv_sample_noalloc) for the same rows."""
    m, v = logits.shape
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    want = torch.full((m,), -1, dtype=torch.int32, device="cuda")
    work = torch.empty(lib.jv_sample_scratch_bytes(c_int(m)), dtype=torch.uint8, device="cuda")
    assert lib.jv_sample(_ptr(want), _ptr(logits), c_longlong(logits.stride(0)), c_int(m), c_int(v), _ptr(temperature),
                         _ptr(keys), _ptr(work), stream) == 0
    got = torch.full((m,), -1, dtype=torch.int32, device="cuda")
    code = lib.jv_sample_noalloc(_ptr(got), _ptr(logits), c_longlong(logits.stride(0)), c_int(m), c_int(v),
                                 _ptr(temperature), _ptr(keys), stream)
    assert code == 0, lib.jv_sample_noalloc_last_error().decode()
    assert lib.jv_sample_noalloc_last_error() == b""
    torch.cuda.synchronize()
    return want.cpu(), got.cpu()


def test_two_calls_in_a_row_the_second_smaller_match_the_workspace_variant():
    lib = _lib()
    assert lib.jv_sample_noalloc_init() == 0
    g = torch.Generator().manual_seed(5)
    # a large call first: 37 rows over a vocabulary that takes many chunks and is no power of two;
    # then a smaller one (fewer rows, fewer chunks): what the first left in the array must not show
    for rows, vocab in ((37, 151_936), (5, 9_001), (1, 777)):
        logits = (3.0 * torch.randn(rows, vocab, generator=g)).cuda()
        logits[0, vocab - 1] = 50.0                       # the last column wins row 0
        want, got = _both(lib, logits, None, None)
        assert torch.equal(want, got) and int(got[0]) == vocab - 1
        assert torch.equal(got.long(), logits.cpu().argmax(dim=-1))
        # sampled rows beside greedy ones: same draws as with the workspace
        temperature = torch.tensor([0.0 if r % 3 == 0 else 0.5 + 0.1 * r for r in range(rows)], dtype=torch.float32).cuda()
        keys = torch.arange(1000, 1000 + rows, dtype=torch.int64).cuda()
        want, got = _both(lib, logits, temperature, keys)
        assert torch.equal(want, got)
        assert int(got.min()) >= 0 and int(got.max()) < vocab


def test_the_largest_call_fits_and_a_larger_one_is_refused_with_a_sentence():
    lib = _lib()
    most = 1024
    logits = torch.randn(most, 300, generator=torch.Generator().manual_seed(6)).cuda()
    want, got = _both(lib, logits, None, None)
    assert torch.equal(want, got)
    out = torch.full((most + 1,), -7, dtype=torch.int32, device="cuda")
    more = torch.zeros(most + 1, 300, device="cuda")
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    code = lib.jv_sample_noalloc(_ptr(out), _ptr(more), c_longlong(300), c_int(most + 1), c_int(300), None, None, stream)
    assert code == 1
    msg = lib.jv_sample_noalloc_last_error().decode()
    assert "1025 rows exceed the maximum of 1024" in msg
    torch.cuda.synchronize()
    assert int(out.min()) == int(out.max()) == -7          # nothing ran
    assert lib.jv_sample_noalloc(_ptr(out), _ptr(more), c_longlong(300), c_int(0), c_int(300), None, None, stream) == 0
