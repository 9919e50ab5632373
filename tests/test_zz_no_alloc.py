"""The sampling entry point that allocates nothing (``lev_sample_static``: its scratch memory is a ``__device__``
array of the library) gives what ``lev_sample`` gives with a workspace from the caller. Called through ``ctypes``,
twice in a row, the second time with fewer rows and a smaller vocabulary, so that the array still holds the first
call's candidates. Collected last: it must pass alone in a fresh process and after every other test."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

c_void_p, c_int, c_long = ctypes.c_void_p, ctypes.c_int, ctypes.c_long


def _library():
    from levanter_amd.kernels import build

    lib = ctypes.CDLL(build.ensure_built("core"), mode=ctypes.RTLD_GLOBAL)
    lib.lev_last_error.restype = ctypes.c_char_p
    lib.lev_sample_workspace.argtypes = [c_int]
    lib.lev_sample_workspace.restype = c_long
    lib.lev_sample.argtypes = [c_void_p, c_long] + [c_void_p] * 6 + [c_int, c_int, c_void_p]
    lib.lev_sample.restype = c_int
    lib.lev_sample_static.argtypes = [c_void_p, c_long] + [c_void_p] * 5 + [c_int, c_int, c_void_p]
    lib.lev_sample_static.restype = c_int
    lib.lev_sample_static_init.restype = c_int
    lib.lev_sample_static_max_rows.restype = c_int
    return lib


def _inputs(rows, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(rows, vocab, generator=g) * 3).cuda()
    temps = torch.tensor([0.0 if r % 3 == 0 else 0.7 + 0.1 * r for r in range(rows)], dtype=torch.float32).cuda()
    keys = torch.randint(-2**31, 2**31 - 1, (rows, 2), generator=g, dtype=torch.int64).to(torch.int32).cuda()
    positions = torch.randint(0, 5000, (rows,), generator=g, dtype=torch.int64).to(torch.int32).cuda()
    return logits, temps, keys, positions


def _run(lib, fn, inputs, workspace):
    logits, temps, keys, positions = inputs
    rows, vocab = logits.shape
    tokens = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
    logprobs = torch.full((rows,), 123.0, dtype=torch.float32, device="cuda")
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: c_void_p(t.data_ptr())
    if workspace is None:
        rc = lib.lev_sample_static(p(logits), logits.stride(0), p(temps), p(keys), p(positions), p(tokens), p(logprobs), rows, vocab, stream)
    else:
        rc = lib.lev_sample(p(logits), logits.stride(0), p(temps), p(keys), p(positions), p(tokens), p(logprobs), p(workspace), rows, vocab, stream)
    assert rc == 0, lib.lev_last_error().decode()
    torch.cuda.synchronize()
    return tokens.cpu(), logprobs.cpu()


def test_sampling_from_the_library_s_own_scratch_array_equals_sampling_with_a_workspace():
    lib = _library()
    assert lib.lev_sample_static_init() == 0, lib.lev_last_error().decode()
    most = lib.lev_sample_static_max_rows()
    assert most >= 64
    workspace = torch.empty(lib.lev_sample_workspace(most), dtype=torch.uint8, device="cuda")
    for rows, vocab, seed in ((most, 50257, 0), (5, 1000, 1)):  # the second call finds the first one's candidates in the array
        inputs = _inputs(rows, vocab, seed)
        want_tokens, want_logprobs = _run(lib, "lev_sample", inputs, workspace)
        got_tokens, got_logprobs = _run(lib, "lev_sample_static", inputs, None)
        assert torch.equal(got_tokens, want_tokens)
        assert torch.equal(got_logprobs, want_logprobs)
        assert int(got_tokens.min()) >= 0 and int(got_tokens.max()) < vocab
        greedy = torch.arange(rows) % 3 == 0
        assert torch.equal(got_tokens[greedy].long(), inputs[0].cpu()[greedy].argmax(-1))
    # beyond the array: refused with a message, nothing launched
    inputs = _inputs(most + 1, 64, 2)
    logits, temps, keys, positions = inputs
    out_t = torch.zeros(most + 1, dtype=torch.int32, device="cuda")
    out_l = torch.zeros(most + 1, dtype=torch.float32, device="cuda")
    p = lambda t: c_void_p(t.data_ptr())
    rc = lib.lev_sample_static(p(logits), logits.stride(0), p(temps), p(keys), p(positions), p(out_t), p(out_l), most + 1, 64,
                               c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc != 0 and b"more than" in lib.lev_last_error()
