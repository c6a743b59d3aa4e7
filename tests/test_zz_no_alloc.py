"""The sampler's entry point that allocates nothing (csrc/sampling.h,
gfa_sample_split_static), called through ctypes as a caller without an allocator would:
its tokens and probabilities must equal those of gfa_sample_split with a workspace from the
caller, on two calls in a row of which the second is smaller, greedy and sampled."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _library():
    from gpt_fast_amd.csrc import build
    build.ensure(["sampling"])
    lib = ctypes.CDLL(build.library_path("sampling"))
    lib.gfa_sample_split_workspace.restype = ctypes.c_size_t
    lib.gfa_sampling_last_error.restype = ctypes.c_char_p
    return lib


def _args(logits, temperature, top_k, seed, keys, pos, out, probs):
    p = lambda t: ctypes.c_void_p(0 if t is None else t.data_ptr())
    B, V = logits.shape
    return [p(logits), ctypes.c_size_t(logits.stride(0)), ctypes.c_int(B), ctypes.c_int(V),
            ctypes.c_float(temperature), ctypes.c_int(top_k), ctypes.c_uint64(seed), p(None),
            p(keys), p(pos), ctypes.c_int(1), p(out), p(probs)]


def _both(lib, B, V, temperature, top_k, seed, gen):
    """(tokens, probabilities) of the entry point with a caller's workspace and of the one
    without, on the same logits."""
    logits = torch.randn(B, V, generator=gen, device=DEV) * 3
    keys = torch.arange(B, dtype=torch.int32, device=DEV) + 5
    pos = torch.arange(B, dtype=torch.int32, device=DEV) * 7
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    got = []
    for static in (False, True):
        out = torch.full((B,), -1, dtype=torch.int32, device=DEV)
        probs = torch.zeros(B, V, device=DEV) if temperature > 0 else None
        args = _args(logits, temperature, top_k, seed, keys, pos, out, probs)
        if static:
            rc = lib.gfa_sample_split_static(*args, stream)
        else:
            ws = torch.zeros(lib.gfa_sample_split_workspace(ctypes.c_int(B), ctypes.c_int(V)) // 4,
                             dtype=torch.int32, device=DEV)
            rc = lib.gfa_sample_split(*args, ctypes.c_void_p(ws.data_ptr()), stream)
        assert rc == 0, (static, rc, lib.gfa_sampling_last_error())
        torch.cuda.synchronize()
        got.append((out.cpu(), None if probs is None else probs.cpu()))
    return got


def test_the_sampler_that_allocates_nothing_equals_the_one_with_a_workspace():
    lib = _library()
    torch.cuda.set_device(0)
    assert lib.gfa_sampling_init() == 0
    gen = torch.Generator(device=DEV).manual_seed(11)
    # two calls in a row on the same array, the second smaller in both sizes; then a larger
    # one again, whose histograms lie where the calls before left other data
    for B, V, temperature, top_k in ((8, 128256, 0.8, 50), (3, 50000, 0.8, 7), (5, 9000, 0.0, 0),
                                     (24, 40000, 1.3, 200), (2, 128256, 0.7, 0), (64, 262144, 0.9, 40)):
        (tok_ws, p_ws), (tok_st, p_st) = _both(lib, B, V, temperature, top_k, 1234 + B, gen)
        assert torch.equal(tok_ws, tok_st), (B, V, temperature, top_k)
        assert int(tok_st.min()) >= 0 and int(tok_st.max()) < V
        if p_ws is not None:
            assert torch.equal(p_ws, p_st)
            assert torch.allclose(p_st.sum(1), torch.ones(B), atol=1e-4)
            if top_k:
                assert int((p_st > 0).sum(1).max()) <= top_k + 2      # ties with the k-th stay


def test_the_sampler_that_allocates_nothing_refuses_what_exceeds_its_array():
    lib = _library()
    gen = torch.Generator(device=DEV).manual_seed(3)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for B, V in ((65, 1000), (2, 262145)):
        logits = torch.randn(B, V, generator=gen, device=DEV)
        keys = torch.zeros(B, dtype=torch.int32, device=DEV)
        out = torch.full((B,), -1, dtype=torch.int32, device=DEV)
        rc = lib.gfa_sample_split_static(*_args(logits, 0.8, 5, 1, keys, keys, out, None), stream)
        assert rc != 0
        msg = lib.gfa_sampling_last_error().decode()
        assert "at most 64 rows" in msg and "262144" in msg, msg
        torch.cuda.synchronize()
        assert int(out.max()) == -1                       # nothing ran
