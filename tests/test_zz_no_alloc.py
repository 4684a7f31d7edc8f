"""The sampling entry point that allocates nothing, called through ctypes.

`pae_sample_static` keeps its chunk results in a buffer inside the library's image on the GPU.
Two calls in a row, the second with fewer rows and a shorter vocabulary (so that it finds the first
call's leftovers in the buffer), must give exactly what `pae_sample` gives with a workspace of the
caller's; sizes beyond the buffer are refused with a message; no device memory is taken from
the driver by the calls (by the driver's own count of free memory); and the call can be recorded
into a graph once the buffer's address is known.
"""

import ctypes

import pytest
import torch

from paged_attention_engine_amd.kernels import lib as K

pytestmark = pytest.mark.gpu


def _reference(logits, temperature, uniform):
    tokens = torch.full((logits.shape[0],), -7, dtype=torch.int32, device=logits.device)
    K.sample(tokens, logits, temperature, uniform)
    return tokens


def _static(lib, logits, temperature, uniform):
    rows, vocab = logits.shape
    tokens = torch.full((rows,), -7, dtype=torch.int32, device=logits.device)
    stream = torch.cuda.current_stream().cuda_stream
    code = lib.pae_sample_static(ctypes.c_void_p(tokens.data_ptr()), ctypes.c_void_p(logits.data_ptr()),
                                 ctypes.c_int64(logits.stride(0)),
                                 ctypes.c_void_p(temperature.data_ptr()) if temperature is not None else None,
                                 ctypes.c_void_p(uniform.data_ptr()) if uniform is not None else None,
                                 ctypes.c_int(rows), ctypes.c_int(vocab), ctypes.c_void_p(stream))
    return code, tokens


def _case(rows, vocab, seed, device):
    gen = torch.Generator(device="cpu").manual_seed(seed)
    logits = (torch.randn(rows, vocab, generator=gen) * 3.0).to(device)
    temperature = torch.tensor([0.0 if r % 3 == 0 else 0.5 + 0.25 * (r % 4) for r in range(rows)],
                               dtype=torch.float32, device=device)
    uniform = torch.rand(rows, generator=gen).to(device)
    return logits, temperature, uniform


def test_sampling_without_a_workspace_matches_sampling_with_one():
    device = torch.device("cuda:0")
    lib = K.library()
    assert lib.pae_sample_static_slots() >= 64 * lib.pae_sample_chunks(152064)
    # first call: many rows, a long vocabulary that is no multiple of the chunk size
    first = _case(37, 151_937, 5, device)
    # second call, right after: fewer rows, fewer and shorter chunks, so most of the buffer still
    # holds what the first call wrote
    second = _case(5, 3_333, 6, device)
    want_first = _reference(*first)
    want_second = _reference(*second)
    want_greedy = _reference(second[0], None, None)
    want_argmax = second[0].argmax(dim=1)
    # the buffer's address is looked up once per device (the runtime may take memory of its own for that,
    # once); from then on a call takes nothing
    assert lib.pae_sample_static_prepare() == 0, lib.pae_last_error()
    code, _ = _static(lib, *_case(3, 1_000, 4, device))
    assert code == 0, lib.pae_last_error()
    torch.cuda.synchronize()
    # what the driver itself says is free: torch's own counters cannot see a hipMalloc inside the library
    held = torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0]

    code, got_first = _static(lib, *first)
    assert code == 0, lib.pae_last_error()
    code, got_second = _static(lib, *second)
    assert code == 0, lib.pae_last_error()
    code, got_greedy = _static(lib, second[0], None, None)
    assert code == 0, lib.pae_last_error()
    torch.cuda.synchronize()
    # nothing was taken from the driver, neither by torch (the outputs' few bytes come out of blocks it
    # already holds) nor behind its back by the library
    after = torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0]
    assert after[0] == held[0]
    assert after[1] == held[1], f"{held[1] - after[1]} bytes of device memory went during the calls"
    assert torch.equal(got_first, want_first)
    assert torch.equal(got_second, want_second)
    assert torch.equal(got_greedy, want_greedy)
    assert int(got_first.min()) >= 0 and int(got_first.max()) < 151_937
    # greedy rows are the first maximum
    assert torch.equal(got_greedy.long(), want_argmax)


def test_the_call_can_be_recorded_into_a_graph_after_a_first_call_outside():
    """The buffer's address is looked up at the first call on a device, which must not fall inside a
    capture; after it, the call records like any kernel launch.  Every replay is checked against the
    eager result, with eager work and synchronisation between the replays."""
    device = torch.device("cuda:0")
    lib = K.library()
    assert lib.pae_sample_static_prepare() == 0, lib.pae_last_error()
    logits, temperature, uniform = _case(9, 50_021, 11, device)
    tokens = torch.full((9,), -7, dtype=torch.int32, device=device)
    K.sample_static(tokens, logits, temperature, uniform)  # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        K.sample_static(tokens, logits, temperature, uniform)
    for seed in (12, 13, 14):
        fresh = _case(9, 50_021, seed, device)
        want = _reference(*fresh)
        for dst, src in zip((logits, temperature, uniform), fresh):
            dst.copy_(src)
        tokens.fill_(-7)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(tokens, want), seed


def test_sizes_beyond_the_buffer_are_refused():
    device = torch.device("cuda:0")
    lib = K.library()
    slots = lib.pae_sample_static_slots()
    vocab = 200_000
    chunks = lib.pae_sample_chunks(vocab)
    rows = slots // chunks + 1
    logits = torch.zeros((rows, vocab), dtype=torch.float32, device=device)
    tokens = torch.full((rows,), -7, dtype=torch.int32, device=device)
    code = lib.pae_sample_static(ctypes.c_void_p(tokens.data_ptr()), ctypes.c_void_p(logits.data_ptr()),
                                 ctypes.c_int64(vocab), None, None, ctypes.c_int(rows), ctypes.c_int(vocab),
                                 ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert code != 0
    message = lib.pae_last_error().decode()
    assert "chunk slots" in message and str(slots) in message
    torch.cuda.synchronize()
    assert int(tokens.min()) == -7 and int(tokens.max()) == -7  # nothing ran
    with pytest.raises(K.KernelError):
        K.sample_static(tokens, logits, None, None)
