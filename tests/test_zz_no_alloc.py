"""The sampling entry point that allocates nothing, called through ctypes the way a
caller without torch would, against `mlr_sample` with a scratch buffer of the caller."""

import ctypes

import pytest
import torch

from mini_llm_runtime_amd.kernels import build

pytestmark = pytest.mark.gpu

_VP, _I = ctypes.c_void_p, ctypes.c_int


def _library():
    lib = ctypes.CDLL(str(build.ensure_module(build.CORE)))
    lib.mlr_last_error.restype = ctypes.c_char_p
    lib.mlr_sample_scratch.argtypes = [_I, _I]
    lib.mlr_sample_scratch.restype = ctypes.c_int64
    lib.mlr_sample.argtypes = [_VP, _VP, _VP, _VP, _VP, _I, _I, _VP]
    lib.mlr_sample_static.argtypes = [_VP, _VP, _VP, _VP, _I, _I, _VP]
    lib.mlr_sample_static_capacity.restype = ctypes.c_int64
    return lib


def _both(lib, rows, vocab, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    logits = (torch.randn(rows, vocab, generator=g) * 3).cuda()
    temperature = torch.where(torch.arange(rows) % 3 == 0, 0.0, 0.7 + 0.1 * (torch.arange(rows) % 5)).float().cuda()
    uniform = torch.rand(rows, generator=g).cuda()
    stream = _VP(torch.cuda.current_stream().cuda_stream)
    expected = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    scratch = torch.empty(lib.mlr_sample_scratch(rows, vocab), dtype=torch.float32, device="cuda")
    got = torch.full((rows,), -2, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    status = lib.mlr_sample(
        logits.data_ptr(), temperature.data_ptr(), uniform.data_ptr(), expected.data_ptr(), scratch.data_ptr(),
        rows, vocab, stream,
    )
    assert status == 0, lib.mlr_last_error()
    # Device memory as the driver counts it (an allocation inside the library would not show in
    # torch's own counters), and torch's counter for whatever went through its allocator.
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    status = lib.mlr_sample_static(
        logits.data_ptr(), temperature.data_ptr(), uniform.data_ptr(), got.data_ptr(), rows, vocab, stream
    )
    assert status == 0, lib.mlr_last_error()
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, f"the call changed free device memory by {free_before - free_after} bytes"
    assert (expected >= 0).all() and (expected < vocab).all()
    assert torch.equal(got, expected)
    greedy = temperature.cpu() == 0
    assert torch.equal(got.cpu()[greedy].long(), logits.cpu()[greedy].argmax(-1))


def test_static_scratch_sampling_equals_the_one_with_a_buffer():
    lib = _library()
    _both(lib, rows=37, vocab=151_936, seed=1)  # 38 segments a row
    _both(lib, rows=5, vocab=5_003, seed=2)  # then a smaller one over what the first left behind
    _both(lib, rows=1, vocab=17, seed=3)


@torch.inference_mode()  # as the engine records its steps (torch's capture state was made under it by then)
def test_static_scratch_sampling_inside_a_graph_capture():
    """A capture forbids allocation: the call is recorded after one call outside (the address of
    the array is looked up at the first call), then replayed with new logits each time and
    compared with the entry point that takes a buffer, run unrecorded between the replays."""
    lib = _library()
    rows, vocab = 9, 33_001
    g = torch.Generator(device="cpu").manual_seed(7)
    logits = (torch.randn(rows, vocab, generator=g) * 3).cuda()
    temperature = torch.where(torch.arange(rows) % 2 == 0, 0.0, 0.9).float().cuda()
    uniform = torch.rand(rows, generator=g).cuda()
    got = torch.full((rows,), -2, dtype=torch.int32, device="cuda")
    scratch = torch.empty(lib.mlr_sample_scratch(rows, vocab), dtype=torch.float32, device="cuda")
    expected = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    arguments = (logits.data_ptr(), temperature.data_ptr(), uniform.data_ptr(), got.data_ptr(), rows, vocab)
    assert lib.mlr_sample_static(*arguments, _VP(torch.cuda.current_stream().cuda_stream)) == 0, lib.mlr_last_error()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        status = lib.mlr_sample_static(*arguments, _VP(torch.cuda.current_stream().cuda_stream))
    assert status == 0, lib.mlr_last_error()
    for turn in range(3):
        logits.copy_((torch.randn(rows, vocab, generator=g) * 3).cuda())
        uniform.copy_(torch.rand(rows, generator=g).cuda())
        got.fill_(-2)
        graph.replay()
        status = lib.mlr_sample(
            logits.data_ptr(), temperature.data_ptr(), uniform.data_ptr(), expected.data_ptr(), scratch.data_ptr(),
            rows, vocab, _VP(torch.cuda.current_stream().cuda_stream),
        )
        assert status == 0, lib.mlr_last_error()
        torch.cuda.synchronize()
        assert torch.equal(got, expected), f"replay {turn}"


def test_static_scratch_refuses_what_does_not_fit():
    lib = _library()
    rows = int(lib.mlr_sample_static_capacity()) // (38 * 3) + 1
    logits = torch.zeros(1, device="cuda")
    tokens = torch.zeros(1, dtype=torch.int32, device="cuda")
    stream = _VP(torch.cuda.current_stream().cuda_stream)
    status = lib.mlr_sample_static(logits.data_ptr(), None, None, tokens.data_ptr(), rows, 151_936, stream)
    assert status == -1
    message = lib.mlr_last_error().decode()
    assert "floats of scratch" in message and str(rows) in message
