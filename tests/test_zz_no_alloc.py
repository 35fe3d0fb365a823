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
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    status = lib.mlr_sample_static(
        logits.data_ptr(), temperature.data_ptr(), uniform.data_ptr(), got.data_ptr(), rows, vocab, stream
    )
    assert status == 0, lib.mlr_last_error()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
    torch.cuda.synchronize()
    assert (expected >= 0).all() and (expected < vocab).all()
    assert torch.equal(got, expected)
    greedy = temperature.cpu() == 0
    assert torch.equal(got.cpu()[greedy].long(), logits.cpu()[greedy].argmax(-1))


def test_static_scratch_sampling_equals_the_one_with_a_buffer():
    lib = _library()
    _both(lib, rows=37, vocab=151_936, seed=1)  # 38 segments a row
    _both(lib, rows=5, vocab=5_003, seed=2)  # then a smaller one over what the first left behind
    _both(lib, rows=1, vocab=17, seed=3)


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
