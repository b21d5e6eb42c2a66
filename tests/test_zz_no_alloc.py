"""The sampling entry point that allocates nothing (`me_sample_static`: its partial results live in a
device array of the library) against the one that takes a workspace (`me_sample`), through ctypes:
two calls in a row, the second with a smaller input, so that the array still holds the first call's
partial results when the second runs."""
import ctypes
from ctypes import c_int, c_int64, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from mini_engine_amd.kernels import build
    lib = ctypes.CDLL(build.core_library())
    lib.me_last_error.restype = ctypes.c_char_p
    lib.me_sample.argtypes = [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]
    lib.me_sample.restype = c_int
    lib.me_sample_static.argtypes = [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]
    lib.me_sample_static.restype = c_int
    return lib


def _case(S, V, seed, ld=None):
    g = torch.Generator().manual_seed(seed)
    ld = ld or V
    logits = (torch.randn(S, ld, generator=g) * 3).cuda()
    temps = torch.tensor([0.0 if i % 3 == 0 else 0.5 + 0.25 * (i % 5) for i in range(S)], dtype=torch.float32).cuda()
    keys = torch.randint(-2**31, 2**31 - 1, (S, 2), generator=g, dtype=torch.int64).to(torch.int32).cuda()
    return logits, temps, keys


def _both(lib, logits, temps, keys, V):
    S = logits.shape[0]
    stream = torch.cuda.current_stream().cuda_stream
    want = torch.full((S,), -7, dtype=torch.int32, device="cuda")
    work = torch.empty(2 * S * 32, dtype=torch.int32, device="cuda")
    rc = lib.me_sample(logits.data_ptr(), logits.stride(0), temps.data_ptr(), keys.data_ptr(), want.data_ptr(),
                       work.data_ptr(), S, V, stream)
    assert rc == 0, lib.me_last_error().decode()
    got = torch.full((S,), -7, dtype=torch.int32, device="cuda")
    rc = lib.me_sample_static(logits.data_ptr(), logits.stride(0), temps.data_ptr(), keys.data_ptr(), got.data_ptr(),
                              S, V, stream)
    assert rc == 0, lib.me_last_error().decode()
    torch.cuda.synchronize()
    return got.cpu(), want.cpu()


def test_static_scratch_sampling_equals_the_workspace_form_twice_in_a_row():
    lib = _library()
    # a large call first (32 chunks per row, 300 rows), then a smaller one (fewer rows, 4 chunks per row,
    # a row stride beyond the vocabulary): the second finds the first's partial results in the array
    for S, V, ld, seed in ((300, 20011, None, 1), (7, 3001, 3008, 2)):
        logits, temps, keys = _case(S, V, seed, ld)
        got, want = _both(lib, logits, temps, keys, V)
        assert (want >= 0).all() and (want < V).all()
        assert torch.equal(got, want), (S, V)
        greedy = (temps.cpu() == 0).nonzero().flatten()
        assert torch.equal(got[greedy].long(), logits[:, :V].argmax(-1).cpu()[greedy])


def test_static_scratch_sampling_refuses_more_rows_than_it_holds():
    lib = _library()
    S, V = 1025, 64
    logits, temps, keys = _case(S, V, 3)
    out = torch.full((S,), -7, dtype=torch.int32, device="cuda")
    rc = lib.me_sample_static(logits.data_ptr(), logits.stride(0), temps.data_ptr(), keys.data_ptr(), out.data_ptr(),
                              S, V, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc != 0 and "1024" in lib.me_last_error().decode()
    assert (out.cpu() == -7).all()          # nothing ran
