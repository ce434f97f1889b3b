"""The entry point that allocates nothing (csrc/no_alloc.h): ``lc_sample_static`` called through
ctypes against ``lc_sample`` with a workspace of the caller's, on two calls in a row, the second
with a smaller input, so that the library's own array still holds the first call's values."""
import ctypes

import pytest
import torch

from lucciola_amd.kernels import ops

pytestmark = pytest.mark.gpu


def _library():
    lib = ctypes.CDLL(ops.library_file())
    lib.lc_last_error.restype = ctypes.c_char_p
    p, i = ctypes.c_void_p, ctypes.c_int
    lib.lc_sample_static.restype = i
    lib.lc_sample_static.argtypes = [p, p, p, p, i, i, p]
    lib.lc_sample.restype = i
    lib.lc_sample.argtypes = [p, p, p, p, p, i, i, p]
    lib.lc_sample_workspace.restype = i
    lib.lc_sample_workspace.argtypes = [i]
    lib.lc_sample_static_max_rows.restype = i
    return lib


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


def test_sampling_without_an_allocation():
    lib = _library()
    dev = torch.device("cuda:0")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    gen = torch.Generator(device="cpu").manual_seed(3)
    assert lib.lc_sample_static_max_rows() == 1024
    for R, V, sampled in ((37, 151936, True), (5, 331, True), (64, 4099, False), (1, 7, True)):
        logits = (torch.randn(R, V, generator=gen) * 3).to(dev)
        temperature = uniform = None
        if sampled:     # greedy rows among sampled ones
            temperature = torch.tensor([0.0 if r % 3 == 0 else 0.5 + 0.1 * r for r in range(R)],
                                       dtype=torch.float32, device=dev)
            uniform = torch.rand(R, generator=gen).to(dev)
        want = torch.full((R,), -1, dtype=torch.int32, device=dev)
        got = torch.full((R,), -2, dtype=torch.int32, device=dev)
        workspace = torch.empty(lib.lc_sample_workspace(R), dtype=torch.float32, device=dev)
        rc = lib.lc_sample(_ptr(logits), _ptr(temperature), _ptr(uniform), _ptr(want), _ptr(workspace),
                           R, V, stream)
        assert rc == 0, lib.lc_last_error()
        # the first call on the device looks the array's address up; what is measured is the calls
        # after it, by the runtime's own count of free device memory (torch's allocator would
        # not see a hipMalloc inside the library)
        rc = lib.lc_sample_static(_ptr(logits), _ptr(temperature), _ptr(uniform), _ptr(got), R, V, stream)
        assert rc == 0, lib.lc_last_error()
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info(dev)[0]
        for _ in range(4):
            got.fill_(-2)
            rc = lib.lc_sample_static(_ptr(logits), _ptr(temperature), _ptr(uniform), _ptr(got), R, V, stream)
            assert rc == 0, lib.lc_last_error()
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info(dev)[0] == free_before
        assert torch.equal(got, want), (R, V)
        assert int(got.min()) >= 0 and int(got.max()) < V
        if not sampled:
            assert torch.equal(got.long(), logits.argmax(dim=1))
        else:
            # against the definition, on the host in float64: greedy rows are the argmax, the others
            # the first token whose cumulative probability exceeds the row's uniform number (a
            # pick at a boundary that float32 sums could move may be its neighbour)
            host, temps, us = logits.double().cpu(), temperature.cpu().tolist(), uniform.cpu().tolist()
            for r in range(R):
                if temps[r] <= 0:
                    assert int(got[r]) == int(host[r].argmax())
                    continue
                cdf = torch.softmax(host[r] / temps[r], 0).cumsum(0)
                pick = min(int(torch.searchsorted(cdf, torch.tensor(us[r], dtype=torch.float64), right=True)), V - 1)
                if int(got[r]) != pick:
                    assert abs(int(got[r]) - pick) == 1 and abs(float(cdf[min(int(got[r]), pick)]) - us[r]) < 1e-5, (r, pick)
    # more rows than the library's array holds: refused, nothing launched
    big = torch.zeros(1025, 8, device=dev)
    out = torch.full((1025,), -5, dtype=torch.int32, device=dev)
    assert lib.lc_sample_static(_ptr(big), None, None, _ptr(out), 1025, 8, stream) != 0
    assert b"1025 rows" in lib.lc_last_error()
    torch.cuda.synchronize()
    assert int(out.max()) == -5
