"""The sampling entry point that allocates nothing (ga_sample_rows_static), called through ctypes as a caller outside
the package would, against ga_sample_rows with scratch memory of the caller's."""
import ctypes

import pytest
import torch

from ginfer_amd.kernels import build

pytestmark = pytest.mark.gpu

_vp, _i, _i64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64


def _library():
    lib = ctypes.CDLL(build.load("sampling")._name)      # the built file, opened as any C caller would
    lib.ga_sample_scratch_floats.restype = _i64
    lib.ga_sample_rows_static_error.restype = ctypes.c_char_p
    return lib


def _stream():
    return _vp(torch.cuda.current_stream().cuda_stream)


def _both(lib, logits, temperature, uniform):
    """(tokens by the entry point that takes scratch memory, tokens by the one that allocates nothing)."""
    R, V = logits.shape
    ptr = lambda t: _vp(t.data_ptr()) if t is not None else _vp(0)
    scratch = torch.empty(max(1, lib.ga_sample_scratch_floats(_i(R), _i(V))), dtype=torch.float32, device=logits.device)
    want = torch.full((R,), -1, dtype=torch.int32, device=logits.device)
    got = torch.full((R,), -1, dtype=torch.int32, device=logits.device)
    torch.cuda.synchronize()
    assert lib.ga_sample_rows(ptr(want), ptr(logits), _i64(logits.stride(0)), _i(R), _i(V), ptr(temperature), ptr(uniform),
                              ptr(scratch), _stream()) == 0
    # what the driver itself has free, with the device idle on both sides of the call: torch's own counters would not see
    # an allocation that the library made behind its back
    torch.cuda.synchronize()
    before = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    rc = lib.ga_sample_rows_static(ptr(got), ptr(logits), _i64(logits.stride(0)), _i(R), _i(V), ptr(temperature),
                                   ptr(uniform), _stream())
    assert rc == 0, lib.ga_sample_rows_static_error(_i(rc))
    torch.cuda.synchronize()
    assert (torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == before
    return want.cpu().tolist(), got.cpu().tolist()


def test_sampling_without_allocation_equals_sampling_with_scratch_memory():
    dev = torch.device("cuda", 0)
    lib = _library()
    assert lib.ga_sample_rows_static_init() == 0
    assert lib.ga_sample_rows_static_max_rows() == 256
    g = torch.Generator().manual_seed(5)
    # two calls in a row, the second smaller in rows and in vocabulary: it must not see what the first one left
    for R, V in ((200, 151936), (7, 777), (256, 5000), (1, 128)):
        logits = (torch.randn(R, V, generator=g) * 3).to(dev)
        temps = torch.where(torch.arange(R) % 3 == 0, torch.zeros(R), torch.rand(R, generator=g) + 0.3).to(dev)
        uni = torch.rand(R, generator=g).to(dev)
        want, got = _both(lib, logits, temps, uni)
        assert got == want and all(0 <= t < V for t in got), (R, V)
        want, got = _both(lib, logits, None, None)           # all rows greedy
        assert got == want == logits.argmax(dim=1).cpu().tolist(), (R, V)


def test_sampling_without_allocation_refuses_more_rows_than_it_holds():
    dev = torch.device("cuda", 0)
    lib = _library()
    logits = torch.zeros(257, 64, device=dev)
    out = torch.full((257,), -7, dtype=torch.int32, device=dev)
    rc = lib.ga_sample_rows_static(_vp(out.data_ptr()), _vp(logits.data_ptr()), _i64(64), _i(257), _i(64), _vp(0), _vp(0),
                                   _stream())
    torch.cuda.synchronize()
    assert rc == -2 and b"256 rows" in lib.ga_sample_rows_static_error(_i(rc))
    assert out.cpu().tolist() == [-7] * 257                  # nothing was launched
    assert lib.ga_sample_rows_static(_vp(out.data_ptr()), _vp(logits.data_ptr()), _i64(64), _i(4), _i(0), _vp(0), _vp(0),
                                     _stream()) == -1
