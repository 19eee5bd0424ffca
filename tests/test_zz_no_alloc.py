"""The sampling entry point that allocates nothing, called through ctypes beside the one with a workspace."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from sprout_lm_amd.ops import library
    lib = library()
    c_void, c_int = ctypes.c_void_p, ctypes.c_int
    lib.sp_sample_static.argtypes = [c_void, c_void, c_void, c_void, c_void, c_void, c_int, c_int]
    lib.sp_sample_static.restype = c_int
    lib.sp_sample_static_max_floats.argtypes = []
    lib.sp_sample_static_max_floats.restype = c_int
    return lib


def _both(lib, logits, temperature=None, seed=None, counter=None):
    """(tokens of sp_sample, tokens of sp_sample_static) for the same rows."""
    rows, vocab = logits.shape
    stream = torch.cuda.current_stream().cuda_stream
    ptr = lambda t: None if t is None else t.data_ptr()
    with_ws = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
    static = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
    ws = torch.empty(max(1, lib.sp_sample_workspace_floats(rows, vocab)), dtype=torch.float32, device="cuda")
    assert lib.sp_sample(stream, logits.data_ptr(), ptr(temperature), ptr(seed), ptr(counter), with_ws.data_ptr(),
                         ws.data_ptr(), rows, vocab) == 0, lib.sp_last_error()
    assert lib.sp_sample_static(stream, logits.data_ptr(), ptr(temperature), ptr(seed), ptr(counter), static.data_ptr(),
                                rows, vocab) == 0, lib.sp_last_error()
    torch.cuda.synchronize()
    return with_ws.cpu().numpy(), static.cpu().numpy()


def test_sampling_without_allocation_gives_what_sampling_with_a_workspace_gives():
    lib = _library()
    limit = lib.sp_sample_static_max_floats()
    assert 0 < limit <= (1 << 20)
    rng = np.random.default_rng(3)
    # two calls in a row, the second with a smaller input: what the first left in the array must not be seen
    first = torch.from_numpy(rng.standard_normal((37, 151_936)).astype(np.float32)).cuda()
    second = torch.from_numpy(rng.standard_normal((5, 4_099)).astype(np.float32)).cuda()
    second[2, 17] = float("nan")                      # a non-finite row yields -1 in both
    second[3, 1000:1003] = 9.0                        # ties: the lowest index
    for logits in (first, second):
        want, got = _both(lib, logits)
        assert np.array_equal(got, want) and np.array_equal(want >= 0, ~torch.isnan(logits).any(1).cpu().numpy())
        assert np.array_equal(want[want >= 0], logits.argmax(1).cpu().numpy()[want >= 0])
    want, got = _both(lib, second)
    assert want[2] == -1 and want[3] == 1000 and np.array_equal(got, want)
    # with temperature: the same draws
    rows = first.shape[0]
    temperature = torch.linspace(0.0, 1.5, rows, device="cuda")
    seed = torch.arange(rows, dtype=torch.int64, device="cuda") * 77 + 5
    counter = torch.arange(rows, dtype=torch.int32, device="cuda")
    want, got = _both(lib, first, temperature, seed, counter)
    assert np.array_equal(got, want) and (want != first.argmax(1).cpu().numpy()).any()
    want, got = _both(lib, second[:2].contiguous(), temperature[:2].contiguous() + 0.5, seed[:2].contiguous(), counter[:2].contiguous())
    assert np.array_equal(got, want)


def test_sizes_beyond_the_static_array_are_refused():
    lib = _library()
    limit = lib.sp_sample_static_max_floats()
    vocab = 151_936
    rows = limit // (2 * (-(-vocab // 2048))) + 1        # one row more than fits
    logits = torch.zeros((rows, vocab), dtype=torch.float32, device="cuda")
    out = torch.zeros(rows, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.sp_sample_static(stream, logits.data_ptr(), None, None, None, out.data_ptr(), rows, vocab) != 0
    assert b"static array holds" in lib.sp_last_error()
    assert lib.sp_sample_static(stream, logits.data_ptr(), None, None, None, out.data_ptr(), rows - 1, vocab) == 0
    torch.cuda.synchronize()
    assert (out[:rows - 1] == 0).all()                   # all logits equal: the lowest index
