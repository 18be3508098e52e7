"""The sampler's entry point that allocates nothing (``ms_sample_rows_static``), called through ctypes
as a foreign caller would, against the entry point it is a variant of (``ms_sample_rows`` with a
scratch buffer of the caller's): two calls in a row on the same GPU, the second with a smaller input,
so that what the first call left in the library's array must not show."""

import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _case(torch, rows, vocab, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    logits = torch.randn((rows, vocab), generator=g, device="cuda", dtype=torch.float32) * 3
    kinds = np.arange(rows) % 3  # greedy, temperature, temperature with a nucleus
    temperature = torch.tensor(np.where(kinds == 0, 0.0, 0.7 + 0.1 * (np.arange(rows) % 5)), dtype=torch.float32, device="cuda")
    top_p = torch.tensor(np.where(kinds == 2, 0.8, 1.0), dtype=torch.float32, device="cuda")
    seeds = torch.arange(rows, dtype=torch.int32, device="cuda") * 7919 + seed
    counter = torch.arange(rows, dtype=torch.int32, device="cuda") + 11
    return logits, temperature, top_p, seeds, counter


def test_sampler_without_allocation_matches_the_sampler_with_a_scratch_buffer():
    import torch

    from miniserve_amd.kernels import ops

    lib = ctypes.CDLL(ops.library_path())
    vp, ci, cll = ctypes.c_void_p, ctypes.c_int, ctypes.c_longlong
    lib.ms_sample_rows.argtypes = [vp, ci, ci, cll, vp, vp, vp, vp, vp, vp, vp]
    lib.ms_sample_rows_static.argtypes = [vp, ci, ci, cll, vp, vp, vp, vp, vp, vp]
    lib.ms_sample_scratch_bytes.argtypes = [ci]
    most = lib.ms_sample_rows_static_max_rows()
    assert most == 256
    stream = torch.cuda.current_stream().cuda_stream

    # the first call fills the library's array for many rows; the second, smaller one must not see it
    for rows, vocab, seed in ((most, 1531, 1), (5, 379, 2)):
        logits, temperature, top_p, seeds, counter = _case(torch, rows, vocab, seed)
        want = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        got = torch.full((rows,), -2, dtype=torch.int32, device="cuda")
        scratch = torch.empty((lib.ms_sample_scratch_bytes(rows),), dtype=torch.uint8, device="cuda")
        args = (logits.data_ptr(), rows, vocab, vocab, temperature.data_ptr(), top_p.data_ptr(), seeds.data_ptr(),
                counter.data_ptr())
        assert lib.ms_sample_rows(*args, scratch.data_ptr(), want.data_ptr(), stream) == 0
        torch.cuda.synchronize()
        if rows == most:  # a warm call: what the first launch of a kernel loads is no allocation of the entry point's
            assert lib.ms_sample_rows_static(*args, got.data_ptr(), stream) == 0
            torch.cuda.synchronize()
            got.fill_(-2)
            torch.cuda.synchronize()
        # neither torch's allocator (which a hipMalloc inside the library would pass by) nor the driver's count
        # of free bytes on the device may move across the call
        before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
        assert lib.ms_sample_rows_static(*args, got.data_ptr(), stream) == 0
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.cuda.mem_get_info()[0] == free_before, "device memory was taken or given back inside the call"
        assert got.tolist() == want.tolist(), f"{rows} rows of {vocab}"
        assert 0 <= min(got.tolist()) and max(got.tolist()) < vocab
        # all rows greedy (no parameters at all)
        assert lib.ms_sample_rows_static(logits.data_ptr(), rows, vocab, vocab, None, None, None, None, got.data_ptr(), stream) == 0
        torch.cuda.synchronize()
        assert got.tolist() == logits.argmax(dim=1).tolist()

    # beyond the maximum: refused with the "unsupported size" code, nothing is launched or written
    rows = most + 1
    logits = torch.zeros((rows, 64), dtype=torch.float32, device="cuda")
    got = torch.full((rows,), -2, dtype=torch.int32, device="cuda")
    assert lib.ms_sample_rows_static(logits.data_ptr(), rows, 64, 64, None, None, None, None, got.data_ptr(), stream) == 2
    torch.cuda.synchronize()
    assert set(got.tolist()) == {-2}
    with pytest.raises(ValueError, match="at most 256 rows"):
        ops.sample_rows_static(logits, got)
    # the Python call of the same entry point
    small = torch.randn((3, 100), device="cuda")
    out = torch.empty((3,), dtype=torch.int32, device="cuda")
    assert ops.sample_rows_static(small, out).tolist() == small.argmax(dim=1).tolist()
