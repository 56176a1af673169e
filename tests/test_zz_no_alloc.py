"""The sampling entry point that allocates nothing (``psamd_sample_static``), called through
ctypes as a caller without torch would, against the entry point that takes a scratch buffer."""

from __future__ import annotations

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _lib():
    from prefixserve_amd.build import ensure_kernels

    lib = ensure_kernels()
    vp, i32 = ctypes.c_void_p, ctypes.c_int
    lib.psamd_sample.argtypes = [vp, vp, vp, vp, vp, vp, i32, i32]
    lib.psamd_sample.restype = i32
    lib.psamd_sample_static.argtypes = [vp, vp, vp, vp, vp, i32, i32]
    lib.psamd_sample_static.restype = i32
    lib.psamd_sample_static_max_rows.argtypes = []
    lib.psamd_sample_static_max_rows.restype = i32
    lib.psamd_sample_scratch_floats.argtypes = [i32]
    lib.psamd_sample_scratch_floats.restype = ctypes.c_int64
    lib.psamd_last_error.restype = ctypes.c_char_p
    return lib


def _inputs(rows: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(rows, vocab, generator=g) * 3.0).to(DEV)
    temps = torch.tensor([0.0, 0.8, 1.3][:1] * rows, dtype=torch.float32)
    temps[1::3] = 0.8
    temps[2::3] = 1.3
    us = torch.rand(rows, generator=g)
    return logits, temps.to(DEV), us.to(DEV)


def test_sampling_without_allocation_equals_sampling_with_a_buffer():
    lib = _lib()
    assert lib.psamd_sample_static_max_rows() == 256
    stream = torch.cuda.current_stream(DEV).cuda_stream
    # The first call on a device looks up the array's address there; it is made here, before
    # anything is measured, as a caller would make it at set-up.
    logits, temps, us = _inputs(2, 2048, 0)
    first = torch.empty(2, dtype=torch.int32, device=DEV)
    assert lib.psamd_sample_static(stream, logits.data_ptr(), temps.data_ptr(), us.data_ptr(), first.data_ptr(), 2, 2048) == 0
    torch.cuda.synchronize()
    # Two calls in a row share the library's array; the second is smaller in rows and vocabulary,
    # so it must not read what the first left behind.
    for rows, vocab, seed in ((200, 50021, 1), (7, 3001, 2)):
        logits, temps, us = _inputs(rows, vocab, seed)
        want = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        got = torch.full((rows,), -2, dtype=torch.int32, device=DEV)
        scratch = torch.empty(int(lib.psamd_sample_scratch_floats(rows)), dtype=torch.float32, device=DEV)
        torch.cuda.synchronize()
        rc = lib.psamd_sample(stream, logits.data_ptr(), temps.data_ptr(), us.data_ptr(), want.data_ptr(),
                              scratch.data_ptr(), rows, vocab)
        assert rc == 0, lib.psamd_last_error().decode()
        torch.cuda.synchronize()
        # The driver's own count of free bytes on the device: it sees an allocation by anybody
        # (hipMalloc in the library, torch's allocator), which torch's statistics would not.
        free_before = torch.cuda.mem_get_info(DEV)[0]
        reserved_before = torch.cuda.memory_reserved(DEV)
        rc = lib.psamd_sample_static(stream, logits.data_ptr(), temps.data_ptr(), us.data_ptr(), got.data_ptr(),
                                     rows, vocab)
        assert rc == 0, lib.psamd_last_error().decode()
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info(DEV)[0] == free_before and torch.cuda.memory_reserved(DEV) == reserved_before
        assert torch.equal(got, want), (rows, vocab)
        assert int(got.min()) >= 0 and int(got.max()) < vocab
        greedy = torch.argmax(logits[0::3], dim=-1).to(torch.int32)
        assert torch.equal(got[0::3], greedy)


def test_sampling_without_allocation_under_graph_capture():
    """One of the callers it is for: the call recorded into a graph (after one call outside any
    capture, which looks up the array's address), replayed with other work between the replays
    and with new inputs in the same buffers; every replay equals the entry point with a buffer."""
    lib = _lib()
    rows, vocab = 33, 10007
    logits, temps, us = _inputs(rows, vocab, 5)
    got = torch.full((rows,), -2, dtype=torch.int32, device=DEV)
    stream = torch.cuda.current_stream(DEV).cuda_stream
    assert lib.psamd_sample_static(stream, logits.data_ptr(), temps.data_ptr(), us.data_ptr(), got.data_ptr(), rows, vocab) == 0
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        inner = torch.cuda.current_stream(DEV).cuda_stream
        rc = lib.psamd_sample_static(inner, logits.data_ptr(), temps.data_ptr(), us.data_ptr(), got.data_ptr(), rows, vocab)
    assert rc == 0, lib.psamd_last_error().decode()
    scratch = torch.empty(int(lib.psamd_sample_scratch_floats(rows)), dtype=torch.float32, device=DEV)
    want = torch.empty(rows, dtype=torch.int32, device=DEV)
    for seed in (6, 7, 8):
        new_logits, _t, new_us = _inputs(rows, vocab, seed)
        logits.copy_(new_logits)
        us.copy_(new_us)
        got.fill_(-2)
        graph.replay()
        stream = torch.cuda.current_stream(DEV).cuda_stream
        assert lib.psamd_sample(stream, logits.data_ptr(), temps.data_ptr(), us.data_ptr(), want.data_ptr(),
                                scratch.data_ptr(), rows, vocab) == 0
        torch.cuda.synchronize()
        assert torch.equal(got, want), seed


def test_sampling_without_allocation_refuses_more_rows_than_its_array_holds():
    lib = _lib()
    rows, vocab = 257, 64
    logits, temps, us = _inputs(rows, vocab, 3)
    out = torch.full((rows,), -3, dtype=torch.int32, device=DEV)
    stream = torch.cuda.current_stream(DEV).cuda_stream
    rc = lib.psamd_sample_static(stream, logits.data_ptr(), temps.data_ptr(), us.data_ptr(), out.data_ptr(), rows, vocab)
    assert rc != 0 and b"256" in lib.psamd_last_error()
    torch.cuda.synchronize()
    assert int(out.max()) == -3        # nothing was launched
