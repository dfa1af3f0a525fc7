"""The entry point that allocates nothing (csrc/hip/no_alloc.h): arg-max over long
rows with its partial results in a file-scope array of device memory.  Called
through ctypes, twice in a row, the second time with fewer and shorter rows, so
that what the first call left in the array lies beside what the second one
writes; both are compared with the existing entry point (scratch from the
caller) and with torch."""
import ctypes
from ctypes import c_int, c_size_t, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu


def _lib():
    from llm_rs_amd.csrc.build import load_hip
    lib = load_hip()
    lib.llmrs_argmax_rows_static.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]
    lib.llmrs_argmax_rows_static.restype = c_int
    lib.llmrs_argmax_rows.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_size_t]
    lib.llmrs_argmax_rows.restype = c_int
    lib.llmrs_hip_error.restype = ctypes.c_char_p
    return lib


def _logits(rows, V, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn(rows, V, generator=g, device="cuda", dtype=torch.float32)
    # equal maxima in some rows: the lowest index must win in both entry points
    x[0, V - 3] = x[0, 5] = 9.0
    if rows > 2:
        x[2, V - 1] = 11.0
    return x


def test_argmax_rows_static_follows_argmax_rows():
    lib = _lib()
    stream = torch.cuda.current_stream().cuda_stream
    for rows, V, seed in ((37, 128256, 1), (5, 9001, 2)):      # the second call is smaller
        x = _logits(rows, V, seed)
        want = torch.empty(rows, dtype=torch.int32, device="cuda")
        got = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        caller_scratch = torch.empty(rows * 32 * 8, dtype=torch.uint8, device="cuda")
        rc = lib.llmrs_argmax_rows(stream, x.data_ptr(), x.stride(0), rows, V, want.data_ptr(),
                                   caller_scratch.data_ptr(), caller_scratch.numel())
        assert rc == 0, lib.llmrs_hip_error().decode()
        torch.cuda.synchronize()
        # the driver's own figure of free memory: it moves with any hipMalloc or hipFree, whoever calls it
        # (torch's counters see only what goes through torch's allocator)
        before = torch.cuda.mem_get_info()[0]
        rc = lib.llmrs_argmax_rows_static(stream, x.data_ptr(), x.stride(0), rows, V, got.data_ptr())
        assert rc == 0, lib.llmrs_hip_error().decode()
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == before
        assert torch.equal(got, want), (rows, V)
        first_max = (x == x.max(dim=1, keepdim=True).values).int().argmax(dim=1).to(torch.int32)
        assert torch.equal(got, first_max)


def test_argmax_rows_static_inside_a_recorded_graph():
    """The use the entry point is there for: one call with no rows before the recording (it looks the array's
    address up), then calls while a stream is being captured, where any allocation would end the capture with an
    error.  The graph is replayed on new logits, with other work and synchronisations between the replays, and
    every replay compared with the existing entry point."""
    lib = _lib()
    rows, V = 19, 50000
    x = _logits(rows, V, 5)
    got = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    want = torch.empty(rows, dtype=torch.int32, device="cuda")
    caller_scratch = torch.empty(rows * 32 * 8, dtype=torch.uint8, device="cuda")
    assert lib.llmrs_argmax_rows_static(torch.cuda.current_stream().cuda_stream, None, V, 0, V, None) == 0
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = lib.llmrs_argmax_rows_static(torch.cuda.current_stream().cuda_stream, x.data_ptr(), x.stride(0), rows, V, got.data_ptr())
    assert rc == 0, lib.llmrs_hip_error().decode()
    for replay in range(4):
        x.copy_(_logits(rows, V, 10 + replay))
        rc = lib.llmrs_argmax_rows(torch.cuda.current_stream().cuda_stream, x.data_ptr(), x.stride(0), rows, V, want.data_ptr(),
                                   caller_scratch.data_ptr(), caller_scratch.numel())
        assert rc == 0, lib.llmrs_hip_error().decode()
        got.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {replay}"


def test_argmax_rows_static_refuses_more_rows_than_its_array_holds():
    lib = _lib()
    stream = torch.cuda.current_stream().cuda_stream
    x = torch.zeros(8, 8192, device="cuda")
    out = torch.zeros(2048, dtype=torch.int32, device="cuda")
    assert lib.llmrs_argmax_rows_static(stream, x.data_ptr(), 0, 1025, 8192, out.data_ptr()) != 0   # ld < V is refused first
    rc = lib.llmrs_argmax_rows_static(stream, x.data_ptr(), 8192, 1025, 8192, out.data_ptr())
    assert rc != 0 and "1024" in lib.llmrs_hip_error().decode()
    torch.cuda.synchronize()
