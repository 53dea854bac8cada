"""The arg-max entry point that allocates nothing (``rl_argmax_static``), called through
``ctypes`` as a caller without an allocator would, against the arg-max the engine uses."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _lib():
    from rapid_llm_amd.kernels import build

    lib = build.load(build.core_library())
    lib.rl_argmax_static.restype = ctypes.c_int
    lib.rl_argmax_static.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                     ctypes.c_int, ctypes.c_void_p]
    return lib


def _call(lib, logits, out, row_index=None):
    stream = torch.cuda.current_stream().cuda_stream
    return lib.rl_argmax_static(
        logits.data_ptr(), 0 if row_index is None else row_index.data_ptr(), out.data_ptr(),
        out.shape[0], logits.shape[1], stream,
    )


def test_two_calls_in_a_row_match_the_engines_arg_max():
    from rapid_llm_amd.kernels import ops

    lib = _lib()
    assert lib.rl_argmax_static_prepare() == 0
    gen = torch.Generator().manual_seed(3)
    # the second call is smaller in both directions: what the first left in the array
    # (more rows, more slices per row) must not reach its result
    for rows, vocab in ((48, 151936), (5, 9001)):
        logits = torch.randn((rows, vocab), generator=gen).cuda()
        logits[1, vocab - 1] = 50.0  # the last column of the last slice
        logits[2, 4096] = logits[2, 4095] = 60.0  # equal maxima across a slice's edge: the lower index
        want = torch.empty(rows, dtype=torch.int32, device="cuda")
        ops.argmax(logits, want)
        got = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        assert _call(lib, logits, got) == 0
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        assert torch.equal(got.cpu().long(), logits.cpu().argmax(dim=1))
        assert got[1] == vocab - 1 and got[2] == 4095
        # rows chosen through an index, as the sampler passes them
        index = torch.tensor([rows - 1, 0, 2], dtype=torch.int32, device="cuda")
        got3 = torch.full((3,), -1, dtype=torch.int32, device="cuda")
        assert _call(lib, logits, got3, index) == 0
        torch.cuda.synchronize()
        assert torch.equal(got3, want[index.long()])


def test_sizes_beyond_the_array_are_refused():
    lib = _lib()
    limit = lib.rl_argmax_static_limit()
    vocab = 151936
    slices = -(-vocab // 4096)
    rows = limit // slices + 1
    logits = torch.zeros((rows, vocab), device="cuda")
    out = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
    assert _call(lib, logits, out) == 1  # an argument the entry point refuses; nothing ran
    torch.cuda.synchronize()
    assert (out == -7).all()
    ok_rows = limit // slices
    assert _call(lib, logits[:ok_rows], out[:ok_rows]) == 0
    torch.cuda.synchronize()
    assert (out[:ok_rows] == 0).all()


def test_it_runs_under_graph_capture_and_leaves_the_devices_memory_as_it_was():
    """What the entry point is for: after ``rl_argmax_static_prepare()`` a call may be recorded
    into a HIP graph (an allocation, or the lookup of the array's address, would fail the
    capture), and eager calls change nothing in the device's free memory.  The graph is replayed
    several times with other logits and eager work in between; every replay must be right."""
    lib = _lib()
    assert lib.rl_argmax_static_prepare() == 0
    gen = torch.Generator().manual_seed(5)
    rows, vocab = 6, 9001
    logits = torch.randn((rows, vocab), generator=gen).cuda()
    out = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    assert _call(lib, logits, out) == 0  # the kernels' code is loaded before anything is measured
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        assert _call(lib, logits, out) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.equal(out.cpu().long(), logits.cpu().argmax(dim=1))

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        code = _call(lib, logits, out)  # the current stream is the capturing one
    assert code == 0
    for _ in range(3):
        fresh = torch.randn((rows, vocab), generator=gen)
        logits.copy_(fresh.cuda())
        out.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.cpu().long(), fresh.argmax(dim=1))
