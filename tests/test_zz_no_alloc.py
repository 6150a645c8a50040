"""The entry point that allocates nothing (qe_argmax_static), called through ctypes as a caller
without torch's allocator would: its output equals qe_argmax's on two calls in a row, the second
with a smaller input, and sizes beyond its fixed buffer are refused with a clear error."""
import ctypes

import pytest
import torch

import qwen_engine_amd  # noqa: F401

pytestmark = pytest.mark.gpu


def _library():
    from qwen_engine_amd.kernels import build
    lib = ctypes.CDLL(str(build.library_path(verbose=False)))
    vp, i32, i64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_long
    lib.qe_argmax_static.argtypes = [vp, vp, i32, i32, vp]
    lib.qe_argmax_static.restype = i32
    lib.qe_argmax.argtypes = [vp, vp, i32, i32, vp, i64, vp]
    lib.qe_argmax.restype = i32
    lib.qe_argmax_workspace_bytes.argtypes = [i32, i32]
    lib.qe_argmax_workspace_bytes.restype = i64
    lib.qe_argmax_static_max_bytes.restype = i64
    lib.qe_last_error.restype = ctypes.c_char_p
    return lib


def test_argmax_without_allocation_equals_argmax_with_a_workspace():
    lib = _library()
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(12)
    stream = torch.cuda.current_stream().cuda_stream
    # every buffer exists before the calls: the entry point itself must not allocate
    cases = [(8, 151936), (3, 10007)]          # the second call is smaller and finds the first one's leftovers
    inputs = []
    for R, V in cases:
        logits = torch.randn(R, V, generator=g).to(dev)
        logits[0, V - 1] = 50.0                                      # the last column wins a row
        logits[R - 1, 4097] = logits[R - 1, 9000] = 60.0             # a tie across two spans: the lower index
        nbytes = lib.qe_argmax_workspace_bytes(R, V)
        assert 0 < nbytes <= lib.qe_argmax_static_max_bytes()        # (the path that uses the buffer)
        inputs.append((logits, torch.full((R,), -7, dtype=torch.int32, device=dev),
                       torch.full((R,), -7, dtype=torch.int32, device=dev),
                       torch.empty(nbytes, dtype=torch.uint8, device=dev), nbytes))
    # one call before the counts are taken: it asks for the address of this device's copy of the buffer,
    # once per process (whatever the runtime sets up for that is not the entry point's own allocation)
    warm = torch.zeros(2, 5000, device=dev)
    assert lib.qe_argmax_static(warm.data_ptr(), torch.empty(2, dtype=torch.int32, device=dev).data_ptr(), 2, 5000, stream) == 0
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(dev)
    free_before = torch.cuda.mem_get_info(dev)[0]        # the driver's count of free bytes: sees a hipMalloc that torch's count cannot
    for (R, V), (logits, got, want, ws, nbytes) in zip(cases, inputs):
        rc = lib.qe_argmax_static(logits.data_ptr(), got.data_ptr(), R, V, stream)
        assert rc == 0, lib.qe_last_error().decode()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(dev)[0] == free_before
    assert torch.cuda.memory_allocated(dev) == before
    for (R, V), (logits, got, want, ws, nbytes) in zip(cases, inputs):
        rc = lib.qe_argmax(logits.data_ptr(), want.data_ptr(), R, V, ws.data_ptr(), nbytes, stream)
        assert rc == 0, lib.qe_last_error().decode()
    torch.cuda.synchronize()
    for (R, V), (logits, got, want, _, _) in zip(cases, inputs):
        assert got.tolist() == want.tolist()
        assert got.tolist() == logits.argmax(dim=1).tolist()
        assert got[0].item() == V - 1 and got[R - 1].item() == 4097
    # a narrow vocabulary needs no buffer at all
    small = torch.randn(5, 300, generator=g).to(dev)
    out = torch.empty(5, dtype=torch.int32, device=dev)
    assert lib.qe_argmax_static(small.data_ptr(), out.data_ptr(), 5, 300, stream) == 0
    torch.cuda.synchronize()
    assert out.tolist() == small.argmax(dim=1).tolist()


def test_sizes_beyond_the_fixed_buffer_are_refused():
    lib = _library()
    dev = torch.device("cuda:0")
    R, V = 437, 151936                       # 437 * 75 spans * 8 bytes is just over 256 KiB
    assert lib.qe_argmax_workspace_bytes(R, V) > lib.qe_argmax_static_max_bytes()
    assert lib.qe_argmax_workspace_bytes(R - 1, V) <= lib.qe_argmax_static_max_bytes()
    logits = torch.zeros(1, dtype=torch.float32, device=dev)     # never read: the call is refused on the host
    out = torch.full((R,), -7, dtype=torch.int32, device=dev)
    rc = lib.qe_argmax_static(logits.data_ptr(), out.data_ptr(), R, V, torch.cuda.current_stream().cuda_stream)
    assert rc == -1
    msg = lib.qe_last_error().decode()
    assert "static buffer" in msg and "437" in msg
    torch.cuda.synchronize()
    assert out.tolist() == [-7] * R


def test_argmax_without_allocation_inside_a_graph_capture():
    """Under stream capture an allocation is an error of the capture; the entry point records its two
    kernels and nothing else.  Replayed three times with other logits and the program's own work between
    the replays, each replay against the eager result."""
    lib = _library()
    dev = torch.device("cuda:0")
    R, V = 8, 151936
    g = torch.Generator().manual_seed(13)
    logits = torch.randn(R, V, generator=g).to(dev)
    out = torch.full((R,), -7, dtype=torch.int32, device=dev)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        assert lib.qe_argmax_static(logits.data_ptr(), out.data_ptr(), R, V, stream.cuda_stream) == 0   # (the address is known now)
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        rc = lib.qe_argmax_static(logits.data_ptr(), out.data_ptr(), R, V, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.qe_last_error().decode()
    for rep in range(3):
        logits.copy_(torch.randn(R, V, generator=g))
        out.fill_(-7)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert out.tolist() == logits.argmax(dim=1).tolist(), rep
