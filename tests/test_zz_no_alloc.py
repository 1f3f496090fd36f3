"""The entry point that allocates nothing (csrc/no_alloc.h): ptl_argmax_static, called through
ctypes as a caller without torch's wrappers would, against ptl_argmax with a workspace from
the caller: two calls in a row, the second with a smaller input, so that what the first call
left in the library's own array must not show."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _lib():
    from pytriton_llama_amd.ops import library
    lib = library.load("sampling")
    lib.ptl_argmax_static.restype = ctypes.c_int
    lib.ptl_argmax.restype = ctypes.c_int
    return lib


def _ptr(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _existing(lib, logits):
    R, V = logits.shape
    chunks = -(-V // 4096)
    out = torch.full((R,), -7, dtype=torch.int32, device=logits.device)
    ws_val = torch.empty((R, chunks), dtype=torch.float32, device=logits.device)
    ws_idx = torch.empty((R, chunks), dtype=torch.int32, device=logits.device)
    rc = lib.ptl_argmax(_ptr(out), _ptr(logits), R, V, ctypes.c_long(logits.stride(0)),
                        _ptr(ws_val), _ptr(ws_idx), None, _stream())
    assert rc == 0
    return out


def _static(lib, logits, out):
    R, V = logits.shape
    return lib.ptl_argmax_static(_ptr(out), _ptr(logits), R, V, ctypes.c_long(logits.stride(0)),
                                 None, _stream())


def test_argmax_static_matches_argmax_on_two_calls_in_a_row(gpu_device):
    lib = _lib()
    g = torch.Generator().manual_seed(5)
    big = torch.randn((48, 128256), generator=g).to(gpu_device)
    big[3, 100000] = 50.0                       # a far maximum, in the last chunks
    big[4, 17] = big[4, 90000] = 60.0           # a tie: the lower index wins
    big[5, 5] = float("nan")
    small = torch.randn((5, 9001), generator=g).to(gpu_device)     # three chunks, the last one short
    small[0, 9000] = 40.0                       # the very last logit
    small[1, 4096] = 40.0                       # first logit of the second chunk
    for logits in (big, small):                 # the second call is the smaller one
        out = torch.full((logits.shape[0],), -7, dtype=torch.int32, device=gpu_device)
        assert _static(lib, logits, out) == 0
        want = _existing(lib, logits)
        torch.cuda.synchronize()
        assert torch.equal(out.cpu(), want.cpu())
        ref = torch.nan_to_num(logits, nan=float("-inf")).argmax(dim=-1).to(torch.int32)
        assert torch.equal(out.cpu(), ref.cpu())
    assert int(out[0]) == 9000 and int(out[1]) == 4096
    # a strided view of a wider buffer, and the choices written to pinned host memory as well
    wide = torch.randn((6, 20000), generator=g).to(gpu_device)
    view = wide[:, :12345]
    out = torch.empty((6,), dtype=torch.int32, device=gpu_device)
    host = torch.full((6,), -1, dtype=torch.int32).pin_memory()
    rc = lib.ptl_argmax_static(_ptr(out), _ptr(view), 6, 12345, ctypes.c_long(view.stride(0)),
                               ctypes.c_void_p(host.data_ptr()), _stream())
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), view.argmax(dim=-1).to(torch.int32).cpu())
    assert torch.equal(host, out.cpu())


def test_argmax_static_refuses_what_exceeds_its_array(gpu_device):
    lib = _lib()
    out = torch.full((8,), -7, dtype=torch.int32, device=gpu_device)
    logits = torch.zeros((8, 16), dtype=torch.float32, device=gpu_device)
    # 16,384 partial results at most: 513 rows of 128,256 logits (32 chunks a row) are too many,
    # and so is one row of 70 million; nothing is launched and ``out`` stays as it was
    assert lib.ptl_argmax_static(_ptr(out), _ptr(logits), 513, 128256, ctypes.c_long(128256), None,
                                 _stream()) == -1
    assert lib.ptl_argmax_static(_ptr(out), _ptr(logits), 1, 70_000_000, ctypes.c_long(70_000_000),
                                 None, _stream()) == -1
    assert lib.ptl_argmax_static(_ptr(out), _ptr(logits), 8, 16, ctypes.c_long(8), None, _stream()) == -1
    assert lib.ptl_argmax_static(None, _ptr(logits), 8, 16, ctypes.c_long(16), None, _stream()) == -1
    torch.cuda.synchronize()
    assert out.cpu().eq(-7).all()
    assert lib.ptl_argmax_static(_ptr(out), _ptr(logits), 8, 16, ctypes.c_long(16), None, _stream()) == 0
    torch.cuda.synchronize()
    assert out.cpu().eq(0).all()                 # all equal: the lowest index


def test_argmax_static_recorded_into_a_graph(gpu_device):
    """For callers under graph capture: after ptl_argmax_static_init (the look-up of the
    library's array is no work for a capturing stream) the call is recorded into a HIP graph and
    replayed on two different inputs, with eager work in between; every replay gives what the
    existing entry point gives."""
    lib = _lib()
    lib.ptl_argmax_static_init.restype = ctypes.c_int
    assert lib.ptl_argmax_static_init() == 0
    g = torch.Generator().manual_seed(8)
    logits = torch.zeros((7, 50000), dtype=torch.float32, device=gpu_device)
    out = torch.full((7,), -7, dtype=torch.int32, device=gpu_device)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        assert _static(lib, logits, out) == 0                  # (warm-up on the side stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = _static(lib, logits, out)
    assert rc == 0
    for seed in (1, 2, 3):
        fresh = torch.randn((7, 50000), generator=g).to(gpu_device)
        fresh[seed, 49999 - seed] = 30.0
        logits.copy_(fresh)
        out.fill_(-7)
        graph.replay()
        torch.cuda.synchronize()
        want = _existing(lib, logits)                          # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(out.cpu(), want.cpu()) and int(out[seed]) == 49999 - seed
