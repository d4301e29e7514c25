"""The argmax entry point that allocates nothing (dlgo_argmax_noalloc), called through ctypes as a caller
that cannot allocate would, against the entry point that takes its scratch as an argument."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

NOALLOC_ROWS = 256     # DLGO_ARGMAX_NOALLOC_ROWS of csrc/sampling.h


def _entry_points():
    from dlgo_amd.kernels import build
    lib = build.load("sampling")
    lib.dlgo_argmax.restype = ctypes.c_char_p
    lib.dlgo_argmax_noalloc.restype = ctypes.c_char_p
    lib.dlgo_argmax_noalloc_init.restype = ctypes.c_char_p
    return lib


def _with_scratch(lib, logits, stream):
    n, v = logits.shape
    scratch = torch.empty(max(n, 1) * 512, dtype=torch.uint8, device=logits.device)
    out = torch.full((n,), -7, dtype=torch.int32, device=logits.device)
    err = lib.dlgo_argmax(ctypes.c_void_p(logits.data_ptr()), logits.stride(0), n, v, ctypes.c_void_p(scratch.data_ptr()),
                          ctypes.c_longlong(scratch.numel()), ctypes.c_void_p(out.data_ptr()), stream)
    assert err is None, err
    return out


def _without(lib, logits, out, stream):
    n, v = logits.shape
    return lib.dlgo_argmax_noalloc(ctypes.c_void_p(logits.data_ptr()), logits.stride(0), n, v, ctypes.c_void_p(out.data_ptr()), stream)


def test_argmax_without_allocation_matches_on_two_calls_in_a_row():
    lib = _entry_points()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    g = torch.Generator(device="cpu").manual_seed(11)
    # the second call is smaller in rows and in width: what the first left in the array must not show
    shapes = [(37, 5003), (5, 517)]
    inputs = [torch.randn(s, generator=g).to(dev) for s in shapes]
    inputs[0][3, 4999] = 50.0           # a maximum in the row's last, short chunk
    inputs[1][2, 0] = 50.0
    inputs[1][4, 100] = inputs[1][4, 300] = 60.0     # a tie: the first index wins
    outs = [torch.full((s[0],), -7, dtype=torch.int32, device=dev) for s in shapes]
    assert lib.dlgo_argmax_noalloc_init() is None          # the array's address on this device: asked once, here
    torch.cuda.synchronize()
    # what the device itself says is free, not torch's own count: a hipMalloc inside the entry point would show here
    before_torch, (before_free, _) = torch.cuda.memory_allocated(dev), torch.cuda.mem_get_info(dev)
    for x, o in zip(inputs, outs):
        err = _without(lib, x, o, stream)
        assert err is None, err
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before_torch
    assert torch.cuda.mem_get_info(dev)[0] == before_free
    for x, o in zip(inputs, outs):
        want = _with_scratch(lib, x, stream)
        torch.cuda.synchronize()
        assert torch.equal(o, want)
        assert torch.equal(o.cpu().long(), x.cpu().argmax(dim=1))
    assert outs[0][3].item() == 4999 and outs[1][2].item() == 0 and outs[1][4].item() == 100


def test_argmax_without_allocation_refuses_what_exceeds_its_array():
    lib = _entry_points()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    x = torch.zeros((NOALLOC_ROWS + 1, 64), device=dev)
    out = torch.zeros(NOALLOC_ROWS + 1, dtype=torch.int32, device=dev)
    err = _without(lib, x, out, stream)
    assert err is not None and b"at most 256 rows" in err
    full = torch.randn((NOALLOC_ROWS, 64), device=dev)
    err = _without(lib, full, out[:NOALLOC_ROWS], stream)
    assert err is None, err
    torch.cuda.synchronize()
    assert torch.equal(out[:NOALLOC_ROWS].cpu().long(), full.cpu().argmax(dim=1))


def test_argmax_without_allocation_under_capture():
    """The use its header names: recorded into a HIP graph (after one call outside any capture, which resolves the
    array's address), then replayed several times with other work and waits between the replays; every replay gives
    what the entry point with a scratch argument gives for the logits of that moment."""
    lib = _entry_points()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    assert lib.dlgo_argmax_noalloc_init() is None
    g = torch.Generator(device="cpu").manual_seed(5)
    x = torch.randn((9, 4001), generator=g).to(dev)
    out = torch.full((9,), -7, dtype=torch.int32, device=dev)
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        err = _without(lib, x, out, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert err is None, err
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for replay in range(4):
        x.copy_(torch.randn((9, 4001), generator=g))
        x[replay, 4000 - replay] = 40.0
        other = _with_scratch(lib, torch.randn((300, 700), generator=g).to(dev), stream)      # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = _with_scratch(lib, x, stream)
        torch.cuda.synchronize()
        assert torch.equal(out, want) and out[replay].item() == 4000 - replay and other.shape == (300,)
