"""The entry point that allocates nothing (`xi_argmax_static`, csrc/kernels/no_alloc.h), called
through ctypes as a caller without torch would, against `xi_argmax`, the entry point it is a
variant of.  Two calls in a row, the second with a smaller input: the fixed scratch keeps the
first call's contents, which must not show in the second."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from xinfer_amd.csrc.build import build_kernels
    lib = ctypes.CDLL(build_kernels())
    lib.xi_last_error.restype = ctypes.c_char_p
    lib.xi_argmax_static.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    lib.xi_argmax.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                              ctypes.c_void_p, ctypes.c_void_p]
    return lib


def _both(lib, logits):
    """(static entry point's result, existing entry point's result) for float32 [rows, V] logits."""
    rows, V = logits.shape
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out_static = torch.full((rows,), -7, dtype=torch.int32, device=logits.device)
    out_plain = torch.full((rows,), -9, dtype=torch.int32, device=logits.device)
    chunks = int(lib.xi_argmax_chunks(V))
    pval = torch.empty((rows, chunks), dtype=torch.float32, device=logits.device)
    pidx = torch.empty((rows, chunks), dtype=torch.int32, device=logits.device)
    torch.cuda.synchronize()
    rc = lib.xi_argmax_static(logits.data_ptr(), rows, V, out_static.data_ptr(), stream)
    assert rc == 0, lib.xi_last_error().decode()
    rc = lib.xi_argmax(logits.data_ptr(), rows, V, out_plain.data_ptr(), pval.data_ptr(), pidx.data_ptr(), stream)
    assert rc == 0, lib.xi_last_error().decode()
    torch.cuda.synchronize()
    return out_static.cpu(), out_plain.cpu()


def test_static_argmax_equals_argmax_on_two_calls_in_a_row():
    lib = _library()
    dev = torch.device("cuda:0")
    gen = torch.Generator(device="cpu").manual_seed(11)
    # first call: many rows of a large vocabulary (32 chunks a row), the winners placed in late chunks
    big = torch.randn((48, 151936), generator=gen, dtype=torch.float32)
    for r in range(48):
        big[r, 151936 - 1 - 37 * r] = 50.0 + r
    # second call: fewer rows, a smaller vocabulary that still takes the two-stage form, the
    # winners early and twice in a row (the lower index wins); what the first call left in the
    # scratch (large values, late indices) would win every comparison if it were read
    small = torch.randn((5, 20011), generator=gen, dtype=torch.float32)
    for r in range(5):
        small[r, 3 + r] = 9.0
        small[r, 9000 + r] = 9.0
    got, want = _both(lib, big.to(dev))
    assert torch.equal(got, want), (got, want)
    assert got.tolist() == [151936 - 1 - 37 * r for r in range(48)]
    got, want = _both(lib, small.to(dev))
    assert torch.equal(got, want), (got, want)
    assert got.tolist() == [3, 4, 5, 6, 7]
    # the one-stage form (small vocabularies) uses no scratch and goes the same way
    tiny = torch.randn((7, 509), generator=gen, dtype=torch.float32)
    got, want = _both(lib, tiny.to(dev))
    assert torch.equal(got, want) and torch.equal(got.long(), tiny.argmax(dim=1))


def test_static_argmax_refuses_sizes_beyond_its_scratch():
    lib = _library()
    most = int(lib.xi_argmax_static_max_rows())
    assert most == 256
    dev = torch.device("cuda:0")
    logits = torch.zeros((most + 1, 16384), dtype=torch.float32, device=dev)
    out = torch.zeros((most + 1,), dtype=torch.int32, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.xi_argmax_static(logits.data_ptr(), most + 1, 16384, out.data_ptr(), stream)
    assert rc != 0 and "more than" in lib.xi_last_error().decode()
    # the largest size it takes
    logits[:, 16000] = 1.0
    rc = lib.xi_argmax_static(logits.data_ptr(), most, 16384, out.data_ptr(), stream)
    assert rc == 0, lib.xi_last_error().decode()
    torch.cuda.synchronize()
    assert out[:most].tolist() == [16000] * most


def test_static_argmax_recorded_in_a_graph():
    """After `xi_argmax_static_init` (outside the capture) the two-stage form is recorded into a HIP
    graph, which holds two kernels and no memset, and replayed with other logits in place, with
    eager work between the replays; every replay against `xi_argmax`."""
    lib = _library()
    dev = torch.device("cuda:0")
    assert lib.xi_argmax_static_init() == 0, lib.xi_last_error().decode()
    gen = torch.Generator(device="cpu").manual_seed(12)
    rows, V = 9, 151936
    logits = torch.randn((rows, V), generator=gen, dtype=torch.float32).to(dev)
    out = torch.full((rows,), -1, dtype=torch.int32, device=dev)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):                 # (the capture runs on a stream of its own)
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = lib.xi_argmax_static(logits.data_ptr(), rows, V, out.data_ptr(), stream)
    assert rc == 0, lib.xi_last_error().decode()
    for k in range(3):
        fresh = torch.randn((rows, V), generator=gen, dtype=torch.float32)
        fresh[k, V - 1 - k] = 40.0
        logits.copy_(fresh.to(dev))
        out.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        _, want = _both(lib, logits)              # eager calls of both entry points between the replays
        assert torch.equal(out.cpu(), want) and int(out[k]) == V - 1 - k, k
