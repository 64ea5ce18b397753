"""The greedy choice through the entry point that allocates nothing (``hfa_argmax_static``, called
through ctypes with raw device pointers) against ``hfa_argmax`` with a workspace: two calls in a row,
the second with fewer and shorter rows, so that what the first call left in the library's own buffer
lies beside and behind what the second one writes; and the refusal of more rows than the buffer holds."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(lib, ops, logits):
    rows, vocab = logits.shape
    out = torch.full((rows,), -7, dtype=torch.int32, device=logits.device)
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.hfa_argmax_static(ctypes.c_void_p(logits.data_ptr()), logits.stride(0), ctypes.c_void_p(out.data_ptr()),
                               rows, vocab, ctypes.c_void_p(stream))
    assert rc == 0, lib.hfa_last_error().decode()
    want = ops.argmax(logits)
    torch.cuda.synchronize()
    return out.cpu().numpy(), want.cpu().numpy()


def _static(lib, logits, out):
    return lib.hfa_argmax_static(ctypes.c_void_p(logits.data_ptr()), logits.stride(0), ctypes.c_void_p(out.data_ptr()),
                                 logits.shape[0], logits.shape[1], ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))


def test_argmax_static_inside_a_captured_graph():
    """The first call on a device resolves the address of the library's own buffer, which is no stream
    operation: made under a capture it is refused with a message that says what to do (in a process that
    has already called it eagerly the address is known and the call is simply recorded). After one eager
    call the entry point is captured into a graph, and the graph is replayed on changed logits with eager
    work of the program between the replays; every replay gives what hfa_argmax gives."""
    from hf_cpu_amd.kernels import Ops
    from hf_cpu_amd.kernels.lib import library
    ops = Ops(torch.float32)
    lib = library()
    g = torch.Generator(device="cpu").manual_seed(5)
    logits = torch.randn((12, 5001), generator=g).cuda()
    out = torch.full((12,), -7, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    cold = torch.cuda.CUDAGraph()
    with torch.cuda.graph(cold):
        rc = _static(lib, logits, out)
    if rc != 0:
        msg = lib.hfa_last_error().decode()
        assert "eagerly" in msg and "captured" in msg
    del cold
    assert _static(lib, logits, out) == 0, lib.hfa_last_error().decode()          # the eager call
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), logits.cpu().numpy().argmax(axis=1))
    graph = torch.cuda.CUDAGraph()
    out.fill_(-7)
    with torch.cuda.graph(graph):
        rc = _static(lib, logits, out)
    assert rc == 0, lib.hfa_last_error().decode()
    for i in range(3):
        fresh = torch.randn((12, 5001), generator=g)
        fresh[i, 4000 + i] = 50.0
        logits.copy_(fresh.cuda())
        want = ops.argmax(logits).cpu().numpy()            # eager work and a synchronisation between the replays
        graph.replay()
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        assert np.array_equal(got, want) and got[i] == 4000 + i, f"replay {i}"


def test_argmax_static_matches_argmax_on_two_calls_in_a_row():
    from hf_cpu_amd.kernels import Ops
    from hf_cpu_amd.kernels.lib import library
    ops = Ops(torch.float32)
    lib = library()
    g = torch.Generator(device="cpu").manual_seed(11)
    big = torch.randn((64, 152064), generator=g).cuda()
    big[3, 100:5000] = big[3].max() + 1.0            # a long tie: the lowest id wins
    big[7, -1] = 1e9                                 # the last column of the last slice
    got, want = _both(lib, ops, big)
    assert np.array_equal(got, want)
    assert got[3] == 100 and got[7] == 152063
    assert np.array_equal(got, big.cpu().numpy().argmax(axis=1))
    small = torch.randn((5, 1000), generator=g).cuda()[:, :777]       # rows with a stride, a vocabulary that is no power of two
    got, want = _both(lib, ops, small)
    assert np.array_equal(got, want)
    assert np.array_equal(got, small.cpu().numpy().argmax(axis=1))
    got, want = _both(lib, ops, big[:9])             # and the first call's rows again
    assert np.array_equal(got, want)


def test_argmax_static_refuses_more_rows_than_its_buffer_holds():
    from hf_cpu_amd.kernels.lib import library
    lib = library()
    x = torch.zeros((300, 8), device="cuda")
    out = torch.zeros((300,), dtype=torch.int32, device="cuda")
    rc = lib.hfa_argmax_static(ctypes.c_void_p(x.data_ptr()), 8, ctypes.c_void_p(out.data_ptr()), 300, 8, None)
    assert rc != 0 and "256" in lib.hfa_last_error().decode()
