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
