"""The entry point that allocates nothing: ``gl3_argmax_static`` against ``gl3_argmax``.

Called through ``ctypes`` on the library's own handle, twice in a row, the second call with a
smaller input: the library's array keeps the first call's partial results, which the second
must not read.
"""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _calls():
    from gpullama3_java_amd.csrc import lib as K
    lib = K.library()
    static = lib.gl3_argmax_static
    static.argtypes = [ctypes.c_void_p, ctypes.c_long, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    static.restype = ctypes.c_int
    return K, lib, static


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def test_static_argmax_matches_the_workspace_one_on_two_calls_in_a_row():
    K, lib, static = _calls()
    dev = "cuda:0"
    g = torch.Generator(device="cpu").manual_seed(5)
    with torch.cuda.device(dev):
        for rows, vocab in ((37, 5003), (3, 257)):          # the second call is the smaller one
            logits = torch.randn(rows, vocab, generator=g).to(dev)
            # ties, and a greatest value in the last place of a row and in the first of another
            logits[0, 11] = logits[0, 97] = 9.0
            logits[1, vocab - 1] = 11.0
            logits[2, 0] = 12.0
            want = torch.empty(rows, dtype=torch.int32, device=dev)
            work = torch.empty(K.sample_work_size(rows, vocab), dtype=torch.float32, device=dev)
            K.argmax(logits, work, want)
            got = torch.full((rows,), -1, dtype=torch.int32, device=dev)
            rc = static(logits.data_ptr(), logits.stride(0), got.data_ptr(), rows, vocab, _stream())
            assert rc == 0, lib.gl3_last_error().decode()
            torch.cuda.synchronize()
            assert got.tolist() == want.tolist()
            assert got[0].item() == 11 and got[1].item() == vocab - 1 and got[2].item() == 0


def test_static_argmax_refuses_more_rows_than_its_array_holds():
    K, lib, static = _calls()
    with torch.cuda.device("cuda:0"):
        logits = torch.zeros(300, 16, device="cuda:0")
        out = torch.zeros(300, dtype=torch.int32, device="cuda:0")
        rc = static(logits.data_ptr(), logits.stride(0), out.data_ptr(), 300, 16, _stream())
        assert rc != 0 and "exceed" in lib.gl3_last_error().decode()
