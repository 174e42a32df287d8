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
            # an answer that no kernel of the library had a hand in (no ties beyond row 0's)
            assert got[1:].tolist() == torch.argmax(logits[1:], dim=1).tolist()


def test_static_argmax_at_the_edges_of_its_array_and_of_a_row():
    """On one stream, after a large call that fills the library's array: as many rows as the array holds
    (the last row's partial results lie at its very end), a strided view of wider rows, and a row shorter
    than the 64 slices it is cut into (most slices are empty). Checked against ``torch.argmax``."""
    K, lib, static = _calls()
    dev = "cuda:0"
    g = torch.Generator(device="cpu").manual_seed(6)
    with torch.cuda.device(dev):
        cases = []
        full = torch.randn(256, 3001, generator=g).to(dev)
        cases.append(full)
        wide = torch.randn(9, 700, generator=g).to(dev)
        cases.append(wide[:, :333])                              # rows 700 floats apart, 333 of them read
        wide[:, 333:] = 100.0                                    # what lies beyond a row's end must not win
        cases.append(torch.randn(5, 41, generator=g).to(dev))    # fewer columns than slices
        cases.append(torch.randn(2, 1, generator=g).to(dev))
        for logits in cases:
            rows, vocab = logits.shape
            got = torch.full((rows,), -1, dtype=torch.int32, device=dev)
            rc = static(logits.data_ptr(), logits.stride(0), got.data_ptr(), rows, vocab, _stream())
            assert rc == 0, lib.gl3_last_error().decode()
            torch.cuda.synchronize()
            assert got.tolist() == torch.argmax(logits, dim=1).tolist(), (rows, vocab)


def test_static_argmax_refuses_more_rows_than_its_array_holds():
    K, lib, static = _calls()
    with torch.cuda.device("cuda:0"):
        logits = torch.zeros(300, 16, device="cuda:0")
        out = torch.zeros(300, dtype=torch.int32, device="cuda:0")
        rc = static(logits.data_ptr(), logits.stride(0), out.data_ptr(), 300, 16, _stream())
        assert rc != 0 and "exceed" in lib.gl3_last_error().decode()
