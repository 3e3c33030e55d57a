"""shk_argmax_static, the argmax entry point that allocates nothing (its chunk
results live in an array the library holds on the GPU), called through ctypes
and compared with shk_argmax on two calls in a row, the second with a smaller
input; sizes beyond the array are refused."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from shrike_amd.csrc.build import ensure_built

    lib = ctypes.CDLL(str(ensure_built()))
    P, I = ctypes.c_void_p, ctypes.c_int
    lib.shk_argmax_static.argtypes = [P, P, I, I, I, P]
    lib.shk_argmax_static.restype = I
    lib.shk_argmax.argtypes = [P, P, I, I, I, P, P]
    lib.shk_argmax.restype = I
    lib.shk_argmax_scratch_floats.argtypes = [I, I]
    lib.shk_argmax_scratch_floats.restype = I
    lib.shk_argmax_static_max_floats.argtypes = []
    lib.shk_argmax_static_max_floats.restype = I
    lib.shk_last_error.restype = ctypes.c_char_p
    return lib


def test_argmax_from_the_library_s_own_scratch_equals_argmax_with_a_workspace():
    lib = _library()
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    gen = torch.Generator(device="cpu").manual_seed(3)
    stream = torch.cuda.current_stream().cuda_stream
    # the second call is smaller in rows and in width: it finds the first call's
    # chunk results in the array and must not read them
    for rows, vocab in [(37, 152064), (5, 50001)]:
        logits = torch.randn(rows, vocab, generator=gen).to(device)
        # equal maxima: the lowest index wins in both entry points
        logits[0, 4095] = logits[0, 4096] = logits[0, vocab - 1] = 50.0
        logits[rows - 1, vocab - 1] = 60.0
        need = lib.shk_argmax_scratch_floats(rows, vocab)
        assert 0 < need <= lib.shk_argmax_static_max_floats()
        workspace = torch.empty(need, dtype=torch.float32, device=device)
        want = torch.full((rows,), -1, dtype=torch.int32, device=device)
        got = torch.full((rows,), -2, dtype=torch.int32, device=device)
        rc = lib.shk_argmax(logits.data_ptr(), want.data_ptr(), rows, vocab, logits.stride(0),
                            workspace.data_ptr(), stream)
        assert rc == 0, lib.shk_last_error().decode()
        before = torch.cuda.memory_allocated(device)
        rc = lib.shk_argmax_static(logits.data_ptr(), got.data_ptr(), rows, vocab, logits.stride(0),
                                   stream)
        assert rc == 0, lib.shk_last_error().decode()
        torch.cuda.synchronize(device)
        assert torch.cuda.memory_allocated(device) == before
        assert torch.equal(got, want)
        assert torch.equal(got.cpu().long(), logits.cpu().argmax(dim=1))
        assert int(got[0]) == 4095 and int(got[rows - 1]) == vocab - 1


def test_sizes_beyond_the_array_are_refused():
    lib = _library()
    device = torch.device("cuda:0")
    limit = lib.shk_argmax_static_max_floats()
    vocab = 152064
    rows = limit // lib.shk_argmax_scratch_floats(1, vocab) + 1
    logits = torch.zeros(1, vocab, device=device)  # never read: the call is refused on the host
    out = torch.zeros(rows, dtype=torch.int32, device=device)
    rc = lib.shk_argmax_static(logits.data_ptr(), out.data_ptr(), rows, vocab, vocab,
                               torch.cuda.current_stream().cuda_stream)
    assert rc != 0
    assert "use shk_argmax with a workspace" in lib.shk_last_error().decode()
