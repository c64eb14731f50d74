"""The entry point that allocates nothing (blm_argmax_static, declared in csrc/no_alloc.h), called
through ctypes as a caller without torch would: its output against the existing blm_argmax's on two
calls in a row, the second with a smaller input, so that what the first call left in the library's
own scratch array would show if it were read."""
import ctypes

import pytest

pytestmark = pytest.mark.gpu


def _lib():
    from burn_lm_amd.csrc import build
    lib = ctypes.CDLL(build.ensure_built())
    lib.blm_last_error.restype = ctypes.c_char_p
    vp, ci = ctypes.c_void_p, ctypes.c_int
    lib.blm_argmax_static.argtypes = [vp, vp, ci, ci, ci, vp]
    lib.blm_argmax_static.restype = ci
    lib.blm_argmax.argtypes = [vp, vp, ci, ci, ci, vp, vp, vp]
    lib.blm_argmax.restype = ci
    lib.blm_static_scratch_init.argtypes = []
    lib.blm_static_scratch_init.restype = ci
    return lib


def test_argmax_without_workspaces_equals_argmax_with_them_twice_in_a_row():
    import torch
    lib = _lib()
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(5)
    stream = torch.cuda.current_stream(dev).cuda_stream
    assert lib.blm_static_scratch_init() == 0, lib.blm_last_error().decode()
    # the second call is smaller in rows and in vocabulary, and its maxima lie elsewhere
    for R, V, ld in ((37, 128256, 128256), (5, 1001, 1008)):
        logits = torch.randn(R, ld, generator=g).to(dev)
        for r in range(R):      # a tie in every row: the lower index must win in both
            a, b = sorted(int(x) for x in torch.randint(0, V, (2,), generator=g))
            logits[r, a] = logits[r, b] = 50.0
        logits[:, V:] = 100.0   # beyond the vocabulary: never looked at
        want = torch.full((R,), -1, dtype=torch.int32, device=dev)
        val = torch.empty(R * 32, dtype=torch.float32, device=dev)
        idx = torch.empty(R * 32, dtype=torch.int32, device=dev)
        rc = lib.blm_argmax(logits.data_ptr(), want.data_ptr(), R, V, ld, val.data_ptr(), idx.data_ptr(), stream)
        assert rc == 0, lib.blm_last_error().decode()
        got = torch.full((R,), -1, dtype=torch.int32, device=dev)
        before = torch.cuda.memory_allocated(dev)
        rc = lib.blm_argmax_static(logits.data_ptr(), got.data_ptr(), R, V, ld, stream)
        assert rc == 0, lib.blm_last_error().decode()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated(dev) == before
        assert got.tolist() == want.tolist()
        assert all(float(logits[r, got[r]]) == 50.0 for r in range(R))


def test_argmax_without_workspaces_refuses_more_rows_than_its_array_holds():
    import torch
    lib = _lib()
    dev = torch.device("cuda:0")
    logits = torch.zeros(1025, 8, device=dev)
    out = torch.zeros(1025, dtype=torch.int32, device=dev)
    rc = lib.blm_argmax_static(logits.data_ptr(), out.data_ptr(), 1025, 8, 8, torch.cuda.current_stream(dev).cuda_stream)
    assert rc != 0 and "1024" in lib.blm_last_error().decode()
    torch.cuda.synchronize()
