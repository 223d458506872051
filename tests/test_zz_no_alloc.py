"""The library's entry point that allocates nothing (egpt_argmax_static), called through ctypes and compared
with the entry point it is a variant of (egpt_argmax, which takes its workspace from the caller)."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def library():
    from easy_gpt.cpp_amd.csrc import build

    lib = ctypes.CDLL(build.ensure_built())
    vp, i = ctypes.c_void_p, ctypes.c_int
    lib.egpt_error_string.restype = ctypes.c_char_p
    lib.egpt_error_string.argtypes = [i]
    lib.egpt_argmax.argtypes = [vp, vp, vp, i, i, vp]
    lib.egpt_argmax_static.argtypes = [vp, vp, i, i, vp]
    lib.egpt_argmax_static_init.argtypes = []
    for name in ("egpt_argmax", "egpt_argmax_static", "egpt_argmax_static_init"):
        getattr(lib, name).restype = i
    return lib


def rows_of_logits(rows, vocab, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    logits = torch.randn(rows, vocab, generator=g, device="cuda", dtype=torch.float32)
    # equal maxima far apart in some rows: the lowest index must win in both stages
    for r in range(0, rows, 3):
        top = float(logits[r].max()) + 1.0
        logits[r, vocab - 1 - r] = top
        logits[r, (7 * r + 5) % vocab] = top
    return logits


def test_argmax_without_allocation_equals_argmax_with_a_workspace():
    lib = library()
    torch.cuda.set_device(0)
    assert lib.egpt_argmax_static_init() == 0
    stream = torch.cuda.current_stream().cuda_stream
    # two calls in a row on the same GPU's buffer, the second smaller in both sizes (what the first left must not
    # show), then a vocabulary so narrow that one stage does it, then the largest number of rows
    for rows, vocab, seed in ((64, 151936, 0), (5, 9001, 1), (3, 777, 2), (1024, 8192, 3)):
        logits = rows_of_logits(rows, vocab, seed)
        print(f"egpt_argmax_static rows={rows} vocab={vocab}", flush=True)
        want = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        workspace = torch.empty(rows * 64, dtype=torch.float32, device="cuda")
        assert lib.egpt_argmax(logits.data_ptr(), want.data_ptr(), workspace.data_ptr(), rows, vocab, stream) == 0
        got = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        code = lib.egpt_argmax_static(logits.data_ptr(), got.data_ptr(), rows, vocab, stream)
        assert code == 0, lib.egpt_error_string(code).decode()
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        assert torch.equal(got.long(), torch.argmax(logits, dim=-1))       # (the library's first maximum, too)


def test_argmax_without_allocation_refuses_what_its_buffer_cannot_hold():
    lib = library()
    torch.cuda.set_device(0)
    stream = torch.cuda.current_stream().cuda_stream
    logits = torch.zeros(8, 16, device="cuda")
    out = torch.full((8,), -7, dtype=torch.int32, device="cuda")
    code = lib.egpt_argmax_static(logits.data_ptr(), out.data_ptr(), 1025, 8192, stream)
    assert code != 0 and "at most 1024 rows" in lib.egpt_error_string(code).decode()
    assert lib.egpt_argmax_static(None, out.data_ptr(), 8, 16, stream) != 0
    torch.cuda.synchronize()
    assert out.tolist() == [-7] * 8                                         # nothing was launched
