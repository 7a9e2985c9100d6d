"""The greedy choice that allocates nothing (ic_argmax_static), called through ctypes as a
caller without torch would, against ic_argmax on the same logits: two calls in a row, the
second with fewer and shorter rows, so stale partial results of the first call would show."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from infinicore_infer_amd.kernels import build as kbuild
    path = kbuild.find_library() or kbuild.build()
    lib = ctypes.CDLL(path)
    P, I, LL = ctypes.c_void_p, ctypes.c_int, ctypes.c_longlong
    lib.ic_argmax.argtypes = [P, LL, I, I, P, P, P, P]
    lib.ic_argmax.restype = I
    lib.ic_argmax_static.argtypes = [P, LL, I, I, P, P]
    lib.ic_argmax_static.restype = I
    lib.ic_argmax_static_max_rows.argtypes = []
    lib.ic_argmax_static_max_rows.restype = I
    return lib


def _both(lib, logits):
    R, V = logits.shape
    stream = torch.cuda.current_stream().cuda_stream
    val = torch.empty(64 * R, dtype=torch.float32, device=logits.device)
    idx = torch.empty(64 * R, dtype=torch.int32, device=logits.device)
    want = torch.full((R,), -1, dtype=torch.int32, device=logits.device)
    got = torch.full((R,), -2, dtype=torch.int32, device=logits.device)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    assert lib.ic_argmax_static(logits.data_ptr(), logits.stride(0), R, V, got.data_ptr(), stream) == 0
    assert torch.cuda.memory_allocated() == before
    assert lib.ic_argmax(logits.data_ptr(), logits.stride(0), R, V, val.data_ptr(), idx.data_ptr(),
                         want.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    return got.cpu(), want.cpu()


def test_argmax_static_equals_argmax_on_two_calls_in_a_row():
    lib = _library()
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(11)
    first = torch.randn(37, 122753, generator=g).to(dev)
    first[5, 70001] = first[5, 12] = 50.0            # equal maxima: the lower index wins
    got, want = _both(lib, first)
    assert torch.equal(got, want)
    assert torch.equal(got.long(), first.cpu().argmax(dim=1)) or got[5] == 12
    assert got[5] == 12
    # the second call: fewer rows, a shorter vocabulary that leaves most chunks of the first call's
    # partial results untouched unless the first stage rewrites them
    second = torch.randn(3, 509, generator=g).to(dev) - 100.0      # every value below the first call's maxima
    got2, want2 = _both(lib, second)
    assert torch.equal(got2, want2)
    assert torch.equal(got2.long(), second.cpu().argmax(dim=1))
    # a strided view (rows of a wider buffer)
    wide = torch.randn(4, 1000, generator=g).to(dev)
    got3, want3 = _both(lib, wide[:, :777])
    assert torch.equal(got3, want3) and torch.equal(got3.long(), wide[:, :777].cpu().argmax(dim=1))


def test_argmax_static_refuses_more_rows_than_it_holds():
    lib = _library()
    dev = torch.device("cuda:0")
    cap = lib.ic_argmax_static_max_rows()
    assert cap == 1024
    logits = torch.zeros(cap + 1, 8, dtype=torch.float32, device=dev)
    out = torch.full((cap + 1,), -7, dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.ic_argmax_static(logits.data_ptr(), 8, cap + 1, 8, out.data_ptr(), stream) == -5
    torch.cuda.synchronize()
    assert bool((out == -7).all())                  # nothing was launched
    logits[:, 3] = 1.0
    assert lib.ic_argmax_static(logits.data_ptr(), 8, cap, 8, out.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    assert bool((out[:cap] == 3).all()) and int(out[cap]) == -7


def test_argmax_static_through_the_package():
    from infinicore_infer_amd.kernels import ops
    dev = torch.device("cuda:0")
    logits = torch.randn(9, 4099, generator=torch.Generator().manual_seed(2)).to(dev)
    out = torch.empty(9, dtype=torch.int32, device=dev)
    ops.argmax_static(logits, out)
    assert torch.equal(out.cpu().long(), logits.cpu().argmax(dim=1))
    with pytest.raises(ops.KernelError):
        ops.argmax_static(torch.zeros(1025, 4, device=dev), torch.empty(1025, dtype=torch.int32, device=dev))
