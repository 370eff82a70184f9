"""The entry point that allocates nothing, called through ctypes as a caller outside
Python would: li_argmax_rows_noalloc against li_argmax_rows (which takes its buffers from
the caller), on two calls in a row, the second with a smaller input, so that what the
first left in the library's scratch array lies beside and behind what the second uses."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _lib():
    from litinfer_amd.kernels import build
    path = build.find_built("sampling")
    assert path is not None, "the sampling library is not built"
    lib = ctypes.CDLL(str(path))
    P, I = ctypes.c_void_p, ctypes.c_int
    lib.li_argmax_rows.argtypes, lib.li_argmax_rows.restype = [P, P, P, P, I, I, P], I
    lib.li_argmax_rows_noalloc.argtypes, lib.li_argmax_rows_noalloc.restype = [P, P, I, I, P], I
    lib.li_argmax_rows_noalloc_init.argtypes, lib.li_argmax_rows_noalloc_init.restype = [], I
    lib.li_argmax_rows_noalloc_max_rows.argtypes, lib.li_argmax_rows_noalloc_max_rows.restype = [], I
    lib.li_argmax_rows_noalloc_error.argtypes, lib.li_argmax_rows_noalloc_error.restype = [], ctypes.c_char_p
    return lib


def test_argmax_without_allocation_equals_the_one_with_buffers_twice_in_a_row():
    lib = _lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.li_argmax_rows_noalloc_init() == 0, lib.li_argmax_rows_noalloc_error().decode()
    g = torch.Generator().manual_seed(5)
    # a first small call of both entry points: what the runtime sets up at a kernel's first launch
    # (its code, its queue) is in place before free memory is compared
    warm = torch.randn(2, 64, generator=g).to(dev)
    w_out = torch.empty(2, dtype=torch.int32, device=dev)
    w_sv, w_si = torch.empty(64, dtype=torch.float32, device=dev), torch.empty(64, dtype=torch.int32, device=dev)
    assert lib.li_argmax_rows(warm.data_ptr(), w_out.data_ptr(), w_sv.data_ptr(), w_si.data_ptr(), 2, 64, stream) == 0
    assert lib.li_argmax_rows_noalloc(warm.data_ptr(), w_out.data_ptr(), 2, 64, stream) == 0
    torch.cuda.synchronize()
    for n, v in ((64, 152064), (5, 301)):                     # the second call is the smaller one
        logits = torch.randn(n, v, generator=g).to(dev)
        logits[1, min(7, v - 1)] = logits[1, v - 1] = 50.0    # a tie: the lower index wins
        want = torch.empty(n, dtype=torch.int32, device=dev)
        sv = torch.empty(n * 32, dtype=torch.float32, device=dev)
        si = torch.empty(n * 32, dtype=torch.int32, device=dev)
        got = torch.full((n,), -7, dtype=torch.int32, device=dev)
        assert lib.li_argmax_rows(logits.data_ptr(), want.data_ptr(), sv.data_ptr(), si.data_ptr(), n, v, stream) == 0
        torch.cuda.synchronize()
        # the device's own count of free memory sees any hipMalloc or hipFree, also one made inside the
        # library; torch's counter sees its own allocator only
        before, free_before = torch.cuda.memory_allocated(dev), torch.cuda.mem_get_info(dev)[0]
        rc = lib.li_argmax_rows_noalloc(logits.data_ptr(), got.data_ptr(), n, v, stream)
        assert rc == 0, lib.li_argmax_rows_noalloc_error().decode()
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info(dev)[0] == free_before, "the device's free memory changed during the call"
        assert torch.cuda.memory_allocated(dev) == before
        assert torch.equal(got, want)
        assert torch.equal(got.cpu().long(), torch.argmax(logits.cpu(), dim=1))
        assert int(got[1]) == min(7, v - 1)
    # more rows than the scratch array holds: refused with a text, nothing launched
    cap = lib.li_argmax_rows_noalloc_max_rows()
    assert cap == 1024
    assert lib.li_argmax_rows_noalloc(logits.data_ptr(), got.data_ptr(), cap + 1, 8, stream) == 2
    assert b"more than the 1024" in lib.li_argmax_rows_noalloc_error()
    assert lib.li_argmax_rows_noalloc(logits.data_ptr(), got.data_ptr(), 0, 8, stream) == 2
    torch.cuda.synchronize()
