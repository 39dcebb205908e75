"""The entry point that allocates nothing (w4a16_gemv_noalloc_bf16: split-K slots in a device array inside the
library) against w4a16_gemv_bf16, through the C ABI: same kernels, so the outputs must agree bit for bit, on two
calls in a row, the second with a smaller input; shapes beyond the array are refused."""
import numpy as np
import pytest
import torch

from helpers import make_awq, make_x

pytestmark = pytest.mark.gpu


def dev(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)
    return torch.from_numpy(a).cuda()


def bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def _both(lib, _lib, K, N, seed):
    print(f"noalloc gemv K={K} N={N} seed={seed}", flush=True)
    qw, qz, s = (dev(t) for t in make_awq(K, N, seed=seed))
    x = dev(make_x((K,), seed=seed + 1))
    st = torch.cuda.current_stream().cuda_stream
    want = torch.full((N,), 7.0, dtype=torch.bfloat16, device="cuda")
    ws = torch.empty(int(lib.w4a16_gemm_workspace_bytes(1, K, N)), dtype=torch.uint8, device="cuda")
    _lib.check(lib.w4a16_workspace_init(ws.data_ptr(), ws.numel(), st))
    _lib.check(lib.w4a16_gemv_bf16(x.data_ptr(), qw.data_ptr(), qz.data_ptr(), s.data_ptr(), want.data_ptr(), K, N, 128,
                                   ws.data_ptr(), ws.numel(), st))
    got = torch.full((N,), -3.0, dtype=torch.bfloat16, device="cuda")
    _lib.check(lib.w4a16_gemv_noalloc_bf16(x.data_ptr(), qw.data_ptr(), qz.data_ptr(), s.data_ptr(), got.data_ptr(), K, N,
                                           128, st))
    torch.cuda.synchronize()
    assert np.array_equal(bits(got), bits(want)), f"K={K} N={N}"


def test_two_calls_in_a_row_second_smaller():
    from air_hip import _lib
    lib = _lib.load_library()
    _both(lib, _lib, 4096, 11008, seed=1)
    _both(lib, _lib, 1024, 544, seed=2)
    _both(lib, _lib, 4096, 11008, seed=3)     # and back to the larger shape on the same array


def test_largest_shape_and_beyond():
    from air_hip import _lib
    lib = _lib.load_library()
    _both(lib, _lib, 256, 32768, seed=4)
    K, N = 128, 32768 + 32
    qw, qz, s = (dev(t) for t in make_awq(K, N, seed=5))
    x, y = dev(make_x((K,), seed=6)), torch.empty((N,), dtype=torch.bfloat16, device="cuda")
    rc = lib.w4a16_gemv_noalloc_bf16(x.data_ptr(), qw.data_ptr(), qz.data_ptr(), s.data_ptr(), y.data_ptr(), K, N, 128, None)
    assert rc == _lib.ERR_TOO_LARGE
    assert b"allocates nothing" in lib.w4a16_strerror(rc)
