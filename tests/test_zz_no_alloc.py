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


def test_first_use_under_capture_is_refused_and_the_array_is_ready_for_every_stream():
    """A first use of the array on this GPU under stream capture launches nothing and returns W4A16_ERR_NOT_PREPARED (the
    array cannot be prepared and waited for there); after one use outside capture (here on another stream) captured
    calls work, and replays equal the eager result bit for bit."""
    from air_hip import _lib, ops
    lib = _lib.load_library()
    K, N = 2048, 4096
    qw, qz, s = (dev(t) for t in make_awq(K, N, seed=11))
    x = dev(make_x((K,), seed=12))
    want = ops.w4a16_gemv(x, qw, qz, s)
    torch.cuda.synchronize()
    ops.tune("noalloc_forget", 1)   # as in a process that has not used the entry point yet
    y = torch.zeros((N,), dtype=torch.bfloat16, device="cuda")
    args = (x.data_ptr(), qw.data_ptr(), qz.data_ptr(), s.data_ptr(), y.data_ptr(), K, N, 128)
    st, st2 = torch.cuda.Stream(), torch.cuda.Stream()
    print("noalloc: first use under capture", flush=True)
    with torch.cuda.stream(st):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=st):
            y.zero_()
            rc = lib.w4a16_gemv_noalloc_bf16(*args, st.cuda_stream)
        assert rc == _lib.ERR_NOT_PREPARED
        assert b"w4a16_noalloc_check" in lib.w4a16_strerror(rc)
        g.replay()
        st.synchronize()
        assert not y.any()   # nothing but the zero fill was captured
    print("noalloc: eager use on a second stream, then captured", flush=True)
    with torch.cuda.stream(st2):
        _lib.check(lib.w4a16_gemv_noalloc_bf16(*args, st2.cuda_stream))
        st2.synchronize()
    assert np.array_equal(bits(y), bits(want))
    with torch.cuda.stream(st):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=st):
            y.zero_()
            _lib.check(lib.w4a16_gemv_noalloc_bf16(*args, st.cuda_stream))
        for _ in range(3):
            g.replay()
            st.synchronize()
            assert np.array_equal(bits(y), bits(want))
    # prepared through the check entry instead: a captured first call then works
    ops.tune("noalloc_forget", 1)
    assert lib.w4a16_noalloc_check(None) == 0
    with torch.cuda.stream(st):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=st):
            y.zero_()
            _lib.check(lib.w4a16_gemv_noalloc_bf16(*args, st.cuda_stream))
        g.replay()
        st.synchronize()
    assert np.array_equal(bits(y), bits(want))


def test_reducer_timeout_in_the_library_array_is_reported_and_repaired():
    """Host-forced fault: producers do not publish, every reducer runs into a tiny poll bound and flags the array's
    header (all waves exit normally).  w4a16_noalloc_check reports it once and empties the array; ops.check_health
    sees the same array; the next call is bit-exact again."""
    from air_hip import _lib, ops
    lib = _lib.load_library()
    K, N = 4096, 1024
    qw, qz, s = (dev(t) for t in make_awq(K, N, seed=21))
    x = dev(make_x((K,), seed=22))
    want = ops.w4a16_gemv(x, qw, qz, s)
    assert torch.equal(ops.w4a16_gemv_noalloc(x, qw, qz, s).view(torch.int16), want.view(torch.int16))
    assert lib.w4a16_noalloc_check(None) == 0
    print("noalloc: forced reducer timeout", flush=True)
    try:
        ops.tune("gemv_skip_publish", 1)
        ops.tune("gemv_spin_limit", 8)
        ops.w4a16_gemv_noalloc(x, qw, qz, s)
        assert lib.w4a16_noalloc_check(None) == _lib.ERR_TIMEOUT
        assert lib.w4a16_noalloc_check(None) == 0          # reported once, array emptied
        ops.w4a16_gemv_noalloc(x, qw, qz, s)
        with pytest.raises(_lib.W4A16Error) as e:
            ops.check_health()
        assert e.value.code == _lib.ERR_TIMEOUT
    finally:
        ops.tune("gemv_skip_publish", 0)
        ops.tune("gemv_spin_limit", 0)
    ops.check_health()
    assert torch.equal(ops.w4a16_gemv_noalloc(x, qw, qz, s).view(torch.int16), want.view(torch.int16))
    ops.check_health()
