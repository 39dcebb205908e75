"""The single-kernel decode FFN against the two-launch path of the same entry point.

Both run the same arithmetic in the same order (per-wave units, LDS combine, partials added in
slice order), so h and y must agree bit for bit; the two-launch path itself is checked against the
oracle in test_gpu_parity.py.  Repeated calls catch races in the cross-workgroup protocol (while the
kernel was being written, a reducer sporadically accepted stale registers as filled slots: from
one call in two down to one in a thousand, depending on the variant), the workspace must be left
clean, and the kernel must replay from a HIP graph.
"""
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


@pytest.fixture(scope="module")
def ops():
    from air_hip import ops
    yield ops
    ops.tune("ffn_fused", 0)   # the library's default: the persistent kernel is opt-in


def _weights(K, H, seed):
    return (tuple(map(dev, make_awq(K, H, seed=seed))), tuple(map(dev, make_awq(K, H, seed=seed + 1))),
            tuple(map(dev, make_awq(H, K, seed=seed + 2))))


def _both(ops, x, g, u, d):
    ops.tune("ffn_fused", 0)
    y0, h0 = ops.ffn_swiglu(x, g, u, d, return_h=True)
    ops.tune("ffn_fused", 1)
    y1, h1 = ops.ffn_swiglu(x, g, u, d, return_h=True)
    torch.cuda.synchronize()
    return (bits(y0), bits(h0)), (bits(y1), bits(h1))


def test_fused_equals_two_launches_config4(ops):
    print("ffn fused vs two launches K=4096 H=14336", flush=True)
    K, H = 4096, 14336
    g, u, d = _weights(K, H, 1)
    x = dev(make_x((K,), seed=4))
    (y0, h0), (y1, h1) = _both(ops, x, g, u, d)
    assert np.array_equal(h1, h0)
    assert np.array_equal(y1, y0)


def test_fused_repeated_calls_stay_bit_exact_and_leave_the_workspace_clean(ops):
    print("ffn fused repeated", flush=True)
    from air_hip import _lib
    K, H = 4096, 14336
    g, u, d = _weights(K, H, 11)
    x = dev(make_x((K,), seed=14))
    (y0, h0), _ = _both(ops, x, g, u, d)
    y0t, h0t = dev(y0), dev(h0)
    bad = torch.zeros((), dtype=torch.int64, device="cuda")
    for _ in range(5000):
        y, h = ops.ffn_swiglu(x, g, u, d, return_h=True)
        bad += (y.view(torch.int16) != y0t.view(torch.int16)).sum() + (h.view(torch.int16) != h0t.view(torch.int16)).sum()
    y = ops.ffn_swiglu(x, g, u, d)          # h kept inside the kernel
    torch.cuda.synchronize()
    assert int(bad) == 0
    assert np.array_equal(bits(y), y0)
    lib = _lib.load_library()
    ws = ops.workspace(1, x.device, ("ffn", K, H))
    assert lib.w4a16_workspace_check(ws.data_ptr(), None) == 0
    # everything behind the header is slots again, except the h buffer the two-launch path keeps at the end
    tail = (2 * H + 255) // 256 * 256
    assert int((ws[256:ws.numel() - tail].view(torch.int32) != -1).sum()) == 0


@pytest.mark.parametrize("K,H", [(256, 512), (2048, 8192), (4096, 11008), (1024, 2048 + 128)])
def test_shapes_the_single_kernel_does_not_take_fall_back(ops, K, H):
    """Either path must give the same result whatever the planner decides for the shape."""
    print(f"ffn fused / fallback K={K} H={H}", flush=True)
    g, u, d = _weights(K, H, K + H)
    x = dev(make_x((K,), seed=K))
    (y0, h0), (y1, h1) = _both(ops, x, g, u, d)
    assert np.array_equal(h1, h0) and np.array_equal(y1, y0)


def test_fused_replays_from_a_hip_graph(ops):
    print("ffn fused graph", flush=True)
    from air_hip import _lib
    lib = _lib.load_library()
    K, H = 4096, 14336
    g, u, d = _weights(K, H, 21)
    x = dev(make_x((K,), seed=24))
    y_eager = ops.ffn_swiglu(x, g, u, d)
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    ws = torch.empty(int(lib.w4a16_ffn_workspace_bytes(K, H)), dtype=torch.uint8, device="cuda")
    y = torch.empty(K, dtype=torch.bfloat16, device="cuda")
    with torch.cuda.stream(stream):
        _lib.check(lib.w4a16_workspace_init(ws.data_ptr(), ws.numel(), stream.cuda_stream))
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            ptrs = [t.data_ptr() for w in (g, u, d) for t in w]
            _lib.check(lib.w4a16_ffn_swiglu_bf16(x.data_ptr(), *ptrs, y.data_ptr(), None, K, H, 128, ws.data_ptr(), ws.numel(),
                                                 stream.cuda_stream))
        for _ in range(4):
            y.zero_()
            stream.synchronize()
            graph.replay()
            stream.synchronize()
            assert np.array_equal(bits(y), bits(y_eager))
            torch.cuda.synchronize()
