"""GPU parity of the stream-order path (through the C ABI): the device re-pack against the host packer bit for
bit, and the whole-K decode GEMV (plain, + residual, SwiGLU pair) against the float64 oracle.

Tolerance: one bf16 rounding of an fp32-accumulated sum -> within 1 bf16 ulp of the float64 value plus 2e-3
absolute, and inside the reference's own gate (rtol 0.1, atol 0.05, r >= 0.999)."""
import numpy as np
import pytest
import torch

from helpers import assert_bf16_close, dense_f64, make_awq, make_x
from oracle import awq as oawq, reference as oref
from oracle.bf16 import bf16_bits_to_f32, f32_to_bf16_bits

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
    return ops


def _stream_weight(ops, qw, qz, s):
    return ops.repack_stream(dev(qw), dev(qz), dev(s))


@pytest.mark.parametrize("K,N", [(128, 16), (256, 48), (2048, 64), (128 * 19, 32), (4096, 4096)])
def test_device_repack_equals_host_packer(ops, K, N):
    print(f"repack K={K} N={N}", flush=True)
    from air_hip import awq, bf16
    qw, qz, s = make_awq(K, N, seed=K + N)
    w = _stream_weight(ops, qw, qz, s)
    torch.cuda.synchronize()
    want = awq.repack_stream(qw, qz, bf16.from_bits(s))
    got = w.buf.cpu().numpy().view(np.uint32).reshape(want.shape)
    assert np.array_equal(got, want)


def _gemv_case(ops, K, N, seed, residual=False):
    print(f"gemv stream K={K} N={N} seed={seed} residual={residual}", flush=True)
    qw, qz, s = make_awq(K, N, seed=seed)
    x = make_x((K,), seed=seed + 1)
    r = make_x((N,), seed=seed + 2) if residual else None
    w = _stream_weight(ops, qw, qz, s)
    y = ops.w4a16_gemv_stream(dev(x), w, residual=dev(r) if residual else None)
    torch.cuda.synchronize()
    got = bits(y)
    want = bf16_bits_to_f32(x).astype(np.float64) @ dense_f64(qw, qz, s)
    if residual:
        want = want + bf16_bits_to_f32(r).astype(np.float64)
    assert_bf16_close(got, want, ulps=1.0, atol=2e-3, what=f"gemv stream K={K} N={N}")
    assert oref.check_outputs(bf16_bits_to_f32(got), bf16_bits_to_f32(f32_to_bf16_bits(want.astype(np.float32))),
                              rtol=0.1, atol=0.05, min_correlation=0.999 if want.size > 8 else None)
    return got


# K = 128 .. 14336: one short block, whole blocks, a short last block (19 and 86 groups), 7 blocks
@pytest.mark.parametrize("K,N", [(128, 16), (256, 544), (1024, 512), (128 * 19, 48), (2048, 8192), (4096, 4096),
                                 (11008, 512), (14336, 4096)])
def test_gemv_stream_shapes(ops, K, N):
    _gemv_case(ops, K, N, seed=K + N)


def test_gemv_stream_config1(ops):
    _gemv_case(ops, 4096, 11008, seed=1)


@pytest.mark.parametrize("K,N", [(512, 64), (4096, 4096), (14336, 4096)])
def test_gemv_stream_residual(ops, K, N):
    _gemv_case(ops, K, N, seed=3 * K + N, residual=True)


def test_gemv_stream_zero_weights_return_the_residual_bit_for_bit(ops):
    K, N = 512, 256
    qw, qz, s = make_awq(K, N, seed=9)
    w = _stream_weight(ops, qw, qz, np.zeros_like(s))
    x, r = make_x((K,), seed=10), make_x((N,), seed=11)
    y = ops.w4a16_gemv_stream(dev(x), w, residual=dev(r))
    torch.cuda.synchronize()
    assert np.array_equal(bits(y), r)


def test_gemv_stream_one_hot_x_is_a_dequantised_row(ops):
    """x = e_k selects row k: (q - z) * s has at most 13 significant bits, so the fp32 sum is exact and the single
    rounding must reproduce the dense dequant bit for bit - every row position of a cell, both blocks."""
    K, N = 4096, 64
    qw, qz, s = make_awq(K, N, seed=3)
    dense = oawq.dequant_to_bf16(qw, qz, s, 128)
    w = _stream_weight(ops, qw, qz, s)
    for k0 in (0, 1, 2, 7, 8, 31, 32, 127, 128, 1000, 2047, 2048, 4095):
        x = np.zeros(K, np.uint16)
        x[k0] = 0x3F80
        y = ops.w4a16_gemv_stream(dev(x), w)
        torch.cuda.synchronize()
        assert np.array_equal(bits(y), dense[k0]), k0


def test_gemv_stream_config1_one_hot_rows(ops):
    K, N = 4096, 11008
    qw, qz, s = make_awq(K, N, seed=1)
    dense = oawq.dequant_to_bf16(qw, qz, s, 128)
    w = _stream_weight(ops, qw, qz, s)
    for k0 in (5, 1234, 4095):
        x = np.zeros(K, np.uint16)
        x[k0] = 0x3F80
        y = ops.w4a16_gemv_stream(dev(x), w)
        torch.cuda.synchronize()
        assert np.array_equal(bits(y), dense[k0]), k0


def test_gemv_stream_power_of_two_scaling_is_exact(ops):
    K, N = 2048, 512
    qw, qz, s = make_awq(K, N, seed=21)
    x = make_x((K,), seed=22)
    w = _stream_weight(ops, qw, qz, s)
    y1 = bits(ops.w4a16_gemv_stream(dev(x), w))
    x8 = f32_to_bf16_bits(bf16_bits_to_f32(x) * 8.0)
    y8 = bits(ops.w4a16_gemv_stream(dev(x8), w))
    assert np.array_equal(bf16_bits_to_f32(y1) * 8.0, bf16_bits_to_f32(y8))


@pytest.mark.parametrize("ct,waves", [(4, 0), (16, 0), (8, 1), (8, 3)])
def test_gemv_stream_launch_shapes_agree(ops, ct, waves):
    """Other task sizes and fewer waves than tasks (a wave then walks several tasks) change the summation order only."""
    base = _gemv_case(ops, 128 * 23, 272, seed=50)
    ops.tune("gemv_ws_ct", ct)
    ops.tune("gemv_ws_waves", waves)
    try:
        got = _gemv_case(ops, 128 * 23, 272, seed=50)
    finally:
        ops.tune("gemv_ws_ct", 0)
        ops.tune("gemv_ws_waves", 0)
    d = np.abs(bf16_bits_to_f32(got).astype(np.float64) - bf16_bits_to_f32(base).astype(np.float64))
    assert np.all(d <= 2.0 ** (np.floor(np.log2(np.maximum(np.abs(bf16_bits_to_f32(base)), 1e-30))) - 7) + 2e-3)


@pytest.mark.parametrize("K,H", [(256, 64), (2048, 8192), (4096, 14336)])
def test_swiglu_stream(ops, K, H):
    print(f"swiglu stream K={K} H={H}", flush=True)
    g, u = make_awq(K, H, seed=K + 1), make_awq(K, H, seed=K + 2)
    x = make_x((K,), seed=K + 3)
    h = ops.w4a16_swiglu_stream(dev(x), _stream_weight(ops, *g), _stream_weight(ops, *u))
    torch.cuda.synchronize()
    xf = bf16_bits_to_f32(x).astype(np.float64)
    gate, up = xf @ dense_f64(*g), xf @ dense_f64(*u)
    gb = bf16_bits_to_f32(f32_to_bf16_bits(gate.astype(np.float32)))
    ub = bf16_bits_to_f32(f32_to_bf16_bits(up.astype(np.float32)))
    want = oref.silu_tanh_f32(gb).astype(np.float64) * ub
    # gate / up each carry one bf16 rounding that may flip by one ulp against the float64 sum: 1 ulp on each
    # moves h by up to ~3 ulp (silu' <= 1.1)
    assert_bf16_close(bits(h), want, ulps=4.0, atol=2e-3, what=f"swiglu stream K={K} H={H}")
    assert oref.check_outputs(bf16_bits_to_f32(bits(h)), bf16_bits_to_f32(f32_to_bf16_bits(want.astype(np.float32))),
                              rtol=0.15, atol=0.5, min_correlation=0.99)


def _gemm_case(ops, M, K, N, seed):
    print(f"gemm stream M={M} K={K} N={N} seed={seed}", flush=True)
    qw, qz, s = make_awq(K, N, seed=seed)
    x = make_x((M, K), seed=seed + 1)
    y = ops.w4a16_gemm_stream(dev(x), _stream_weight(ops, qw, qz, s))
    torch.cuda.synchronize()
    got = bits(y)
    want = bf16_bits_to_f32(x).astype(np.float64) @ dense_f64(qw, qz, s)
    assert_bf16_close(got, want, ulps=1.0, atol=2e-3, what=f"gemm stream M={M} K={K} N={N}")
    assert oref.check_outputs(bf16_bits_to_f32(got), bf16_bits_to_f32(f32_to_bf16_bits(want.astype(np.float32))),
                              rtol=0.1, atol=0.05, max_mismatch_percentage=0.05, min_correlation=0.999)
    return got


# rows 2..16 and beyond, one / two / four tiles per workgroup (N = 14336 and 6400 pick 4 and 2),
# K with a short last task (19 groups) and more tasks than waves (K = 14336: 28 tasks on 8 waves)
@pytest.mark.parametrize("M,K,N", [(2, 128, 16), (3, 256, 544), (7, 1152, 544), (16, 512, 1056), (5, 128 * 19, 48),
                                   (16, 4096, 6400), (9, 14336, 4096), (40, 1024, 512), (16, 2048, 2048)])
def test_gemm_stream_shapes(ops, M, K, N):
    _gemm_case(ops, M, K, N, seed=M + K + N)


# 17 .. 64 rows run as one launch of two or four row tiles, more rows as launches of 64 and a rest: ragged last row tile,
# a rest of one row, short last task (19 groups in tasks of two), more tasks than waves, one / two / four tiles per workgroup
@pytest.mark.parametrize("M,K,N", [(17, 256, 64), (32, 1024, 544), (33, 512, 1056), (48, 128 * 19, 48), (64, 4096, 6400),
                                   (65, 1024, 512), (96, 2048, 2048), (30, 128 * 19, 528), (64, 2048, 14336), (20, 14336, 4096)])
def test_gemm_stream_more_than_sixteen_rows(ops, M, K, N):
    _gemm_case(ops, M, K, N, seed=M + K + N)


@pytest.mark.parametrize("M,K,N", [(17, 256, 64), (32, 1024, 544), (48, 128 * 19, 48), (64, 4096, 6400), (65, 1024, 512),
                                   (128, 2048, 2048), (30, 128 * 19, 528), (64, 4096, 14336), (20, 14336, 4096), (33, 128, 272)])
def test_gemm_stream_split_k_against_whole_k(ops, M, K, N):
    """17 .. 128 rows through ops.w4a16_gemm_stream run split along K where that is the faster way (256-column
    workgroups, x through LDS, the slices added by a second launch), else as the whole-K launches of
    w4a16_gemm_stream_bf16; here each way is forced in turn.  Both are within one ulp of the float64 product (checked
    by _gemm_case) and differ from each other by summation order only.  Shapes: one slice (K = 128), ragged column sets
    (N = 48, 272, 528, 544), a short last quad of groups (19), two launches of rows (65, 128), both row-tile counts."""
    try:
        ops.tune("gemm_splitk", 1)
        split = bf16_bits_to_f32(_gemm_case(ops, M, K, N, seed=M + K + N)).astype(np.float64)
        ops.tune("gemm_splitk", 2)
        whole = bf16_bits_to_f32(_gemm_case(ops, M, K, N, seed=M + K + N)).astype(np.float64)
    finally:
        ops.tune("gemm_splitk", 0)
    assert np.all(np.abs(split - whole) <= 2.0 ** (np.floor(np.log2(np.maximum(np.abs(whole), 1e-30))) - 7) + 2e-3)
    assert np.mean(split != whole) < 0.05


def test_gemm_stream_split_k_scratch_contract(ops):
    """The split-K entry point: scratch size by shape (none below 17 rows, above 128, or for a single slice), a short or
    missing scratch buffer is refused before any launch, and the result does not depend on what the scratch held."""
    from air_hip import _lib
    lib = _lib.load_library()
    K, N, M = 1024, 512, 40
    # by shape: long K, enough rows, and not where the whole-K workgroups are 64 columns wide already
    assert lib.w4a16_gemm_stream_scratch_bytes(64, 14336, 4096) == 14 * 64 * 4096 * 4       # 112 groups in slices of 8
    assert lib.w4a16_gemm_stream_scratch_bytes(64, 4096, 4096) > 0 and lib.w4a16_gemm_stream_scratch_bytes(32, 4096, 4096) == 0
    assert lib.w4a16_gemm_stream_scratch_bytes(64, 2048, 8192) == 0 and lib.w4a16_gemm_stream_scratch_bytes(64, 4096, 14336) == 0
    assert lib.w4a16_gemm_stream_scratch_bytes(M, K, N) == 0
    ops.tune("gemm_splitk", 1)
    try:
        _split_k_scratch_contract(ops, lib, M, K, N)
    finally:
        ops.tune("gemm_splitk", 0)


def _split_k_scratch_contract(ops, lib, M, K, N):
    from air_hip import _lib
    assert lib.w4a16_gemm_stream_scratch_bytes(16, K, N) == 0 and lib.w4a16_gemm_stream_scratch_bytes(129, K, N) == 0
    assert lib.w4a16_gemm_stream_scratch_bytes(M, 128, N) == 0                 # one group: one slice
    need = lib.w4a16_gemm_stream_scratch_bytes(M, K, N)
    assert need == 2 * M * N * 4                                              # 8 groups in slices of 4
    assert lib.w4a16_gemm_stream_scratch_bytes(128, K, N) == 2 * 64 * N * 4   # launches of 64 rows share it
    qw, qz, s = make_awq(K, N, seed=91)
    w = _stream_weight(ops, qw, qz, s)
    x = dev(make_x((M, K), seed=92))
    y = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    scratch = torch.full((need,), 0xFF, dtype=torch.uint8, device="cuda")     # NaN patterns: must all be overwritten
    p = lambda t: t.data_ptr()
    assert lib.w4a16_gemm_stream_scratch_bf16(p(x), p(w.buf), p(y), M, K, N, 128, None, 0, st) == _lib.ERR_WORKSPACE
    assert lib.w4a16_gemm_stream_scratch_bf16(p(x), p(w.buf), p(y), M, K, N, 128, p(scratch), need - 1, st) == _lib.ERR_WORKSPACE
    assert lib.w4a16_gemm_stream_scratch_bf16(p(x), p(w.buf), p(y), M, K, N, 128, p(scratch) + 4, need, st) == _lib.ERR_ALIGN
    torch.cuda.synchronize()
    assert not y.any()
    _lib.check(lib.w4a16_gemm_stream_scratch_bf16(p(x), p(w.buf), p(y), M, K, N, 128, p(scratch), need, st))
    y2 = ops.w4a16_gemm_stream(x, w)
    torch.cuda.synchronize()
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16)) and torch.isfinite(y.float()).all()
    # rows outside the split range go to the same launches as w4a16_gemm_stream_bf16, scratch or not
    x16 = x[:16].contiguous()
    ya, yb = torch.zeros((16, N), dtype=torch.bfloat16, device="cuda"), torch.zeros((16, N), dtype=torch.bfloat16, device="cuda")
    _lib.check(lib.w4a16_gemm_stream_scratch_bf16(p(x16), p(w.buf), p(ya), 16, K, N, 128, None, 0, st))
    _lib.check(lib.w4a16_gemm_stream_bf16(p(x16), p(w.buf), p(yb), 16, K, N, 128, st))
    torch.cuda.synchronize()
    assert torch.equal(ya.view(torch.int16), yb.view(torch.int16))


@pytest.mark.parametrize("rows", [16, 32])
def test_gemm_stream_rows_per_launch_agree_up_to_summation_order(ops, rows):
    """The rows a launch takes change only how a column's groups are dealt to the waves: the same sums in another order."""
    M, K, N = 64, 2048, 1024
    base = bf16_bits_to_f32(_gemm_case(ops, M, K, N, seed=90)).astype(np.float64)
    ops.tune("gemm_ws_rows", rows)
    try:
        other = bf16_bits_to_f32(_gemm_case(ops, M, K, N, seed=90)).astype(np.float64)
    finally:
        ops.tune("gemm_ws_rows", 0)
    assert np.all(np.abs(base - other) <= 2.0 ** (np.floor(np.log2(np.maximum(np.abs(base), 1e-30))) - 7) + 2e-3)
    assert np.mean(base != other) < 0.02


def test_gemm_stream_config2(ops):
    _gemm_case(ops, 16, 4096, 14336, seed=2)


@pytest.mark.parametrize("cb", [1, 2, 4])
def test_gemm_stream_tiles_per_workgroup_agree(ops, cb):
    """The number of tiles a workgroup owns changes nothing about a column's arithmetic: same bits."""
    base = _gemm_case(ops, 11, 1024, 1024, seed=70)
    ops.tune("gemm_ws_cb", cb)
    try:
        assert np.array_equal(_gemm_case(ops, 11, 1024, 1024, seed=70), base)
    finally:
        ops.tune("gemm_ws_cb", 0)


def test_gemm_stream_rows_equal_the_gemv_up_to_summation_order(ops):
    K, N = 2048, 1024
    qw, qz, s = make_awq(K, N, seed=81)
    x = make_x((6, K), seed=82)
    w = _stream_weight(ops, qw, qz, s)
    y = bf16_bits_to_f32(bits(ops.w4a16_gemm_stream(dev(x), w))).astype(np.float64)
    for m in range(6):
        v = bf16_bits_to_f32(bits(ops.w4a16_gemv_stream(dev(x[m]), w))).astype(np.float64)
        assert np.all(np.abs(y[m] - v) <= 2.0 ** (np.floor(np.log2(np.maximum(np.abs(v), 1e-30))) - 7) + 2e-3)


def _prefill_case(ops, M, K, N, seed):
    """The tiled prefill kernel multiplies bf16-rounded weights W = bf16_rne((q - z) * s): within 1 bf16 ulp of the
    float64 product on those weights, and inside the reference's gate against the unrounded product
    (matmul_int4_packed.cpu_reference, matmul_int4_packed.py:89-105: rtol 0.1, atol 0.05, 0.05 % budget, r >= 0.999)."""
    print(f"prefill stream M={M} K={K} N={N} seed={seed}", flush=True)
    qw, qz, s = make_awq(K, N, seed=seed)
    x = make_x((M, K), seed=seed + 1)
    ops.tune("prefill_min_m", 17)   # (by itself the tiled kernel runs from M = 129 on)
    try:
        y = ops.w4a16_gemm_stream(dev(x), _stream_weight(ops, qw, qz, s))
        torch.cuda.synchronize()
    finally:
        ops.tune("prefill_min_m", 0)
    got = bits(y)
    xf = bf16_bits_to_f32(x).astype(np.float64)
    assert_bf16_close(got, xf @ dense_f64(qw, qz, s, rounded=True), ulps=1.0, atol=2e-3, what=f"prefill stream M={M} K={K} N={N}")
    want_u = xf @ dense_f64(qw, qz, s)
    assert oref.check_outputs(bf16_bits_to_f32(got), bf16_bits_to_f32(f32_to_bf16_bits(want_u.astype(np.float32))),
                              rtol=0.1, atol=0.05, max_mismatch_percentage=0.05, min_correlation=0.999)
    return got


# N = 64 U is cut into 256-wide and 192-wide column tiles (4 a + 3 b = U): wide only (U = 4, 16), narrow only (3, 6),
# mixed (7, 14, 28), ragged M, one row tile and several, two groups (no steady-state trip of the K loop) and many
@pytest.mark.parametrize("M,K,N", [(128, 256, 448), (200, 512, 896), (97, 1024, 256), (300, 512, 1024), (512, 2048, 1792),
                                   (100, 256, 192), (257, 768, 384)])
def test_prefill_stream_shapes(ops, M, K, N):
    _prefill_case(ops, M, K, N, seed=M + K + N)


@pytest.mark.parametrize("tile,N", [(1, 1024), (2, 768), (3, 896), (4, 448)])
def test_prefill_stream_forced_tile_width_agrees(ops, tile, N):
    """The same product through one tile width only (tuning knob: 256, 192, 128, 64 columns) and through the width
    chosen by shape: same bits (a column's sum does not depend on the tile it sits in)."""
    want = _prefill_case(ops, 300, 512, N, seed=N)
    ops.tune("prefill_tile", tile)
    try:
        got = _prefill_case(ops, 300, 512, N, seed=N)
    finally:
        ops.tune("prefill_tile", 0)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("tile", [1, 2])
def test_prefill_stream_wide_tiles_on_many_groups(ops, tile):
    """Small matrices pick the 64-column tiling by themselves; the 256- and 192-column tiles on a long K, forced."""
    ops.tune("prefill_tile", tile)
    try:
        _prefill_case(ops, 257, 2048, 768, seed=40 + tile)
    finally:
        ops.tune("prefill_tile", 0)


def test_prefill_stream_small_m_through_the_tiled_kernel(ops):
    _prefill_case(ops, 17, 256, 448, seed=5)
    _prefill_case(ops, 40, 512, 512, seed=6)


def test_gemm_stream_hands_over_to_the_tiled_kernel_above_128_rows(ops):
    """M = 128 is two launches of the batched kernel (unrounded weights), M = 129 the tiled kernel (bf16-rounded
    weights): row 0 of x gives the batched kernel's bits in the first case and the tiled kernel's in the second."""
    K, N = 1024, 512
    qw, qz, s = make_awq(K, N, seed=55)
    w = _stream_weight(ops, qw, qz, s)
    x = make_x((129, K), seed=56)
    y128 = bits(ops.w4a16_gemm_stream(dev(x[:128]), w))
    y129 = bits(ops.w4a16_gemm_stream(dev(x), w))
    ops.tune("prefill_min_m", 17)
    try:
        tiled = bits(ops.w4a16_gemm_stream(dev(x[:128]), w))
    finally:
        ops.tune("prefill_min_m", 0)
    batched = bits(ops.w4a16_gemm_stream(dev(x[:16]), w))
    torch.cuda.synchronize()
    assert np.array_equal(y129[:128], tiled) and not np.array_equal(y128, tiled)
    xf = bf16_bits_to_f32(x).astype(np.float64)
    assert_bf16_close(y128, xf[:128] @ dense_f64(qw, qz, s), ulps=1.0, atol=2e-3, what="M = 128 on the batched kernel")
    assert np.mean(y128[:16] != batched) < 0.02   # the same sums in another order


def test_prefill_stream_config3(ops):
    _prefill_case(ops, 2048, 4096, 14336, seed=3)


def test_prefill_stream_one_hot_rows_reproduce_the_dequant(ops):
    """x = e_k in every row k of a 256-row tile: row k of y is the dense dequant's row k bit for bit."""
    K, N = 256, 448
    qw, qz, s = make_awq(K, N, seed=9)
    x = np.zeros((K, K), np.uint16)
    x[np.arange(K), np.arange(K)] = 0x3F80
    y = ops.w4a16_gemm_stream(dev(x), _stream_weight(ops, qw, qz, s))
    torch.cuda.synchronize()
    assert np.array_equal(bits(y), oawq.dequant_to_bf16(qw, qz, s, 128))


def test_prefill_sized_m_on_a_shape_the_tiled_kernel_does_not_take(ops):
    """K = 384 (an odd number of groups) and N = 80: M = 200 runs the batched kernel in launches of 64 rows and a rest."""
    M, K, N = 200, 384, 80
    qw, qz, s = make_awq(K, N, seed=31)
    x = make_x((M, K), seed=32)
    y = ops.w4a16_gemm_stream(dev(x), _stream_weight(ops, qw, qz, s))
    torch.cuda.synchronize()
    want = bf16_bits_to_f32(x).astype(np.float64) @ dense_f64(qw, qz, s)
    assert_bf16_close(bits(y), want, ulps=1.0, atol=2e-3, what="gemm stream fallback")


def test_stream_entry_points_reject_bad_arguments(ops):
    """Argument checks come before the first launch: negative codes, nothing written."""
    from air_hip import _lib
    lib = _lib.load_library()
    K, N = 256, 64
    qw, qz, s = make_awq(K, N, seed=33)
    w = _stream_weight(ops, qw, qz, s)
    x = dev(make_x((K,), seed=34))
    y = torch.zeros((N,), dtype=torch.bfloat16, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    p = lambda t: t.data_ptr()
    assert lib.w4a16_gemv_stream_bf16(None, p(w.buf), p(y), K, N, 128, st) == _lib.ERR_NULL
    assert lib.w4a16_gemv_stream_bf16(p(x), p(w.buf), p(y), K, N, 64, st) == _lib.ERR_GROUP
    assert lib.w4a16_gemv_stream_bf16(p(x), p(w.buf), p(y), K + 64, N, 128, st) == _lib.ERR_SHAPE
    assert lib.w4a16_gemv_stream_bf16(p(x), p(w.buf), p(y), K, N + 8, 128, st) == _lib.ERR_SHAPE
    assert lib.w4a16_gemv_stream_bf16(p(x) + 2, p(w.buf), p(y), K, N, 128, st) == _lib.ERR_ALIGN
    assert lib.w4a16_gemm_stream_bf16(p(x), p(w.buf), p(y), 0, K, N, 128, st) == _lib.ERR_SHAPE
    assert lib.w4a16_gemv_add_stream_bf16(p(x), p(w.buf), None, p(y), K, N, 128, st) == _lib.ERR_NULL
    assert lib.w4a16_repack_stream(p(dev(qw)), p(dev(qz)), p(dev(s)), None, K, N, 128, st) == _lib.ERR_NULL
    assert lib.w4a16_stream_bytes(K + 1, N) == 0 and lib.w4a16_stream_bytes(K, N) == w.buf.numel()
    torch.cuda.synchronize()
    assert not y.any()


def test_hip_graph_replays_of_the_stream_kernels_match_eager(ops):
    """The GEMV, the batched kernels (up to 16 rows, and four row tiles) and the tiled prefill kernel captured in one HIP graph: every replay, with eager
    work and synchronisations in between, equals the eager results bit for bit (nothing kept between launches)."""
    K, N = 1024, 1792
    qw, qz, s = make_awq(K, N, seed=61)
    w = _stream_weight(ops, qw, qz, s)
    shapes = {"gemv": (K,), "gemm": (12, K), "rows": (40, K), "prefill": (300, K)}
    inputs = {k: [dev(make_x(shp, seed=70 + 3 * i + j)) for j in range(3)] for i, (k, shp) in enumerate(shapes.items())}
    cur = {k: v[0].clone() for k, v in inputs.items()}
    st = torch.cuda.Stream()
    with torch.cuda.stream(st):
        outs = {k: ops.w4a16_gemm_stream(cur[k], w) for k in shapes}   # warm-up: outputs allocated outside the graph
        st.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=st):
            for k in shapes:
                ops.w4a16_gemm_stream(cur[k], w, out=outs[k] if cur[k].dim() == 2 else outs[k].unsqueeze(0))
        for j in range(3):
            for k in shapes:
                cur[k].copy_(inputs[k][j])
            g.replay()
            st.synchronize()
            for k in shapes:
                want = ops.w4a16_gemm_stream(inputs[k][j], w)
                st.synchronize()
                assert torch.equal(outs[k].view(torch.int16), want.view(torch.int16)), (k, j)


def test_stream_entry_points_from_two_threads_on_two_streams(ops):
    """The stream-order entry points keep no state: two host threads, each on its own stream, calling the GEMV, the
    batched kernel and the SwiGLU front half at the same time get the bits a single thread gets."""
    import threading
    K, N = 2048, 1792
    w = [_stream_weight(ops, *make_awq(K, N, seed=120 + i)) for i in range(2)]
    xs = [dev(make_x((24, K), seed=130 + i)) for i in range(2)]

    def work(i):
        return (ops.w4a16_gemv_stream(xs[i][0], w[i]), ops.w4a16_gemm_stream(xs[i], w[i]),
                ops.w4a16_swiglu_stream(xs[i][1], w[i], w[1 - i]))

    want = [work(i) for i in range(2)]
    torch.cuda.synchronize()
    got, errors = [None, None], []

    def run(i):
        try:
            st = torch.cuda.Stream()
            with torch.cuda.stream(st):
                for _ in range(50):
                    got[i] = work(i)
                st.synchronize()
        except Exception as e:   # surfaced below: an exception in a thread would otherwise pass silently
            errors.append(e)

    threads = [threading.Thread(target=run, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i in range(2):
        for a, b in zip(got[i], want[i]):
            assert torch.equal(a.view(torch.int16), b.view(torch.int16))

