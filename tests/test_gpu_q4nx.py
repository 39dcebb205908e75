"""GPU parity for the Q4NX / Q4_0 block codec: dequant and repack bit-exact against the oracle,
the GEMV within 1 bf16 ulp + 2e-3 of the float64 restatement of the reference kernel's sum
(c += (q.b) * scale + min * sum(b) per 32-column group) and inside the reference's own gate
(rtol 0.1, atol 0.05, r >= 0.999)."""
import numpy as np
import pytest
import torch

from helpers import assert_bf16_close
from oracle import awq as oawq, q4nx as oq, reference as oref
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


def make(M, K, seed, wild=False):
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 16, (M, K), dtype=np.uint8)
    if wild:   # any finite bf16 pattern of moderate exponent, both signs
        s = (rng.integers(0x3000, 0x4200, (M, K // 32)) | (rng.integers(0, 2, (M, K // 32)) << 15)).astype(np.uint16)
        m = (rng.integers(0x3000, 0x4200, (M, K // 32)) | (rng.integers(0, 2, (M, K // 32)) << 15)).astype(np.uint16)
    else:      # what a min/max quantiser of N(0, 0.02) weights produces
        s = f32_to_bf16_bits((np.abs(rng.standard_normal((M, K // 32))) * 0.003 + 1e-3).astype(np.float32))
        m = f32_to_bf16_bits((-np.abs(rng.standard_normal((M, K // 32))) * 0.02 - 0.01).astype(np.float32))
    return q, s, m


@pytest.mark.parametrize("mode", [oq.ADDITIVE, oq.SUBTRACTIVE, oq.Q4_0])
@pytest.mark.parametrize("M,K,wild", [(32, 256, True), (96, 768, False), (512, 2048, True)])
def test_dequant_bit_exact(ops, mode, M, K, wild):
    print(f"q4nx dequant mode={mode} M={M} K={K} wild={wild}", flush=True)
    q, s, m = make(M, K, M + K + mode, wild)
    blocks = oq.pack_matrix(q, s, m)
    out = ops.q4nx_dequant(dev(blocks), M, K, mode)
    torch.cuda.synchronize()
    assert np.array_equal(bits(out), oq.dequant(blocks, M, K, mode))


def test_dequant_bit_exact_llama8b_projection(ops):
    print("q4nx dequant 4096x4096", flush=True)
    M = K = 4096
    q, s, m = make(M, K, 1)
    blocks = oq.pack_matrix(q, s, m)
    out = ops.q4nx_dequant(dev(blocks), M, K, oq.ADDITIVE)
    torch.cuda.synchronize()
    assert np.array_equal(bits(out), oq.dequant(blocks, M, K, oq.ADDITIVE))


@pytest.mark.parametrize("mode", [oq.ADDITIVE, oq.SUBTRACTIVE, oq.Q4_0])
def test_repack_operands(ops, mode):
    print(f"q4nx repack mode={mode}", flush=True)
    M, K = 160, 768
    q, s, m = make(M, K, 20 + mode, wild=True)
    blocks = oq.pack_matrix(q, s, m)
    qw, sc, mn = ops.q4nx_repack(dev(blocks), M, K, mode)
    torch.cuda.synchronize()
    # qweight[k, j] holds rows 8 j .. 8 j + 7 of column k, unsigned, in the AutoAWQ nibble order
    q_u = q ^ 8 if mode == oq.Q4_0 else q
    assert np.array_equal(oawq.unpack_awq_int32(qw.cpu().numpy()), q_u.T)
    assert np.array_equal(bits(sc), s.T)
    sf, mf = bf16_bits_to_f32(s), bf16_bits_to_f32(m)
    want_m = {oq.ADDITIVE: m, oq.SUBTRACTIVE: f32_to_bf16_bits(-(sf * mf)), oq.Q4_0: f32_to_bf16_bits(-8.0 * sf)}[mode]
    assert np.array_equal(bits(mn), want_m.T)


def _gemm_case(ops, rows, M, K, seed, mode=oq.ADDITIVE, residual=False):
    print(f"q4nx gemm rows={rows} M={M} K={K} mode={mode} residual={residual}", flush=True)
    q, s, m = make(M, K, seed)
    rng = np.random.default_rng(seed + 1)
    x = f32_to_bf16_bits(rng.standard_normal((rows, K)).astype(np.float32))
    blocks = dev(oq.pack_matrix(q, s, m))
    qw, sc, mn = ops.q4nx_repack(blocks, M, K, mode)
    res = f32_to_bf16_bits(rng.standard_normal((rows, M)).astype(np.float32)) if residual else None
    y = ops.q4nx_gemm(dev(x), qw, sc, mn, residual=dev(res) if residual else None)
    torch.cuda.synchronize()
    if mode == oq.SUBTRACTIVE:   # the kernel works on the repacked constant term bf16(-s m)
        want = oq.gemv_reference(q, s, bits(mn).T.copy(), x, oq.ADDITIVE)
    else:
        want = oq.gemv_reference(q, s, m, x, mode)
    if residual:
        want = want + bf16_bits_to_f32(res).astype(np.float64)
    got = bits(y)
    assert_bf16_close(got, want, ulps=1.0, atol=2e-3, what=f"q4nx gemm rows={rows} M={M} K={K}")
    assert oref.check_outputs(bf16_bits_to_f32(got), bf16_bits_to_f32(f32_to_bf16_bits(want.astype(np.float32))),
                              rtol=0.1, atol=0.05, min_correlation=0.999)
    return got, want


@pytest.mark.parametrize("rows", [1, 3, 4, 7, 16, 17, 40])
def test_gemm_rows(ops, rows):
    _gemm_case(ops, rows, 512, 1024, seed=rows)


@pytest.mark.parametrize("M,K", [(32, 256), (2048, 2048), (1024, 4096), (4096, 14336), (3104, 1280)])
def test_gemv_shapes(ops, M, K):
    _gemm_case(ops, 1, M, K, seed=M + K)


@pytest.mark.parametrize("mode", [oq.SUBTRACTIVE, oq.Q4_0])
def test_gemv_other_conventions(ops, mode):
    _gemm_case(ops, 1, 2048, 2048, seed=30 + mode, mode=mode)


def test_gemv_with_residual(ops):
    _gemm_case(ops, 1, 4096, 4096, seed=40, residual=True)
    _gemm_case(ops, 5, 1024, 512, seed=41, residual=True)


def test_gemv_llama8b_gate_shape_properties(ops):
    """N = 14336 outputs from K = 4096 inputs (the Q4NX Llama-3.1-8B gate projection): against the
    oracle, then determinism, linearity in x (exact for a power-of-two factor) and column independence."""
    M, K = 14336, 4096
    got, want = _gemm_case(ops, 1, M, K, seed=50)
    q, s, m = make(M, K, 50)
    rng = np.random.default_rng(51)
    x = f32_to_bf16_bits(rng.standard_normal((1, K)).astype(np.float32))
    blocks = dev(oq.pack_matrix(q, s, m))
    qw, sc, mn = ops.q4nx_repack(blocks, M, K, oq.ADDITIVE)
    y1 = bits(ops.q4nx_gemm(dev(x), qw, sc, mn))
    x2 = f32_to_bf16_bits(bf16_bits_to_f32(x) * 2.0)
    y2 = bits(ops.q4nx_gemm(dev(x2), qw, sc, mn))
    torch.cuda.synchronize()
    assert np.array_equal(y1, got)                                                    # deterministic
    assert np.array_equal(bf16_bits_to_f32(y2), bf16_bits_to_f32(y1) * 2.0)
    # the first 2048 output features alone (a different K-split, so a different summation order)
    qw_h, sc_h, mn_h = ops.q4nx_repack(blocks[:(2048 // 32) * (K // 256)].contiguous(), 2048, K, oq.ADDITIVE)
    yh = bits(ops.q4nx_gemm(dev(x), qw_h, sc_h, mn_h))
    torch.cuda.synchronize()
    assert_bf16_close(yh, want[:, :2048], ulps=1.0, atol=2e-3, what="first 2048 features alone")
    assert np.mean(yh == y1[:, :2048]) > 0.98


def test_gemv_equals_dequant_then_dense(ops):
    """Same weights through q4nx_dequant + a float64 product: the two GPU paths agree to bf16 rounding
    of the weights (reference gate), tying the repack to the dequant."""
    M, K = 1024, 2048
    q, s, m = make(M, K, 60)
    rng = np.random.default_rng(61)
    x = f32_to_bf16_bits(rng.standard_normal((1, K)).astype(np.float32))
    blocks = dev(oq.pack_matrix(q, s, m))
    W = bf16_bits_to_f32(bits(ops.q4nx_dequant(blocks, M, K, oq.ADDITIVE))).astype(np.float64)
    y = bits(ops.q4nx_gemm(dev(x), *ops.q4nx_repack(blocks, M, K, oq.ADDITIVE)))
    torch.cuda.synchronize()
    want = bf16_bits_to_f32(x).astype(np.float64) @ W.T
    assert oref.check_outputs(bf16_bits_to_f32(y), want.astype(np.float32), rtol=0.1, atol=0.05, min_correlation=0.999)


def test_argument_errors(ops):
    from air_hip import _lib
    blocks = torch.zeros((1, 5120), dtype=torch.uint8, device="cuda")
    with pytest.raises(ValueError):
        ops.q4nx_dequant(blocks, 64, 256)
    with pytest.raises(_lib.W4A16Error):
        ops.q4nx_dequant(blocks, 32, 256, mode=3)
    lib = _lib.load_library()
    assert lib.q4nx_repack(None, None, None, None, 32, 256, 0, None) == _lib.ERR_NULL
    assert lib.q4nx_dequant_bf16(blocks.data_ptr(), blocks.data_ptr(), 48, 256, 0, None) == _lib.ERR_SHAPE
    assert lib.w4a16_q4nx_gemm_bf16(blocks.data_ptr(), blocks.data_ptr(), blocks.data_ptr(), blocks.data_ptr(), None,
                                    blocks.data_ptr(), 1, 128, 32, None, 0, None) == _lib.ERR_WORKSPACE
