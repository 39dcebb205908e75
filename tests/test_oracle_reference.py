"""Pins oracle/reference.py (GEMV / GEMM / SwiGLU / FFN restatements) with
closed forms and library routines, chosen so that a dropped term, a swapped
nibble, a transposed operand or a wrong group index fails at least one."""
import numpy as np
import torch

import oracle
from oracle import awq, reference as ref
from oracle.bf16 import bf16_bits_to_f32, f32_to_bf16_bits


def _l1(M, K, gs, seed, z_lo=0, z_hi=16):
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 16, size=(M, K), dtype=np.uint8)
    a_q = (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.uint8)
    a_s = f32_to_bf16_bits(rng.uniform(0.005, 0.02, size=(K // gs, M)).astype(np.float32))
    a_z = rng.integers(z_lo, z_hi, size=(K // gs, M), dtype=np.uint8)
    b = f32_to_bf16_bits(rng.standard_normal(K).astype(np.float32))
    return q, a_q, a_s, a_z, b


def test_integer_matrix_special_case_is_exact():
    # z = 0, s = 1, small-integer x: the GEMV is an exact integer product
    M, K, gs = 24, 256, 128
    q, a_q, _, _, _ = _l1(M, K, gs, 0)
    a_s = np.full((K // gs, M), 0x3F80, np.uint16)
    a_z = np.zeros((K // gs, M), np.uint8)
    xi = np.random.default_rng(1).integers(-2, 3, K)
    b = f32_to_bf16_bits(xi.astype(np.float32))
    want = q.astype(np.int64) @ xi
    assert np.array_equal(ref.matvec_f64(a_q, a_s, a_z, b), want.astype(np.float64))
    assert np.array_equal(bf16_bits_to_f32(ref.matvec_cpu_reference_loop(a_q, a_s, a_z, b)),
                          bf16_bits_to_f32(f32_to_bf16_bits(want.astype(np.float32))))


def test_one_hot_x_returns_one_dequantised_row_bit_exact():
    M, K, gs = 16, 256, 128
    q, a_q, a_s, a_z, _ = _l1(M, K, gs, 2)
    qweight, qzeros, s = awq.l1_to_awq(a_q, a_s, a_z)
    w = awq.dequant_to_bf16(qweight, qzeros, s, gs)  # [K, M]
    for k0 in (0, 1, 127, 128, 255):   # even/odd nibble and both groups
        b = np.zeros(K, np.uint16)
        b[k0] = 0x3F80
        assert np.array_equal(ref.matvec_cpu_reference(a_q, a_s, a_z, b), w[k0])
        assert np.array_equal(ref.matvec_cpu_reference_loop(a_q, a_s, a_z, b), w[k0])


def test_constant_q_per_group_closed_form():
    # q constant within each group: y[r] = sum_g (c_g - z[g,r]) * s[g,r] * sum_{k in g} x[k]
    M, K, gs = 8, 384, 128
    rng = np.random.default_rng(3)
    cg = rng.integers(0, 16, K // gs)
    q = np.repeat(cg, gs)[None, :].repeat(M, 0).astype(np.uint8)
    a_q = (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.uint8)
    _, _, a_s, a_z, b = _l1(M, K, gs, 4)
    x = bf16_bits_to_f32(b).astype(np.float64)
    xs = x.reshape(K // gs, gs).sum(1)
    s = bf16_bits_to_f32(a_s).astype(np.float64)
    want = ((cg[:, None] - a_z.astype(np.float64)) * s * xs[:, None]).sum(0)
    assert np.allclose(ref.matvec_f64(a_q, a_s, a_z, b), want, rtol=1e-12, atol=1e-12)


def test_scalar_loop_python_vs_c_and_vs_f64():
    M, K, gs = 12, 256, 128
    _, a_q, a_s, a_z, b = _l1(M, K, gs, 5)
    py = ref.matvec_cpu_reference_loop(a_q, a_s, a_z, b)
    lib = oracle.load_c_oracle()
    out = np.zeros(M, np.uint16)
    lib.oracle_matvec_loop(a_q.ctypes.data, a_s.ctypes.data, a_z.ctypes.data, b.ctypes.data, M, K, gs, out.ctypes.data)
    assert np.array_equal(py, out)
    # sequential float32 accumulation stays within one bf16 ulp of the float64 sum
    f64 = ref.matvec_f64(a_q, a_s, a_z, b)
    assert np.all(np.abs(bf16_bits_to_f32(out) - f64) <= np.abs(f64) * 2.0**-8 + 1e-3)


def test_residual_and_down_projection_rounding_points():
    M, K, gs = 8, 256, 128
    _, a_q, a_s, a_z, b = _l1(M, K, gs, 6)
    r = f32_to_bf16_bits(np.random.default_rng(7).standard_normal(M).astype(np.float32))
    f64 = ref.matvec_f64(a_q, a_s, a_z, b)
    # matvec_add: one rounding after adding R in float32
    want = f32_to_bf16_bits(f64.astype(np.float32) + bf16_bits_to_f32(r))
    assert np.array_equal(ref.matvec_add_cpu_reference(a_q, a_s, a_z, b, r), want)
    # ld: GEMV result is rounded to bf16 BEFORE R is added, then rounded again
    raw = bf16_bits_to_f32(f32_to_bf16_bits(f64.astype(np.float32)))
    assert np.array_equal(ref.ld_cpu_reference(a_q, a_s, a_z, b, r), f32_to_bf16_bits(raw + bf16_bits_to_f32(r)))
    assert np.array_equal(ref.ld_cpu_reference(a_q, a_s, a_z, b, None), ref.matvec_cpu_reference(a_q, a_s, a_z, b))


def test_matmul_matches_matvec_rows_and_torch():
    N, K, gs, M = 32, 256, 128, 5
    _, w_q, w_s, w_z, _ = _l1(N, K, gs, 8)
    a = f32_to_bf16_bits(np.random.default_rng(9).standard_normal((M, K)).astype(np.float32))
    c64 = ref.matmul_cpu_reference(w_q, w_s, w_z, a, accumulate="f64")
    for m in range(M):
        assert np.array_equal(c64[m], ref.matvec_cpu_reference(w_q, w_s, w_z, a[m]))
    # torch float64 matmul of the dense dequantised weights (library routine, [K, N] orientation)
    qweight, qzeros, s = awq.l1_to_awq(w_q, w_s, w_z)
    w = awq.dequant_unrounded_f32(qweight, qzeros, s, gs)
    t = (torch.from_numpy(bf16_bits_to_f32(a)).double() @ torch.from_numpy(w).double()).float().numpy()
    assert np.array_equal(c64, f32_to_bf16_bits(t))
    c32 = ref.matmul_cpu_reference(w_q, w_s, w_z, a)
    assert np.max(np.abs(bf16_bits_to_f32(c32) - bf16_bits_to_f32(c64))) <= 2.0**-7 * np.max(np.abs(bf16_bits_to_f32(c64)))
    # rounded-weight variant multiplies exactly the dequant kernel's output
    wr = bf16_bits_to_f32(awq.dequant_to_bf16(qweight, qzeros, s, gs)).astype(np.float64)
    cr = f32_to_bf16_bits((bf16_bits_to_f32(a).astype(np.float64) @ wr).astype(np.float32))
    assert np.array_equal(ref.matmul_cpu_reference(w_q, w_s, w_z, a, round_weights=True, accumulate="f64"), cr)


def test_silu_identity_and_library_cross_check():
    g = np.linspace(-12, 12, 4001).astype(np.float32)
    got = ref.silu_tanh_f32(g)
    sig = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64)))
    assert np.allclose(got, sig, rtol=2e-6, atol=1e-6)
    t = torch.nn.functional.silu(torch.from_numpy(g)).numpy()
    assert np.allclose(got, t, rtol=4e-6, atol=1e-6)


def test_swiglu_rounding_points_and_interleave():
    H, K, gs = 16, 256, 128
    _, gq, gs_, gz, x = _l1(H, K, gs, 10)
    _, uq, us_, uz, _ = _l1(H, K, gs, 11)
    a_q, a_s, a_z = ref.interleave_gate_up((gq, gs_, gz), (uq, us_, uz))
    assert np.array_equal(a_q[0::2], gq) and np.array_equal(a_q[1::2], uq)
    assert np.array_equal(a_s[:, 1::2], us_) and np.array_equal(a_z[:, 0::2], gz)
    h = ref.swiglu_rms_cpu_reference(a_q, a_s, a_z, x, None)
    g = bf16_bits_to_f32(ref.matvec_cpu_reference(gq, gs_, gz, x))       # bf16 after the GEMV
    u = bf16_bits_to_f32(ref.matvec_cpu_reference(uq, us_, uz, x))
    want = f32_to_bf16_bits(ref.silu_tanh_f32(g) * u)                     # bf16 after silu * up
    assert np.array_equal(h, want)
    # RMSNorm prologue: unit weight and x with mean square 1 leaves x (up to eps) unchanged
    xn = np.where(np.arange(K) % 2 == 0, 0x3F80, 0xBF80).astype(np.uint16)
    ones = np.full(K, 0x3F80, np.uint16)
    assert np.array_equal(f32_to_bf16_bits(ref.rms_norm_bf16(xn, ones)), xn)
    h2 = ref.swiglu_rms_cpu_reference(a_q, a_s, a_z, xn, ones)
    assert np.array_equal(h2, ref.swiglu_rms_cpu_reference(a_q, a_s, a_z, xn, None))


def test_rms_norm_against_library_and_closed_forms():
    K = 512
    rng = np.random.default_rng(40)
    x = f32_to_bf16_bits(rng.standard_normal(K).astype(np.float32))
    w = f32_to_bf16_bits((rng.standard_normal(K) * 0.1 + 1.0).astype(np.float32))
    got = ref.rms_norm_bf16(x, w, eps=1e-5)
    # library routine (float64 so that its own rounding cannot matter), then one bf16 rounding
    t = torch.nn.functional.rms_norm(torch.from_numpy(bf16_bits_to_f32(x)).double(), (K,),
                                     torch.from_numpy(bf16_bits_to_f32(w)).double(), eps=1e-5)
    want = bf16_bits_to_f32(f32_to_bf16_bits(t.float().numpy()))
    assert np.mean(got != want) <= 0.01 and np.max(np.abs(got - want) / np.abs(want)) <= 2.0**-7
    # constant x = c: rstd = 1 / sqrt(c^2 + eps), n = bf16(c * rstd * w); eps matters for small c
    c = np.float32(0.0078125)
    xc = f32_to_bf16_bits(np.full(K, c, np.float32))
    n = ref.rms_norm_bf16(xc, w, eps=1e-5)
    closed = float(c) / np.sqrt(float(c) ** 2 + 1e-5) * bf16_bits_to_f32(w).astype(np.float64)
    assert np.max(np.abs(n - closed) / np.abs(closed)) <= 2.0**-8 * 1.001
    # a dropped eps or a sum instead of a mean would give 1.0 * w and w / sqrt(K)
    assert not np.allclose(n, bf16_bits_to_f32(w), rtol=1e-2)


def test_block_references_agree_and_reduce_to_their_stages():
    E, H, gs = 256, 512, 128
    _, oq, os_, oz, attn = _l1(E, E, gs, 50)
    _, gq, gs_, gz, xres = _l1(H, E, gs, 51)
    _, uq, us_, uz, _ = _l1(H, E, gs, 52)
    _, dq, ds, dz, _ = _l1(E, H, gs, 53)
    rng = np.random.default_rng(54)
    w = f32_to_bf16_bits((rng.standard_normal(E) * 0.1 + 1.0).astype(np.float32))
    res1, h, y = ref.o_gemv_ffn_staged_reference((oq, os_, oz), (gq, gs_, gz), (uq, us_, uz), (dq, ds, dz), attn, xres, w)
    # stage identities
    assert np.array_equal(res1, ref.matvec_add_cpu_reference(oq, os_, oz, attn, xres))
    a_q, a_s, a_z = ref.interleave_gate_up((gq, gs_, gz), (uq, us_, uz))
    assert np.array_equal(h, ref.swiglu_rms_cpu_reference(a_q, a_s, a_z, res1, w))
    # residual: sum + R in float64, one rounding
    want_y = ref.matvec_f64(dq, ds, dz, h) + bf16_bits_to_f32(res1)
    assert np.max(np.abs(bf16_bits_to_f32(y) - want_y)) <= np.max(np.abs(want_y)) * 2.0**-8
    # W = 0 (q == z): matvec_add returns R bit for bit
    zq = np.repeat(oz.T, gs, axis=1)                      # [out, K] nibbles equal to the zero points
    zero_q = (zq[:, 0::2] | (zq[:, 1::2] << 4)).astype(np.uint8)
    assert np.array_equal(ref.matvec_add_cpu_reference(zero_q, os_, oz, attn, xres), xres)
    # the float32 whole-block reference on bf16-dequantised weights lands on the same values
    # within the block's gate (its rounding points differ: res1 and gate/up stay float32)
    deq = lambda q, s, z: f32_to_bf16_bits(ref._dequant_l1_f64(q, s, z, q.shape[1] * 2).astype(np.float32))
    whole = ref.o_gemv_ffn_int4_reference(deq(oq, os_, oz), attn, xres, w, deq(gq, gs_, gz), deq(uq, us_, uz), deq(dq, ds, dz))
    assert ref.check_outputs(bf16_bits_to_f32(y), bf16_bits_to_f32(whole), rtol=0.05, atol=0.05, min_correlation=0.9999)
    # and against an independent float64 evaluation of the block formula
    f = lambda b: bf16_bits_to_f32(b).astype(np.float64)
    r64 = f(deq(oq, os_, oz)) @ f(attn) + f(xres)
    n64 = f(f32_to_bf16_bits((r64 / np.sqrt(np.mean(r64 * r64) + 1e-5) * f(w)).astype(np.float32)))
    g64 = f(deq(gq, gs_, gz)) @ n64
    u64 = f(deq(uq, us_, uz)) @ n64
    s64 = f(f32_to_bf16_bits((g64 / (1 + np.exp(-g64)) * u64).astype(np.float32)))
    y64 = f(deq(dq, ds, dz)) @ s64 + r64
    assert np.max(np.abs(f(whole) - y64)) <= 2.0**-7 * np.max(np.abs(y64))


def test_ffn_chain():
    H, K, gs = 256, 128, 128
    _, gq, gs_, gz, x = _l1(H, K, gs, 12)
    _, uq, us_, uz, _ = _l1(H, K, gs, 13)
    _, dq, ds, dz, _ = _l1(K, H, gs, 14)
    h, y = ref.ffn_swiglu_reference((gq, gs_, gz), (uq, us_, uz), (dq, ds, dz), x)
    assert h.shape == (H,) and y.shape == (K,)
    assert np.array_equal(y, ref.matvec_cpu_reference(dq, ds, dz, h))


def test_check_outputs_semantics():
    e = np.linspace(1, 2, 1000)
    a = e.copy()
    assert ref.check_outputs(a, e, rtol=0.1, atol=0.05, min_correlation=0.999)
    a[:5] += 1.0
    assert not ref.check_outputs(a, e, rtol=0.1, atol=0.05)
    assert ref.check_outputs(a, e, rtol=0.1, atol=0.05, max_mismatch_percentage=0.5)      # int(1000*0.5/100)=5
    assert not ref.check_outputs(a, e, rtol=0.1, atol=0.05, max_mismatch_percentage=0.49)  # int(4.9)=4
    # constant actual -> NaN correlation -> fail
    assert not ref.check_outputs(np.ones(10), np.ones(10), rtol=1, atol=1, min_correlation=0.5)


def test_prefill_block_reference_against_library_and_closed_forms():
    M, E, H, gs = 24, 256, 512, 128
    _, oq, os_, oz, _ = _l1(E, E, gs, 60)
    _, gq, gs_, gz, _ = _l1(H, E, gs, 61)
    _, uq, us_, uz, _ = _l1(H, E, gs, 62)
    _, dq, ds, dz, _ = _l1(E, H, gs, 63)
    rng = np.random.default_rng(64)
    attn = f32_to_bf16_bits(rng.standard_normal((M, E)).astype(np.float32))
    xres = f32_to_bf16_bits(rng.standard_normal((M, E)).astype(np.float32))
    w = f32_to_bf16_bits((rng.standard_normal(E) * 0.1 + 1.0).astype(np.float32))
    wo, wg, wu, wd = (oq, os_, oz), (gq, gs_, gz), (uq, us_, uz), (dq, ds, dz)
    out, res1, h = ref.o_ffn_int4_prefill_reference(wo, wg, wu, wd, attn, xres, w)

    # the same chain with library routines in float64 and one rounding per stage
    def dense(l1, k):
        return torch.from_numpy(ref._dequant_l1_f64(*l1, k).T.copy())          # [K, N] float64

    def rnd(t):
        return torch.from_numpy(bf16_bits_to_f32(f32_to_bf16_bits(t.float().numpy()))).double()

    a, r = torch.from_numpy(bf16_bits_to_f32(attn)).double(), torch.from_numpy(bf16_bits_to_f32(xres)).double()
    res1_t = rnd(rnd(a @ dense(wo, E)) + r)
    n_t = rnd(torch.nn.functional.rms_norm(res1_t, (E,), torch.from_numpy(bf16_bits_to_f32(w)).double(), eps=1e-5))
    g_t, u_t = rnd(n_t @ dense(wg, E)), rnd(n_t @ dense(wu, E))
    h_t = rnd(torch.nn.functional.silu(g_t) * u_t)
    out_t = rnd(rnd(h_t @ dense(wd, H)) + res1_t)
    for got, want, name in ((res1, res1_t, "res1"), (h, h_t, "h"), (out, out_t, "out")):
        g = bf16_bits_to_f32(got).astype(np.float64)
        wv = want.numpy()
        # float32 BLAS sums and one-ulp flips upstream: a few bf16 ulps of the tensor's scale, almost everywhere equal
        assert np.max(np.abs(g - wv)) <= 4 * 2.0**-8 * np.max(np.abs(wv)), name
        assert np.mean(g != wv) < 0.1, name
    # Wo = 0 (z = q): res1 = x_residual exactly; Wdown = 0: out = res1
    zo = (np.zeros_like(oq), os_, np.zeros_like(oz))
    zd = (np.zeros_like(dq), ds, np.zeros_like(dz))
    out0, res10, _ = ref.o_ffn_int4_prefill_reference(zo, wg, wu, zd, attn, xres, w)
    assert np.array_equal(res10, xres) and np.array_equal(out0, xres)
    # rows are independent: a row subset gives the same rows
    out_s, res1_s, h_s = ref.o_ffn_int4_prefill_reference(wo, wg, wu, wd, attn[5:9], xres[5:9], w)
    assert np.array_equal(out_s, out[5:9]) and np.array_equal(h_s, h[5:9])
    # the row-wise norm against its closed form for constant rows (a sum instead of a mean would give 1 / sqrt(E))
    c = np.float32(0.0078125)
    n = bf16_bits_to_f32(ref.rms_norm_rows_bf16(f32_to_bf16_bits(np.full((3, E), c, np.float32)), np.full(E, 0x3F80, np.uint16)))
    assert np.max(np.abs(n - float(c) / np.sqrt(float(c) ** 2 + 1e-5))) <= 2.0**-8
    # gate = 0 gives h = 0 whatever up is (silu(0) = 0); the tanh form used by the decode kernels agrees with this one
    gvals = np.linspace(-8, 8, 101).astype(np.float32)
    assert np.allclose(gvals / (1 + np.exp(-gvals)), ref.silu_tanh_f32(gvals), rtol=1e-5, atol=1e-6)
