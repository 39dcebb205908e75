"""Pins oracle/awq.py: nibble order, exact dequant, repack identities.

Each check is independent of the oracle's own formula: a hand-computed word, a
scalar packer written from the description of the format, exact rational
arithmetic, and the identities the reference's self-test states
(programming_examples/llms/llama32_1b_int4/awq_repacker.py:166-206).
"""
from fractions import Fraction

import numpy as np

from oracle import awq
from oracle.bf16 import bf16_bits_to_f32, f32_to_bf16_bits


def test_known_word_unpacks_to_documented_order():
    # nibble value == its bit-position index; natural column j is at position [0,4,1,5,2,6,3,7][j]
    w = np.array([[0x76543210]], dtype=np.uint32).view(np.int32)
    assert awq.unpack_awq_int32(w).tolist() == [[0, 4, 1, 5, 2, 6, 3, 7]]
    # sign bit set: the top nibble must come out as 0xF, not be sign-smeared
    w = np.array([[0xF0000000]], dtype=np.uint32).view(np.int32)
    assert awq.unpack_awq_int32(w).tolist() == [[0, 0, 0, 0, 0, 0, 0, 15]]


def _scalar_pack(nibs):
    """Bit position 4*i holds column 8*b + ORDER[i] - written as a scalar loop."""
    order = [0, 2, 4, 6, 1, 3, 5, 7]
    rows, n = nibs.shape
    out = np.zeros((rows, n // 8), dtype=np.uint32)
    for r in range(rows):
        for b in range(n // 8):
            word = 0
            for i in range(8):
                word |= int(nibs[r, 8 * b + order[i]]) << (4 * i)
            out[r, b] = word
    return out.view(np.int32)


def test_pack_unpack_round_trip_against_scalar_packer():
    rng = np.random.default_rng(1)
    nibs = rng.integers(0, 16, size=(5, 48), dtype=np.uint8)
    packed = _scalar_pack(nibs)
    assert np.array_equal(awq.pack_awq_int32(nibs), packed)
    assert np.array_equal(awq.unpack_awq_int32(packed), nibs)
    # distinct values per column of one block
    blk = np.arange(8, dtype=np.uint8)[None, :]
    assert np.array_equal(awq.unpack_awq_int32(_scalar_pack(blk)), blk)


def _exact_bf16_rne(fr):
    """Round a Fraction to bf16 (8 significant bits, RNE); returns float."""
    if fr == 0:
        return 0.0
    sign = -1 if fr < 0 else 1
    a = abs(fr)
    e = 0
    while a >= 2:
        a /= 2
        e += 1
    while a < 1:
        a *= 2
        e -= 1
    scaled = a * 128  # in [128, 256)
    lo = scaled.numerator // scaled.denominator
    rem = scaled - lo
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and lo % 2 == 1):
        lo += 1
    return sign * float(Fraction(lo, 128) * Fraction(2) ** e)


def test_dequant_exhaustive_qz_against_exact_rationals():
    # all 16x16 (q, z) pairs x a sweep of scale bit patterns, incl. the tie case 3 * 0x3F81
    scale_bits = np.array([0x3F81, 0x3C23, 0x3CA4, 0x3A83, 0x3D4D, 0x3F80, 0x3BFF, 0x3C01], dtype=np.uint16)
    n = 8 * len(scale_bits)
    K = 16
    q = np.tile(np.arange(16, dtype=np.uint8)[:, None], (1, n))
    for z0 in range(16):
        z = np.full((1, n), z0, dtype=np.uint8)
        s = np.repeat(scale_bits, 8)[None, :]
        out = awq.dequant_to_bf16(awq.pack_awq_int32(q), awq.pack_awq_int32(z), s, K)
        got = bf16_bits_to_f32(out)
        for k in range(16):
            for j, sb in enumerate(scale_bits):
                sv = Fraction(float(bf16_bits_to_f32(np.array([sb], np.uint16))[0]))
                want = _exact_bf16_rne((k - z0) * sv)
                assert got[k, 8 * j] == want, (k, z0, hex(sb))
    # q == z gives +0.0 for a positive scale
    out = awq.dequant_to_bf16(awq.pack_awq_int32(np.full((16, 8), 5, np.uint8)),
                              awq.pack_awq_int32(np.full((1, 8), 5, np.uint8)),
                              np.full((1, 8), 0x3C23, np.uint16), 16)
    assert np.all(out == 0)
    # the documented tie: (q - z) = 3, s = 0x3F81 -> 0x4042
    q3 = np.full((16, 8), 10, np.uint8)
    z3 = np.full((1, 8), 7, np.uint8)
    out = awq.dequant_to_bf16(awq.pack_awq_int32(q3), awq.pack_awq_int32(z3), np.full((1, 8), 0x3F81, np.uint16), 16)
    assert np.all(out == 0x4042)


def _synthetic(K, N, gs, seed):
    rng = np.random.default_rng(seed)
    nibs = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // gs, N), dtype=np.uint8)
    s = f32_to_bf16_bits(rng.uniform(0.005, 0.02, size=(K // gs, N)).astype(np.float32))
    return nibs, z, s


def test_self_test_identities_a_and_b():
    K, N, gs = 512, 128, 128
    nibs, z, s = _synthetic(K, N, gs, 42)
    qweight, qzeros = awq.pack_awq_int32(nibs), awq.pack_awq_int32(z)
    # (a) unpack round trip
    assert np.array_equal(awq.unpack_awq_int32(qweight), nibs)
    assert np.array_equal(awq.unpack_awq_int32(qzeros), z)
    # (b) dense dequant == dequant of the repacked kernel-side arrays, bit for bit
    w_dense = awq.dequant_to_bf16(qweight, qzeros, s, gs)
    a_q, a_s, a_z = awq.repack_hf_awq_linear(qweight, qzeros, s, gs)
    assert a_q.shape == (N, K // 2) and a_s.shape == (K // gs, N) and a_z.shape == (K // gs, N)
    n_from = awq.l1_unpack_nibbles(a_q)
    w_rep = (n_from - np.repeat(a_z.astype(np.int32), gs, axis=0).T).astype(np.float32) * \
        np.repeat(bf16_bits_to_f32(a_s), gs, axis=0).T
    assert np.array_equal(w_dense, f32_to_bf16_bits(w_rep).T)
    # inverse converter
    qw2, qz2, s2 = awq.l1_to_awq(a_q, a_s, a_z)
    assert np.array_equal(qw2, qweight) and np.array_equal(qz2, qzeros) and np.array_equal(s2, s)


def test_dequant_shape_errors_match_reference_behaviour():
    nibs, z, s = _synthetic(256, 16, 128, 3)
    import pytest
    with pytest.raises(ValueError):
        awq.dequant_to_bf16(awq.pack_awq_int32(nibs), awq.pack_awq_int32(z[:1]), s, 128)
    with pytest.raises(ValueError):
        awq.repack_hf_awq_linear(awq.pack_awq_int32(nibs), awq.pack_awq_int32(z), s[:, :8], 128)


def test_dequant_1d_matches_dense_form_and_c_restatement():
    import ctypes
    import oracle
    rng = np.random.default_rng(0)
    n, gs = 1024, 128
    q = rng.integers(0, 16, n).astype(np.uint8)
    s = f32_to_bf16_bits(rng.uniform(0.01, 0.1, n // gs).astype(np.float32))
    z = rng.integers(7, 10, n // gs).astype(np.uint8)
    out = awq.dequant_1d(q, s, z, gs)
    # same numbers laid out as a K x 8 AWQ matrix (every column uses the same scale per group)
    K, N = n, 8
    nibs = np.tile(q[:, None], (1, N))
    w = awq.dequant_to_bf16(awq.pack_awq_int32(nibs), awq.pack_awq_int32(np.tile(z[:, None], (1, N))),
                            np.tile(s[:, None], (1, N)), gs)
    assert np.array_equal(w[:, 3], out)
    lib = oracle.load_c_oracle()
    qw = np.ascontiguousarray(awq.pack_awq_int32(nibs))
    qz = np.ascontiguousarray(awq.pack_awq_int32(np.tile(z[:, None], (1, N))))
    sc = np.ascontiguousarray(np.tile(s[:, None], (1, N)))
    got = np.zeros((K, N), np.uint16)
    lib.oracle_dequant_awq(qw.ctypes.data, qz.ctypes.data, sc.ctypes.data, K, N, gs, got.ctypes.data)
    assert np.array_equal(got, w)


def test_fake_quantize_known_answers_and_bounds():
    """fake_quantize_awq_int4 (awq_pack.py:287-316).  A ramp w_i = (i % 16 - 8) / 4 has min -2, max 1.75, so
    scale = 3.75 / 15 = 1/4 exactly, zero = 8 and q_i = i % 16: every output follows by hand.  Then properties the
    definition fixes for any group that straddles zero: the minimum quantises to 0 and the maximum to 15, and inside
    the representable range the reconstruction error is at most half a step."""
    gs = 128
    ramp = ((np.arange(2 * gs) % 16 - 8) / 4.0).astype(np.float32)
    w = np.stack([ramp, -ramp[::-1] * 0 + ramp * 2])          # row 1: the same ramp doubled (scale 1/2)
    a_q, s_bits, z = awq.fake_quantize_awq_int4_loop(w, gs)
    nib = awq.l1_unpack_nibbles(a_q)
    assert np.array_equal(nib[0], np.arange(2 * gs) % 16) and np.array_equal(nib[1], np.arange(2 * gs) % 16)
    assert s_bits.shape == (2, 2) and z.shape == (2, 2)        # [groups, rows]
    assert np.array_equal(s_bits[:, 0], [0x3E80, 0x3E80]) and np.array_equal(s_bits[:, 1], [0x3F00, 0x3F00])
    assert np.all(z == 8)
    assert a_q[0, 0] == (0 | (1 << 4)) and a_q[0, 7] == (14 | (15 << 4))   # even k in the low nibble
    # the dequantised ramp is the ramp
    back = (nib[0].astype(np.float64) - 8) * 0.25
    assert np.array_equal(back, ramp.astype(np.float64))
    # random groups straddling zero
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((6, 3 * gs)) * rng.uniform(0.01, 3.0, (6, 1))).astype(np.float32)
    a_q, s_bits, z = awq.fake_quantize_awq_int4_loop(w, gs)
    nib = awq.l1_unpack_nibbles(a_q).reshape(6, 3, gs)
    wg = w.reshape(6, 3, gs)
    step = ((wg.max(axis=2) - wg.min(axis=2)) / np.float32(15.0)).astype(np.float64)
    assert np.all(np.take_along_axis(nib, wg.argmin(axis=2)[:, :, None], 2)[:, :, 0] == 0)
    assert np.all(np.take_along_axis(nib, wg.argmax(axis=2)[:, :, None], 2)[:, :, 0] == 15)
    recon = (nib - z.T[:, :, None].astype(np.float64)) * step[:, :, None]
    inside = (nib > 0) & (nib < 15)
    assert np.all(np.abs(recon - wg)[inside] <= 0.5 * np.broadcast_to(step[:, :, None], wg.shape)[inside] * (1 + 1e-5))
    # scales leave as bf16 of the float32 step
    assert np.array_equal(s_bits.T, f32_to_bf16_bits(step.astype(np.float32)))
    # a constant group: step 1e-7, everything clips to one end
    a_q, s_bits, z = awq.fake_quantize_awq_int4_loop(np.full((1, gs), 0.5, np.float32), gs)
    assert s_bits[0, 0] == f32_to_bf16_bits(np.float32([1e-7]))[0] and z[0, 0] == 0 and np.all(awq.l1_unpack_nibbles(a_q) == 15)
    a_q, s_bits, z = awq.fake_quantize_awq_int4_loop(np.full((1, gs), -0.5, np.float32), gs)
    assert z[0, 0] == 15 and np.all(awq.l1_unpack_nibbles(a_q) == 0)
    # an all-positive group: the zero point clips to 0 and the minimum lands above 0
    a_q, s_bits, z = awq.fake_quantize_awq_int4_loop(np.linspace(1.0, 2.5, gs, dtype=np.float32)[None], gs)
    assert z[0, 0] == 0 and awq.l1_unpack_nibbles(a_q)[0, 0] == 10 and awq.l1_unpack_nibbles(a_q)[0, -1] == 15
