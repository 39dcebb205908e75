"""Pins for the decode-block oracle: each check fails for a plausible slip (swapped sin/cos,
wrong sign, interleaved instead of half-split pairing, missing scale, wrong head grouping)."""
import numpy as np
import torch

from oracle import decode as dec
from oracle.bf16 import bf16_bits_to_f32, f32_to_bf16_bits


def test_rope_lut_closed_forms():
    lut = bf16_bits_to_f32(dec.generate_rope_lut(64, 500000.0, 33))
    assert lut.shape == (33, 64)
    assert np.all(lut[0, :32] == 1.0) and np.all(lut[0, 32:] == 0.0)          # position 0: cos 1, sin 0
    r = lambda v: bf16_bits_to_f32(f32_to_bf16_bits(np.float32(v)))
    assert lut[1, 0] == r(np.cos(1.0)) and lut[1, 32] == r(np.sin(1.0))       # index 0: frequency 1
    assert lut[5, 16] == r(np.cos(5.0 * 500000.0 ** -0.5))                     # i = 16: base^(-32/64)
    assert lut[7, 32 + 31] == r(np.sin(7.0 * 500000.0 ** (-62.0 / 64.0)))


def test_rope_is_the_complex_rotation_of_half_split_pairs():
    rng = np.random.default_rng(0)
    x = f32_to_bf16_bits(rng.standard_normal((5, 64)).astype(np.float32))
    lut = dec.generate_rope_lut(64, 10000.0, 40)
    got = bf16_bits_to_f32(dec.rope_halfsplit(x, lut[17]))
    xf = bf16_bits_to_f32(x).astype(np.float64)
    l = bf16_bits_to_f32(lut[17]).astype(np.float64)
    z = (xf[:, :32] + 1j * xf[:, 32:]) * (l[:32] + 1j * l[32:])               # pair (i, i + 32)
    want = np.concatenate([z.real, z.imag], axis=1)
    assert np.max(np.abs(got - want)) <= 2.0**-8 * np.max(np.abs(want)) + 1e-6
    # position 0 is the identity, bit for bit
    assert np.array_equal(dec.rope_halfsplit(x, lut[0]), x)
    # an interleaved pairing (2i, 2i + 1) would differ
    zi = (xf[:, 0::2] + 1j * xf[:, 1::2]) * (l[:32] + 1j * l[32:])
    assert np.max(np.abs(got[:, :32] - zi.real)) > 0.1


def test_attention_against_library_and_closed_forms():
    n_heads, n_kv, hd, max_seq, pos = 8, 2, 64, 48, 36
    rng = np.random.default_rng(1)
    q = f32_to_bf16_bits(rng.standard_normal(n_heads * hd).astype(np.float32))
    k = f32_to_bf16_bits(rng.standard_normal((n_kv, max_seq, hd)).astype(np.float32))
    v = f32_to_bf16_bits(rng.standard_normal((n_kv, max_seq, hd)).astype(np.float32))
    got = bf16_bits_to_f32(dec.decode_attention_cpu(q, k, v, pos, n_heads, n_kv, hd)).reshape(n_heads, hd)
    tq = torch.from_numpy(bf16_bits_to_f32(q)).double().reshape(1, n_heads, 1, hd)
    tk = torch.from_numpy(bf16_bits_to_f32(k[:, :pos + 1])).double().repeat_interleave(n_heads // n_kv, dim=0)[None]
    tv = torch.from_numpy(bf16_bits_to_f32(v[:, :pos + 1])).double().repeat_interleave(n_heads // n_kv, dim=0)[None]
    want = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv)[0, :, 0].numpy()
    assert np.max(np.abs(got - want)) <= 2.0**-8 * np.max(np.abs(want)) + 1e-5
    # positions beyond current_pos are ignored
    k2, v2 = k.copy(), v.copy()
    k2[:, pos + 1:] = 0x7F80
    v2[:, pos + 1:] = 0x7F80
    assert np.array_equal(dec.decode_attention_cpu(q, k2, v2, pos, n_heads, n_kv, hd), f32_to_bf16_bits(got.reshape(-1)))
    # seq_len 1: the output is v[kv head of h][0] for every head
    one = dec.decode_attention_cpu(q, k, v, 0, n_heads, n_kv, hd).reshape(n_heads, hd)
    for h in range(n_heads):
        assert np.array_equal(one[h], v[h // 4, 0])
    # equal keys: uniform softmax, the output is the mean of the values
    ke = np.broadcast_to(k[:, :1], k.shape).copy()
    me = bf16_bits_to_f32(dec.decode_attention_cpu(q, ke, v, pos, n_heads, n_kv, hd)).reshape(n_heads, hd)
    mean = bf16_bits_to_f32(v[:, :pos + 1]).astype(np.float64).mean(axis=1)
    assert np.max(np.abs(me - mean[np.arange(n_heads) // 4])) <= 2.0**-8 * np.abs(mean).max() + 1e-4


def test_lm_head_tail_against_library_and_closed_forms():
    V, E = 96, 512
    rng = np.random.default_rng(70)
    x = f32_to_bf16_bits((rng.standard_normal(E) * 3.0).astype(np.float32))
    nw = f32_to_bf16_bits((rng.standard_normal(E) * 0.1 + 1.0).astype(np.float32))
    W = f32_to_bf16_bits((rng.standard_normal((V, E)) * 0.05).astype(np.float32))
    logits, best = dec.lm_head_reference(x, nw, W, eps=1e-5)
    # library routines in float64, one rounding per stage
    xt, wt = torch.from_numpy(bf16_bits_to_f32(x)).double(), torch.from_numpy(bf16_bits_to_f32(nw)).double()
    n_lib = bf16_bits_to_f32(f32_to_bf16_bits(torch.nn.functional.rms_norm(xt, (E,), wt, eps=1e-5).float().numpy()))
    n_got = bf16_bits_to_f32(dec.final_rms_norm(x, nw))
    assert np.mean(n_got != n_lib) <= 0.01 and np.max(np.abs(n_got - n_lib) / np.abs(n_lib)) <= 2.0**-7
    l_lib = torch.from_numpy(bf16_bits_to_f32(W)).double() @ torch.from_numpy(n_got).double()
    assert np.array_equal(logits, f32_to_bf16_bits(l_lib.float().numpy()))
    assert best == int(torch.argmax(l_lib.float().bfloat16().float()))
    # one-hot rows pick elements of the normalised vector: row v = unit vector e_(5 v mod E)
    idx = (5 * np.arange(V)) % E
    onehot = np.zeros((V, E), np.uint16)
    onehot[np.arange(V), idx] = 0x3F80
    l1, b1 = dec.lm_head_reference(x, nw, onehot)
    assert np.array_equal(l1, dec.final_rms_norm(x, nw)[idx])
    assert b1 == int(np.argmax(n_got[idx]))
    # a transposed operand or a dropped norm would fail here: without the norm the logits are x itself
    l2, _ = dec.lm_head_reference(x, None, onehot)
    assert np.array_equal(l2, x[idx]) and not np.array_equal(l1, l2)
    # constant x = c with unit weight: normed = c / sqrt(c^2 + eps); a sum instead of a mean gives 1 / sqrt(E)
    c = np.float32(0.0078125)
    n = bf16_bits_to_f32(dec.final_rms_norm(f32_to_bf16_bits(np.full(E, c, np.float32)), np.full(E, 0x3F80, np.uint16)))
    closed = float(c) / np.sqrt(float(c) ** 2 + 1e-5)
    assert np.max(np.abs(n - closed)) <= 2.0**-8 * closed * 1.001
    # tied rows: the first of the equal maxima wins, also when the tie is between +0 and -0
    Wt = W.copy()
    Wt[40] = Wt[7]
    Wt[80] = Wt[7]
    lt, _ = dec.lm_head_reference(x, nw, Wt)
    assert lt[40] == lt[7] == lt[80]
    big = f32_to_bf16_bits(bf16_bits_to_f32(dec.final_rms_norm(x, nw)) * np.float32(0.25))   # row = 0.25 * normed: the largest possible logit direction
    Wt[7] = Wt[40] = Wt[80] = big
    assert dec.lm_head_reference(x, nw, Wt)[1] == 7
    zeros = np.zeros((4, E), np.uint16)
    zeros[0, 0] = 0x8000          # -0 * x: logits -0 or +0, all equal as floats
    assert dec.lm_head_reference(x, nw, zeros)[1] == 0


def _l1(M, K, gs, seed):
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 16, size=(M, K), dtype=np.uint8)
    a_q = (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.uint8)
    a_s = f32_to_bf16_bits(rng.uniform(0.005, 0.02, size=(K // gs, M)).astype(np.float32))
    a_z = rng.integers(0, 16, size=(K // gs, M), dtype=np.uint8)
    return a_q, a_s, a_z


def test_prefill_qkv_rope_reference_against_its_stages_and_the_decode_step():
    from oracle import reference as ref

    M, E, nh, nkv, hd, pos0 = 6, 256, 4, 2, 64, 3
    rng = np.random.default_rng(80)
    x = f32_to_bf16_bits(rng.standard_normal((M, E)).astype(np.float32))
    nw = f32_to_bf16_bits((rng.standard_normal(E) * 0.1 + 1.0).astype(np.float32))
    wq, wk, wv = _l1(nh * hd, E, 128, 81), _l1(nkv * hd, E, 128, 82), _l1(nkv * hd, E, 128, 83)
    lut = dec.generate_rope_lut(hd, 500000.0, 16)
    out = dec.prefill_rms_qkv_rope_reference(x, nw, wq, wk, wv, lut, pos0, nh, nkv, hd)
    assert out.shape == (M, (nh + 2 * nkv) * hd)
    # per-row rotation: the complex rotation by that row's angles; equal LUT rows reduce to rope_halfsplit
    xr = f32_to_bf16_bits(rng.standard_normal((5, hd)).astype(np.float32))
    rows = lut[[1, 4, 4, 9, 0]]
    got = bf16_bits_to_f32(dec.rope_rows(xr, rows))
    xf, l = bf16_bits_to_f32(xr).astype(np.float64), bf16_bits_to_f32(rows).astype(np.float64)
    z = (xf[:, :32] + 1j * xf[:, 32:]) * (l[:, :32] + 1j * l[:, 32:])
    assert np.max(np.abs(got - np.concatenate([z.real, z.imag], axis=1))) <= 2.0**-8 * np.max(np.abs(xf)) * 1.5
    assert np.array_equal(dec.rope_rows(xr, np.repeat(lut[7:8], 5, axis=0)), dec.rope_halfsplit(xr, lut[7]))
    assert np.array_equal(dec.rope_rows(xr, rows)[4], xr[4])                      # position 0 is the identity
    # stages: V is the plain product of the normalised rows; Q of row m is rope(product) with LUT row pos0 + m
    normed = ref.rms_norm_rows_bf16(x, nw)
    assert np.array_equal(out[:, (nh + nkv) * hd:], ref.matmul_cpu_reference(*wv, normed))
    qm = ref.matmul_cpu_reference(*wq, normed)
    for m in (0, M - 1):
        assert np.array_equal(out[m, :nh * hd].reshape(nh, hd), dec.rope_halfsplit(qm[m].reshape(nh, hd), lut[pos0 + m]))
    # a single row is what the decode-step reference computes for that token (GEMV = one-row GEMM up to
    # the float32 BLAS summation order and the norm's x * rstd against x / rms: a few one-ulp flips)
    m = 2
    one = dec.rms_qkv_rope_reference(x[m], nw, wq, wk, wv, lut[pos0 + m], nh, nkv, hd)
    a, b = bf16_bits_to_f32(np.concatenate([np.ravel(t) for t in one])), bf16_bits_to_f32(out[m])
    assert a.shape == b.shape and np.max(np.abs(a - b)) <= 2.0**-6 * np.max(np.abs(b)) and np.mean(a != b) < 0.2


def test_prefill_attention_reference_against_library_and_the_decode_reference():
    M, nh, nkv, hd = 23, 4, 2, 64
    rng = np.random.default_rng(90)
    q = f32_to_bf16_bits(rng.standard_normal((M, nh * hd)).astype(np.float32))
    k = f32_to_bf16_bits(rng.standard_normal((M, nkv * hd)).astype(np.float32))
    v = f32_to_bf16_bits(rng.standard_normal((M, nkv * hd)).astype(np.float32))
    got = dec.prefill_attention_reference(q, k, v, nh, nkv)
    t = lambda b, n: torch.from_numpy(bf16_bits_to_f32(b)).double().reshape(M, n, hd).transpose(0, 1)
    want = torch.nn.functional.scaled_dot_product_attention(t(q, nh), t(k, nkv).repeat_interleave(nh // nkv, dim=0),
                                                            t(v, nkv).repeat_interleave(nh // nkv, dim=0), is_causal=True)
    want = want.transpose(0, 1).reshape(M, nh * hd).numpy()
    assert np.max(np.abs(got - want)) <= 1e-5
    # the first token only sees itself: its output is its own V row, for every query head of the group
    assert np.allclose(got[0].reshape(nh, hd), bf16_bits_to_f32(v[0]).reshape(nkv, hd).repeat(nh // nkv, axis=0), atol=1e-6)
    # row m is what the single-query decode attention gives for position m over the cache of rows 0..m
    m = 11
    kc = k.reshape(M, nkv, hd).transpose(1, 0, 2).copy()
    vc = v.reshape(M, nkv, hd).transpose(1, 0, 2).copy()
    one = bf16_bits_to_f32(dec.decode_attention_cpu(q[m], kc, vc, m, nh, nkv, hd))
    assert np.max(np.abs(one - got[m])) <= 2.0**-8 * np.max(np.abs(got[m])) + 1e-6
    # a non-causal softmax would let row 0 see everything
    assert not np.allclose(got[0], got[M - 1])
