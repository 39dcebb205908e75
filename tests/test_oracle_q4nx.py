"""Pins of the Q4NX / Q4_0 oracle (oracle/q4nx.py) and of the host module against it.

None of these retype the oracle's formulas: the block layout is checked against bytes written
one by one from the layout comment of programming_examples/fused_decode/proj_qmm_pack.py:4-9,
the quantisers against their defining properties, the dequant against scalar arithmetic on
Python floats, the stream orders against hand-enumerated cases.
"""
import struct

import numpy as np
import pytest

from oracle import q4nx as oq
from oracle.bf16 import bf16_bits_to_f32, f32_to_bf16_bits


def _rand(M, K, seed):
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 16, (M, K), dtype=np.uint8)
    s = f32_to_bf16_bits((np.abs(rng.standard_normal((M, K // 32))) * 0.01 + 1e-3).astype(np.float32))
    m = f32_to_bf16_bits((rng.standard_normal((M, K // 32)) * 0.05).astype(np.float32))
    return q, s, m


def test_block_size_and_offsets():
    assert oq.BLOCK_BYTES == 5120 == 2 * 2560
    assert oq.N_GROUPS == 8 and oq.ROW_GROUPS == 2


def test_block_bytes_written_by_hand():
    """q[r, c] = (r + 3 c) % 16, scale[r, g] = bits 0x3C00 + 8 g + r, min = 0xBC00 + ... ; every byte
    of the block follows from the documented layout."""
    q = np.fromfunction(lambda r, c: (r + 3 * c) % 16, (32, 256), dtype=np.int64).astype(np.uint8)
    s = np.fromfunction(lambda r, g: 0x3C00 + 32 * g + r, (32, 8), dtype=np.int64).astype(np.uint16)
    m = np.fromfunction(lambda r, g: 0xBC00 + 32 * g + r, (32, 8), dtype=np.int64).astype(np.uint16)
    want = bytearray(5120)
    for g in range(8):
        for r in range(32):
            struct.pack_into("<H", want, 2 * (g * 32 + r), 0x3C00 + 32 * g + r)          # scales[g][r]
            struct.pack_into("<H", want, 512 + 2 * (g * 32 + r), 0xBC00 + 32 * g + r)    # mins[g][r]
    for rg in range(2):
        for c in range(256):
            for kk in range(8):
                even = (16 * rg + 2 * kk + 3 * c) % 16
                odd = (16 * rg + 2 * kk + 1 + 3 * c) % 16
                want[1024 + (rg * 256 + c) * 8 + kk] = (odd << 4) | even
    want = np.frombuffer(bytes(want), dtype=np.uint8)
    assert np.array_equal(oq.pack_block_loop(q, s, m), want)
    assert np.array_equal(oq.pack_matrix(q, s, m)[0], want)


def test_matrix_is_row_block_major_and_matches_loop_packer():
    M, K = 96, 768
    q, s, m = _rand(M, K, 1)
    blocks = oq.pack_matrix(q, s, m)
    assert blocks.shape == (3 * 3, 5120)
    for bi in range(3):
        for bj in range(3):
            one = oq.pack_block_loop(q[32 * bi:32 * bi + 32, 256 * bj:256 * bj + 256], s[32 * bi:32 * bi + 32, 8 * bj:8 * bj + 8],
                                     m[32 * bi:32 * bi + 32, 8 * bj:8 * bj + 8])
            assert np.array_equal(blocks[bi * 3 + bj], one)


def test_unpack_inverts_pack():
    M, K = 64, 512
    q, s, m = _rand(M, K, 2)
    q2, s2, m2 = oq.unpack_matrix(oq.pack_matrix(q, s, m), M, K)
    assert np.array_equal(q2, q) and np.array_equal(s2, s) and np.array_equal(m2, m)


def _bf(bits):
    return struct.unpack("<f", struct.pack("<I", int(bits) << 16))[0]


def _f32(v):
    return struct.unpack("<f", struct.pack("<f", v))[0]


@pytest.mark.parametrize("mode", [oq.ADDITIVE, oq.SUBTRACTIVE, oq.Q4_0])
def test_dequant_against_scalar_arithmetic(mode):
    M, K = 32, 256
    q, s, m = _rand(M, K, 3 + mode)
    got = bf16_bits_to_f32(oq.dequant(oq.pack_matrix(q, s, m), M, K, mode))
    rng = np.random.default_rng(9)
    for _ in range(300):
        r, c = int(rng.integers(M)), int(rng.integers(K))
        sv, mv, qv = _bf(s[r, c // 32]), _bf(m[r, c // 32]), int(q[r, c])
        if mode == oq.ADDITIVE:
            w = _f32(_f32(sv * qv) + mv)
        elif mode == oq.SUBTRACTIVE:
            w = _f32(sv * _f32(qv - mv))
        else:
            w = _f32(sv * (qv - 16 if qv >= 8 else qv))
        want = bf16_bits_to_f32(f32_to_bf16_bits(np.float32(w)))
        assert got[r, c] == want, (r, c, mode)


def test_dequant_special_cases():
    M, K = 32, 256
    q = np.zeros((M, K), np.uint8)
    s = np.full((M, 8), 0x3F80, np.uint16)     # 1.0
    m = np.full((M, 8), 0x4040, np.uint16)     # 3.0
    blocks = oq.pack_matrix(q, s, m)
    assert np.all(bf16_bits_to_f32(oq.dequant(blocks, M, K, oq.ADDITIVE)) == 3.0)       # q = 0 -> min
    assert np.all(bf16_bits_to_f32(oq.dequant(blocks, M, K, oq.SUBTRACTIVE)) == -3.0)   # -zero point
    assert np.all(bf16_bits_to_f32(oq.dequant(blocks, M, K, oq.Q4_0)) == 0.0)
    q[:] = 15
    blocks = oq.pack_matrix(q, s, m)
    assert np.all(bf16_bits_to_f32(oq.dequant(blocks, M, K, oq.ADDITIVE)) == 18.0)
    assert np.all(bf16_bits_to_f32(oq.dequant(blocks, M, K, oq.Q4_0)) == -1.0)          # 0xF is -1


def test_requant_q4k_properties():
    rng = np.random.default_rng(4)
    W = rng.standard_normal((64, 512)).astype(np.float32)
    q, sc, mn = oq.requant_q4k(W)
    Wg = W.reshape(64, 16, 32)
    assert np.array_equal(mn, Wg.min(2))
    assert np.allclose(sc, (Wg.max(2) - Wg.min(2)) / 15.0)
    qg = q.reshape(64, 16, 32)
    assert np.all(qg[np.arange(64)[:, None], np.arange(16)[None], Wg.argmin(2)] == 0)    # the minimum maps to 0
    assert np.all(qg[np.arange(64)[:, None], np.arange(16)[None], Wg.argmax(2)] == 15)   # the maximum to 15
    err = np.abs(qg * sc[..., None] + mn[..., None] - Wg)
    assert np.all(err <= sc[..., None] * 0.5 * (1 + 1e-5))
    q0, sc0, mn0 = oq.requant_q4k(np.full((32, 256), 2.5, np.float32))                    # constant group
    assert np.all(sc0 == 1.0) and np.all(q0 == 0) and np.all(mn0 == 2.5)


def test_requant_q4_0_properties():
    rng = np.random.default_rng(5)
    W = rng.standard_normal((32, 256)).astype(np.float32)
    W[0, :32] = 0.0                       # all-zero group -> scale 1
    W[1, :32] = np.linspace(-1, 1, 32)    # +peak rounds to +8 and clips to +7
    W[2, :32] = -W[1, :32]
    q, sc = oq.requant_q4_0(W)
    signed = q.view(np.int8)
    assert sc[0, 0] == 1.0 and np.all(signed[0, :32] == 0)
    assert np.isclose(sc[1, 0], 1.0 / 8.0) and signed[1, 31] == 7 and signed[1, 0] == -8
    assert signed[2, 0] == 7 and signed[2, 31] == -8
    assert signed.min() >= -8 and signed.max() <= 7
    assert np.allclose(sc, np.where(np.abs(W.reshape(32, 8, 32)).max(2) > 0, np.abs(W.reshape(32, 8, 32)).max(2) / 8, 1.0))
    back = oq.dequant_q4_0(q, sc)
    inner = np.abs(W) < 7.5 * np.repeat(sc, 32, axis=1)         # not clipped
    assert np.all(np.abs(back - W)[inner] <= np.repeat(sc, 32, axis=1)[inner] * 0.5 * (1 + 1e-5))
    # packed as nibbles and dequantised through the block path: same values rounded to bf16
    sb = f32_to_bf16_bits(sc)
    blocks = oq.pack_matrix(q, sb, np.zeros_like(sb))
    want = f32_to_bf16_bits(signed.astype(np.float32) * np.repeat(bf16_bits_to_f32(sb), 32, axis=1))
    assert np.array_equal(oq.dequant(blocks, 32, 256, oq.Q4_0), want)


def test_cascade_order_small_cases_by_hand():
    # 4 row-blocks, 2 col-blocks, 2 x 1 cores: nbi_pc = 2.  Stream [cx][i][j][cy].
    assert oq.cascade_order(4, 2, 2, 1) == [(0, 0), (0, 1), (1, 0), (1, 1), (2, 0), (2, 1), (3, 0), (3, 1)]
    # iteration-major: gi = i * n_cores + cx * ncy + cy
    assert oq.cascade_order(4, 2, 2, 1, iter_major=True) == [(0, 0), (0, 1), (2, 0), (2, 1), (1, 0), (1, 1), (3, 0), (3, 1)]
    # 1 x 2 cores, default: gi = i * ncy + cy, cy innermost
    assert oq.cascade_order(4, 1, 1, 2) == [(0, 0), (1, 0), (2, 0), (3, 0)]
    # core-major: core cy owns rows [2 cy, 2 cy + 2)
    assert oq.cascade_order(4, 1, 1, 2, core_major=True) == [(0, 0), (2, 0), (1, 0), (3, 0)]
    # dual channel: the low half of cy for every step, then the high half
    assert oq.cascade_order(4, 1, 1, 2, dual_chan=True) == [(0, 0), (2, 0), (1, 0), (3, 0)]


@pytest.mark.parametrize("kw", [{}, {"core_major": True}, {"iter_major": True}, {"dual_chan": True},
                                {"iter_major": True, "dual_chan": True}])
def test_cascade_order_is_a_permutation(kw):
    order = oq.cascade_order(16, 3, 4, 2, **kw)
    assert sorted(order) == [(i, j) for i in range(16) for j in range(3)]


@pytest.mark.parametrize("mode", [oq.ADDITIVE, oq.SUBTRACTIVE, oq.Q4_0])
def test_gemv_reference_is_the_dense_product(mode):
    M, K = 64, 512
    q, s, m = _rand(M, K, 7 + mode)
    rng = np.random.default_rng(8)
    x = f32_to_bf16_bits(rng.standard_normal((3, K)).astype(np.float32))
    sv = np.repeat(bf16_bits_to_f32(s).astype(np.float64), 32, axis=1)
    mv = np.repeat(bf16_bits_to_f32(m).astype(np.float64), 32, axis=1)
    if mode == oq.ADDITIVE:
        W = sv * q + mv
    elif mode == oq.SUBTRACTIVE:
        W = sv * (q - mv)
    else:
        W = sv * np.where(q >= 8, q.astype(np.float64) - 16, q)
    want = bf16_bits_to_f32(x).astype(np.float64) @ W.T
    got = oq.gemv_reference(q, s, m, x, mode)
    assert np.allclose(got, want, rtol=1e-12, atol=1e-12)


# ---- host module of the product against the oracle ----

def test_host_module_matches_oracle():
    from air_hip import q4nx as hq
    M, K = 96, 512
    q, s, m = _rand(M, K, 11)
    blocks = hq.pack_blocks(q, s, m)
    assert np.array_equal(blocks, oq.pack_matrix(q, s, m))
    q2, s2, m2 = hq.unpack_blocks(blocks, M, K)
    assert np.array_equal(q2, q) and np.array_equal(s2, s) and np.array_equal(m2, m)
    assert np.array_equal(hq.pack_blocks(q, s)[:, 512:1024], np.zeros((6, 512), np.uint8))   # Q4_0: zero mins
    rng = np.random.default_rng(12)
    W = rng.standard_normal((M, K)).astype(np.float32)
    for a, b in zip(hq.requant_q4k(W), oq.requant_q4k(W)):
        assert np.array_equal(a, b)
    for a, b in zip(hq.requant_q4_0(W), oq.requant_q4_0(W)):
        assert np.array_equal(a, b)
    with pytest.raises(ValueError):
        hq.pack_blocks(q[:40], s[:40], m[:40])


@pytest.mark.parametrize("kw", [{}, {"core_major": True}, {"iter_major": True}, {"dual_chan": True},
                                {"iter_major": True, "dual_chan": True}])
def test_host_cascade_round_trip(kw):
    from air_hip import q4nx as hq
    nbi, nbj, ncx, ncy = 16, 3, 4, 2
    perm = hq.cascade_permutation(nbi, nbj, ncx, ncy, **kw)
    assert perm.tolist() == [gi * nbj + j for gi, j in oq.cascade_order(nbi, nbj, ncx, ncy, **kw)]
    q, s, m = _rand(nbi * 32, nbj * 256, 13)
    blocks = hq.pack_blocks(q, s, m)
    stream = hq.blocks_to_cascade(blocks, nbi, nbj, ncx, ncy, **kw)
    assert stream.dtype == np.int16 and stream.size == nbi * nbj * hq.BLOCK_BF16
    for pos, (gi, j) in enumerate(oq.cascade_order(nbi, nbj, ncx, ncy, **kw)):
        if pos % 7 == 0:
            assert np.array_equal(stream[pos * 2560:(pos + 1) * 2560].view(np.uint8), blocks[gi * nbj + j])
    assert np.array_equal(hq.blocks_from_cascade(stream, nbi, nbj, ncx, ncy, **kw), blocks)


def test_q4nx_bundle_reader(tmp_path):
    """A model.q4nx file written here with both header conventions."""
    import json
    from air_hip import q4nx as hq
    M, K = 64, 256
    q, s, m = _rand(M, K, 14)
    blocks = hq.pack_blocks(q, s, m)
    norm = f32_to_bf16_bits(np.linspace(0.5, 1.5, K).astype(np.float32))
    payload = blocks.tobytes() + blocks.tobytes() + norm.tobytes()
    n = blocks.nbytes
    hdr = {
        "__metadata__": {"format": "pt"},
        "a.weight": {"dtype": "Q4NX", "shape": [M, K], "data_offsets": [0, n]},
        "b.weight": {"dtype": "I8", "shape": [blocks.shape[0], 5120], "data_offsets": [n, 2 * n]},
        "norm.weight": {"dtype": "BF16", "shape": [K], "data_offsets": [2 * n, 2 * n + norm.nbytes]},
    }
    raw = json.dumps(hdr).encode()
    path = tmp_path / "model.q4nx"
    path.write_bytes(struct.pack("<Q", len(raw)) + raw + payload)
    mdl = hq.Q4nxModel(str(tmp_path))
    assert set(mdl.names()) == {"a.weight", "b.weight", "norm.weight"}
    b, mode, M2, K2 = mdl.blocks("a.weight")
    assert mode == hq.SUBTRACTIVE and (M2, K2) == (M, K) and np.array_equal(b, blocks)
    with pytest.raises(ValueError):
        mdl.blocks("b.weight")                       # packed header: the caller must give M and K
    with pytest.raises(ValueError):
        mdl.blocks("b.weight", 32, 256)              # block count does not match
    with pytest.raises(ValueError):
        mdl.blocks("a.weight", K, M)                 # disagrees with the header
    b, mode, _, _ = mdl.blocks("b.weight", M, K)
    assert mode == hq.ADDITIVE and np.array_equal(b, blocks)
    assert np.array_equal(np.asarray(mdl.bf16_bits("norm.weight")), norm)
    with pytest.raises(FileNotFoundError):
        hq.Q4nxModel(str(tmp_path / "missing"))
