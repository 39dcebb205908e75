"""Stream order (the decode kernels' device layout) on the host: size, an element followed by hand to its
byte, nibble and field, the round trip, and what a short last block holds."""
import numpy as np
import pytest

from air_hip import awq, bf16


def _random(K, N, seed):
    rng = np.random.default_rng(seed)
    G = K // 128
    q = rng.integers(0, 16, (K, N), dtype=np.uint8)
    z = rng.integers(0, 16, (G, N), dtype=np.uint8)
    s = rng.integers(0, 65536, (G, N)).astype(np.uint16)
    return q, z, s


@pytest.mark.parametrize("K,N", [(128, 16), (256, 32), (2048, 48), (128 * 19, 64), (4096, 32)])
def test_round_trip_and_size(K, N):
    q, z, s = _random(K, N, K + N)
    buf = awq.repack_stream(awq.pack_int4(q), awq.pack_int4(z), bf16.from_bits(s))
    G = K // 128
    assert buf.nbytes == awq.stream_bytes(K, N) == (N // 16) * (-(-G // 16) + G) * 1024
    q2, z2, s2 = awq.unpack_stream(buf, K, N)
    assert np.array_equal(q, q2) and np.array_equal(z, z2) and np.array_equal(s, s2)


def test_first_cell_written_out_by_hand():
    """K = 128, N = 16: one tile = [1 KiB scales / zeros][1 KiB cell].  Lane 16 lg + ln, dword t, nibble p is row
    32 t + 8 lg + (0, 2, 4, 6, 1, 3, 5, 7)[p] of column ln."""
    K, N = 128, 16
    q = (np.arange(K)[:, None] * 3 + np.arange(N)[None, :] * 5) % 16
    z = (np.arange(N)[None, :] * 7 + 1) % 16
    s = (0x3C00 + np.arange(N)[None, :]).astype(np.uint16)
    raw = awq.repack_stream(awq.pack_int4(q.astype(np.uint8)), awq.pack_int4(z.astype(np.uint8)), bf16.from_bits(s))
    by = raw.view(np.uint8).reshape(-1).astype(np.int64)
    assert by.size == 2048
    # row 77 = 32 * 2 + 8 * 1 + 5 -> t = 2, lg = 1, j = 5 -> nibble p = 6; column 9 -> lane 16 + 9 = 25
    byte = 1024 + 25 * 16 + 2 * 4 + 6 // 2          # cell starts at 1024; dword t = 2; nibble 6 is the low half of byte 3
    assert (by[byte] & 0xF) == q[77, 9]
    # row 0, column 0: very first nibble of the cell
    assert (by[1024] & 0xF) == q[0, 0]
    # row 2 is nibble 1 (high half of byte 0), row 1 is nibble 4 (low half of byte 2)
    assert (by[1024] >> 4) == q[2, 0] and (by[1026] & 0xF) == q[1, 0]
    # scales / zero points of group 0 (lane group 0, dword 0), column 9: lane 9 -> bytes 144..147
    assert by[144] | (by[145] << 8) == s[0, 9]
    assert by[146] | (by[147] << 8) == 0xC300 | z[0, 9]
    # 0xC300 | z is the bf16 value -(128 + z)
    assert bf16.to_f32(np.array([0xC300 | 11], dtype=np.uint16))[0] == -139.0
    # groups 1..15 of the block do not exist: their fields are zero
    md = raw.reshape(-1)[:256].reshape(64, 4)
    assert not md[:, 1:].any() and not md[16:].any()


def test_short_last_block_has_only_its_own_cells():
    """K = 19 groups: block 0 is full (17 KiB), block 1 holds 1 KiB of scales / zeros and 3 cells."""
    K, N = 128 * 19, 16
    q, z, s = _random(K, N, 5)
    buf = awq.repack_stream(awq.pack_int4(q), awq.pack_int4(z), bf16.from_bits(s))
    assert buf.shape == (1, (2 + 19) * 256)
    md1 = buf[0, 17 * 256:18 * 256].reshape(4, 16, 4)       # [lg, ln, i] -> group 16 + 4 lg + i
    assert (md1[0, :, :3] & 0xFFFF).T.tolist() == s[16:19].tolist()
    assert not md1[0, :, 3].any() and not md1[1:].any()


def test_rejects_shapes_outside_the_layout():
    with pytest.raises(ValueError):
        awq.stream_bytes(4096, 24)
    with pytest.raises(ValueError):
        awq.stream_bytes(4000, 32)


def test_q4nx_order_elements_followed_by_hand():
    """Q4NX order, K = 2304 (18 groups: one full block and a short one), N = 32: a tile is (4 * 2 + 18) KiB, block b
    starts 20 b KiB into it; the pair of (row k, column n) sits in KiB t = (k % 128) / 32 of the block's first four,
    lane 16 lg + ln with 4 lg + i = (k / 128) % 16, dword i; the nibble as in the AWQ order behind those 4 KiB."""
    K, N = 2304, 32
    rng = np.random.default_rng(5)
    q = rng.integers(0, 16, (K, N), dtype=np.uint8)
    s = rng.integers(0, 65536, (K // 32, N)).astype(np.uint16)
    m = rng.integers(0, 65536, (K // 32, N)).astype(np.uint16)
    raw = awq.repack_stream_q4nx(q, s, m)
    assert raw.nbytes == (N // 16) * (4 * 2 + 18) * 1024
    by = raw.view(np.uint8).reshape(-1).astype(np.int64)
    tile_bytes = 26 * 1024
    for k, n in ((0, 0), (77, 9), (128 * 5 + 33, 17), (128 * 16 + 100, 31), (2303, 16)):
        tile, ln = n // 16, n % 16
        g, r = k // 128, k % 128
        b, gl = g // 16, g % 16
        t, lg, j = r // 32, (r % 32) // 8, r % 8
        p = (0, 2, 4, 6, 1, 3, 5, 7).index(j)
        blk = tile * tile_bytes + b * 20 * 1024
        # nibble: cell gl of the block, behind the 4 KiB of pairs
        byte = blk + (4 + gl) * 1024 + (16 * lg + ln) * 16 + 4 * t + p // 2
        assert ((by[byte] >> (4 * (p % 2))) & 0xF) == q[k, n], (k, n)
        # pair of this row's 32-row sub-group: KiB t, lane 16 (gl / 4) + ln, dword gl % 4
        word = blk + t * 1024 + (16 * (gl // 4) + ln) * 16 + 4 * (gl % 4)
        got = by[word] | (by[word + 1] << 8) | (by[word + 2] << 16) | (by[word + 3] << 24)
        assert got == (int(s[k // 32, n]) | (int(m[k // 32, n]) << 16)), (k, n)
    # groups 18 .. 31 of the short block do not exist: their pair words are zero
    short = raw[0, 20 * 256:20 * 256 + 4 * 256].reshape(4, 4, 16, 4)      # [t, lg, ln, i] of block 1
    assert np.all(short[:, 1:] == 0) and np.all(short[:, 0, :, 2:] == 0) and np.any(short[:, 0, :, :2] != 0)
    with pytest.raises(ValueError):
        awq.repack_stream_q4nx(q[:100], s[:3], m[:3])
