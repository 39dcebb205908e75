"""TEST INFRASTRUCTURE ONLY - CPU restatement of the reference's AWQ codec.

Follows, function by function (paths relative to the reference root,
PE = programming_examples):

  AWQ_PACK_ORDER / AWQ_UNPACK_PERM   PE/llms/llama32_1b_int4/awq_repacker.py:33-38
                                     (= _AWQ_REORDER_PERM, awq_pack.py:61-63)
  unpack_awq_int32                   awq_repacker.py:41-54 (= awq_pack.py:66-76)
  pack_awq_int32                     awq_repacker.py:155-162 (packer inside
                                     _gen_synthetic_awq)
  dequant_to_bf16                    awq_repacker.py:57-82 (= awq_dequant_layer,
                                     awq_pack.py:84-104)
  repack_hf_awq_linear               awq_repacker.py:85-109
  l1_unpack_nibbles                  matvec_int4_packed.py:282-283 (byte ->
                                     even/odd-k nibble)
  dequant_1d                         PE/dequant_awq/dequant_awq.py:391-396
  pack_inputs_loop                   PE/matrix_vector_multiplication/int4_awq/
                                     matvec_int4_packed.py:57-103 (decode buffer tiling;
                                     pinned by a hand-computed tile and its byte offsets)

bf16 tensors are uint16 bit patterns (see oracle/bf16.py).

Pins (tests/test_oracle_awq.py): the hand-computed word 0x76543210, a scalar
brute-force packer, exhaustive (q, z) x scale-bit-pattern dequant against
exact rational arithmetic, the self-test identities of awq_repacker.py:166-206.
"""

import numpy as np

from .bf16 import bf16_bits_to_f32, f32_to_bf16_bits

# Bit position 4*i of each int32 holds output column 8*block + AWQ_PACK_ORDER[i].
AWQ_PACK_ORDER = np.array([0, 2, 4, 6, 1, 3, 5, 7], dtype=np.int64)
# AWQ_UNPACK_PERM[j] is the bit-position index holding natural column j.
AWQ_UNPACK_PERM = np.argsort(AWQ_PACK_ORDER)


def unpack_awq_int32(packed):
    """int32 [..., N/8] -> uint8 nibbles [..., N] in natural column order."""
    packed64 = np.asarray(packed).astype(np.int64)
    shifts = np.arange(8, dtype=np.int64) * 4
    nibs = ((packed64[..., :, None] >> shifts) & 0xF).astype(np.uint8)
    nibs = nibs[..., AWQ_UNPACK_PERM]
    return nibs.reshape(*packed64.shape[:-1], packed64.shape[-1] * 8)


def pack_awq_int32(nibs):
    """uint8 nibbles [R, N] (natural order) -> int32 [R, N/8] in AWQ order."""
    nibs = np.asarray(nibs)
    rows, n = nibs.shape
    assert n % 8 == 0
    out = np.zeros((rows, n // 8), dtype=np.uint32)
    for i in range(8):
        col = int(AWQ_PACK_ORDER[i])
        out |= (nibs[:, col::8].astype(np.uint32) & 0xF) << np.uint32(4 * i)
    return out.view(np.int32)


def dequant_to_bf16(qweight, qzeros, scales_bits, group_size):
    """AWQ tensors -> dense W[K, N] as bf16 bits.

    W[k, n] = bf16_rne((q[k, n] - z[k // gs, n]) * s[k // gs, n]); the product
    is formed in float32 exactly as the reference does.
    """
    q = unpack_awq_int32(qweight)
    z = unpack_awq_int32(qzeros)
    k, n = q.shape
    n_groups = k // group_size
    if z.shape != (n_groups, n):
        raise ValueError(f"qzeros shape {z.shape} vs expected ({n_groups}, {n})")
    if np.shape(scales_bits) != (n_groups, n):
        raise ValueError(f"scales shape {np.shape(scales_bits)} vs expected ({n_groups}, {n})")
    s = bf16_bits_to_f32(scales_bits)
    z_per_k = np.repeat(z.astype(np.int32), group_size, axis=0)
    s_per_k = np.repeat(s, group_size, axis=0)
    w_f32 = ((q.astype(np.int32) - z_per_k).astype(np.float32)) * s_per_k
    return f32_to_bf16_bits(w_f32)


def dequant_unrounded_f32(qweight, qzeros, scales_bits, group_size):
    """(q - z) * s in float32 without the final bf16 rounding (exact: the
    product has at most 13 significant bits)."""
    q = unpack_awq_int32(qweight).astype(np.int32)
    z = unpack_awq_int32(qzeros).astype(np.int32)
    s = bf16_bits_to_f32(scales_bits)
    return (q - np.repeat(z, group_size, axis=0)).astype(np.float32) * np.repeat(s, group_size, axis=0)


def repack_hf_awq_linear(qweight, qzeros, scales_bits, group_size):
    """AWQ tensors -> the examples' kernel-side arrays
    (A_q u8 [out, K/2], A_s bf16-bits [K/gs, out], A_z u8 [K/gs, out])."""
    q = unpack_awq_int32(qweight)
    z = unpack_awq_int32(qzeros)
    k, n = q.shape
    n_groups = k // group_size
    if z.shape != (n_groups, n):
        raise ValueError(f"qzeros shape {z.shape} vs expected ({n_groups}, {n})")
    if np.shape(scales_bits) != (n_groups, n):
        raise ValueError(f"scales shape {np.shape(scales_bits)} vs expected ({n_groups}, {n})")
    q_mn = np.ascontiguousarray(q.T)
    a_q = ((q_mn[:, 0::2] & 0x0F) | ((q_mn[:, 1::2] & 0x0F) << 4)).astype(np.uint8)
    a_s = np.ascontiguousarray(scales_bits).astype(np.uint16)
    a_z = np.ascontiguousarray(z).astype(np.uint8)
    return a_q, a_s, a_z


def l1_unpack_nibbles(a_q):
    """A_q u8 [out, K/2] -> nibbles int32 [out, K] (even k = low nibble)."""
    a = np.asarray(a_q).astype(np.int32)
    out = np.empty((a.shape[0], a.shape[1] * 2), dtype=np.int32)
    out[:, 0::2] = a & 0x0F
    out[:, 1::2] = (a >> 4) & 0x0F
    return out


def l1_to_awq(a_q, a_s_bits, a_z):
    """Inverse of repack_hf_awq_linear: kernel-side arrays -> AWQ tensors."""
    nibs_kn = np.ascontiguousarray(l1_unpack_nibbles(a_q).T).astype(np.uint8)
    qweight = pack_awq_int32(nibs_kn)
    qzeros = pack_awq_int32(np.asarray(a_z).astype(np.uint8))
    return qweight, qzeros, np.ascontiguousarray(a_s_bits).astype(np.uint16)


def fake_quantize_awq_int4_loop(w_f32, gs):
    """Scalar restatement of fake_quantize_awq_int4 (programming_examples/llms/llama32_1b_int4/awq_pack.py:287-316) on a
    float32 matrix [M, K], one (row, group) at a time: scale = (max - min) / 15 in float32 (1e-7 if zero),
    zero = clip(round(-min / scale), 0, 15), q = clip(round(w / scale + zero), 0, 15), rounding half to even as
    np.round does.  Returns (A_q u8 [M, K / 2], scale bf16 bits [K / gs, M], zero u8 [K / gs, M]).
    Pinned in tests/test_oracle_awq.py by a ramp whose quantisation is exact by hand (scale 1/4, zero 8, q = the ramp
    index), the end points (min -> 0, max -> 15 when the group straddles zero), the error bound |w - (q - z) s| <= s / 2
    inside the representable range, and constant groups."""
    w = np.asarray(w_f32, dtype=np.float32)
    M, K = w.shape
    G = K // gs
    q = np.zeros((M, K), np.uint8)
    scale = np.zeros((G, M), np.float32)
    zero = np.zeros((G, M), np.uint8)
    f = np.float32
    for m in range(M):
        for g in range(G):
            grp = w[m, g * gs:(g + 1) * gs]
            lo, hi = f(min(grp)), f(max(grp))
            sc = f(f(hi - lo) / f(15.0))
            if sc == 0:
                sc = f(1e-7)
            z = min(max(float(np.round(f(-lo) / sc)), 0.0), 15.0)
            scale[g, m], zero[g, m] = sc, int(z)
            for i in range(gs):
                q[m, g * gs + i] = int(min(max(float(np.round(f(f(grp[i] / sc) + f(z)))), 0.0), 15.0))
    a_q = (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.uint8)
    return a_q, f32_to_bf16_bits(scale), zero


def dequant_1d(int4_vals, scales_bits, zeros, group_size):
    """1-D form of the dequant example: out[i] = bf16((q[i] - z[g]) * s[g])
    evaluated in double as the reference's Python floats do."""
    q = np.asarray(int4_vals).astype(np.float64)
    g = np.arange(q.size) // group_size
    z = np.asarray(zeros).astype(np.float64)[g]
    s = bf16_bits_to_f32(scales_bits).astype(np.float64)[g]
    return f32_to_bf16_bits(((q - z) * s).astype(np.float32))


def pack_inputs_1d_loop(int4_vals, scales_bits, zeros, n, group_size, herd_n):
    """Scalar restatement of the 1-D dequant example's tiling (pack_inputs, dequant_awq.py:259-278; tile size
    packed_tile_bytes, :59-69): tile ty = [Q: element pairs, even one in the low nibble][S: bf16 little endian per
    group][Z: one byte per group][zero padding to a multiple of 4 bytes].  One byte at a time."""
    n_tile = n // herd_n
    ng_tile = n_tile // group_size
    q_bytes, s_bytes, z_bytes = n_tile // 2, 2 * ng_tile, ng_tile
    tile_bytes = (q_bytes + s_bytes + z_bytes + 3) & ~3
    out = np.zeros((herd_n, tile_bytes), dtype=np.uint8)
    for ty in range(herd_n):
        for j in range(q_bytes):
            lo, hi = int(int4_vals[ty * n_tile + 2 * j]), int(int4_vals[ty * n_tile + 2 * j + 1])
            out[ty, j] = lo | (hi << 4)
        for g in range(ng_tile):
            bits = int(scales_bits[ty * ng_tile + g])
            out[ty, q_bytes + 2 * g] = bits & 0xFF
            out[ty, q_bytes + 2 * g + 1] = bits >> 8
            out[ty, q_bytes + s_bytes + g] = int(zeros[ty * ng_tile + g])
    return out


def pack_inputs_loop(a_q, a_s_bits, a_z, M, K, GS, M_TILE, K_CHUNK, N_CORES, M_PER_LAUNCH):
    """Scalar restatement of the decode buffer tiling (matvec_int4_packed.py:57-103): one tile per
    (launch, core, M block, K chunk) in that nesting order, each tile
    [Q rows x K_CHUNK/2 bytes][S groups x rows bf16][Z groups x rows u8].  Pure Python loops over
    bytes: small shapes only."""
    n_gpc = K_CHUNK // GS
    q_bytes, s_bytes, z_bytes = M_TILE * (K_CHUNK // 2), n_gpc * M_TILE * 2, n_gpc * M_TILE
    m_core = M_PER_LAUNCH // N_CORES
    tiles = []
    for launch in range(M // M_PER_LAUNCH):
        for core in range(N_CORES):
            for outer in range(m_core // M_TILE):
                row0 = launch * M_PER_LAUNCH + core * m_core + outer * M_TILE
                for kc in range(K // K_CHUNK):
                    t = np.zeros(q_bytes + s_bytes + z_bytes, dtype=np.uint8)
                    for r in range(M_TILE):
                        for b in range(K_CHUNK // 2):
                            t[r * (K_CHUNK // 2) + b] = a_q[row0 + r, kc * (K_CHUNK // 2) + b]
                    for g in range(n_gpc):
                        for r in range(M_TILE):
                            v = int(a_s_bits[kc * n_gpc + g, row0 + r])
                            o = q_bytes + 2 * (g * M_TILE + r)
                            t[o], t[o + 1] = v & 0xFF, v >> 8            # little-endian bf16
                            t[q_bytes + s_bytes + g * M_TILE + r] = a_z[kc * n_gpc + g, row0 + r]
                    tiles.append(t)
    return np.stack(tiles)


def pack_inputs_gemm_loop(w_q, w_s_bits, w_z, K, N, GS, N_TILE, K_CHUNK):
    """Scalar restatement of the prefill GEMM weight tiling (matmul_int4_packed.py:57-86): uint8
    [N / N_TILE, K / K_CHUNK, tile_bytes], tile (n_outer, k_outer) =
    [Q: N_TILE rows x K_CHUNK/2 bytes][S: K_CHUNK/GS groups x N_TILE bf16][Z: K_CHUNK/GS x N_TILE u8].
    Pure Python loops over bytes: small shapes only."""
    n_gpc = K_CHUNK // GS
    q_bytes, s_bytes, z_bytes = N_TILE * (K_CHUNK // 2), n_gpc * N_TILE * 2, n_gpc * N_TILE
    out = np.zeros((N // N_TILE, K // K_CHUNK, q_bytes + s_bytes + z_bytes), dtype=np.uint8)
    for n_outer in range(N // N_TILE):
        for k_outer in range(K // K_CHUNK):
            t = out[n_outer, k_outer]
            for r in range(N_TILE):
                for b in range(K_CHUNK // 2):
                    t[r * (K_CHUNK // 2) + b] = w_q[n_outer * N_TILE + r, k_outer * (K_CHUNK // 2) + b]
            for g in range(n_gpc):
                for r in range(N_TILE):
                    v = int(w_s_bits[k_outer * n_gpc + g, n_outer * N_TILE + r])
                    o = q_bytes + 2 * (g * N_TILE + r)
                    t[o], t[o + 1] = v & 0xFF, v >> 8
                    t[q_bytes + s_bytes + g * N_TILE + r] = w_z[k_outer * n_gpc + g, n_outer * N_TILE + r]
    return out
