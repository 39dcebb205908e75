"""Host-side AWQ layout tools: the device format of this backend is the AutoAWQ
"gemm" checkpoint layout itself, so static weights are written once without a
per-tile repack.

  qweight int32 [K, N/8], qzeros int32 [K/gs, N/8], scales bf16 [K/gs, N];
  bit position 4*i of a word holds column 8*b + PACK_ORDER[i]
  (programming_examples/llms/llama32_1b_int4/awq_repacker.py:33-38).

The examples' kernel-side arrays (A_q u8 [out, K/2], A_s bf16 [K/gs, out],
A_z u8 [K/gs, out]; matvec_int4_packed.py:346-350) convert both ways.
"""

import numpy as np

from . import bf16

PACK_ORDER = (0, 2, 4, 6, 1, 3, 5, 7)
UNPACK_POS = (0, 4, 1, 5, 2, 6, 3, 7)   # bit-position index that holds natural column j
GROUP = 128


def pack_int4(nibs):
    """uint8 [R, N] values 0..15 in natural column order -> int32 [R, N/8]."""
    nibs = np.asarray(nibs)
    if nibs.ndim != 2 or nibs.shape[1] % 8:
        raise ValueError("pack_int4 expects [R, N] with N % 8 == 0")
    blocks = nibs.reshape(nibs.shape[0], -1, 8).astype(np.uint32) & 0xF
    word = np.zeros(blocks.shape[:2], dtype=np.uint32)
    for j in range(8):
        word |= blocks[:, :, j] << np.uint32(4 * UNPACK_POS[j])
    return word.view(np.int32)


def unpack_int4(packed):
    """int32 [R, N/8] -> uint8 [R, N] in natural column order."""
    w = np.ascontiguousarray(np.asarray(packed, dtype=np.int32)).view(np.uint32)
    out = np.empty(w.shape + (8,), dtype=np.uint8)
    for j in range(8):
        out[..., j] = (w >> np.uint32(4 * UNPACK_POS[j])) & np.uint32(0xF)
    return out.reshape(w.shape[0], -1)


def awq_from_l1(A_q, A_s, A_z):
    """Kernel-side arrays of the examples -> (qweight, qzeros, scales) in AWQ layout."""
    A_q = np.asarray(A_q, dtype=np.uint8)
    out, half_k = A_q.shape
    nib = np.empty((out, 2 * half_k), dtype=np.uint8)
    nib[:, 0::2] = A_q & 0x0F
    nib[:, 1::2] = A_q >> 4
    qweight = pack_int4(np.ascontiguousarray(nib.T))
    qzeros = pack_int4(np.asarray(A_z, dtype=np.uint8))
    scales = bf16.from_bits(bf16.bits_of(A_s))
    if qzeros.shape[0] != scales.shape[0] or scales.shape[1] != out:
        raise ValueError(f"A_s {scales.shape} / A_z {np.shape(A_z)} do not match A_q {A_q.shape}")
    return qweight, qzeros, scales


def l1_from_awq(qweight, qzeros, scales):
    """AWQ layout -> (A_q, A_s, A_z) as repack_hf_awq_linear builds them
    (awq_repacker.py:85-109)."""
    q = unpack_int4(qweight)
    z = unpack_int4(qzeros)
    q_mn = np.ascontiguousarray(q.T)
    A_q = ((q_mn[:, 0::2] & 0x0F) | ((q_mn[:, 1::2] & 0x0F) << 4)).astype(np.uint8)
    return A_q, bf16.from_bits(bf16.bits_of(scales)), z


def fake_quantize_awq_int4(W_bf16, gs=GROUP):
    """Asymmetric uint4 quantisation per group of `gs` input features of a weight [M, K] (bf16 bits or floats),
    the quantiser of the stand-alone GEMM example (fake_quantize_awq_int4,
    programming_examples/llms/llama32_1b_int4/awq_pack.py:287-316): per (row, group) scale = (max - min) / 15 in
    float32 (1e-7 for a constant group), zero = round(-min / scale) clipped to 0..15, q = round(w / scale + zero)
    clipped likewise.  Returns the kernel-side arrays pack_inputs takes: W_q u8 [M, K / 2] (even k in the low nibble),
    W_s bf16 [K / gs, M], W_z u8 [K / gs, M]."""
    W = bf16.to_f32(bf16.bits_of(W_bf16)) if bf16.is_bf16(W_bf16) or np.asarray(W_bf16).dtype == np.uint16 else np.asarray(W_bf16, np.float32)
    M, K = W.shape
    if K % gs:
        raise ValueError(f"K={K} not divisible by gs={gs}")
    grouped = W.reshape(M, K // gs, gs)
    lo, hi = grouped.min(axis=2), grouped.max(axis=2)
    scale = ((hi - lo) / np.float32(15.0)).astype(np.float32)
    scale[scale == 0] = np.float32(1e-7)
    zero = np.clip(np.round(-lo / scale), 0, 15).astype(np.uint8)
    q = np.clip(np.round(grouped / scale[:, :, None] + zero.astype(np.float32)[:, :, None]), 0, 15).astype(np.uint8).reshape(M, K)
    return pack_l1_nibbles(q), bf16.from_f32(scale.T), np.ascontiguousarray(zero.T)


def pack_l1_nibbles(q):
    """nibbles u8 [M, K] -> u8 [M, K / 2], even k in the low nibble (the kernel-side A_q of the examples)."""
    q = np.asarray(q, dtype=np.uint8)
    return (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.uint8)


def interleave_rows(gate, up):
    """Row-interleave two kernel-side weight triples (row 2i = gate[i], 2i+1 = up[i]),
    the layout of the decode FFN front half (llama32_1b_int4_weights.py:173-207)."""
    def il(a, b, axis):
        a, b = np.asarray(a), np.asarray(b)
        shape = list(a.shape)
        shape[axis] *= 2
        out = np.empty(shape, dtype=a.dtype)
        sl0 = [slice(None)] * a.ndim
        sl1 = [slice(None)] * a.ndim
        sl0[axis] = slice(0, None, 2)
        sl1[axis] = slice(1, None, 2)
        out[tuple(sl0)] = a
        out[tuple(sl1)] = b
        return out
    return il(gate[0], up[0], 0), il(bf16.bits_of(gate[1]), bf16.bits_of(up[1]), 1).view(bf16.BF16Array), il(gate[2], up[2], 1)


def deinterleave_rows(A_q, A_s, A_z):
    """Inverse of interleave_rows -> (gate triple, up triple)."""
    s = bf16.bits_of(A_s)
    gate = (np.ascontiguousarray(A_q[0::2]), bf16.from_bits(s[:, 0::2]), np.ascontiguousarray(np.asarray(A_z)[:, 0::2]))
    up = (np.ascontiguousarray(A_q[1::2]), bf16.from_bits(s[:, 1::2]), np.ascontiguousarray(np.asarray(A_z)[:, 1::2]))
    return gate, up


# --- the reference's tiled decode buffers -----------------------------------------------

def bo_tile_bytes(GS, M_TILE, K_CHUNK):
    """Bytes of one tile [Q: M_TILE * K_CHUNK / 2][S: K_CHUNK / GS * M_TILE bf16][Z: K_CHUNK / GS * M_TILE u8]
    (matvec_int4_packed.py:63-67)."""
    n_gpc = K_CHUNK // GS
    return M_TILE * (K_CHUNK // 2), n_gpc * M_TILE * 2, n_gpc * M_TILE


def _check_bo_shape(M, K, GS, M_TILE, K_CHUNK, N_CORES, M_PER_LAUNCH):
    if M_PER_LAUNCH is None:
        M_PER_LAUNCH = M
    if K % K_CHUNK or K_CHUNK % GS or M % M_PER_LAUNCH or M_PER_LAUNCH % (N_CORES * M_TILE):
        raise ValueError(f"tiling does not divide the matrix: M={M} K={K} GS={GS} M_TILE={M_TILE} "
                         f"K_CHUNK={K_CHUNK} N_CORES={N_CORES} M_PER_LAUNCH={M_PER_LAUNCH}")
    return M_PER_LAUNCH


def pack_bo_tiles(A_q, A_s, A_z, M, K, GS=GROUP, M_TILE=8, K_CHUNK=2048, N_CORES=8, M_PER_LAUNCH=None):
    """Kernel-side arrays -> uint8 [tiles, tile_bytes] in the reference's decode buffer layout
    (matvec_int4_packed.pack_inputs, matvec_int4_packed.py:57-103).  Tiles are ordered launch ->
    core -> M block -> K chunk; since launches, cores and M blocks each cover consecutive rows,
    that is row-block-major: tile = (row / M_TILE) * (K / K_CHUNK) + k / K_CHUNK."""
    _check_bo_shape(M, K, GS, M_TILE, K_CHUNK, N_CORES, M_PER_LAUNCH)
    A_q = np.ascontiguousarray(A_q, dtype=np.uint8)
    s_bits = np.ascontiguousarray(bf16.bits_of(A_s))
    A_z = np.ascontiguousarray(A_z, dtype=np.uint8)
    if A_q.shape != (M, K // 2) or s_bits.shape != (K // GS, M) or A_z.shape != (K // GS, M):
        raise ValueError("pack_bo_tiles: array shapes do not match M, K, GS")
    rb, kd, gpc = M // M_TILE, K // K_CHUNK, K_CHUNK // GS
    q = A_q.reshape(rb, M_TILE, kd, K_CHUNK // 2).transpose(0, 2, 1, 3).reshape(rb * kd, -1)
    sc = s_bits.reshape(kd, gpc, rb, M_TILE).transpose(2, 0, 1, 3).reshape(rb * kd, -1)
    z = A_z.reshape(kd, gpc, rb, M_TILE).transpose(2, 0, 1, 3).reshape(rb * kd, -1)
    return np.concatenate([q, np.ascontiguousarray(sc).view(np.uint8), z], axis=1)


def unpack_bo_tiles(packed, M, K, GS=GROUP, M_TILE=8, K_CHUNK=2048, N_CORES=8, M_PER_LAUNCH=None):
    """Inverse of pack_bo_tiles: a buffer packed by the reference -> (A_q, A_s, A_z); feed the
    result to awq_from_l1 to obtain this backend's device tensors."""
    _check_bo_shape(M, K, GS, M_TILE, K_CHUNK, N_CORES, M_PER_LAUNCH)
    q_b, s_b, z_b = bo_tile_bytes(GS, M_TILE, K_CHUNK)
    rb, kd, gpc = M // M_TILE, K // K_CHUNK, K_CHUNK // GS
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    if packed.size != rb * kd * (q_b + s_b + z_b):
        raise ValueError(f"buffer has {packed.size} bytes, expected {rb * kd * (q_b + s_b + z_b)}")
    packed = packed.reshape(rb * kd, q_b + s_b + z_b)
    A_q = packed[:, :q_b].reshape(rb, kd, M_TILE, K_CHUNK // 2).transpose(0, 2, 1, 3).reshape(M, K // 2)
    sc = np.ascontiguousarray(packed[:, q_b:q_b + s_b]).view(np.uint16).reshape(rb, kd, gpc, M_TILE)
    A_s = sc.transpose(1, 2, 0, 3).reshape(K // GS, M)
    A_z = packed[:, q_b + s_b:].reshape(rb, kd, gpc, M_TILE).transpose(1, 2, 0, 3).reshape(K // GS, M)
    return np.ascontiguousarray(A_q), bf16.from_bits(np.ascontiguousarray(A_s)), np.ascontiguousarray(A_z)


def pack_gemm_tiles(W_q, W_s, W_z, K, N, GS=GROUP, N_TILE=16, K_CHUNK=128):
    """Kernel-side arrays of a prefill weight (W_q [N, K/2] u8 output-major, W_s, W_z [K/GS, N]) -> uint8
    [N / N_TILE, K / K_CHUNK, tile_bytes] in the layout of the reference's int4 GEMM buffers
    (matmul_int4_packed.pack_inputs, programming_examples/matrix_multiplication/int4_awq/matmul_int4_packed.py:57-86;
    what awq_pack_for_npu emits, llama32_1b_int4/awq_pack.py:112-146).  A tile is the decode tile with
    N_TILE output rows, and tiles are ordered output block, then K chunk."""
    t = pack_bo_tiles(W_q, W_s, W_z, N, K, GS, N_TILE, K_CHUNK, 1, N)
    return t.reshape(N // N_TILE, K // K_CHUNK, -1)


def unpack_gemm_tiles(packed, K, N, GS=GROUP, N_TILE=16, K_CHUNK=128):
    """Inverse of pack_gemm_tiles: a buffer packed by the reference -> (W_q, W_s, W_z)."""
    return unpack_bo_tiles(np.asarray(packed).reshape(-1), N, K, GS, N_TILE, K_CHUNK, 1, N)


# --- single packed buffer ("BO") ------------------------------------------------------

def _round256(v):
    return (v + 255) & ~255


def packed_layout(K, N, gs=GROUP):
    """Byte offsets of the three sections inside one packed weight buffer."""
    q_bytes = K * (N // 8) * 4
    z_bytes = (K // gs) * (N // 8) * 4
    s_bytes = (K // gs) * N * 2
    z_off = _round256(q_bytes)
    s_off = z_off + _round256(z_bytes)
    return {"q_off": 0, "z_off": z_off, "s_off": s_off, "total": s_off + _round256(s_bytes),
            "q_bytes": q_bytes, "z_bytes": z_bytes, "s_bytes": s_bytes}


def pack_buffer(qweight, qzeros, scales):
    """[qweight | qzeros | scales] in one uint8 buffer, sections 256-byte aligned
    (the counterpart of the examples' single packed weight BO)."""
    K, nb = qweight.shape
    N = nb * 8
    gs = K // qzeros.shape[0]
    lay = packed_layout(K, N, gs)
    buf = np.zeros(lay["total"], dtype=np.uint8)
    buf[0:lay["q_bytes"]] = np.ascontiguousarray(qweight).view(np.uint8).reshape(-1)
    buf[lay["z_off"]:lay["z_off"] + lay["z_bytes"]] = np.ascontiguousarray(qzeros).view(np.uint8).reshape(-1)
    buf[lay["s_off"]:lay["s_off"] + lay["s_bytes"]] = bf16.bits_of(scales).view(np.uint8).reshape(-1)
    return buf


def unpack_buffer(buf, K, N, gs=GROUP):
    lay = packed_layout(K, N, gs)
    buf = np.asarray(buf, dtype=np.uint8).reshape(-1)
    if buf.size != lay["total"]:
        raise ValueError(f"packed buffer has {buf.size} bytes, expected {lay['total']} for K={K} N={N}")
    qweight = buf[0:lay["q_bytes"]].view(np.int32).reshape(K, N // 8)
    qzeros = buf[lay["z_off"]:lay["z_off"] + lay["z_bytes"]].view(np.int32).reshape(K // gs, N // 8)
    scales = buf[lay["s_off"]:lay["s_off"] + lay["s_bytes"]].view(np.uint16).reshape(K // gs, N).view(bf16.BF16Array)
    return qweight, qzeros, scales


# --- the 1-D dequant example's tiled buffer ------------------------------------------------------

def packed_tile_bytes_1d(n_tile, group_size):
    """(q_bytes, s_bytes, z_bytes, tile_bytes) of one tile of the 1-D dequant example: Q two elements per byte,
    S bf16 per group, Z u8 per group, the tile padded to a multiple of 4 bytes
    (packed_tile_bytes, programming_examples/dequant_awq/dequant_awq.py:59-69)."""
    ng = n_tile // group_size
    q_bytes, s_bytes, z_bytes = n_tile // 2, 2 * ng, ng
    return q_bytes, s_bytes, z_bytes, -(-(q_bytes + s_bytes + z_bytes) // 4) * 4


def pack_inputs_1d(int4_vals, scales, zeros, n, group_size, herd_n):
    """uint8 [herd_n, tile_bytes]: tile ty holds elements [ty * n / herd_n, (ty + 1) * n / herd_n) as [Q | S | Z | pad],
    element 2 j of a tile in the low nibble of its byte j (pack_inputs, dequant_awq.py:259-278)."""
    if n % herd_n or (n // herd_n) % group_size or group_size % 2:
        raise ValueError("N / herd_n must be divisible by group_size")
    n_tile = n // herd_n
    q_bytes, s_bytes, z_bytes, tile_bytes = packed_tile_bytes_1d(n_tile, group_size)
    q = np.asarray(int4_vals, dtype=np.uint8).reshape(herd_n, n_tile)
    out = np.zeros((herd_n, tile_bytes), dtype=np.uint8)
    out[:, :q_bytes] = (q[:, 0::2] & 0xF) | ((q[:, 1::2] & 0xF) << 4)
    out[:, q_bytes:q_bytes + s_bytes] = np.ascontiguousarray(bf16.bits_of(scales)).reshape(herd_n, -1).view(np.uint8)
    out[:, q_bytes + s_bytes:q_bytes + s_bytes + z_bytes] = np.asarray(zeros, dtype=np.uint8).reshape(herd_n, -1)
    return out


def unpack_inputs_1d(packed, n, group_size, herd_n):
    """Inverse of pack_inputs_1d -> (int4_vals u8 [n], scales bf16 [n / gs], zeros u8 [n / gs])."""
    n_tile = n // herd_n
    q_bytes, s_bytes, z_bytes, tile_bytes = packed_tile_bytes_1d(n_tile, group_size)
    packed = np.asarray(packed, dtype=np.uint8).reshape(herd_n, tile_bytes)
    q = np.empty((herd_n, n_tile), dtype=np.uint8)
    q[:, 0::2] = packed[:, :q_bytes] & 0xF
    q[:, 1::2] = packed[:, :q_bytes] >> 4
    s = np.ascontiguousarray(packed[:, q_bytes:q_bytes + s_bytes]).view(np.uint16).reshape(-1)
    z = np.ascontiguousarray(packed[:, q_bytes + s_bytes:q_bytes + s_bytes + z_bytes]).reshape(-1)
    return q.reshape(-1), bf16.from_bits(s), z


# --- stream order: the device layout of the decode kernels ---------------------------------------
#
# Counterpart of the reference's load-time re-pack into the order its cores consume the weights
# (repack_for_gemv, awq_repacker.py:112-135).  Per 16-column tile one contiguous slab of all K rows:
# blocks of 16 groups, each [1 KiB scales / zero points][one 1 KiB cell per group].  A cell is 64
# lanes x 4 dwords; lane l = 16 lg + ln, dword t, nibble p holds row 128 g + 32 t + 8 lg +
# PACK_ORDER[p] of column 16 tile + ln.  Scales / zero points: lane l, dword i belongs to group
# 16 b + 4 lg + i: bits 0..15 the bf16 scale, bits 16..31 the bf16 value -(128 + z) = 0xC300 | z.

STREAM_TILE_COLS = 16
STREAM_BLOCK_GROUPS = 16


def stream_bytes(K, N):
    """Size of the stream-order buffer of a [K, N] matrix."""
    if K % GROUP or N % STREAM_TILE_COLS:
        raise ValueError("stream order needs K % 128 == 0 and N % 16 == 0")
    G = K // GROUP
    return (N // STREAM_TILE_COLS) * (-(-G // STREAM_BLOCK_GROUPS) + G) * 1024


def repack_stream(qweight, qzeros, scales):
    """AWQ layout -> stream order, uint32 [N/16, (NB + G) * 256] (host twin of w4a16_repack_stream)."""
    q = unpack_int4(qweight)                       # [K, N]
    z = unpack_int4(qzeros)                        # [G, N]
    s = bf16.bits_of(scales).astype(np.uint32)     # [G, N]
    K, N = q.shape
    G = K // GROUP
    if K % GROUP or N % STREAM_TILE_COLS or z.shape != (G, N) or s.shape != (G, N):
        raise ValueError("repack_stream: need K % 128 == 0, N % 16 == 0 and [K/128, N] scales / zeros")
    NB = -(-G // STREAM_BLOCK_GROUPS)
    T = N // STREAM_TILE_COLS
    out = np.zeros((T, (NB + G) * 256), dtype=np.uint32)
    # cells: q[k, n] with k = 128 g + 32 t + 8 lg + PACK_ORDER[p], n = 16 tile + ln
    qv = q.reshape(G, 4, 4, 8, T, 16).astype(np.uint32)          # [g, t, lg, j, tile, ln]
    cells = np.zeros((G, 4, 4, T, 16), dtype=np.uint32)          # [g, t, lg, tile, ln]
    for p, j in enumerate(PACK_ORDER):
        cells |= qv[:, :, :, j] << np.uint32(4 * p)
    cells = cells.transpose(3, 0, 2, 4, 1)                       # [tile, g, lg, ln, t]
    # scales / zero points: dword (lane, i) of block b <- group 16 b + 4 lg + i
    md = s | ((np.uint32(0xC300) | z.astype(np.uint32)) << np.uint32(16))     # [G, N]
    md_pad = np.zeros((NB * STREAM_BLOCK_GROUPS, N), dtype=np.uint32)
    md_pad[:G] = md
    md_pad = md_pad.reshape(NB, 4, 4, T, 16).transpose(3, 0, 1, 4, 2)         # [tile, b, lg, ln, i]
    for b in range(NB):
        g0 = b * STREAM_BLOCK_GROUPS
        ng = min(STREAM_BLOCK_GROUPS, G - g0)
        base = b * (STREAM_BLOCK_GROUPS + 1) * 256
        out[:, base:base + 256] = md_pad[:, b].reshape(T, 256)
        out[:, base + 256:base + 256 * (1 + ng)] = cells[:, g0:g0 + ng].reshape(T, ng * 256)
    return out


def repack_stream_q4nx(q, scale_bits, min_bits):
    """Q4NX stream order, uint32 [N/16, (4 NB + G) * 256], from the values of the affine path: q uint8 [K, N] (unsigned
    nibbles), scale and min' bit patterns uint16 [K/32, N] with w = s q + min' (host twin of w4a16_q4nx_repack_stream,
    whose operands are the same values in q4nx_repack's packing).  Cells as in repack_stream; in front of a block's
    cells 4 KiB of words, KiB t, lane 16 lg + ln, dword i = (scale | min' << 16) of rows 32 t .. 32 t + 31 of group
    16 b + 4 lg + i, column 16 tile + ln."""
    q = np.asarray(q)
    s = np.asarray(scale_bits).astype(np.uint32)
    m = np.asarray(min_bits).astype(np.uint32)
    K, N = q.shape
    G = K // GROUP
    if K % GROUP or N % STREAM_TILE_COLS or s.shape != (K // 32, N) or m.shape != s.shape:
        raise ValueError("repack_stream_q4nx: need K % 128 == 0, N % 16 == 0 and [K/32, N] scales / mins")
    NB = -(-G // STREAM_BLOCK_GROUPS)
    T = N // STREAM_TILE_COLS
    MDK = 4
    out = np.zeros((T, (MDK * NB + G) * 256), dtype=np.uint32)
    qv = q.reshape(G, 4, 4, 8, T, 16).astype(np.uint32)          # [g, t, lg, j, tile, ln]
    cells = np.zeros((G, 4, 4, T, 16), dtype=np.uint32)          # [g, t, lg, tile, ln]
    for p, j in enumerate(PACK_ORDER):
        cells |= qv[:, :, :, j] << np.uint32(4 * p)
    cells = cells.transpose(3, 0, 2, 4, 1)                       # [tile, g, lg, ln, t]
    md = (s | (m << np.uint32(16))).reshape(G, 4, N)             # [g, t, n]
    md_pad = np.zeros((NB * STREAM_BLOCK_GROUPS, 4, N), dtype=np.uint32)
    md_pad[:G] = md
    md_pad = md_pad.reshape(NB, 4, 4, 4, T, 16).transpose(4, 0, 3, 1, 5, 2)   # [tile, b, t, lg, ln, i]
    for b in range(NB):
        g0 = b * STREAM_BLOCK_GROUPS
        ng = min(STREAM_BLOCK_GROUPS, G - g0)
        base = b * (STREAM_BLOCK_GROUPS + MDK) * 256
        out[:, base:base + MDK * 256] = md_pad[:, b].reshape(T, MDK * 256)
        out[:, base + MDK * 256:base + 256 * (MDK + ng)] = cells[:, g0:g0 + ng].reshape(T, ng * 256)
    return out


def unpack_stream(buf, K, N):
    """Stream order -> (q uint8 [K, N], z uint8 [K/128, N], scale bits uint16 [K/128, N])."""
    G = K // GROUP
    NB = -(-G // STREAM_BLOCK_GROUPS)
    T = N // STREAM_TILE_COLS
    buf = np.ascontiguousarray(buf).view(np.uint32).reshape(T, (NB + G) * 256)
    q = np.empty((K, N), dtype=np.uint8)
    z = np.empty((G, N), dtype=np.uint8)
    s = np.empty((G, N), dtype=np.uint16)
    qv = q.reshape(G, 4, 4, 8, T, 16)
    for b in range(NB):
        g0 = b * STREAM_BLOCK_GROUPS
        ng = min(STREAM_BLOCK_GROUPS, G - g0)
        base = b * (STREAM_BLOCK_GROUPS + 1) * 256
        md = buf[:, base:base + 256].reshape(T, 4, 16, 4).transpose(1, 3, 0, 2).reshape(16, N)   # [4 lg + i, n]
        s[g0:g0 + ng] = (md[:ng] & 0xFFFF).astype(np.uint16)
        hi = md[:ng] >> 16
        if np.any((hi & 0xFFF0) != 0xC300):
            raise ValueError("unpack_stream: a zero-point field is not 0xC300 | z")
        z[g0:g0 + ng] = (hi & 0xF).astype(np.uint8)
        cells = buf[:, base + 256:base + 256 * (1 + ng)].reshape(T, ng, 4, 16, 4)               # [tile, g, lg, ln, t]
        for p, j in enumerate(PACK_ORDER):
            qv[g0:g0 + ng, :, :, j] = ((cells >> np.uint32(4 * p)) & 0xF).transpose(1, 4, 2, 0, 3).astype(np.uint8)
    return q, z, s
