"""TEST INFRASTRUCTURE ONLY - CPU restatement of the reference's Q4NX / Q4_0 block codec.
Never imported by the product.

Follows (FD = programming_examples/fused_decode, LLM = programming_examples/llms):

  pack_block_loop        FD/proj_qmm_pack.py:23-58 (pack_q4k_block: the byte layout of one
                         32 x 256 block, scalar loops)
  pack_matrix            the plain (row-block, col-block) block order of a model.q4nx tensor
                         (LLM/llama32_1b_q4nx/llama32_1b_q4nx_weights.py:262-266), vectorised
                         like FD/qwen25_3b_requant.py:151-175
  cascade_order          FD/proj_qmm_pack.py:109-137: the (row-block, col-block) of every
                         block of the device stream [cx][i][j][cy] in its three numberings
                         (default, core_major, iter_major) and the dual-channel split
  unpack_matrix          LLM/llama32_1b_q4nx/llama32_1b_q4nx_weights.py:226-253
  dequant                the same function, :254-266: additive (w = s q + m, "I8" header, the
                         proj_qmm kernel's convention FD/kernels/q4_k.h:9-17) or subtractive
                         (w = s (q - m), "Q4NX" header)
  requant_q4k            LLM/llama32_1b_q4nx/q4nx_requant.py:25-35 (min/max 4-bit per group)
  requant_q4_0           FD/qwen25_3b_requant.py:116-134 (signed, scale = amax / 8)
  dequant_q4_0           LLM/qwen25_3b_q4/qwen25_3b_q4_weights.py:86-95
  gemv_reference         FD/kernels/q4_k.h:39-45 restated exactly: per group
                         c += (sum q b) * scale + min * sum b, in float64
  rms_gemv_reference, block_staged_reference
                         the RMSNorm + GEMV and O + FFN block stagings of oracle/reference.py
                         (rms_norm_bf16, o_gemv_ffn_staged_reference) with gemv_reference as the GEMV

bf16 tensors are uint16 bit patterns.  Pins (tests/test_oracle_q4nx.py): a block written byte
by byte from the layout comment of proj_qmm_pack.py:4-9, loop packer == vectorised packer,
unpack(pack) identity, dequant against a scalar per-element formula, requantisers against
their defining properties (end points, error bound, the +peak clip of Q4_0), the stream orders
against hand-enumerated small cases and as permutations, the GEMV against a dense float64 product.
"""

import numpy as np

from .bf16 import bf16_bits_to_f32, f32_to_bf16_bits

ROW_BLOCK = 32
COL_BLOCK = 256
GROUP = 32
PARALLEL = 16
N_GROUPS = COL_BLOCK // GROUP        # 8
ROW_GROUPS = ROW_BLOCK // PARALLEL   # 2
BLOCK_BYTES = ROW_BLOCK * COL_BLOCK // 2 + 2 * 2 * N_GROUPS * ROW_BLOCK   # 5120

ADDITIVE, SUBTRACTIVE, Q4_0 = 0, 1, 2


def pack_block_loop(q, scale_bits, min_bits):
    """One block, scalar loops.  q uint8 [32, 256] nibbles, scale/min bf16 bits [32, 8]
    (row, group) -> uint8 [5120]."""
    assert q.shape == (ROW_BLOCK, COL_BLOCK) and scale_bits.shape == (ROW_BLOCK, N_GROUPS)
    buf = np.zeros(BLOCK_BYTES, dtype=np.uint8)
    sc = np.zeros((N_GROUPS, ROW_BLOCK), dtype=np.uint16)
    mi = np.zeros((N_GROUPS, ROW_BLOCK), dtype=np.uint16)
    for g in range(N_GROUPS):
        for r in range(ROW_BLOCK):
            sc[g, r] = scale_bits[r, g]
            mi[g, r] = min_bits[r, g]
    buf[0:512] = sc.reshape(-1).view(np.uint8)
    buf[512:1024] = mi.reshape(-1).view(np.uint8)
    off = 1024
    for rg in range(ROW_GROUPS):
        for col in range(COL_BLOCK):
            for kk in range(PARALLEL // 2):
                w0 = int(q[rg * PARALLEL + 2 * kk, col]) & 0xF
                w1 = int(q[rg * PARALLEL + 2 * kk + 1, col]) & 0xF
                buf[off] = (w1 << 4) | w0
                off += 1
    return buf


def pack_matrix(q, scale_bits, min_bits):
    """q uint8 [M, K], scale/min bf16 bits [M, K / 32] -> uint8 [M/32 * K/256, 5120], row-block major."""
    M, K = q.shape
    nbi, nbj = M // ROW_BLOCK, K // COL_BLOCK
    per_block = lambda a: (np.asarray(a, dtype=np.uint16).reshape(nbi, ROW_BLOCK, nbj, N_GROUPS)
                           .transpose(0, 2, 3, 1).reshape(nbi * nbj, -1))
    qv = (np.asarray(q, dtype=np.uint8) & 0xF).reshape(nbi, ROW_GROUPS, PARALLEL // 2, 2, nbj, COL_BLOCK)
    byte = (qv[:, :, :, 1] << 4) | qv[:, :, :, 0]            # [nbi, rg, kk, nbj, col]
    qs = byte.transpose(0, 3, 1, 4, 2).reshape(nbi * nbj, -1)   # [nbi, nbj, rg, col, kk]
    out = np.empty((nbi * nbj, BLOCK_BYTES), dtype=np.uint8)
    out[:, 0:512] = np.ascontiguousarray(per_block(scale_bits)).view(np.uint8)
    out[:, 512:1024] = np.ascontiguousarray(per_block(min_bits)).view(np.uint8)
    out[:, 1024:] = qs
    return out


def cascade_order(nbi, nbj, ncx, ncy, core_major=False, iter_major=False, dual_chan=False):
    """(row-block, col-block) of every block of the device weight stream, in stream order."""
    n_cores = ncx * ncy
    assert nbi % n_cores == 0
    nbi_pc = nbi // n_cores
    steps = [(i, j) for i in range(nbi_pc) for j in range(nbj)]
    if dual_chan:
        assert ncy % 2 == 0
        order = [(i, j, cy) for h in range(2) for (i, j) in steps for cy in range(h * (ncy // 2), (h + 1) * (ncy // 2))]
    else:
        order = [(i, j, cy) for (i, j) in steps for cy in range(ncy)]
    out = []
    for cx in range(ncx):
        for i, j, cy in order:
            if iter_major:
                gi = i * n_cores + cx * ncy + cy
            elif core_major:
                gi = (cx * ncy + cy) * nbi_pc + i
            else:
                gi = cx * (ncy * nbi_pc) + i * ncy + cy
            out.append((gi, j))
    return out


def unpack_matrix(blocks, M, K):
    """uint8 [nb, 5120] (row-block major) -> (q uint8 [M, K], scale bits [M, K/32], min bits [M, K/32])."""
    nbi, nbj = M // ROW_BLOCK, K // COL_BLOCK
    b = np.asarray(blocks, dtype=np.uint8).reshape(nbi, nbj, BLOCK_BYTES)
    hdr = lambda lo: (np.ascontiguousarray(b[:, :, lo:lo + 512]).view(np.uint16)
                      .reshape(nbi, nbj, N_GROUPS, ROW_BLOCK).transpose(0, 3, 1, 2).reshape(M, K // GROUP))
    qs = b[:, :, 1024:].reshape(nbi, nbj, ROW_GROUPS, COL_BLOCK, PARALLEL // 2)
    q = np.empty((nbi, nbj, ROW_GROUPS, PARALLEL // 2, 2, COL_BLOCK), dtype=np.uint8)
    q[:, :, :, :, 0, :] = (qs & 0xF).transpose(0, 1, 2, 4, 3)
    q[:, :, :, :, 1, :] = (qs >> 4).transpose(0, 1, 2, 4, 3)
    q = q.reshape(nbi, nbj, ROW_BLOCK, COL_BLOCK).transpose(0, 2, 1, 3).reshape(M, K)
    return q, hdr(0), hdr(512)


def dequant_values(q, scale_bits, min_bits, mode=ADDITIVE):
    """float32 [M, K] in the reference's operation order (float32 throughout)."""
    s = np.repeat(bf16_bits_to_f32(scale_bits), GROUP, axis=1)
    m = np.repeat(bf16_bits_to_f32(min_bits), GROUP, axis=1)
    if mode == Q4_0:
        signed = (np.asarray(q, dtype=np.uint8) << 4).view(np.int8) >> 4   # two's complement nibble
        return signed.astype(np.float32) * s
    qf = np.asarray(q, dtype=np.float32)
    return s * (qf - m) if mode == SUBTRACTIVE else s * qf + m


def dequant(blocks, M, K, mode=ADDITIVE):
    """Blocks -> bf16 bits [M, K]."""
    return f32_to_bf16_bits(dequant_values(*unpack_matrix(blocks, M, K), mode))


def requant_q4k(W, group=GROUP):
    """float [M, K] -> (q uint8, scale float32 [M, K/group], min float32): per-group min/max."""
    M, K = W.shape
    Wg = np.asarray(W, dtype=np.float32).reshape(M, K // group, group)
    mn = Wg.min(2)
    mx = Wg.max(2)
    sc = (mx - mn) / 15.0
    sc = np.where(sc <= 0, 1.0, sc).astype(np.float32)
    q = np.clip(np.round((Wg - mn[..., None]) / sc[..., None]), 0, 15).astype(np.uint8)
    return q.reshape(M, K), sc, mn.astype(np.float32)


def requant_q4_0(W, group=GROUP):
    """float [M, K] -> (two's-complement codes uint8 [M, K], scale float32): w ~ q * scale, q in [-8, 7]."""
    M, K = W.shape
    Wg = np.asarray(W, dtype=np.float32).reshape(M, K // group, group)
    amax = np.abs(Wg).max(2)
    sc = np.where(amax <= 0, 1.0, amax / 8.0).astype(np.float32)
    q = np.clip(np.rint(Wg / sc[..., None]), -8, 7).astype(np.int8)
    return q.reshape(M, K).view(np.uint8), sc


def dequant_q4_0(q_u8, scale, group=GROUP):
    """One signed code per byte, scale [M, K/group] -> float32 [M, K]."""
    return q_u8.view(np.int8).astype(np.float32) * np.repeat(scale, group, axis=1)


def gemv_reference(q, scale_bits, min_bits, x_bits, mode=ADDITIVE):
    """y[M_rows_of_x, M] float64 for x bf16 bits [rows, K]: per group (sum q x) * s + m * sum x."""
    s = bf16_bits_to_f32(scale_bits).astype(np.float64)       # [M, K/32]
    m = bf16_bits_to_f32(min_bits).astype(np.float64)
    x = bf16_bits_to_f32(np.atleast_2d(x_bits)).astype(np.float64)
    M, K = q.shape
    ng = K // GROUP
    if mode == Q4_0:
        qv = ((np.asarray(q, dtype=np.uint8) << 4).view(np.int8) >> 4).astype(np.float64)
        m = np.zeros_like(s)
    else:
        qv = np.asarray(q, dtype=np.float64)
        if mode == SUBTRACTIVE:
            m = -s * m
    qg = qv.reshape(M, ng, GROUP)
    xg = x.reshape(x.shape[0], ng, GROUP)
    dot = np.einsum("mgk,rgk->rmg", qg, xg)                   # sum q x per group
    xsum = xg.sum(2)                                          # [rows, ng]
    return (dot * s[None] + m[None] * xsum[:, None, :]).sum(2)


def rms_gemv_reference(w, x_bits, norm_w_bits, eps=1e-5):
    """bf16 bits [M]: the GEMV on bf16((x * rstd) * norm_w).  w = (q, scale bits, min bits) of W[M, K]."""
    from . import reference as ref
    normed = f32_to_bf16_bits(ref.rms_norm_bf16(x_bits, norm_w_bits, eps))
    return f32_to_bf16_bits(gemv_reference(*w, normed)[0].astype(np.float32))


def block_staged_reference(wo, wg, wu, wd, attn_out_bits, x_residual_bits, ffn_norm_w_bits, eps=1e-5):
    """The O + FFN decode block in the staging of the int4 path (oracle/reference.py
    o_gemv_ffn_staged_reference), on affine-codec weights: res1 = bf16(attn . Wo + x),
    h = bf16(silu(bf16(n . Wg)) * bf16(n . Wu)) with n = bf16 RMSNorm of res1, y = bf16(h . Wd + res1).
    Returns (res1 bits, h bits, y bits)."""
    from . import reference as ref
    res1 = f32_to_bf16_bits((gemv_reference(*wo, attn_out_bits)[0]
                             + bf16_bits_to_f32(x_residual_bits).astype(np.float64)).astype(np.float32))
    normed = f32_to_bf16_bits(ref.rms_norm_bf16(res1, ffn_norm_w_bits, eps))
    gate = bf16_bits_to_f32(f32_to_bf16_bits(gemv_reference(*wg, normed)[0].astype(np.float32)))
    up = bf16_bits_to_f32(f32_to_bf16_bits(gemv_reference(*wu, normed)[0].astype(np.float32)))
    h = f32_to_bf16_bits(ref.silu_tanh_f32(gate) * up)
    y = f32_to_bf16_bits((gemv_reference(*wd, h)[0] + bf16_bits_to_f32(res1).astype(np.float64)).astype(np.float32))
    return res1, h, y
