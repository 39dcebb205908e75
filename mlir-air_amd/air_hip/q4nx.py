"""Q4NX / Q4_0 block codec on the host: block layout, quantisers, stream orders and the reader of
a local `model.q4nx` bundle.

One block is 32 rows (output features) x 256 columns (input features) of W[M, K], 5120 bytes:
bf16 scales[8 groups][32 rows] | bf16 mins[8][32] | uint8 qs[2 row groups][256 cols][8], byte kk
of (rg, col) = (q[16 rg + 2 kk + 1][col] << 4) | q[16 rg + 2 kk][col]
(programming_examples/fused_decode/proj_qmm_pack.py:4-9).  A tensor is its blocks in
(row-block, col-block) order; the reference's decode additionally permutes the blocks into a
per-core stream order (`pack_q4k_cascade`, proj_qmm_pack.py:61-140), which `cascade_permutation`
reproduces so that such a stream can be read back (`blocks_from_cascade`) or written
(`blocks_to_cascade`).

The GPU side (dequant, repack into GEMV operands, the GEMV itself) is in `ops`:
`q4nx_dequant`, `q4nx_repack`, `q4nx_gemm`.  bf16 values are uint16 bit patterns on the host.
"""

import json
import os

import numpy as np

from . import bf16

ROW_BLOCK = 32
COL_BLOCK = 256
GROUP = 32
PARALLEL = 16
N_GROUPS = COL_BLOCK // GROUP
ROW_GROUPS = ROW_BLOCK // PARALLEL
BLOCK_BYTES = 5120
BLOCK_BF16 = BLOCK_BYTES // 2

# value conventions (include/w4a16.h)
ADDITIVE, SUBTRACTIVE, Q4_0 = 0, 1, 2


def pack_blocks(q, scale_bits, min_bits=None):
    """q uint8 [M, K] (low nibble used), scale / min bf16 bits [M, K / 32] -> uint8
    [M/32 * K/256, 5120] in (row-block, col-block) order.  `min_bits` None writes zero mins
    (Q4_0, pack_q4k_cascade_fast, programming_examples/fused_decode/qwen25_3b_requant.py:137-175)."""
    q = np.asarray(q)
    M, K = q.shape
    if M % ROW_BLOCK or K % COL_BLOCK:
        raise ValueError(f"Q4NX needs M % {ROW_BLOCK} == 0 and K % {COL_BLOCK} == 0, got {(M, K)}")
    nbi, nbj = M // ROW_BLOCK, K // COL_BLOCK
    scale_bits = np.asarray(scale_bits).view(np.uint16)
    if scale_bits.shape != (M, K // GROUP):
        raise ValueError(f"scales must be [{M}, {K // GROUP}], got {scale_bits.shape}")
    min_bits = np.zeros_like(scale_bits) if min_bits is None else np.asarray(min_bits).view(np.uint16)

    def header(a):   # [M, K/32] -> [block][group][row]
        return np.ascontiguousarray(a.reshape(nbi, ROW_BLOCK, nbj, N_GROUPS).transpose(0, 2, 3, 1)).reshape(nbi * nbj, -1)

    nib = (q.astype(np.uint8) & 0xF).reshape(nbi, ROW_GROUPS, PARALLEL // 2, 2, nbj, COL_BLOCK)
    pair = (nib[:, :, :, 1] << 4) | nib[:, :, :, 0]                       # [nbi, rg, kk, nbj, col]
    out = np.empty((nbi * nbj, BLOCK_BYTES), dtype=np.uint8)
    out[:, :512] = header(scale_bits).view(np.uint8)
    out[:, 512:1024] = header(min_bits).view(np.uint8)
    out[:, 1024:] = pair.transpose(0, 3, 1, 4, 2).reshape(nbi * nbj, -1)  # [nbi, nbj, rg, col, kk]
    return out


def unpack_blocks(blocks, M, K):
    """Inverse of pack_blocks: (q uint8 [M, K], scale bits [M, K/32], min bits [M, K/32])."""
    nbi, nbj = M // ROW_BLOCK, K // COL_BLOCK
    b = np.asarray(blocks).view(np.uint8).reshape(nbi, nbj, BLOCK_BYTES)

    def header(lo):
        h = np.ascontiguousarray(b[:, :, lo:lo + 512]).view(np.uint16)
        return np.ascontiguousarray(h.reshape(nbi, nbj, N_GROUPS, ROW_BLOCK).transpose(0, 3, 1, 2)).reshape(M, K // GROUP)

    qs = b[:, :, 1024:].reshape(nbi, nbj, ROW_GROUPS, COL_BLOCK, PARALLEL // 2)
    q = np.empty((nbi, ROW_GROUPS, PARALLEL // 2, 2, nbj, COL_BLOCK), dtype=np.uint8)
    q[:, :, :, 0] = (qs & 0xF).transpose(0, 2, 4, 1, 3)
    q[:, :, :, 1] = (qs >> 4).transpose(0, 2, 4, 1, 3)
    return q.reshape(M, K), header(0), header(512)


def requant_q4k(W, group=GROUP):
    """Per-group min/max 4-bit quantisation of float W[M, K]: (q uint8, scale, min) float32 with
    w ~ q * scale + min (_requant_q4k, programming_examples/llms/llama32_1b_q4nx/q4nx_requant.py:25-35).
    Round scale and min to bf16 (bf16.from_f32) before packing, as the packer does."""
    M, K = W.shape
    Wg = np.asarray(W, dtype=np.float32).reshape(M, K // group, group)
    lo, hi = Wg.min(2), Wg.max(2)
    sc = (hi - lo) / 15.0
    sc = np.where(sc <= 0, 1.0, sc).astype(np.float32)
    q = np.clip(np.round((Wg - lo[..., None]) / sc[..., None]), 0, 15).astype(np.uint8)
    return q.reshape(M, K), sc, lo.astype(np.float32)


def requant_q4_0(W, group=GROUP):
    """Symmetric signed 4-bit quantisation: (two's-complement codes uint8 [M, K], scale float32)
    with w ~ q * scale, q in [-8, 7], scale = amax / 8 and 1 for an all-zero group
    (programming_examples/fused_decode/qwen25_3b_requant.py:116-134)."""
    M, K = W.shape
    Wg = np.asarray(W, dtype=np.float32).reshape(M, K // group, group)
    amax = np.abs(Wg).max(2)
    sc = np.where(amax <= 0, 1.0, amax / 8.0).astype(np.float32)
    q = np.clip(np.rint(Wg / sc[..., None]), -8, 7).astype(np.int8)
    return q.reshape(M, K).view(np.uint8), sc


def cascade_permutation(nbi, nbj, ncx, ncy, core_major=False, iter_major=False, dual_chan=False):
    """Index into the (row-block, col-block) ordered block list for every position of the
    reference's device stream [cx][i][j][cy] (pack_q4k_cascade, proj_qmm_pack.py:109-137;
    pack_q4k_cascade_fast is the iter_major case, qwen25_3b_requant.py:177-196)."""
    n_cores = ncx * ncy
    if nbi % n_cores:
        raise ValueError("row-blocks must split evenly across cores")
    nbi_pc = nbi // n_cores
    cx, i, j, cy = np.meshgrid(np.arange(ncx), np.arange(nbi_pc), np.arange(nbj), np.arange(ncy), indexing="ij")
    if iter_major:
        gi = i * n_cores + cx * ncy + cy
    elif core_major:
        gi = (cx * ncy + cy) * nbi_pc + i
    else:
        gi = cx * (ncy * nbi_pc) + i * ncy + cy
    idx = gi * nbj + j                                   # [cx, i, j, cy]
    if dual_chan:                                        # row half (= shim channel) outermost inside cx
        if ncy % 2:
            raise ValueError("dual_chan needs an even NCY")
        idx = idx.reshape(ncx, nbi_pc, nbj, 2, ncy // 2).transpose(0, 3, 1, 2, 4)
    return np.ascontiguousarray(idx).reshape(-1)


def blocks_to_cascade(blocks, nbi, nbj, ncx, ncy, **order):
    """Plain-order blocks [nbi * nbj, 5120] -> the reference's stream (int16 [nb * 2560])."""
    perm = cascade_permutation(nbi, nbj, ncx, ncy, **order)
    return np.ascontiguousarray(np.asarray(blocks).view(np.uint8).reshape(nbi * nbj, BLOCK_BYTES)[perm]).view(np.int16).reshape(-1)


def blocks_from_cascade(stream, nbi, nbj, ncx, ncy, **order):
    """A stream written by pack_q4k_cascade -> plain-order blocks uint8 [nbi * nbj, 5120]."""
    perm = cascade_permutation(nbi, nbj, ncx, ncy, **order)
    src = np.ascontiguousarray(np.asarray(stream)).view(np.uint8).reshape(nbi * nbj, BLOCK_BYTES)
    out = np.empty_like(src)
    out[perm] = src
    return out


class Q4nxModel:
    """Reader of a local `model.q4nx` (a safetensors container with the custom tensor types
    "Q4NX" and "I8"; Q4nxModel, programming_examples/llms/llama32_1b_q4nx/llama32_1b_q4nx_weights.py:148-266).

    A quantised tensor comes back as (blocks uint8 [nb, 5120], mode): "Q4NX" headers carry the
    logical [M, K] and the subtractive convention, "I8" headers carry [n_blocks, 5120], need M and K
    from the model configuration and are additive.  Nothing is downloaded: `path` is a file or a
    directory that contains model.q4nx.
    """

    def __init__(self, path):
        if os.path.isdir(path):
            path = os.path.join(path, "model.q4nx")
        if not os.path.isfile(path):
            raise FileNotFoundError(f"'{path}' not found; downloading bundles is not supported here")
        self._mm = np.memmap(path, dtype=np.uint8, mode="r")
        hlen = int(np.frombuffer(self._mm[:8].tobytes(), dtype="<u8")[0])
        self._hdr = json.loads(self._mm[8:8 + hlen].tobytes())
        self._base = 8 + hlen

    def names(self):
        return [k for k in self._hdr if k != "__metadata__"]

    def has(self, name):
        return name in self._hdr

    def _raw(self, name):
        o0, o1 = self._hdr[name]["data_offsets"]
        return np.asarray(self._mm[self._base + o0:self._base + o1])

    def bf16_bits(self, name):
        """A BF16 tensor as uint16 bit patterns in its declared shape."""
        e = self._hdr[name]
        if e["dtype"] != "BF16":
            raise TypeError(f"{name} is {e['dtype']}, not BF16")
        return bf16.from_bits(self._raw(name).view(np.uint16).reshape(e["shape"]))

    def dims(self, name):
        """Logical (M, K) of a quantised tensor, or None when the header does not carry it."""
        e = self._hdr[name]
        return tuple(e["shape"]) if e.get("dtype") == "Q4NX" else None

    def blocks(self, name, M=None, K=None):
        """(blocks uint8 [nb, 5120], mode, M, K) of a quantised tensor."""
        e = self._hdr[name]
        hdr_dims = self.dims(name)
        if hdr_dims is None:
            if M is None or K is None:
                raise ValueError(f"{name}: packed header {e['shape']} does not carry the logical shape; pass M and K")
        else:
            if M is not None and (M, K) != hdr_dims:
                raise ValueError(f"{name}: caller says {(M, K)}, header {hdr_dims}")
            M, K = hdr_dims
        if M % ROW_BLOCK or K % COL_BLOCK:
            raise ValueError(f"{name}: [M, K] = {[M, K]} is not a whole number of {ROW_BLOCK} x {COL_BLOCK} blocks")
        nb = (M // ROW_BLOCK) * (K // COL_BLOCK)
        raw = self._raw(name)
        if raw.size != nb * BLOCK_BYTES or (hdr_dims is None and e["shape"][0] != nb):
            raise ValueError(f"{name}: holds {raw.size // BLOCK_BYTES} blocks but [M, K] = {[M, K]} needs {nb}")
        return raw.reshape(nb, BLOCK_BYTES), (SUBTRACTIVE if hdr_dims is not None else ADDITIVE), M, K
