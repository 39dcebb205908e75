"""Operator-level wrappers over the C ABI for torch (ROCm) tensors.

torch is used for device memory and streams only.  Every function launches on
the current torch stream of the tensors' device and returns without
synchronising.  There is no CPU path: tensors must live on the GPU.
"""

import torch

from . import _lib

GROUP = 128
_workspaces = {}
_checked = False


def _ptr(t):
    return t.data_ptr()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _need_cuda(*tensors):
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("air_hip ops need GPU tensors; there is no CPU fallback")
        if not t.is_contiguous():
            raise ValueError("air_hip ops need contiguous tensors")


def _bits(t):
    """bf16 tensors are passed as their 16-bit patterns."""
    if t.dtype == torch.bfloat16:
        return t
    if t.dtype in (torch.int16, torch.uint16):
        return t
    raise TypeError(f"expected a bf16 tensor (or its int16 bits), got {t.dtype}")


def workspace(nbytes, device, use="gemm"):
    """Cleared workspace per (device, stream, use), grown on demand.  `use` names the entry point and
    shape: the FFN and block entry points keep plain intermediates (h, res1) behind their slot area,
    so a buffer is only shared between calls that lay it out the same way."""
    lib = _lib.load_library()
    key = (device.index, _stream(), use)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(int(nbytes), dtype=torch.uint8, device=device)
        _lib.check(lib.w4a16_workspace_init(_ptr(ws), ws.numel(), _stream()))
        _workspaces[key] = ws
    return ws


def check_health():
    """Synchronise the device and look at every split-K workspace that this module handed out: if a reducer of an
    earlier call gave up waiting for a partial result (its output is then invalid), re-initialise that workspace, so
    that the next call works, and raise W4A16Error(ERR_TIMEOUT).  The launches themselves never synchronise, so this is
    the place where such a failure becomes visible: callers that read results back on the host (the backends, the
    token loop) call it there (counterpart of the run-state check after a kernel run,
    python/air/backend/xrt.py:204-218).  The stream-order entry points keep no such state and cannot time out."""
    lib = _lib.load_library()
    torch.cuda.synchronize()
    failed = []
    for key, ws in _workspaces.items():
        if lib.w4a16_workspace_check(_ptr(ws), None) == _lib.ERR_TIMEOUT:
            _lib.check(lib.w4a16_workspace_init(_ptr(ws), ws.numel(), None))
            failed.append(key)
    if _noalloc_used and lib.w4a16_noalloc_check(None) == _lib.ERR_TIMEOUT:   # (the array inside the library)
        failed.append((None, None, "no-alloc array"))
    if failed:
        torch.cuda.synchronize()
        raise _lib.W4A16Error(_lib.ERR_TIMEOUT, "a split-K reducer gave up waiting for a partial result; the outputs of the calls "
                              f"since the last check are invalid (workspaces {[k[2] for k in failed]} re-initialised)")


_noalloc_used = False


def w4a16_gemv_noalloc(x, qweight, qzeros, scales, group=GROUP, out=None):
    """w4a16_gemv on the library's own split-K array (w4a16_gemv_noalloc_bf16): no workspace from this module.
    check_health() looks at that array as well once this has been called."""
    global _noalloc_used
    lib = _lib.load_library()
    _need_cuda(x, qweight, qzeros, scales)
    K, N = x.numel(), qweight.shape[1] * 8
    if qweight.shape[0] != K:
        raise ValueError(f"x has K={K} but qweight has {qweight.shape[0]} rows")
    if out is None:
        out = torch.empty((N,), dtype=torch.bfloat16, device=x.device)
    _lib.check(lib.w4a16_gemv_noalloc_bf16(_ptr(_bits(x)), _ptr(qweight), _ptr(qzeros), _ptr(_bits(scales)), _ptr(out), K, N,
                                           group, _stream()))
    _noalloc_used = True
    _after_workspace_call()
    return out


def set_checked(on):
    """Checked mode: every call that uses a split-K workspace synchronises and runs check_health() before it returns
    (for tests and for hunting a failure down to one call; off by default)."""
    global _checked
    _checked = bool(on)


def _after_workspace_call():
    if _checked:
        check_health()


def awq_dequant(qweight, qzeros, scales, group=GROUP, out=None):
    """Dense W[K, N] bf16 from AWQ tensors (int32 [K, N/8], int32 [K/g, N/8], bf16 [K/g, N])."""
    lib = _lib.load_library()
    _need_cuda(qweight, qzeros, scales)
    K, nb = qweight.shape
    N = nb * 8
    if out is None:
        out = torch.empty((K, N), dtype=torch.bfloat16, device=qweight.device)
    _lib.check(lib.awq_dequant_bf16(_ptr(qweight), _ptr(qzeros), _ptr(_bits(scales)), _ptr(out), K, N, group, _stream()))
    return out


def awq_dequant_1d(packed, n, group=GROUP, herd_n=4, out=None):
    """1-D dequant of the reference example's tiled buffer (uint8 [herd_n * tile_bytes]) -> bf16 [n]."""
    lib = _lib.load_library()
    _need_cuda(packed)
    tile_bytes = lib.awq_dequant_1d_tile_bytes(n, group, herd_n)
    if tile_bytes == 0 or packed.numel() != herd_n * tile_bytes:
        raise ValueError(f"awq_dequant_1d: n={n}, group={group}, herd_n={herd_n} needs {herd_n} tiles of {tile_bytes} bytes")
    if out is None:
        out = torch.empty((n,), dtype=torch.bfloat16, device=packed.device)
    _lib.check(lib.awq_dequant_1d_bf16(_ptr(packed), _ptr(out), n, group, herd_n, _stream()))
    return out


def w4a16_gemm(x, qweight, qzeros, scales, group=GROUP, out=None):
    """y[M, N] = bf16(x[M, K] . W); x may also be a vector [K] (returns [N])."""
    lib = _lib.load_library()
    _need_cuda(x, qweight, qzeros, scales)
    vec = x.dim() == 1
    x2 = x.unsqueeze(0) if vec else x
    M, K = x2.shape
    if qweight.shape[0] != K:
        raise ValueError(f"x has K={K} but qweight has {qweight.shape[0]} rows")
    N = qweight.shape[1] * 8
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    nbytes = lib.w4a16_gemm_workspace_bytes(M, K, N)
    ws = workspace(nbytes, x.device)
    _lib.check(lib.w4a16_gemm_bf16(_ptr(_bits(x2)), _ptr(qweight), _ptr(qzeros), _ptr(_bits(scales)), _ptr(out),
                                   M, K, N, group, _ptr(ws), ws.numel(), _stream()))
    _after_workspace_call()
    return out.squeeze(0) if vec else out


def w4a16_gemv(x, qweight, qzeros, scales, group=GROUP, out=None):
    """Decode GEMV: y[N] = bf16(x[K] . W)."""
    lib = _lib.load_library()
    _need_cuda(x, qweight, qzeros, scales)
    K = x.numel()
    if qweight.shape[0] != K:
        raise ValueError(f"x has K={K} but qweight has {qweight.shape[0]} rows")
    N = qweight.shape[1] * 8
    if out is None:
        out = torch.empty((N,), dtype=torch.bfloat16, device=x.device)
    ws = workspace(lib.w4a16_gemm_workspace_bytes(1, K, N), x.device)
    _lib.check(lib.w4a16_gemv_bf16(_ptr(_bits(x)), _ptr(qweight), _ptr(qzeros), _ptr(_bits(scales)), _ptr(out),
                                   K, N, group, _ptr(ws), ws.numel(), _stream()))
    _after_workspace_call()
    return out


def w4a16_swiglu(x, gate, up, group=GROUP):
    """Decode FFN front half: h[H] = bf16(silu(bf16(x Wg)) * bf16(x Wu)); gate/up are (qweight, qzeros, scales)."""
    lib = _lib.load_library()
    _need_cuda(x, *gate, *up)
    K = x.numel()
    H = gate[0].shape[1] * 8
    if gate[0].shape[0] != K or up[0].shape != gate[0].shape:
        raise ValueError("w4a16_swiglu: gate and up must both be [K, H/8]")
    h = torch.empty((H,), dtype=torch.bfloat16, device=x.device)
    ws = workspace(lib.w4a16_ffn_workspace_bytes(K, H), x.device, ("ffn", K, H))
    _lib.check(lib.w4a16_gemv_swiglu_bf16(
        _ptr(_bits(x)), _ptr(gate[0]), _ptr(gate[1]), _ptr(_bits(gate[2])),
        _ptr(up[0]), _ptr(up[1]), _ptr(_bits(up[2])), _ptr(h), K, H, group, _ptr(ws), ws.numel(), _stream()))
    _after_workspace_call()
    return h


def ffn_swiglu(x, gate, up, down, group=GROUP, return_h=False):
    """Decode FFN: y = Wd(silu(x Wg) * (x Wu)); gate/up/down are (qweight, qzeros, scales)."""
    lib = _lib.load_library()
    _need_cuda(x, *gate, *up, *down)
    K = x.numel()
    H = gate[0].shape[1] * 8
    if gate[0].shape[0] != K or up[0].shape != gate[0].shape or down[0].shape[0] != H or down[0].shape[1] * 8 != K:
        raise ValueError("ffn_swiglu: gate/up must be [K, H/8] and down [H, K/8]")
    y = torch.empty((K,), dtype=torch.bfloat16, device=x.device)
    h = torch.empty((H,), dtype=torch.bfloat16, device=x.device) if return_h else None
    ws = workspace(lib.w4a16_ffn_workspace_bytes(K, H), x.device, ("ffn", K, H))
    _lib.check(lib.w4a16_ffn_swiglu_bf16(
        _ptr(_bits(x)),
        _ptr(gate[0]), _ptr(gate[1]), _ptr(_bits(gate[2])),
        _ptr(up[0]), _ptr(up[1]), _ptr(_bits(up[2])),
        _ptr(down[0]), _ptr(down[1]), _ptr(_bits(down[2])),
        _ptr(y), _ptr(h) if h is not None else None, K, H, group, _ptr(ws), ws.numel(), _stream()))
    _after_workspace_call()
    return (y, h) if return_h else y


def _wptrs(w):
    return [_ptr(w[0]), _ptr(w[1]), _ptr(_bits(w[2]))]


class StreamWeight:
    """One AWQ matrix in stream order (the device layout of the decode kernels), made once at load time
    by `repack_stream`: the counterpart of the reference's per-layer packed decode buffers
    (repack_for_gemv, programming_examples/llms/llama32_1b_int4/awq_repacker.py:112-135)."""

    __slots__ = ("buf", "K", "N", "order")

    def __init__(self, buf, K, N, order="awq"):
        self.buf, self.K, self.N, self.order = buf, K, N, order   # order: "awq", or "q4nx" (q4nx_repack_stream)


def _need_order(order, *weights):
    """The two orders are read by different kernels (a Q4NX-order kernel on an AWQ-order buffer would run past its end)."""
    for w in weights:
        if w is not None and w.order != order:
            raise ValueError(f"this op takes StreamWeights in {order} order, got one in {w.order} order")


def repack_stream(qweight, qzeros, scales, group=GROUP):
    """AWQ tensors on the GPU -> StreamWeight (one kernel, no host round trip)."""
    lib = _lib.load_library()
    _need_cuda(qweight, qzeros, scales)
    K, nb = qweight.shape
    N = nb * 8
    nbytes = lib.w4a16_stream_bytes(K, N)
    if nbytes == 0:
        raise ValueError(f"stream order needs K % 128 == 0 and N % 16 == 0, got K={K}, N={N}")
    buf = torch.empty(int(nbytes), dtype=torch.uint8, device=qweight.device)
    _lib.check(lib.w4a16_repack_stream(_ptr(qweight), _ptr(qzeros), _ptr(_bits(scales)), _ptr(buf), K, N, group, _stream()))
    return StreamWeight(buf, K, N)


def w4a16_gemv_stream(x, w, residual=None, group=GROUP, out=None):
    """Decode GEMV on a StreamWeight: y[N] = bf16(x[K] . W), with `residual` y = bf16(x . W + R).
    Stateless (no workspace)."""
    lib = _lib.load_library()
    _need_cuda(x, w.buf)
    _need_order("awq", w)
    if x.numel() != w.K:
        raise ValueError(f"x has K={x.numel()} but the matrix has {w.K} rows")
    if out is None:
        out = torch.empty((w.N,), dtype=torch.bfloat16, device=x.device)
    if residual is not None:
        _need_cuda(residual)
        if residual.numel() != w.N:
            raise ValueError(f"residual has {residual.numel()} elements, expected N={w.N}")
        _lib.check(lib.w4a16_gemv_add_stream_bf16(_ptr(_bits(x)), _ptr(w.buf), _ptr(_bits(residual)), _ptr(out), w.K, w.N,
                                                  group, _stream()))
    else:
        _lib.check(lib.w4a16_gemv_stream_bf16(_ptr(_bits(x)), _ptr(w.buf), _ptr(out), w.K, w.N, group, _stream()))
    return out


_gemm_scratch = {}


def w4a16_gemm_stream(x, w, group=GROUP, out=None):
    """y[M, N] = bf16(x[M, K] . W) on a StreamWeight; x may be a vector [K].  Batches of 17 to 128 rows run split along
    K with their partial sums in a scratch buffer of this module (plain scratch per device and stream, grown on
    demand, nothing kept in it between calls)."""
    lib = _lib.load_library()
    _need_cuda(x, w.buf)
    _need_order("awq", w)
    vec = x.dim() == 1
    x2 = x.unsqueeze(0) if vec else x
    M, K = x2.shape
    if K != w.K:
        raise ValueError(f"x has K={K} but the matrix has {w.K} rows")
    if out is None:
        out = torch.empty((M, w.N), dtype=torch.bfloat16, device=x.device)
    need = lib.w4a16_gemm_stream_scratch_bytes(M, K, w.N)
    if need:
        key = (x.device.index, _stream())
        scratch = _gemm_scratch.get(key)
        if scratch is None or scratch.numel() < need:
            scratch = _gemm_scratch[key] = torch.empty(int(need), dtype=torch.uint8, device=x.device)
        _lib.check(lib.w4a16_gemm_stream_scratch_bf16(_ptr(_bits(x2)), _ptr(w.buf), _ptr(out), M, K, w.N, group, _ptr(scratch),
                                                      scratch.numel(), _stream()))
    else:
        _lib.check(lib.w4a16_gemm_stream_bf16(_ptr(_bits(x2)), _ptr(w.buf), _ptr(out), M, K, w.N, group, _stream()))
    return out.squeeze(0) if vec else out


def w4a16_swiglu_stream(x, gate, up, group=GROUP, out=None):
    """Decode FFN front half on two StreamWeights: h[H] = bf16(silu(bf16(x Wg)) * bf16(x Wu))."""
    lib = _lib.load_library()
    _need_cuda(x, gate.buf, up.buf)
    _need_order("awq", gate, up)
    if x.numel() != gate.K or (up.K, up.N) != (gate.K, gate.N):
        raise ValueError("w4a16_swiglu_stream: gate and up must both be [K, H]")
    if out is None:
        out = torch.empty((gate.N,), dtype=torch.bfloat16, device=x.device)
    _lib.check(lib.w4a16_gemv_swiglu_stream_bf16(_ptr(_bits(x)), _ptr(gate.buf), _ptr(up.buf), _ptr(out), gate.K, gate.N,
                                                 group, _stream()))
    return out


def w4a16_gemv_add(x, qweight, qzeros, scales, residual, group=GROUP, out=None):
    """Decode GEMV with residual: y[N] = bf16(x[K] . W + R[N]) (one rounding)."""
    lib = _lib.load_library()
    _need_cuda(x, qweight, qzeros, scales, residual)
    K = x.numel()
    if qweight.shape[0] != K:
        raise ValueError(f"x has K={K} but qweight has {qweight.shape[0]} rows")
    N = qweight.shape[1] * 8
    if residual.numel() != N:
        raise ValueError(f"residual has {residual.numel()} elements, expected N={N}")
    if out is None:
        out = torch.empty((N,), dtype=torch.bfloat16, device=x.device)
    ws = workspace(lib.w4a16_gemm_workspace_bytes(1, K, N), x.device)
    _lib.check(lib.w4a16_gemv_add_bf16(_ptr(_bits(x)), *_wptrs((qweight, qzeros, scales)), _ptr(_bits(residual)),
                                       _ptr(out), K, N, group, _ptr(ws), ws.numel(), _stream()))
    _after_workspace_call()
    return out


def w4a16_rms_gemv(x, norm_weight, qweight, qzeros, scales, eps=1e-5, group=GROUP, x_sumsq=None):
    """y[N] = bf16(rms_norm(x, norm_weight) . W), the normalised vector rounded to bf16 first.  x_sumsq: float32
    partial sums of x^2 (at most 64) left by the call that produced x (decode_attn_o_gemv_ffn), used for the mean
    instead of a pass over x."""
    lib = _lib.load_library()
    _need_cuda(x, norm_weight, qweight, qzeros, scales)
    K = x.numel()
    if qweight.shape[0] != K or norm_weight.numel() != K:
        raise ValueError("w4a16_rms_gemv: x, norm_weight must have K elements and qweight K rows")
    N = qweight.shape[1] * 8
    out = torch.empty((N,), dtype=torch.bfloat16, device=x.device)
    ws = workspace(lib.w4a16_gemm_workspace_bytes(1, K, N), x.device)
    if x_sumsq is not None:
        if x_sumsq.dtype != torch.float32 or not x_sumsq.is_cuda or not x_sumsq.is_contiguous():
            raise ValueError("x_sumsq must be a contiguous float32 GPU tensor")
        _lib.check(lib.w4a16_rms_gemv_sumsq_bf16(_ptr(_bits(x)), _ptr(x_sumsq), x_sumsq.numel(), _ptr(_bits(norm_weight)),
                                                 float(eps), *_wptrs((qweight, qzeros, scales)), _ptr(out), K, N, group,
                                                 _ptr(ws), ws.numel(), _stream()))
        return out
    _lib.check(lib.w4a16_rms_gemv_bf16(_ptr(_bits(x)), _ptr(_bits(norm_weight)), float(eps),
                                       *_wptrs((qweight, qzeros, scales)), _ptr(out), K, N, group,
                                       _ptr(ws), ws.numel(), _stream()))
    _after_workspace_call()
    return out


def w4a16_rms_swiglu(x, norm_weight, gate, up, eps=1e-5, group=GROUP):
    """h[H] = bf16(silu(bf16(n Wg)) * bf16(n Wu)) with n = bf16((x * rstd) * norm_weight)."""
    lib = _lib.load_library()
    _need_cuda(x, norm_weight, *gate, *up)
    K = x.numel()
    H = gate[0].shape[1] * 8
    if gate[0].shape[0] != K or up[0].shape != gate[0].shape or norm_weight.numel() != K:
        raise ValueError("w4a16_rms_swiglu: gate and up must both be [K, H/8], norm_weight [K]")
    h = torch.empty((H,), dtype=torch.bfloat16, device=x.device)
    ws = workspace(lib.w4a16_ffn_workspace_bytes(K, H), x.device, ("ffn", K, H))
    _lib.check(lib.w4a16_rms_gemv_swiglu_bf16(_ptr(_bits(x)), _ptr(_bits(norm_weight)), float(eps),
                                              *_wptrs(gate), *_wptrs(up), _ptr(h), K, H, group,
                                              _ptr(ws), ws.numel(), _stream()))
    _after_workspace_call()
    return h


def o_gemv_ffn(attn_out, x_residual, ffn_norm_weight, wo, gate, up, down, eps=1e-5, group=GROUP,
               return_intermediates=False):
    """Decode block: res1 = Wo(attn_out) + x_residual; y = Wd(swiglu(rms_norm(res1))) + res1.

    wo/gate/up/down are (qweight, qzeros, scales).  Returns y, or (y, res1, h).
    """
    lib = _lib.load_library()
    _need_cuda(attn_out, x_residual, ffn_norm_weight, *wo, *gate, *up, *down)
    E = attn_out.numel()
    H = gate[0].shape[1] * 8
    if (wo[0].shape[0] != E or wo[0].shape[1] * 8 != E or gate[0].shape[0] != E or up[0].shape != gate[0].shape
            or down[0].shape[0] != H or down[0].shape[1] * 8 != E or x_residual.numel() != E
            or ffn_norm_weight.numel() != E):
        raise ValueError("o_gemv_ffn: wo must be [E, E/8], gate/up [E, H/8], down [H, E/8], vectors [E]")
    dev = attn_out.device
    y = torch.empty((E,), dtype=torch.bfloat16, device=dev)
    res1 = torch.empty((E,), dtype=torch.bfloat16, device=dev) if return_intermediates else None
    h = torch.empty((H,), dtype=torch.bfloat16, device=dev) if return_intermediates else None
    ws = workspace(lib.w4a16_block_workspace_bytes(E, H), dev, ("block", E, H))
    _lib.check(lib.w4a16_o_gemv_ffn_bf16(
        _ptr(_bits(attn_out)), _ptr(_bits(x_residual)), _ptr(_bits(ffn_norm_weight)), float(eps),
        *_wptrs(wo), *_wptrs(gate), *_wptrs(up), *_wptrs(down), _ptr(y),
        _ptr(res1) if res1 is not None else None, _ptr(h) if h is not None else None,
        E, H, group, _ptr(ws), ws.numel(), _stream()))
    _after_workspace_call()
    return (y, res1, h) if return_intermediates else y


_attn_ws = {}


def decode_attention(qkv, rope_lut_row, k_cache, v_cache, pos, n_heads, out=None):
    """RoPE on Q and K of the new token, KV-cache append at `pos`, single-query GQA attention.

    qkv bf16 [n_heads * hd + 2 * n_kv * hd]; rope_lut_row bf16 [hd]; caches bf16 [n_kv, max_seq, hd]
    (updated in place).  Returns attn_out bf16 [n_heads * hd]."""
    lib = _lib.load_library()
    _need_cuda(qkv, rope_lut_row, k_cache, v_cache)
    n_kv, max_seq, hd = k_cache.shape
    if v_cache.shape != k_cache.shape or qkv.numel() != (n_heads + 2 * n_kv) * hd or rope_lut_row.numel() != hd:
        raise ValueError("decode_attention: qkv must be [(n_heads + 2 n_kv) * hd], caches [n_kv, max_seq, hd], lut row [hd]")
    if out is None:
        out = torch.empty((n_heads * hd,), dtype=torch.bfloat16, device=qkv.device)
    key = (qkv.device.index, _stream(), n_heads, hd)
    ws = _attn_ws.get(key)
    if ws is None:
        ws = torch.empty(int(lib.w4a16_attention_workspace_bytes(n_heads, hd)), dtype=torch.uint8, device=qkv.device)
        _attn_ws[key] = ws
    _lib.check(lib.w4a16_decode_attention_bf16(_ptr(_bits(qkv)), _ptr(_bits(rope_lut_row)), _ptr(_bits(k_cache)),
                                               _ptr(_bits(v_cache)), _ptr(out), int(pos), max_seq, n_heads, n_kv, hd,
                                               _ptr(ws), ws.numel(), _stream()))
    return out


def decode_attn_o_gemv_ffn(qkv, rope_lut_row, k_cache, v_cache, pos, n_heads, x_residual, ffn_norm_weight, wo, gate, up, down,
                           eps=1e-5, group=GROUP, return_sumsq=False):
    """decode_attention followed by o_gemv_ffn in one call; over several sequence chunks the O projection merges the
    attention partials itself (one launch fewer), with the same result bit for bit.  Returns y bf16 [E], with
    return_sumsq also float32 [E / 256]: the sum of squares of y per 256-column tile for the next layer's
    w4a16_rms_gemv (None where E is not a multiple of 256)."""
    lib = _lib.load_library()
    _need_cuda(qkv, rope_lut_row, k_cache, v_cache, x_residual, ffn_norm_weight, *wo, *gate, *up, *down)
    n_kv, max_seq, hd = k_cache.shape
    E = n_heads * hd
    H = gate[0].shape[1] * 8
    if v_cache.shape != k_cache.shape or qkv.numel() != (n_heads + 2 * n_kv) * hd or rope_lut_row.numel() != hd:
        raise ValueError("decode_attn_o_gemv_ffn: qkv must be [(n_heads + 2 n_kv) * hd], caches [n_kv, max_seq, hd], lut row [hd]")
    if (wo[0].shape[0] != E or wo[0].shape[1] * 8 != E or gate[0].shape[0] != E or up[0].shape != gate[0].shape
            or down[0].shape[0] != H or down[0].shape[1] * 8 != E or x_residual.numel() != E or ffn_norm_weight.numel() != E):
        raise ValueError("decode_attn_o_gemv_ffn: wo must be [E, E/8], gate/up [E, H/8], down [H, E/8], vectors [E]")
    dev = qkv.device
    y = torch.empty((E,), dtype=torch.bfloat16, device=dev)
    attn_out = torch.empty((E,), dtype=torch.bfloat16, device=dev)
    key = (dev.index, _stream(), n_heads, hd)
    aws = _attn_ws.get(key)
    if aws is None:
        aws = torch.empty(int(lib.w4a16_attention_workspace_bytes(n_heads, hd)), dtype=torch.uint8, device=dev)
        _attn_ws[key] = aws
    ws = workspace(lib.w4a16_block_workspace_bytes(E, H), dev, ("block", E, H))
    sumsq = torch.empty((E // 256,), dtype=torch.float32, device=dev) if return_sumsq and E % 256 == 0 and E <= 16384 else None
    _lib.check(lib.w4a16_decode_attn_o_gemv_ffn_bf16(
        _ptr(_bits(qkv)), _ptr(_bits(rope_lut_row)), _ptr(_bits(k_cache)), _ptr(_bits(v_cache)), _ptr(attn_out), int(pos),
        max_seq, n_heads, n_kv, hd, _ptr(aws), aws.numel(), _ptr(_bits(x_residual)), _ptr(_bits(ffn_norm_weight)), float(eps),
        *_wptrs(wo), *_wptrs(gate), *_wptrs(up), *_wptrs(down), _ptr(y), _ptr(sumsq) if sumsq is not None else None, E, H, group,
        _ptr(ws), ws.numel(), _stream()))
    _after_workspace_call()
    return (y, sumsq) if return_sumsq else y


_block_scratch = {}


def _block_stream_scratch(E, H, device):
    """Plain scratch of the stream-order block (res1, h, sums of squares): nothing is kept in it between calls."""
    lib = _lib.load_library()
    key = (device.index, _stream(), E, H)
    ws = _block_scratch.get(key)
    if ws is None:
        ws = torch.empty(int(lib.w4a16_block_stream_workspace_bytes(E, H)), dtype=torch.uint8, device=device)
        _block_scratch[key] = ws
    return ws


def w4a16_rms_gemv_stream(x, norm_weight, w, eps=1e-5, group=GROUP, x_sumsq=None):
    """y[N] = bf16(rms_norm(x, norm_weight) . W) on a StreamWeight.  x_sumsq: float32 partial sums of x^2 left by the
    call that produced x (o_gemv_ffn_stream / decode_attn_o_gemv_ffn_stream with return_sumsq)."""
    lib = _lib.load_library()
    _need_cuda(x, norm_weight, w.buf)
    _need_order("awq", w)
    if x.numel() != w.K or norm_weight.numel() != w.K:
        raise ValueError("w4a16_rms_gemv_stream: x and norm_weight must have K elements")
    out = torch.empty((w.N,), dtype=torch.bfloat16, device=x.device)
    if x_sumsq is not None and (x_sumsq.dtype != torch.float32 or not x_sumsq.is_cuda or not x_sumsq.is_contiguous()):
        raise ValueError("x_sumsq must be a contiguous float32 GPU tensor")
    _lib.check(lib.w4a16_rms_gemv_stream_bf16(_ptr(_bits(x)), _ptr(x_sumsq) if x_sumsq is not None else None,
                                              x_sumsq.numel() if x_sumsq is not None else 0, _ptr(_bits(norm_weight)), float(eps),
                                              _ptr(w.buf), _ptr(out), w.K, w.N, group, _stream()))
    return out


def w4a16_rms_swiglu_stream(x, norm_weight, gate, up, eps=1e-5, group=GROUP):
    """h[H] = bf16(silu(bf16(n Wg)) * bf16(n Wu)), n = bf16((x * rstd) * norm_weight), on two StreamWeights."""
    lib = _lib.load_library()
    _need_cuda(x, norm_weight, gate.buf, up.buf)
    _need_order("awq", gate, up)
    if x.numel() != gate.K or (up.K, up.N) != (gate.K, gate.N) or norm_weight.numel() != gate.K:
        raise ValueError("w4a16_rms_swiglu_stream: gate and up must both be [K, H], x and norm_weight [K]")
    h = torch.empty((gate.N,), dtype=torch.bfloat16, device=x.device)
    _lib.check(lib.w4a16_rms_gemv_swiglu_stream_bf16(_ptr(_bits(x)), _ptr(_bits(norm_weight)), float(eps), _ptr(gate.buf),
                                                     _ptr(up.buf), _ptr(h), gate.K, gate.N, group, _stream()))
    return h


def ffn_swiglu_stream(x, gate, up, down, group=GROUP, return_h=False):
    """Decode FFN on StreamWeights: y = Wd(silu(x Wg) * (x Wu)); two whole-K launches, no workspace."""
    lib = _lib.load_library()
    _need_cuda(x, gate.buf, up.buf, down.buf)
    _need_order("awq", gate, up, down)
    K, H = gate.K, gate.N
    if x.numel() != K or (up.K, up.N) != (K, H) or (down.K, down.N) != (H, K):
        raise ValueError("ffn_swiglu_stream: gate/up must be [K, H] and down [H, K]")
    y = torch.empty((K,), dtype=torch.bfloat16, device=x.device)
    h = torch.empty((H,), dtype=torch.bfloat16, device=x.device)
    _lib.check(lib.w4a16_ffn_swiglu_stream_bf16(_ptr(_bits(x)), _ptr(gate.buf), _ptr(up.buf), _ptr(down.buf), _ptr(y), _ptr(h),
                                                K, H, group, _stream()))
    return (y, h) if return_h else y


def _check_block_stream(E, H, wo, gate, up, down, *vectors):
    if ((wo.K, wo.N) != (E, E) or (gate.K, gate.N) != (E, H) or (up.K, up.N) != (E, H) or (down.K, down.N) != (H, E)
            or any(v.numel() != E for v in vectors)):
        raise ValueError("stream-order block: wo must be [E, E], gate/up [E, H], down [H, E], vectors [E]")


def o_gemv_ffn_stream(attn_out, x_residual, ffn_norm_weight, wo, gate, up, down, eps=1e-5, group=GROUP,
                      return_intermediates=False, return_sumsq=False):
    """Decode block on StreamWeights: res1 = Wo(attn_out) + x_residual; y = Wd(swiglu(rms_norm(res1))) + res1.
    Returns y, or (y, res1, h); with return_sumsq the sum of squares of y per 16 columns (float32 [E / 16]) is
    appended for the next layer's w4a16_rms_gemv_stream."""
    lib = _lib.load_library()
    _need_cuda(attn_out, x_residual, ffn_norm_weight, wo.buf, gate.buf, up.buf, down.buf)
    _need_order("awq", wo, gate, up, down)
    E, H = wo.K, gate.N
    _check_block_stream(E, H, wo, gate, up, down, attn_out, x_residual, ffn_norm_weight)
    dev = attn_out.device
    y = torch.empty((E,), dtype=torch.bfloat16, device=dev)
    res1 = torch.empty((E,), dtype=torch.bfloat16, device=dev) if return_intermediates else None
    h = torch.empty((H,), dtype=torch.bfloat16, device=dev) if return_intermediates else None
    sumsq = torch.empty((E // 16,), dtype=torch.float32, device=dev) if return_sumsq else None
    ws = _block_stream_scratch(E, H, dev)
    opt = lambda t: _ptr(t) if t is not None else None
    _lib.check(lib.w4a16_o_gemv_ffn_stream_bf16(
        _ptr(_bits(attn_out)), _ptr(_bits(x_residual)), _ptr(_bits(ffn_norm_weight)), float(eps), _ptr(wo.buf), _ptr(gate.buf),
        _ptr(up.buf), _ptr(down.buf), _ptr(y), opt(res1), opt(h), opt(sumsq), E, H, group, _ptr(ws), ws.numel(), _stream()))
    out = (y, res1, h) if return_intermediates else (y,)
    if return_sumsq:
        out = out + (sumsq,)
    return out if len(out) > 1 else y


def decode_attn_o_gemv_ffn_stream(qkv, rope_lut_row, k_cache, v_cache, pos, n_heads, x_residual, ffn_norm_weight, wo, gate, up,
                                  down, eps=1e-5, group=GROUP, return_sumsq=False):
    """decode_attention followed by o_gemv_ffn_stream as one call.  Returns y bf16 [E], with return_sumsq also the sum
    of squares of y per 16 columns (float32 [E / 16])."""
    lib = _lib.load_library()
    _need_cuda(qkv, rope_lut_row, k_cache, v_cache, x_residual, ffn_norm_weight, wo.buf, gate.buf, up.buf, down.buf)
    _need_order("awq", wo, gate, up, down)
    n_kv, max_seq, hd = k_cache.shape
    E, H = n_heads * hd, gate.N
    if v_cache.shape != k_cache.shape or qkv.numel() != (n_heads + 2 * n_kv) * hd or rope_lut_row.numel() != hd:
        raise ValueError("decode_attn_o_gemv_ffn_stream: qkv must be [(n_heads + 2 n_kv) * hd], caches [n_kv, max_seq, hd], lut row [hd]")
    _check_block_stream(E, H, wo, gate, up, down, x_residual, ffn_norm_weight)
    dev = qkv.device
    y = torch.empty((E,), dtype=torch.bfloat16, device=dev)
    attn_out = torch.empty((E,), dtype=torch.bfloat16, device=dev)
    key = (dev.index, _stream(), n_heads, hd)
    aws = _attn_ws.get(key)
    if aws is None:
        aws = torch.empty(int(lib.w4a16_attention_workspace_bytes(n_heads, hd)), dtype=torch.uint8, device=dev)
        _attn_ws[key] = aws
    ws = _block_stream_scratch(E, H, dev)
    sumsq = torch.empty((E // 16,), dtype=torch.float32, device=dev) if return_sumsq else None
    _lib.check(lib.w4a16_decode_attn_o_gemv_ffn_stream_bf16(
        _ptr(_bits(qkv)), _ptr(_bits(rope_lut_row)), _ptr(_bits(k_cache)), _ptr(_bits(v_cache)), _ptr(attn_out), int(pos),
        max_seq, n_heads, n_kv, hd, _ptr(aws), aws.numel(), _ptr(_bits(x_residual)), _ptr(_bits(ffn_norm_weight)), float(eps),
        _ptr(wo.buf), _ptr(gate.buf), _ptr(up.buf), _ptr(down.buf), _ptr(y), _ptr(sumsq) if sumsq is not None else None, E, H,
        group, _ptr(ws), ws.numel(), _stream()))
    return (y, sumsq) if return_sumsq else y


def rope_halfsplit(x, lut):
    """Half-split RoPE of x bf16 [rows, dim] with one LUT row (cos then sin) per row: lut bf16 [rows, dim]."""
    lib = _lib.load_library()
    _need_cuda(x, lut)
    if x.dim() != 2 or lut.shape != x.shape:
        raise ValueError("rope_halfsplit: x and lut must both be [rows, dim]")
    rows, dim = x.shape
    out = torch.empty_like(x)
    _lib.check(lib.rope_halfsplit_bf16(_ptr(_bits(x)), _ptr(_bits(lut)), _ptr(out), rows, dim, _stream()))
    return out


def rms_norm_rows(x, norm_weight, eps=1e-5):
    """out[m, :] = bf16((x[m, :] / sqrt(mean(x[m, :]^2) + eps)) * norm_weight) for x bf16 [M, K]."""
    lib = _lib.load_library()
    _need_cuda(x, norm_weight)
    M, K = x.shape
    out = torch.empty_like(x)
    _lib.check(lib.rms_norm_rows_bf16(_ptr(_bits(x)), _ptr(_bits(norm_weight)), float(eps), _ptr(out), M, K, _stream()))
    return out


def prefill_rms_qkv_rope(x, attn_norm_weight, wqkv, rope_lut, pos0, n_heads, n_kv_heads, head_dim, eps=1e-5, group=GROUP):
    """RMSNorm + fused Q|K|V projection + RoPE on the Q and K heads for M tokens at positions pos0..:
    x bf16 [M, E] -> bf16 [M, (n_heads + 2 n_kv_heads) * head_dim].  wqkv is the AWQ triple of the
    concatenated weights, rope_lut bf16 [positions, head_dim]."""
    lib = _lib.load_library()
    _need_cuda(x, attn_norm_weight, rope_lut)
    M, E = x.shape
    N = (n_heads + 2 * n_kv_heads) * head_dim
    out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    key = (x.device.index, _stream(), "prefill_qkv", M, E)
    ws = _attn_ws.get(key)
    if ws is None:
        ws = torch.empty(int(lib.w4a16_prefill_qkv_workspace_bytes(M, E)), dtype=torch.uint8, device=x.device)
        _attn_ws[key] = ws
    _lib.check(lib.w4a16_prefill_rms_qkv_rope_bf16(_ptr(_bits(x)), _ptr(_bits(attn_norm_weight)), float(eps), *_wptrs(wqkv),
                                                   _ptr(_bits(rope_lut)), rope_lut.shape[0], int(pos0), _ptr(out), M, E,
                                                   n_heads, n_kv_heads, head_dim, group, _ptr(ws), ws.numel(), _stream()))
    return out


def prefill_attention(qkv, n_heads, n_kv_heads, head_dim):
    """Causal GQA attention over the M rows of qkv bf16 [M, (n_heads + 2 n_kv_heads) * head_dim] (roped Q | roped K | V):
    returns bf16 [M, n_heads * head_dim]."""
    lib = _lib.load_library()
    _need_cuda(qkv)
    M = qkv.shape[0]
    if qkv.shape[1] != (n_heads + 2 * n_kv_heads) * head_dim:
        raise ValueError("qkv must be [M, (n_heads + 2 n_kv_heads) * head_dim]")
    out = torch.empty((M, n_heads * head_dim), dtype=torch.bfloat16, device=qkv.device)
    _lib.check(lib.w4a16_prefill_attention_bf16(_ptr(_bits(qkv)), _ptr(out), M, n_heads, n_kv_heads, head_dim, _stream()))
    return out


def prefill_o_ffn(attn_out, x_residual, ffn_norm_weight, wo, gate, up, down, eps=1e-5, group=GROUP,
                  return_intermediates=False):
    """Prefill O projection + residual + RMSNorm + SwiGLU FFN + residual for M tokens: bf16 [M, E] -> [M, E].
    Every weight is an AWQ triple (qweight, qzeros, scales).  With return_intermediates also res1 [M, E]
    and h [M, H]."""
    lib = _lib.load_library()
    _need_cuda(attn_out, x_residual, ffn_norm_weight)
    M, E = attn_out.shape
    H = gate[0].shape[1] * 8
    y = torch.empty((M, E), dtype=torch.bfloat16, device=attn_out.device)
    res1 = torch.empty((M, E), dtype=torch.bfloat16, device=attn_out.device) if return_intermediates else None
    h = torch.empty((M, H), dtype=torch.bfloat16, device=attn_out.device) if return_intermediates else None
    key = (attn_out.device.index, _stream(), "prefill_block", M, E, H)
    ws = _attn_ws.get(key)
    if ws is None:
        ws = torch.empty(int(lib.w4a16_prefill_block_workspace_bytes(M, E, H)), dtype=torch.uint8, device=attn_out.device)
        _attn_ws[key] = ws
    _lib.check(lib.w4a16_prefill_o_ffn_bf16(_ptr(_bits(attn_out)), _ptr(_bits(x_residual)), _ptr(_bits(ffn_norm_weight)),
                                            float(eps), *_wptrs(wo), *_wptrs(gate), *_wptrs(up), *_wptrs(down), _ptr(y),
                                            _ptr(res1) if res1 is not None else None, _ptr(h) if h is not None else None,
                                            M, E, H, group, _ptr(ws), ws.numel(), _stream()))
    return (y, res1, h) if return_intermediates else y


def prefill_rms_qkv_rope_stream(x, attn_norm_weight, wqkv, rope_lut, pos0, n_heads, n_kv_heads, head_dim, eps=1e-5, group=GROUP,
                                codec="awq"):
    """prefill_rms_qkv_rope on a StreamWeight (the re-pack of the concatenated Q|K|V matrix): the tiled stream-order
    GEMM with the RoPE epilogue in place of the checkpoint-layout GEMM, same rounding points.  codec "q4nx": the
    StreamWeight is in Q4NX order (q4nx_repack_stream)."""
    lib = _lib.load_library()
    _need_cuda(x, attn_norm_weight, rope_lut, wqkv.buf)
    _need_order(codec, wqkv)
    M, E = x.shape
    N = (n_heads + 2 * n_kv_heads) * head_dim
    if (wqkv.K, wqkv.N) != (E, N):
        raise ValueError(f"wqkv is [{wqkv.K}, {wqkv.N}], the block needs [{E}, {N}]")
    out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    key = (x.device.index, _stream(), "prefill_qkv", M, E)
    ws = _attn_ws.get(key)
    if ws is None:
        ws = torch.empty(int(lib.w4a16_prefill_qkv_workspace_bytes(M, E)), dtype=torch.uint8, device=x.device)
        _attn_ws[key] = ws
    if codec == "q4nx":
        _lib.check(lib.w4a16_q4nx_prefill_rms_qkv_rope_stream_bf16(_ptr(_bits(x)), _ptr(_bits(attn_norm_weight)), float(eps),
                                                                   _ptr(wqkv.buf), _ptr(_bits(rope_lut)), rope_lut.shape[0], int(pos0),
                                                                   _ptr(out), M, E, n_heads, n_kv_heads, head_dim, _ptr(ws), ws.numel(),
                                                                   _stream()))
        return out
    _lib.check(lib.w4a16_prefill_rms_qkv_rope_stream_bf16(_ptr(_bits(x)), _ptr(_bits(attn_norm_weight)), float(eps), _ptr(wqkv.buf),
                                                          _ptr(_bits(rope_lut)), rope_lut.shape[0], int(pos0), _ptr(out), M, E,
                                                          n_heads, n_kv_heads, head_dim, group, _ptr(ws), ws.numel(), _stream()))
    return out


def prefill_o_ffn_stream(attn_out, x_residual, ffn_norm_weight, wo, gate, up, down, eps=1e-5, group=GROUP,
                         return_intermediates=False, codec="awq"):
    """prefill_o_ffn on four StreamWeights: bf16 [M, E] -> [M, E]; with return_intermediates also res1 [M, E] and h [M, H].
    codec "q4nx": the StreamWeights are in Q4NX order (q4nx_repack_stream)."""
    lib = _lib.load_library()
    _need_cuda(attn_out, x_residual, ffn_norm_weight, wo.buf, gate.buf, up.buf, down.buf)
    _need_order(codec, wo, gate, up, down)
    M, E = attn_out.shape
    H = gate.N
    if (wo.K, wo.N) != (E, E) or (gate.K, up.K, up.N) != (E, E, H) or (down.K, down.N) != (H, E):
        raise ValueError("prefill_o_ffn_stream: wo [E, E], gate and up [E, H], down [H, E]")
    y = torch.empty((M, E), dtype=torch.bfloat16, device=attn_out.device)
    res1 = torch.empty((M, E), dtype=torch.bfloat16, device=attn_out.device) if return_intermediates else None
    h = torch.empty((M, H), dtype=torch.bfloat16, device=attn_out.device) if return_intermediates else None
    key = (attn_out.device.index, _stream(), "prefill_block", M, E, H)
    ws = _attn_ws.get(key)
    if ws is None:
        ws = torch.empty(int(lib.w4a16_prefill_block_workspace_bytes(M, E, H)), dtype=torch.uint8, device=attn_out.device)
        _attn_ws[key] = ws
    args = (_ptr(_bits(attn_out)), _ptr(_bits(x_residual)), _ptr(_bits(ffn_norm_weight)), float(eps), _ptr(wo.buf), _ptr(gate.buf),
            _ptr(up.buf), _ptr(down.buf), _ptr(y), _ptr(res1) if res1 is not None else None, _ptr(h) if h is not None else None,
            M, E, H)
    if codec == "q4nx":
        _lib.check(lib.w4a16_q4nx_prefill_o_ffn_stream_bf16(*args, _ptr(ws), ws.numel(), _stream()))
    else:
        _lib.check(lib.w4a16_prefill_o_ffn_stream_bf16(*args, group, _ptr(ws), ws.numel(), _stream()))
    return (y, res1, h) if return_intermediates else y


def lm_head(x, lm_head_weight, norm_weight=None, eps=1e-5, return_argmax=True, argmax_out=None):
    """Tail of a decode step: logits bf16 [V] = lm_head_weight [V, E] . rms_norm(x) (x itself when
    norm_weight is None), and the index of the largest logit as a device int32 tensor [1]
    (`argmax_out`: written there instead of into a new tensor, e.g. a slot of the generated-ids buffer)."""
    lib = _lib.load_library()
    _need_cuda(x, lm_head_weight)
    V, E = lm_head_weight.shape
    if x.numel() != E:
        raise ValueError(f"x has {x.numel()} elements but lm_head has E={E}")
    if not lm_head_weight.is_contiguous():
        raise ValueError("lm_head must be contiguous [V, E]")
    logits = torch.empty((V,), dtype=torch.bfloat16, device=x.device)
    best = None
    if return_argmax:
        best = argmax_out if argmax_out is not None else torch.empty((1,), dtype=torch.int32, device=x.device)
        if best.dtype != torch.int32 or best.numel() != 1 or not best.is_cuda:
            raise ValueError("argmax_out must be a device int32 tensor of one element")
    key = (x.device.index, _stream(), "lm_head", V)
    ws = _attn_ws.get(key)
    if ws is None:
        ws = torch.empty(int(lib.lm_head_workspace_bytes(V)), dtype=torch.uint8, device=x.device)
        _attn_ws[key] = ws
    _lib.check(lib.lm_head_gemv_bf16(_ptr(_bits(x)), _ptr(_bits(norm_weight)) if norm_weight is not None else None,
                                     float(eps), _ptr(_bits(lm_head_weight)), _ptr(logits),
                                     _ptr(best) if return_argmax else None, V, E, _ptr(ws), ws.numel(), _stream()))
    return (logits, best) if return_argmax else logits


def q4nx_dequant(blocks, M, K, mode=0, out=None):
    """Dense W[M, K] bf16 from Q4NX / Q4_0 blocks (uint8 [M/32 * K/256, 5120] on the GPU);
    mode 0 w = s q + m, 1 w = s (q - m), 2 signed q with w = s q."""
    lib = _lib.load_library()
    _need_cuda(blocks)
    if blocks.numel() * blocks.element_size() != (M // 32) * (K // 256) * 5120:
        raise ValueError(f"blocks hold {blocks.numel() * blocks.element_size()} bytes, [M, K] = {[M, K]} needs {(M // 32) * (K // 256) * 5120}")
    if out is None:
        out = torch.empty((M, K), dtype=torch.bfloat16, device=blocks.device)
    _lib.check(lib.q4nx_dequant_bf16(_ptr(blocks), _ptr(out), M, K, mode, _stream()))
    return out


def q4nx_repack(blocks, M, K, mode=0):
    """Blocks -> (qweight int32 [K, M/8], scales bf16 [K/32, M], mins bf16 [K/32, M]), the
    operands of q4nx_repack_stream; done once per tensor at load time."""
    lib = _lib.load_library()
    _need_cuda(blocks)
    if blocks.numel() * blocks.element_size() != (M // 32) * (K // 256) * 5120:
        raise ValueError(f"blocks hold {blocks.numel() * blocks.element_size()} bytes, [M, K] = {[M, K]} needs {(M // 32) * (K // 256) * 5120}")
    qweight = torch.empty((K, M // 8), dtype=torch.int32, device=blocks.device)
    scales = torch.empty((K // 32, M), dtype=torch.bfloat16, device=blocks.device)
    mins = torch.empty((K // 32, M), dtype=torch.bfloat16, device=blocks.device)
    _lib.check(lib.q4nx_repack(_ptr(blocks), _ptr(qweight), _ptr(scales), _ptr(mins), M, K, mode, _stream()))
    return qweight, scales, mins


def q4nx_gemm(x, qweight, scales, mins, residual=None, out=None):
    """y = bf16(x . W + residual) for the operands of q4nx_repack; x [rows, K] or a vector [K].  Re-packs W into Q4NX
    stream order on every call: a caller that multiplies more than once keeps the result of q4nx_repack_stream and
    calls q4nx_gemm_stream."""
    return q4nx_gemm_stream(x, q4nx_repack_stream(qweight, scales, mins), residual=residual, out=out)


def q4nx_rms_gemv(x, norm_weight, qweight, scales, mins, eps=1e-5):
    """y[N] = bf16(rms_norm(x, norm_weight) . W) for the operands of q4nx_repack (re-packed on every call, as q4nx_gemm)."""
    return q4nx_rms_gemv_stream(x, norm_weight, q4nx_repack_stream(qweight, scales, mins), eps=eps)


def q4nx_o_gemv_ffn(attn_out, x_residual, ffn_norm_weight, wo, gate, up, down, eps=1e-5, return_intermediates=False):
    """o_gemv_ffn for the affine codec: wo/gate/up/down are (qweight, scales, mins) from q4nx_repack (re-packed on every
    call, as q4nx_gemm)."""
    sw = [q4nx_repack_stream(*w) for w in (wo, gate, up, down)]
    return q4nx_o_gemv_ffn_stream(attn_out, x_residual, ffn_norm_weight, *sw, eps=eps, return_intermediates=return_intermediates)


def q4nx_repack_stream(qweight, scales, mins):
    """Operands of q4nx_repack (qweight int32 [K, N / 8], scales and mins bf16 [K / 32, N]) -> StreamWeight in Q4NX
    order, the form the whole-K decode kernels read; once per tensor at load time."""
    lib = _lib.load_library()
    _need_cuda(qweight, scales, mins)
    K, N = qweight.shape[0], qweight.shape[1] * 8
    if scales.shape != (K // 32, N) or mins.shape != scales.shape:
        raise ValueError("q4nx_repack_stream: scales and mins must be [K / 32, N]")
    nbytes = lib.w4a16_q4nx_stream_bytes(K, N)
    if nbytes == 0:
        raise ValueError(f"Q4NX stream order needs K % 128 == 0 and N % 16 == 0, got K={K}, N={N}")
    buf = torch.empty(int(nbytes), dtype=torch.uint8, device=qweight.device)
    _lib.check(lib.w4a16_q4nx_repack_stream(_ptr(qweight), _ptr(_bits(scales)), _ptr(_bits(mins)), _ptr(buf), K, N, _stream()))
    return StreamWeight(buf, K, N, "q4nx")


def q4nx_blocks_to_stream(blocks, M, K, mode=0):
    """Blocks of W[M, K] (uint8 [n_blocks, 5120] on the GPU) -> StreamWeight in Q4NX order of the [K, N = M] matrix, in
    one pass (the same bytes as q4nx_repack followed by q4nx_repack_stream); once per tensor at load time."""
    lib = _lib.load_library()
    _need_cuda(blocks)
    if blocks.numel() != (M // 32) * (K // 256) * 5120:
        raise ValueError(f"blocks must hold {(M // 32) * (K // 256)} blocks of 5120 bytes for W[{M}, {K}]")
    nbytes = lib.w4a16_q4nx_stream_bytes(K, M)
    if nbytes == 0 or M % 32 or K % 256:
        raise ValueError(f"Q4NX blocks need M % 32 == 0 and K % 256 == 0, got M={M}, K={K}")
    buf = torch.empty(int(nbytes), dtype=torch.uint8, device=blocks.device)
    _lib.check(lib.w4a16_q4nx_blocks_to_stream(_ptr(blocks), _ptr(buf), M, K, int(mode), _stream()))
    return StreamWeight(buf, K, M, "q4nx")


def q4nx_gemv_stream(x, w, residual=None, out=None):
    """y[N] = bf16(x[K] . W (+ residual)) on a Q4NX-order StreamWeight; stateless, no workspace."""
    lib = _lib.load_library()
    _need_cuda(x, w.buf)
    _need_order("q4nx", w)
    if x.numel() != w.K or (residual is not None and residual.numel() != w.N):
        raise ValueError("q4nx_gemv_stream: x must have K elements, residual N")
    if out is None:
        out = torch.empty((w.N,), dtype=torch.bfloat16, device=x.device)
    _lib.check(lib.w4a16_q4nx_gemv_stream_bf16(_ptr(_bits(x)), _ptr(w.buf), _ptr(_bits(residual)) if residual is not None else None,
                                               _ptr(out), w.K, w.N, _stream()))
    return out


def q4nx_gemm_stream(x, w, residual=None, out=None):
    """y[M, N] = bf16(x[M, K] . W (+ residual [M, N])) on a Q4NX-order StreamWeight; x may be a vector [K]."""
    lib = _lib.load_library()
    _need_cuda(x, w.buf)
    _need_order("q4nx", w)
    vec = x.dim() == 1
    x2 = x.unsqueeze(0) if vec else x
    M, K = x2.shape
    if K != w.K or (residual is not None and residual.numel() != M * w.N):
        raise ValueError("q4nx_gemm_stream: x must be [M, K], residual [M, N]")
    if out is None:
        out = torch.empty((M, w.N), dtype=torch.bfloat16, device=x.device)
    _lib.check(lib.w4a16_q4nx_gemm_stream_bf16(_ptr(_bits(x2)), _ptr(w.buf), _ptr(_bits(residual)) if residual is not None else None,
                                               _ptr(out), M, K, w.N, _stream()))
    return out.squeeze(0) if vec else out


def q4nx_rms_gemv_stream(x, norm_weight, w, eps=1e-5, x_sumsq=None):
    """y[N] = bf16(rms_norm(x, norm_weight) . W) on a Q4NX-order StreamWeight (x_sumsq as in w4a16_rms_gemv_stream)."""
    lib = _lib.load_library()
    _need_cuda(x, norm_weight, w.buf)
    _need_order("q4nx", w)
    if x.numel() != w.K or norm_weight.numel() != w.K:
        raise ValueError("q4nx_rms_gemv_stream: x and norm_weight must have K elements")
    out = torch.empty((w.N,), dtype=torch.bfloat16, device=x.device)
    if x_sumsq is not None and (x_sumsq.dtype != torch.float32 or not x_sumsq.is_cuda or not x_sumsq.is_contiguous()):
        raise ValueError("x_sumsq must be a contiguous float32 GPU tensor")
    _lib.check(lib.w4a16_q4nx_rms_gemv_stream_bf16(_ptr(_bits(x)), _ptr(x_sumsq) if x_sumsq is not None else None,
                                                   x_sumsq.numel() if x_sumsq is not None else 0, _ptr(_bits(norm_weight)),
                                                   float(eps), _ptr(w.buf), _ptr(out), w.K, w.N, _stream()))
    return out


def q4nx_o_gemv_ffn_stream(attn_out, x_residual, ffn_norm_weight, wo, gate, up, down, eps=1e-5, return_intermediates=False,
                           return_sumsq=False):
    """o_gemv_ffn_stream on Q4NX-order StreamWeights: same stages, outputs and scratch."""
    lib = _lib.load_library()
    _need_cuda(attn_out, x_residual, ffn_norm_weight, wo.buf, gate.buf, up.buf, down.buf)
    _need_order("q4nx", wo, gate, up, down)
    E, H = wo.K, gate.N
    _check_block_stream(E, H, wo, gate, up, down, attn_out, x_residual, ffn_norm_weight)
    dev = attn_out.device
    y = torch.empty((E,), dtype=torch.bfloat16, device=dev)
    res1 = torch.empty((E,), dtype=torch.bfloat16, device=dev) if return_intermediates else None
    h = torch.empty((H,), dtype=torch.bfloat16, device=dev) if return_intermediates else None
    sumsq = torch.empty((E // 16,), dtype=torch.float32, device=dev) if return_sumsq else None
    ws = _block_stream_scratch(E, H, dev)
    opt = lambda t: _ptr(t) if t is not None else None
    _lib.check(lib.w4a16_q4nx_o_gemv_ffn_stream_bf16(
        _ptr(_bits(attn_out)), _ptr(_bits(x_residual)), _ptr(_bits(ffn_norm_weight)), float(eps), _ptr(wo.buf), _ptr(gate.buf),
        _ptr(up.buf), _ptr(down.buf), _ptr(y), opt(res1), opt(h), opt(sumsq), E, H, _ptr(ws), ws.numel(), _stream()))
    out = (y, res1, h) if return_intermediates else (y,)
    if return_sumsq:
        out = out + (sumsq,)
    return out if len(out) > 1 else y


def tune(key, value):
    lib = _lib.load_library()
    _lib.check(lib.w4a16_tune(key.encode(), int(value)))
