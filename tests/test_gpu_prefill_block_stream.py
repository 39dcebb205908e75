"""GPU parity of the two prompt-pass blocks on stream-order weights (RMSNorm + Q|K|V GEMM + RoPE; O projection +
residual + RMSNorm + SwiGLU FFN + residual), which run the tiled stream-order GEMM with fused epilogues.

Two kinds of check per stage.  Against the library's own plain product (w4a16_gemm_stream through the same tiled
kernel): the epilogues work on the bf16 product, so residual adds and rotations must come out bit for bit.  Against the
oracle: each stage on the kernel's own input to it within the roundings of that stage, and the whole block against the
restated CPU reference under the reference's gate.
"""
import numpy as np
import pytest
import torch

from helpers import bf16_ulp, dense_f64, make_awq, make_x
from oracle import awq as oawq, reference as oref
from oracle.bf16 import bf16_bits_to_f32, f32_to_bf16_bits

pytestmark = pytest.mark.gpu


def dev(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)
    return torch.from_numpy(a).cuda()


def bits(t):
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


@pytest.fixture(scope="module")
def ops():
    from air_hip import ops
    return ops


@pytest.fixture
def tiled_gemm(ops):
    """w4a16_gemm_stream runs the tiled kernel from M = 17 on (by itself it does from M = 97 on), so that its output
    is the product inside the fused calls bit for bit."""
    ops.tune("prefill_min_m", 17)
    yield
    ops.tune("prefill_min_m", 0)


def _scaled(K, N, seed, scale):
    qw, qz, s = make_awq(K, N, seed=seed)
    return qw, qz, f32_to_bf16_bits(bf16_bits_to_f32(s) * np.float32(scale))


def _weights(E, H, seed, scale=1.0):
    return [_scaled(K, N, seed + i, scale) for i, (K, N) in enumerate(((E, E), (E, H), (E, H), (H, E)))]


def _sw(ops, w):
    return ops.repack_stream(*map(dev, w))


def _norm_w(E, seed):
    rng = np.random.default_rng(seed)
    return f32_to_bf16_bits((rng.standard_normal(E) * 0.1 + 1.0).astype(np.float32))


def _add_rounded(prod, add):
    return (prod.float() + add.float()).to(torch.bfloat16)


def _close_sum(got_bits, prod64, add32, what):
    want = prod64 + add32
    err = np.abs(bf16_bits_to_f32(got_bits).astype(np.float64) - want)
    tol = bf16_ulp(want) + bf16_ulp(prod64) + 2e-3
    assert np.all(err <= tol), f"{what}: worst {np.max(err - tol):.4g} over tolerance at {np.unravel_index(np.argmax(err - tol), err.shape)}"


@pytest.mark.parametrize("M,E,H", [(40, 256, 512), (300, 512, 1280), (17, 256, 256), (260, 1024, 2048)])
def test_prefill_block_stream_stage_by_stage(ops, tiled_gemm, M, E, H):
    print(f"prefill block (stream order) M={M} E={E} H={H}", flush=True)
    wo, wg, wu, wd = _weights(E, H, seed=M + E, scale=0.25)
    so, sg, su, sd = (_sw(ops, w) for w in (wo, wg, wu, wd))
    attn, xres, nw = make_x((M, E), seed=M), make_x((M, E), seed=M + 1), _norm_w(E, M + 2)
    y, res1, h = ops.prefill_o_ffn_stream(dev(attn), dev(xres), dev(nw), so, sg, su, sd, return_intermediates=True)
    y2 = ops.prefill_o_ffn_stream(dev(attn), dev(xres), dev(nw), so, sg, su, sd)
    torch.cuda.synchronize()
    y_b, res1_b, h_b = bits(y), bits(res1), bits(h)
    assert np.array_equal(bits(y2), y_b), "intermediates kept in the workspace give another result"
    f = lambda b: bf16_bits_to_f32(b).astype(np.float64)
    # 1. O projection + residual: the epilogue on the plain product, and the float64 product
    assert torch.equal(res1.view(torch.int16), _add_rounded(ops.w4a16_gemm_stream(dev(attn), so), dev(xres)).view(torch.int16))
    _close_sum(res1_b, f(attn) @ dense_f64(*wo, rounded=True), f(xres), "res1")
    # 2. row-wise RMSNorm of the kernel's res1
    normed = ops.rms_norm_rows(res1, dev(nw))
    n_gpu = bits(normed)
    n_ref = oref.rms_norm_rows_bf16(res1_b, nw)
    nd = np.abs(f(n_gpu) - f(n_ref))
    assert np.all(nd <= bf16_ulp(f(n_ref))) and np.mean(n_gpu != n_ref) < 0.01, (nd.max(), np.mean(n_gpu != n_ref))
    # 3. gate / up + SwiGLU: on the library's own bf16 products within one rounding (+ the exponential's last bits),
    #    and on float64 products of the kernel's normalised rows
    gb, ub = f(bits(ops.w4a16_gemm_stream(normed, sg))), f(bits(ops.w4a16_gemm_stream(normed, su)))
    h_exact = gb / (1.0 + np.exp(-gb)) * ub
    assert np.all(np.abs(f(h_b) - h_exact) <= 0.51 * bf16_ulp(h_exact) + 1e-6 * np.abs(h_exact) + 1e-30), \
        np.max(np.abs(f(h_b) - h_exact) / bf16_ulp(h_exact))
    G, U = f(n_gpu) @ dense_f64(*wg, rounded=True), f(n_gpu) @ dense_f64(*wu, rounded=True)
    g64, u64 = f(f32_to_bf16_bits(G.astype(np.float32))), f(f32_to_bf16_bits(U.astype(np.float32)))
    h_want = g64 / (1.0 + np.exp(-g64)) * u64
    h_tol = 4 * bf16_ulp(h_want) + 1.2 * bf16_ulp(g64) * np.abs(u64) + bf16_ulp(u64) * np.abs(g64) + 1e-3
    assert np.all(np.abs(f(h_b) - h_want) <= h_tol), np.max(np.abs(f(h_b) - h_want) - h_tol)
    # 4. down projection + residual on the kernel's h and res1
    assert torch.equal(y.view(torch.int16), _add_rounded(ops.w4a16_gemm_stream(h, sd), res1).view(torch.int16))
    _close_sum(y_b, f(h_b) @ dense_f64(*wd, rounded=True), f(res1_b), "y")
    # the whole block against the restated CPU reference, under the reference's gate and a tighter one
    l1 = [oawq.repack_hf_awq_linear(*w, 128) for w in (wo, wg, wu, wd)]
    want, _, _ = oref.o_ffn_int4_prefill_reference(*l1, attn, xres, nw)
    got_f, want_f = bf16_bits_to_f32(y_b), bf16_bits_to_f32(want)
    assert oref.check_outputs(got_f, want_f, rtol=0.5, atol=10.0, max_mismatch_percentage=0.5, min_correlation=0.99)
    assert np.max(np.abs(got_f - want_f)) <= 8 * 2.0**-8 * np.max(np.abs(want_f)), np.max(np.abs(got_f - want_f))


def test_prefill_block_stream_zero_projections_are_exact(ops):
    """q == z makes a projection exactly zero: res1 is the residual and y is res1, bit for bit."""
    M, E, H = 200, 256, 512
    wo, wg, wu, wd = _weights(E, H, seed=90)
    zero = lambda w: (w[1].repeat(128, axis=0), w[1], w[2])      # every q row equals its group's z row
    attn, xres, nw = make_x((M, E), seed=91), make_x((M, E), seed=92), _norm_w(E, 93)
    print("prefill block (stream order), zero O and down projections", flush=True)
    y, res1, h = ops.prefill_o_ffn_stream(dev(attn), dev(xres), dev(nw), _sw(ops, zero(wo)), _sw(ops, wg), _sw(ops, wu),
                                          _sw(ops, zero(wd)), return_intermediates=True)
    torch.cuda.synchronize()
    assert np.array_equal(bits(res1), xres) and np.array_equal(bits(y), xres)
    _, _, h0 = ops.prefill_o_ffn_stream(dev(attn), dev(xres), dev(nw), _sw(ops, wo), _sw(ops, zero(wg)), _sw(ops, wu),
                                        _sw(ops, wd), return_intermediates=True)
    assert np.all((bits(h0) & 0x7FFF) == 0)


@pytest.mark.parametrize("M,E,H,tile", [(300, 512, 1280, 0), (300, 512, 1024, 1), (130, 256, 768, 3), (2048, 2048, 8192, 0),
                                        (300, 512, 1280, 5), (260, 256, 1792, 5)])
def test_prefill_block_stream_paired_gate_up_launch_equals_two_launches(ops, M, E, H, tile):
    """Gate and up in one launch (a tile holds the same columns of both products) against the gate launch followed by
    the up launch with the SwiGLU epilogue: the same bits in h and y, at the tile width chosen by shape and forced."""
    ws = _weights(E, H, seed=70 + tile, scale=0.25)
    sws = [_sw(ops, w) for w in ws]
    attn, xres, nw = make_x((M, E), seed=71), make_x((M, E), seed=72), _norm_w(E, 73)
    print(f"prefill block (stream order), one launch for gate and up against two, M={M} E={E} H={H} tile={tile}", flush=True)
    ops.tune("prefill_tile", tile)
    try:
        y1, _, h1 = ops.prefill_o_ffn_stream(dev(attn), dev(xres), dev(nw), *sws, return_intermediates=True)
        ops.tune("prefill_swiglu_split", 1)
        y2, _, h2 = ops.prefill_o_ffn_stream(dev(attn), dev(xres), dev(nw), *sws, return_intermediates=True)
        torch.cuda.synchronize()
    finally:
        ops.tune("prefill_swiglu_split", 0)
        ops.tune("prefill_tile", 0)
    assert torch.equal(h1.view(torch.int16), h2.view(torch.int16)) and torch.equal(y1.view(torch.int16), y2.view(torch.int16))
    assert float(h1.float().abs().max()) > 0


def test_prefill_block_stream_agrees_with_the_checkpoint_layout_block(ops):
    """The same block on the checkpoint tensors (another kernel, another summation order inside a product): the
    outputs differ by roundings only."""
    M, E, H = 300, 512, 1024
    ws = _weights(E, H, seed=60, scale=0.25)
    attn, xres, nw = make_x((M, E), seed=61), make_x((M, E), seed=62), _norm_w(E, 63)
    print("prefill block, stream order against checkpoint layout", flush=True)
    a = ops.prefill_o_ffn_stream(dev(attn), dev(xres), dev(nw), *(_sw(ops, w) for w in ws))
    b = ops.prefill_o_ffn(dev(attn), dev(xres), dev(nw), *(tuple(map(dev, w)) for w in ws))
    err = (a.double() - b.double()).abs()
    assert float(err.max()) <= 4 * 2.0**-8 * float(b.double().abs().max()), float(err.max())


@pytest.mark.parametrize("M,E,H", [(2048, 2048, 8192), (512, 4096, 14336)])
def test_prefill_block_stream_model_sizes(ops, M, E, H):
    """Llama-3.2-1B's dimensions at the reference example's sequence length, and Llama-3-8B's at 512 tokens: the
    epilogues against the library's own products bit for bit, the products against float64 on the GPU."""
    print(f"prefill block (stream order) M={M} E={E} H={H}", flush=True)
    wo, wg, wu, wd = _weights(E, H, seed=7, scale=0.1)
    so, sg, su, sd = (_sw(ops, w) for w in (wo, wg, wu, wd))
    attn, xres, nw = make_x((M, E), seed=8), make_x((M, E), seed=9), _norm_w(E, 10)
    y, res1, h = ops.prefill_o_ffn_stream(dev(attn), dev(xres), dev(nw), so, sg, su, sd, return_intermediates=True)
    torch.cuda.synchronize()
    assert torch.equal(res1.view(torch.int16), _add_rounded(ops.w4a16_gemm_stream(dev(attn), so), dev(xres)).view(torch.int16))
    assert torch.equal(y.view(torch.int16), _add_rounded(ops.w4a16_gemm_stream(h, sd), res1).view(torch.int16))
    d64 = lambda w: torch.from_numpy(dense_f64(*w, rounded=True)).cuda()
    rnd = lambda t: t.to(torch.bfloat16).double()
    res1_t = rnd(rnd(dev(attn).double() @ d64(wo)) + dev(xres).double())
    err = (res1.double() - res1_t).abs()
    assert float(err.max()) <= 2.0**-7 * float(res1_t.abs().max()) and float((err > 0).double().mean()) < 0.02
    n_t = rnd(torch.nn.functional.rms_norm(res1.double(), (E,), dev(nw).double(), eps=1e-5))
    g_t, u_t = rnd(n_t @ d64(wg)), rnd(n_t @ d64(wu))
    h_t = rnd(torch.nn.functional.silu(g_t) * u_t)
    herr = (h.double() - h_t).abs()
    assert float(herr.max()) <= 8 * 2.0**-8 * float(h_t.abs().max()) and float((herr > 0).double().mean()) < 0.1
    y_t = rnd(rnd(h.double() @ d64(wd)) + res1.double())
    yerr = (y.double() - y_t).abs()
    assert float(yerr.max()) <= 2.0**-7 * float(y_t.abs().max()) and float((yerr > 0).double().mean()) < 0.02


def test_prefill_block_stream_rejects_bad_arguments(ops):
    from air_hip import _lib
    lib = _lib.load_library()
    ws = lib.w4a16_prefill_block_workspace_bytes(32, 256, 256)
    wsq = lib.w4a16_prefill_qkv_workspace_bytes(32, 256)
    zeros = torch.zeros(1 << 18, dtype=torch.int32, device="cuda")
    out = torch.zeros(1 << 18, dtype=torch.int32, device="cuda")
    scratch = torch.zeros(max(ws, wsq), dtype=torch.uint8, device="cuda")
    P, Y, W = zeros.data_ptr(), out.data_ptr(), scratch.data_ptr()
    args = [P, P, P, 1e-5] + [P] * 4 + [Y, None, None, 32, 256, 256, 128, W, ws, None]
    assert lib.w4a16_prefill_o_ffn_stream_bf16(*args) == 0
    torch.cuda.synchronize()
    bad = list(args); bad[16] = ws - 1
    assert lib.w4a16_prefill_o_ffn_stream_bf16(*bad) == _lib.ERR_WORKSPACE
    bad = list(args); bad[12] = 128            # E must be a multiple of 256
    assert lib.w4a16_prefill_o_ffn_stream_bf16(*bad) == _lib.ERR_SHAPE
    bad = list(args); bad[13] = 320            # and so must H
    assert lib.w4a16_prefill_o_ffn_stream_bf16(*bad) == _lib.ERR_SHAPE
    bad = list(args); bad[14] = 64
    assert lib.w4a16_prefill_o_ffn_stream_bf16(*bad) == _lib.ERR_GROUP
    bad = list(args); bad[5] = None
    assert lib.w4a16_prefill_o_ffn_stream_bf16(*bad) == _lib.ERR_NULL
    bad = list(args); bad[0] = P + 2
    assert lib.w4a16_prefill_o_ffn_stream_bf16(*bad) == _lib.ERR_ALIGN
    qargs = [P, P, 1e-5, P, P, 64, 0, Y, 32, 256, 2, 1, 64, 128, W, wsq, None]
    assert lib.w4a16_prefill_rms_qkv_rope_stream_bf16(*qargs) == 0
    torch.cuda.synchronize()
    bad = list(qargs); bad[6] = 33             # positions 33 .. 64 of a 64-row table
    assert lib.w4a16_prefill_rms_qkv_rope_stream_bf16(*bad) == _lib.ERR_SHAPE
    bad = list(qargs); bad[12] = 32            # head_dim
    assert lib.w4a16_prefill_rms_qkv_rope_stream_bf16(*bad) == _lib.ERR_SHAPE
    bad = list(qargs); bad[15] = wsq - 1
    assert lib.w4a16_prefill_rms_qkv_rope_stream_bf16(*bad) == _lib.ERR_WORKSPACE
    bad = list(qargs); bad[3] = None
    assert lib.w4a16_prefill_rms_qkv_rope_stream_bf16(*bad) == _lib.ERR_NULL


def _qkv_weights(E, nh, nkv, hd, seed, scale=0.25):
    parts = [_scaled(E, N, seed + i, scale) for i, N in enumerate((nh * hd, nkv * hd, nkv * hd))]
    fused = tuple(np.concatenate([p[j] for p in parts], axis=1) for j in range(3))
    return parts, fused


# head widths 64 and 128 through every tile width that holds whole heads (tile 0: the width chosen by shape, which for
# these small matrices is 64 or 128 columns; 1: 256, 2: 192, 3: 128, 4: 64, 5: 256 mixed with 128), ragged M, one row
# tile and two
@pytest.mark.parametrize("M,E,nh,nkv,hd,pos0,tile", [(40, 256, 4, 2, 64, 0, 0), (300, 512, 8, 8, 64, 7, 0), (130, 256, 2, 1, 128, 100, 0),
                                                      (17, 256, 3, 1, 64, 1, 0), (270, 512, 1, 1, 128, 3, 0), (300, 256, 4, 2, 64, 5, 1),
                                                      (100, 256, 4, 1, 64, 2, 2), (260, 512, 2, 1, 128, 9, 1), (64, 256, 4, 2, 64, 0, 3),
                                                      (33, 256, 2, 1, 64, 11, 4), (270, 256, 4, 1, 128, 6, 5), (100, 512, 3, 2, 128, 0, 5)])
def test_prefill_rms_qkv_rope_stream(ops, tiled_gemm, M, E, nh, nkv, hd, pos0, tile):
    from oracle import decode as odec
    print(f"prefill qkv rope (stream order) M={M} E={E} heads {nh}/{nkv} hd={hd} pos0={pos0} tile={tile}", flush=True)
    parts, fused = _qkv_weights(E, nh, nkv, hd, seed=M + E)
    x, nw = make_x((M, E), seed=M + 3), _norm_w(E, M + 4)
    lut = odec.generate_rope_lut(hd, 500000.0, pos0 + M + 5)
    sw = _sw(ops, fused)
    ops.tune("prefill_tile", tile)
    try:
        out = ops.prefill_rms_qkv_rope_stream(dev(x), dev(nw), sw, dev(lut), pos0, nh, nkv, hd)
        torch.cuda.synchronize()
    finally:
        ops.tune("prefill_tile", 0)
    normed = ops.rms_norm_rows(dev(x), dev(nw))
    plain = ops.w4a16_gemm_stream(normed, sw)
    torch.cuda.synchronize()
    got = bits(out)
    f = lambda b: bf16_bits_to_f32(b).astype(np.float64)
    nq, nk = nh * hd, nkv * hd
    # V columns are the plain product, bit for bit the GEMM entry point's
    assert np.array_equal(got[:, nq + nk:], bits(plain)[:, nq + nk:])
    # Q and K: the rotation of the kernel's own bf16 product is reproduced exactly by the oracle's rotation
    rows = lut[pos0:pos0 + M]
    for lo, n in ((0, nh), (nq, nkv)):
        prod = bits(plain)[:, lo:lo + n * hd].reshape(M * n, hd)
        want = odec.rope_rows(prod, np.repeat(rows, n, axis=0)).reshape(M, n * hd)
        assert np.array_equal(got[:, lo:lo + n * hd], want)
    # and the whole call against the restated CPU reference (float32 BLAS products, one-ulp flips upstream)
    l1 = [oawq.repack_hf_awq_linear(*w, 128) for w in parts]
    ref_out = odec.prefill_rms_qkv_rope_reference(x, nw, *l1, lut, pos0, nh, nkv, hd)
    err = np.abs(f(got) - f(ref_out))
    assert np.max(err) <= 4 * 2.0**-8 * np.max(np.abs(f(ref_out))), err.max()
    ref_r = odec.prefill_rms_qkv_rope_reference(x, nw, *l1, lut, pos0, nh, nkv, hd, round_weights=True)
    assert np.mean(got != ref_r) < 0.1, np.mean(got != ref_r)


def test_prefill_rms_qkv_rope_stream_position_zero_is_the_identity(ops, tiled_gemm):
    """Every row at position 0 (a one-row table, cos = 1, sin = 0) leaves Q and K unrotated: the fused call equals
    RMSNorm + plain GEMM bit for bit; and shifting pos0 equals shifting the table."""
    from oracle import decode as odec
    E, nh, nkv, hd = 256, 4, 2, 64
    _, fused = _qkv_weights(E, nh, nkv, hd, seed=5)
    sw = _sw(ops, fused)
    nw = _norm_w(E, 6)
    lut = odec.generate_rope_lut(hd, 500000.0, 64)
    x = make_x((40, E), seed=7)
    print("prefill qkv rope (stream order), position 0 and shifted tables", flush=True)
    plain = ops.w4a16_gemm_stream(ops.rms_norm_rows(dev(x), dev(nw)), sw)
    for m in (0, 17, 39):
        one = ops.prefill_rms_qkv_rope_stream(dev(x[m:m + 1]), dev(nw), sw, dev(lut[:1]), 0, nh, nkv, hd)
        assert torch.equal(one.view(torch.int16), plain[m:m + 1].view(torch.int16))
    a = ops.prefill_rms_qkv_rope_stream(dev(x), dev(nw), sw, dev(lut), 9, nh, nkv, hd)
    b = ops.prefill_rms_qkv_rope_stream(dev(x), dev(nw), sw, dev(lut[9:]), 0, nh, nkv, hd)
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))


@pytest.mark.parametrize("M,E,nh,nkv,hd", [(2048, 2048, 32, 8, 64), (1024, 4096, 32, 8, 128)])
def test_prefill_rms_qkv_rope_stream_model_sizes(ops, M, E, nh, nkv, hd):
    """Llama-3.2-1B's and Llama-3-8B's projections (tiles of 256 and 192 columns for the first, 256 only for the
    second, whose heads are 128 wide)."""
    from oracle import decode as odec
    print(f"prefill qkv rope (stream order) M={M} E={E} {nh}/{nkv} heads of {hd}", flush=True)
    _, fused = _qkv_weights(E, nh, nkv, hd, seed=15, scale=0.1)
    sw = _sw(ops, fused)
    x, nw = make_x((M, E), seed=16), _norm_w(E, 17)
    lut = odec.generate_rope_lut(hd, 500000.0, M)
    out = ops.prefill_rms_qkv_rope_stream(dev(x), dev(nw), sw, dev(lut), 0, nh, nkv, hd)
    plain = ops.w4a16_gemm_stream(ops.rms_norm_rows(dev(x), dev(nw)), sw)
    torch.cuda.synchronize()
    got, prod = bits(out), bits(plain)
    nq, nk = nh * hd, nkv * hd
    want_q = odec.rope_rows(prod[:, :nq].reshape(M * nh, hd), np.repeat(lut, nh, axis=0)).reshape(M, nq)
    assert np.array_equal(got[:, :nq], want_q)
    want_k = odec.rope_rows(prod[:, nq:nq + nk].reshape(M * nkv, hd), np.repeat(lut, nkv, axis=0)).reshape(M, nk)
    assert np.array_equal(got[:, nq:nq + nk], want_k)
    assert np.array_equal(got[:, nq + nk:], prod[:, nq + nk:])
    # rotations preserve the norm of every (i, i + head_dim / 2) pair up to the bf16 roundings
    g = bf16_bits_to_f32(got[:, :nq]).reshape(M, nh, 2, hd // 2).astype(np.float64)
    p = bf16_bits_to_f32(prod[:, :nq]).reshape(M, nh, 2, hd // 2).astype(np.float64)
    n_g, n_p = np.sqrt((g**2).sum(axis=2)), np.sqrt((p**2).sum(axis=2))
    assert np.max(np.abs(n_g - n_p)) <= 2.0**-6 * np.max(n_p)


def test_prompt_layer_on_stream_order_weights_replays_from_a_hip_graph(ops):
    """RMSNorm + Q|K|V + RoPE, causal attention and the O + FFN block (the tiled kernel raises its LDS limit by a
    function attribute at every launch) captured in one HIP graph: every replay, with eager work and
    synchronisations in between, equals the eager results bit for bit."""
    from oracle import decode as odec
    M, E, H, nh, nkv, hd = 300, 512, 1280, 8, 2, 64
    print(f"prompt layer graph M={M} E={E} H={H}", flush=True)
    _, fused = _qkv_weights(E, nh, nkv, hd, seed=2100)
    wqkv = _sw(ops, fused)
    wo, wg, wu, wd = (_sw(ops, w) for w in _weights(E, H, seed=2110, scale=0.5))
    nw_a, nw_f = dev(_norm_w(E, 2120)), dev(_norm_w(E, 2121))
    lut = dev(odec.generate_rope_lut(hd, 500000.0, M))
    xs = [dev(make_x((M, E), seed=2130 + j)) for j in range(3)]
    cur = xs[0].clone()

    def layer(x):
        qkv = ops.prefill_rms_qkv_rope_stream(x, nw_a, wqkv, lut, 0, nh, nkv, hd)
        attn = ops.prefill_attention(qkv, nh, nkv, hd)
        return qkv, attn, ops.prefill_o_ffn_stream(attn, x, nw_f, wo, wg, wu, wd)

    st = torch.cuda.Stream()
    with torch.cuda.stream(st):
        layer(cur)   # warm-up: workspaces and function attributes outside the graph
        st.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=st):
            outs = layer(cur)
        for j in range(3):
            cur.copy_(xs[j])
            g.replay()
            st.synchronize()
            want = layer(xs[j])
            st.synchronize()
            for name, a, b in zip(("qkv", "attention", "block"), outs, want):
                assert torch.isfinite(a.float()).all(), (name, j)
                assert torch.equal(a.view(torch.int16), b.view(torch.int16)), (name, j)
