"""GPU parity of the prefill O projection + FFN block (four GEMMs with fused epilogues + one
row-wise RMSNorm) against the oracle, stage by stage.

Every stage is checked on the kernel's own input to that stage, so that a one-ulp flip upstream
does not have to be propagated through a GEMM: res1 and y are bf16(bf16(P) + R) with P a float64
product (tolerance: one ulp of the sum, one ulp of P, 2e-3 absolute), the RMSNorm rows may flip
one ulp where fp32 sums differ in their last bit, and h = silu(bf16(G)) * bf16(U) moves by up to
~3 ulp when G and U flip (silu' <= 1.1).  The whole block also passes the reference's own gate.
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
    """w4a16_gemm runs the tiled prefill kernel for every M > 16, so that its output can be compared bit for bit
    with the product inside the fused prefill calls (the streaming kernel sums in another order)."""
    ops.tune("gemm_stream_max_m", 16)
    yield
    ops.tune("gemm_stream_max_m", 0)


def _weights(E, H, seed, scale=1.0):
    out = []
    for i, (K, N) in enumerate(((E, E), (E, H), (E, H), (H, E))):
        qw, qz, s = make_awq(K, N, seed=seed + i)
        out.append((qw, qz, f32_to_bf16_bits(bf16_bits_to_f32(s) * np.float32(scale))))
    return out


def _norm_w(E, seed):
    rng = np.random.default_rng(seed)
    return f32_to_bf16_bits((rng.standard_normal(E) * 0.1 + 1.0).astype(np.float32))


def _close_sum(got_bits, prod64, add32, what):
    """got = bf16(bf16(prod) + add) up to one ulp of each rounding."""
    want = prod64 + add32
    err = np.abs(bf16_bits_to_f32(got_bits).astype(np.float64) - want)
    tol = bf16_ulp(want) + bf16_ulp(prod64) + 2e-3
    assert np.all(err <= tol), f"{what}: worst {np.max(err - tol):.4g} over tolerance at {np.unravel_index(np.argmax(err - tol), err.shape)}"


@pytest.mark.parametrize("M,E,H", [(40, 256, 512), (300, 512, 1152), (17, 128, 128), (260, 1024, 2048)])
def test_prefill_block_stage_by_stage(ops, M, E, H):
    print(f"prefill block M={M} E={E} H={H}", flush=True)
    wo, wg, wu, wd = _weights(E, H, seed=M + E, scale=0.25)
    attn, xres, nw = make_x((M, E), seed=M), make_x((M, E), seed=M + 1), _norm_w(E, M + 2)
    y, res1, h = ops.prefill_o_ffn(dev(attn), dev(xres), dev(nw), tuple(map(dev, wo)), tuple(map(dev, wg)),
                                   tuple(map(dev, wu)), tuple(map(dev, wd)), return_intermediates=True)
    y2 = ops.prefill_o_ffn(dev(attn), dev(xres), dev(nw), tuple(map(dev, wo)), tuple(map(dev, wg)),
                           tuple(map(dev, wu)), tuple(map(dev, wd)))
    torch.cuda.synchronize()
    y_b, res1_b, h_b = bits(y), bits(res1), bits(h)
    assert np.array_equal(bits(y2), y_b), "intermediates kept in the workspace give another result"
    f = lambda b: bf16_bits_to_f32(b).astype(np.float64)
    # 1. O projection + residual
    _close_sum(res1_b, f(attn) @ dense_f64(*wo, rounded=True), f(xres), "res1")
    # 2. row-wise RMSNorm of the kernel's res1
    n_gpu = bits(ops.rms_norm_rows(res1, dev(nw)))
    n_ref = oref.rms_norm_rows_bf16(res1_b, nw)
    nd = np.abs(f(n_gpu) - f(n_ref))
    assert np.all(nd <= bf16_ulp(f(n_ref))) and np.mean(n_gpu != n_ref) < 0.01, (nd.max(), np.mean(n_gpu != n_ref))
    # 3. gate / up + SwiGLU on the kernel's normalised rows
    G, U = f(n_gpu) @ dense_f64(*wg, rounded=True), f(n_gpu) @ dense_f64(*wu, rounded=True)
    gb, ub = f(f32_to_bf16_bits(G.astype(np.float32))), f(f32_to_bf16_bits(U.astype(np.float32)))
    h_want = gb / (1.0 + np.exp(-gb)) * ub
    h_tol = 4 * bf16_ulp(h_want) + 1.2 * bf16_ulp(gb) * np.abs(ub) + bf16_ulp(ub) * np.abs(gb) + 1e-3
    assert np.all(np.abs(f(h_b) - h_want) <= h_tol), np.max(np.abs(f(h_b) - h_want) - h_tol)
    # 4. down projection + residual on the kernel's h and res1
    _close_sum(y_b, f(h_b) @ dense_f64(*wd, rounded=True), f(res1_b), "y")
    # the whole block against the restated CPU reference, under the reference's gate and a tighter one
    l1 = [oawq.repack_hf_awq_linear(*w, 128) for w in (wo, wg, wu, wd)]
    want, _, _ = oref.o_ffn_int4_prefill_reference(*l1, attn, xres, nw)
    got_f, want_f = bf16_bits_to_f32(y_b), bf16_bits_to_f32(want)
    assert oref.check_outputs(got_f, want_f, rtol=0.5, atol=10.0, max_mismatch_percentage=0.5, min_correlation=0.99)
    assert np.max(np.abs(got_f - want_f)) <= 8 * 2.0**-8 * np.max(np.abs(want_f)), np.max(np.abs(got_f - want_f))


def test_prefill_block_zero_projections_are_exact(ops):
    """q == z makes a projection exactly zero: res1 is the residual and y is res1, bit for bit."""
    M, E, H = 200, 256, 512
    wo, wg, wu, wd = _weights(E, H, seed=90)
    zero = lambda w: (w[1].repeat(128, axis=0), w[1], w[2])      # every q row equals its group's z row
    attn, xres, nw = make_x((M, E), seed=91), make_x((M, E), seed=92), _norm_w(E, 93)
    print("prefill block, zero O and down projections", flush=True)
    y, res1, h = ops.prefill_o_ffn(dev(attn), dev(xres), dev(nw), tuple(map(dev, zero(wo))), tuple(map(dev, wg)),
                                   tuple(map(dev, wu)), tuple(map(dev, zero(wd))), return_intermediates=True)
    torch.cuda.synchronize()
    assert np.array_equal(bits(res1), xres) and np.array_equal(bits(y), xres)
    # a zero gate projection gives h = 0 whatever up is
    _, _, h0 = ops.prefill_o_ffn(dev(attn), dev(xres), dev(nw), tuple(map(dev, wo)), tuple(map(dev, zero(wg))),
                                 tuple(map(dev, wu)), tuple(map(dev, wd)), return_intermediates=True)
    assert np.all((bits(h0) & 0x7FFF) == 0)


def test_prefill_block_llama32_1b_size(ops):
    """The reference example's dimensions (seq 2048, emb 2048, hidden 8192) against a float64 chain on the GPU."""
    M, E, H = 2048, 2048, 8192
    print("prefill block M=2048 E=2048 H=8192", flush=True)
    wo, wg, wu, wd = _weights(E, H, seed=7, scale=0.1)
    attn, xres, nw = make_x((M, E), seed=8), make_x((M, E), seed=9), _norm_w(E, 10)
    y, res1, h = ops.prefill_o_ffn(dev(attn), dev(xres), dev(nw), tuple(map(dev, wo)), tuple(map(dev, wg)),
                                   tuple(map(dev, wu)), tuple(map(dev, wd)), return_intermediates=True)
    torch.cuda.synchronize()
    d64 = lambda w: torch.from_numpy(dense_f64(*w, rounded=True)).cuda()
    rnd = lambda t: t.to(torch.bfloat16).double()
    res1_t = rnd(rnd(dev(attn).double() @ d64(wo)) + dev(xres).double())
    err = (res1.double() - res1_t).abs()
    assert float(err.max()) <= 2.0**-7 * float(res1_t.abs().max()) and float((err > 0).double().mean()) < 0.02
    # the later stages on the kernel's own intermediates
    n_t = rnd(torch.nn.functional.rms_norm(res1.double(), (E,), dev(nw).double(), eps=1e-5))
    g_t, u_t = rnd(n_t @ d64(wg)), rnd(n_t @ d64(wu))
    h_t = rnd(torch.nn.functional.silu(g_t) * u_t)
    herr = (h.double() - h_t).abs()
    assert float(herr.max()) <= 8 * 2.0**-8 * float(h_t.abs().max()) and float((herr > 0).double().mean()) < 0.1
    y_t = rnd(rnd(h.double() @ d64(wd)) + res1.double())
    yerr = (y.double() - y_t).abs()
    assert float(yerr.max()) <= 2.0**-7 * float(y_t.abs().max()) and float((yerr > 0).double().mean()) < 0.02


def test_prefill_block_rejects_bad_arguments(ops):
    from air_hip import _lib
    lib = _lib.load_library()
    P = torch.zeros(1 << 16, dtype=torch.int32, device="cuda").data_ptr()
    ws = lib.w4a16_prefill_block_workspace_bytes(32, 128, 128)
    args = [P, P, P, 1e-5] + [P] * 12 + [P, None, None, 32, 128, 128, 128, P, ws, None]
    bad = list(args); bad[24] = ws - 1
    assert lib.w4a16_prefill_o_ffn_bf16(*bad) == _lib.ERR_WORKSPACE
    bad = list(args); bad[20] = 100
    assert lib.w4a16_prefill_o_ffn_bf16(*bad) == _lib.ERR_SHAPE
    bad = list(args); bad[0] = None
    assert lib.w4a16_prefill_o_ffn_bf16(*bad) == _lib.ERR_NULL
    assert lib.rms_norm_rows_bf16(P, P, 1e-5, P, 4, 8200, None) == _lib.ERR_SHAPE


def _qkv_weights(E, nh, nkv, hd, seed, scale=0.25):
    parts = []
    for i, N in enumerate((nh * hd, nkv * hd, nkv * hd)):
        qw, qz, s = make_awq(E, N, seed=seed + i)
        parts.append((qw, qz, f32_to_bf16_bits(bf16_bits_to_f32(s) * np.float32(scale))))
    fused = tuple(np.concatenate([p[j] for p in parts], axis=1) for j in range(3))
    return parts, fused


@pytest.mark.parametrize("M,E,nh,nkv,hd,pos0", [(40, 256, 4, 2, 64, 0), (300, 512, 8, 8, 64, 7), (130, 256, 2, 1, 128, 100),
                                                 (17, 128, 3, 1, 64, 1)])
def test_prefill_rms_qkv_rope(ops, tiled_gemm, M, E, nh, nkv, hd, pos0):
    from oracle import decode as odec
    print(f"prefill qkv rope M={M} E={E} heads {nh}/{nkv} hd={hd} pos0={pos0}", flush=True)
    parts, fused = _qkv_weights(E, nh, nkv, hd, seed=M + E)
    x, nw = make_x((M, E), seed=M + 3), _norm_w(E, M + 4)
    lut = odec.generate_rope_lut(hd, 500000.0, pos0 + M + 5)
    dw = tuple(map(dev, fused))
    out = ops.prefill_rms_qkv_rope(dev(x), dev(nw), dw, dev(lut), pos0, nh, nkv, hd)
    normed = ops.rms_norm_rows(dev(x), dev(nw))
    plain = ops.w4a16_gemm(normed, *dw)
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
    # with the weights rounded to bf16 first, as the kernel's tiles hold them, most outputs agree bit for bit
    ref_r = odec.prefill_rms_qkv_rope_reference(x, nw, *l1, lut, pos0, nh, nkv, hd, round_weights=True)
    assert np.mean(got != ref_r) < 0.1, np.mean(got != ref_r)


def test_prefill_rms_qkv_rope_position_zero_is_the_identity(ops, tiled_gemm):
    """Every row at position 0 (a one-row table, cos = 1, sin = 0) leaves Q and K unrotated: the fused call equals
    RMSNorm + plain GEMM bit for bit; and shifting pos0 equals shifting the table."""
    from oracle import decode as odec
    E, nh, nkv, hd = 256, 4, 2, 64
    _, fused = _qkv_weights(E, nh, nkv, hd, seed=5)
    dw = tuple(map(dev, fused))
    nw = _norm_w(E, 6)
    lut = odec.generate_rope_lut(hd, 500000.0, 64)
    x = make_x((40, E), seed=7)
    print("prefill qkv rope, position 0 and shifted tables", flush=True)
    plain = ops.w4a16_gemm(ops.rms_norm_rows(dev(x), dev(nw)), *dw)
    for m in (0, 17, 39):
        one = ops.prefill_rms_qkv_rope(dev(x[m:m + 1]), dev(nw), dw, dev(lut[:1]), 0, nh, nkv, hd)
        assert torch.equal(one.view(torch.int16), plain[m:m + 1].view(torch.int16))
    a = ops.prefill_rms_qkv_rope(dev(x), dev(nw), dw, dev(lut), 9, nh, nkv, hd)
    b = ops.prefill_rms_qkv_rope(dev(x), dev(nw), dw, dev(lut[9:]), 0, nh, nkv, hd)
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))


def test_prefill_rms_qkv_rope_llama32_1b_size(ops, tiled_gemm):
    from oracle import decode as odec
    M, E, nh, nkv, hd = 2048, 2048, 32, 8, 64
    print("prefill qkv rope M=2048 E=2048 32/8 heads", flush=True)
    _, fused = _qkv_weights(E, nh, nkv, hd, seed=15, scale=0.1)
    dw = tuple(map(dev, fused))
    x, nw = make_x((M, E), seed=16), _norm_w(E, 17)
    lut = odec.generate_rope_lut(hd, 500000.0, M)
    out = ops.prefill_rms_qkv_rope(dev(x), dev(nw), dw, dev(lut), 0, nh, nkv, hd)
    plain = ops.w4a16_gemm(ops.rms_norm_rows(dev(x), dev(nw)), *dw)
    torch.cuda.synchronize()
    got, prod = bits(out), bits(plain)
    nq = nh * hd
    want_q = odec.rope_rows(prod[:, :nq].reshape(M * nh, hd), np.repeat(lut, nh, axis=0)).reshape(M, nq)
    assert np.array_equal(got[:, :nq], want_q)
    assert np.array_equal(got[:, nq + nkv * hd:], prod[:, nq + nkv * hd:])
    # rotations preserve the norm of every (i, i + 32) pair up to the bf16 roundings
    g = bf16_bits_to_f32(got[:, :nq]).reshape(M, nh, 2, hd // 2).astype(np.float64)
    p = bf16_bits_to_f32(prod[:, :nq]).reshape(M, nh, 2, hd // 2).astype(np.float64)
    n_g, n_p = np.sqrt((g**2).sum(axis=2)), np.sqrt((p**2).sum(axis=2))
    assert np.max(np.abs(n_g - n_p)) <= 2.0**-6 * np.max(n_p)


# query heads per KV head 1, 2, 3, 4, 8 (a workgroup takes 4, 2 or 1 heads of a group); one item, an odd and an even
# number of items (the kernel pairs the longest with the shortest), M not a multiple of the 32 queries of a wave
@pytest.mark.parametrize("M,nh,nkv,hd", [(40, 4, 2, 64), (64, 2, 2, 64), (65, 4, 1, 128), (300, 8, 2, 64), (1, 2, 1, 64),
                                         (200, 8, 1, 128), (33, 3, 3, 64), (257, 6, 2, 64), (500, 4, 1, 64), (129, 8, 2, 128),
                                         (700, 2, 1, 128), (96, 4, 1, 64)])
def test_prefill_attention(ops, M, nh, nkv, hd):
    from oracle import decode as odec
    print(f"prefill attention M={M} heads {nh}/{nkv} hd={hd}", flush=True)
    rng = np.random.default_rng(M + nh + hd)
    qkv = f32_to_bf16_bits(rng.standard_normal((M, (nh + 2 * nkv) * hd)).astype(np.float32))
    out = ops.prefill_attention(dev(qkv), nh, nkv, hd)
    torch.cuda.synchronize()
    nq, nk = nh * hd, nkv * hd
    want = odec.prefill_attention_reference(qkv[:, :nq], qkv[:, nq:nq + nk], qkv[:, nq + nk:], nh, nkv)
    got = bf16_bits_to_f32(bits(out)).astype(np.float64)
    # probabilities are rounded to bf16 before the P.V product: each of up to M terms carries 2^-9 relative error
    # (errors of random sign), plus the output rounding
    tol = bf16_ulp(want) + 2.0**-8 * np.max(np.abs(bf16_bits_to_f32(qkv[:, nq + nk:]))) + 1e-3
    assert np.all(np.abs(got - want) <= tol), np.max(np.abs(got - want) - tol)
    # the first token attends to itself only: its output is its V row, bit for bit (P = 1)
    v0 = qkv[0, nq + nk:].reshape(nkv, hd).repeat(nh // nkv, axis=0).reshape(-1)
    assert np.array_equal(bits(out)[0], v0)


def test_prefill_attention_scores_of_wide_range(ops):
    """Scores spread over hundreds of log2 units: the kernel's reference maximum, which follows the true one in steps,
    must not lose the small terms or overflow; and a second call returns the same bits."""
    from oracle import decode as odec
    M, nh, nkv, hd = 400, 4, 1, 64
    rng = np.random.default_rng(11)
    qkv = rng.standard_normal((M, (nh + 2 * nkv) * hd)).astype(np.float32)
    qkv[:, :(nh + nkv) * hd] *= 4.0                               # |q . k| / 8 up to ~100
    qkv[::7, nh * hd:(nh + nkv) * hd] *= 0.05                     # and keys that hardly count
    qkv = f32_to_bf16_bits(qkv)
    print("prefill attention, wide score range", flush=True)
    out = ops.prefill_attention(dev(qkv), nh, nkv, hd)
    again = ops.prefill_attention(dev(qkv), nh, nkv, hd)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), again.view(torch.int16))
    nq, nk = nh * hd, nkv * hd
    want = odec.prefill_attention_reference(qkv[:, :nq], qkv[:, nq:nq + nk], qkv[:, nq + nk:], nh, nkv)
    got = bf16_bits_to_f32(bits(out)).astype(np.float64)
    tol = bf16_ulp(want) + 2.0**-8 * np.max(np.abs(bf16_bits_to_f32(qkv[:, nq + nk:]))) + 1e-3
    assert np.all(np.isfinite(got)) and np.all(np.abs(got - want) <= tol), np.max(np.abs(got - want) - tol)


def test_prefill_attention_matches_the_decode_kernel_row_by_row(ops):
    """Row m of the prefill attention against the single-query decode kernel at position m over the same keys
    (that kernel applies RoPE itself, so it is fed unrotated rows and a position-0 table row)."""
    from oracle import decode as odec
    M, nh, nkv, hd = 150, 8, 2, 64
    rng = np.random.default_rng(3)
    qkv = f32_to_bf16_bits(rng.standard_normal((M, (nh + 2 * nkv) * hd)).astype(np.float32))
    print("prefill attention vs decode attention", flush=True)
    out = ops.prefill_attention(dev(qkv), nh, nkv, hd)
    ident = dev(odec.generate_rope_lut(hd, 500000.0, 1)[0])          # cos = 1, sin = 0
    nq, nk = nh * hd, nkv * hd
    kc = torch.zeros((nkv, M, hd), dtype=torch.bfloat16, device="cuda")
    vc = torch.zeros((nkv, M, hd), dtype=torch.bfloat16, device="cuda")
    d = dev(qkv)
    for m in range(M):
        one = ops.decode_attention(d[m].contiguous(), ident, kc, vc, m, nh)
        if m in (0, 63, 64, 149):
            err = (one.float() - out[m].float()).abs().max().item()
            assert err <= 2.0**-6 * out[m].float().abs().max().item(), (m, err)
    # the decode kernel filled the caches with exactly the K and V columns
    assert torch.equal(kc.transpose(0, 1).reshape(M, nk), d[:, nq:nq + nk]) and torch.equal(vc.transpose(0, 1).reshape(M, nk), d[:, nq + nk:])


def test_prefill_attention_llama32_1b_size(ops):
    M, nh, nkv, hd = 2048, 32, 8, 64
    print("prefill attention M=2048 32/8 heads", flush=True)
    g = torch.Generator(device="cuda").manual_seed(4)
    qkv = torch.randn((M, (nh + 2 * nkv) * hd), device="cuda", generator=g).to(torch.bfloat16)
    out = ops.prefill_attention(qkv, nh, nkv, hd)
    nq, nk = nh * hd, nkv * hd
    t = lambda x, n: x.double().reshape(M, n, hd).transpose(0, 1)
    want = torch.nn.functional.scaled_dot_product_attention(t(qkv[:, :nq], nh), t(qkv[:, nq:nq + nk], nkv).repeat_interleave(nh // nkv, dim=0),
                                                            t(qkv[:, nq + nk:], nkv).repeat_interleave(nh // nkv, dim=0), is_causal=True)
    want = want.transpose(0, 1).reshape(M, nq)
    err = (out.double() - want).abs()
    assert float(err.max()) <= 2.0**-7 * float(qkv[:, nq + nk:].float().abs().max()), float(err.max())
