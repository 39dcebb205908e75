"""Host logic of the product package (no GPU): layout tools against the oracle, the runner's
comparator, backend argument checks, and the C ABI's symbols and error paths."""
import ctypes
import os
import re

import numpy as np
import pytest

from air_hip import _lib, awq, bf16
from air_hip.backend import AirBackendError, HIPBackend, HIPRunner, HipModule
from air_hip.examples import dequant_awq, matmul_int4_packed, matvec_int4_packed, matvec_int4_swiglu_rms, o_gemv_ffn_int4
from oracle import awq as oawq, reference as oref
from oracle.bf16 import f32_to_bf16_bits

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bf16_helpers_match_oracle():
    rng = np.random.default_rng(0)
    a = np.concatenate([rng.standard_normal(50000).astype(np.float32) * 3, np.array([3.0234375, 0.0, -0.0, np.inf], np.float32)])
    assert np.array_equal(np.asarray(bf16.from_f32(a)), f32_to_bf16_bits(a))
    assert np.array_equal(bf16.to_f32(bf16.from_f32(a)), oawq.bf16_bits_to_f32(f32_to_bf16_bits(a)))
    assert bf16.is_bf16(bf16.from_f32(a)) and not bf16.is_bf16(a)


def test_pack_unpack_and_layout_converters_match_oracle():
    rng = np.random.default_rng(1)
    nib = rng.integers(0, 16, size=(256, 64), dtype=np.uint8)
    assert np.array_equal(awq.pack_int4(nib), oawq.pack_awq_int32(nib))
    assert np.array_equal(awq.unpack_int4(awq.pack_int4(nib)), nib)
    z = rng.integers(0, 16, size=(2, 64), dtype=np.uint8)
    s = f32_to_bf16_bits(rng.uniform(0.005, 0.02, size=(2, 64)).astype(np.float32))
    qw, qz = awq.pack_int4(nib), awq.pack_int4(z)
    a_q, a_s, a_z = awq.l1_from_awq(qw, qz, s)
    o_q, o_s, o_z = oawq.repack_hf_awq_linear(qw, qz, s, 128)
    assert np.array_equal(a_q, o_q) and np.array_equal(np.asarray(a_s), o_s) and np.array_equal(a_z, o_z)
    qw2, qz2, s2 = awq.awq_from_l1(a_q, a_s, a_z)
    assert np.array_equal(qw2, qw) and np.array_equal(qz2, qz) and np.array_equal(np.asarray(s2), s)
    with pytest.raises(ValueError):
        awq.pack_int4(nib[:, :60])


def test_packed_buffer_round_trip_and_alignment():
    rng = np.random.default_rng(2)
    K, N = 256, 96
    qw = awq.pack_int4(rng.integers(0, 16, size=(K, N), dtype=np.uint8))
    qz = awq.pack_int4(rng.integers(0, 16, size=(K // 128, N), dtype=np.uint8))
    s = f32_to_bf16_bits(rng.uniform(0.005, 0.02, size=(K // 128, N)).astype(np.float32))
    buf = awq.pack_buffer(qw, qz, s)
    lay = awq.packed_layout(K, N)
    assert buf.size == lay["total"] and lay["z_off"] % 256 == 0 and lay["s_off"] % 256 == 0
    q2, z2, s2 = awq.unpack_buffer(buf, K, N)
    assert np.array_equal(q2, qw) and np.array_equal(z2, qz) and np.array_equal(np.asarray(s2), s)
    with pytest.raises(ValueError):
        awq.unpack_buffer(buf[:-1], K, N)


def test_interleave_round_trip_matches_oracle():
    rng = np.random.default_rng(3)
    def l1(rows):
        q = rng.integers(0, 256, size=(rows, 64), dtype=np.uint8)
        return q, bf16.from_bits(rng.integers(0, 2**15, size=(1, rows)).astype(np.uint16)), rng.integers(0, 16, size=(1, rows), dtype=np.uint8)
    g, u = l1(8), l1(8)
    a_q, a_s, a_z = awq.interleave_rows(g, u)
    o_q, o_s, o_z = oref.interleave_gate_up((g[0], np.asarray(g[1]), g[2]), (u[0], np.asarray(u[1]), u[2]))
    assert np.array_equal(a_q, o_q) and np.array_equal(np.asarray(a_s), o_s) and np.array_equal(a_z, o_z)
    g2, u2 = awq.deinterleave_rows(a_q, a_s, a_z)
    assert np.array_equal(g2[0], g[0]) and np.array_equal(np.asarray(u2[1]), np.asarray(u[1])) and np.array_equal(u2[2], u[2])


def test_examples_draw_order_and_packing():
    a = matvec_int4_packed.parse_args(["--m", "64", "--k", "256"])
    A_q, A_s, A_z, B = matvec_int4_packed.draw_inputs(a)
    f = np.load(os.path.join(ROOT, "tests", "golden", "gemv_m64_k256_seed42.npz"))
    assert np.array_equal(A_q, f["A_q"]) and np.array_equal(np.asarray(A_s), f["A_s"]) and np.array_equal(A_z, f["A_z"])
    assert np.array_equal(np.asarray(B), f["B"])
    buf = matvec_int4_packed.pack_inputs(A_q, A_s, A_z, 64, 256, 128)
    qw, qz, s = awq.unpack_buffer(buf, 256, 64)
    assert np.array_equal(qw, f["qweight"]) and np.array_equal(qz, f["qzeros"])
    assert str(matvec_int4_packed.build_module(64, 256)) == "hip.module @matvec_int4 {M = 1, K = 256, N = 64, gs = 128}"
    assert matmul_int4_packed.build_module(32, 256, 64, 128, 16, 128, 128, 16, 2, 4) == HipModule("matmul_int4", K=256, N=64, M=32)
    assert matvec_int4_swiglu_rms.build_module(128, 256).N == 64
    d = dequant_awq.parse_args([])
    q, sc, z = dequant_awq.draw_inputs(d)
    g = np.load(os.path.join(ROOT, "tests", "golden", "dequant1d_n1024_seed0.npz"))
    assert np.array_equal(q, g["int4_vals"]) and np.array_equal(np.asarray(sc), g["scales"]) and np.array_equal(z, g["zeros"])
    # the fused RMSNorm example hands RMS_in (x row, weight row) to the kernel unchanged
    assert matvec_int4_swiglu_rms.build_module(128, 256).op == "matvec_int4_swiglu_rms"
    args = matvec_int4_swiglu_rms.parse_args(["--m", "32", "--k", "256"])
    *_, RMS_in = matvec_int4_swiglu_rms.draw_inputs(args)
    assert bf16.bits_of(RMS_in).shape == (2, 256)
    # block example: reference argument names, weight generator seeds and shapes
    a = o_gemv_ffn_int4.parse_args(["--emb-dim", "256", "--hidden-dim", "512"])
    wo, gu, wd, attn_out, x_residual, ffn_norm_w = o_gemv_ffn_int4.draw_inputs(a)
    assert wo[0].shape == (256, 128) and gu[0].shape == (1024, 128) and wd[0].shape == (256, 256)
    assert wd[1].shape == (4, 256) and set(np.unique(wo[2])) <= {7, 8}
    assert o_gemv_ffn_int4.build_module(256, 512) == HipModule("o_gemv_ffn_int4", K=256, N=512)
    rng = np.random.default_rng(100)
    q = rng.integers(0, 16, size=(256, 256), dtype=np.uint8)
    assert np.array_equal(wo[0], q[:, 0::2] | (q[:, 1::2] << 4))


def test_example_scripts_cli_without_a_gpu(tmp_path, capsys):
    """The stand-alone entry points: -p prints the module, compile-only validates it, a run without --expected or with
    a file written for other arguments returns 2 before anything touches the GPU."""
    import json
    import sys
    from air_hip.examples import _common
    assert matvec_int4_packed.main(["-p", "--m", "256", "--k", "512"]) == 0
    assert "hip.module @matvec_int4 {M = 1, K = 512, N = 256, gs = 128}" in capsys.readouterr().out
    assert matmul_int4_packed.main(["--compile-mode", "compile-only", "--output-format", "xclbin"]) == 0
    with pytest.raises(AirBackendError):
        matvec_int4_packed.main(["--compile-mode", "compile-only", "--k", "100"])
    assert o_gemv_ffn_int4.main([]) == 2
    assert "--expected" in capsys.readouterr().err
    args = dequant_awq.parse_args(["--n", "256"])
    path = str(tmp_path / "e.npz")
    _common.save_expected(path, args, np.zeros(256, np.uint16))
    with np.load(path) as f:
        assert json.loads(str(f["params"])) == {"group_size": 128, "herd_n": 4, "n": 256}
    assert dequant_awq.main(["--n", "512", "--expected", path]) == 2
    assert "was computed for" in capsys.readouterr().err
    sys.path.insert(0, os.path.join(os.path.dirname(__file__), "golden"))
    try:
        import make_expected
    finally:
        sys.path.pop(0)
    path = make_expected.write_expected("matvec_int4_packed", ["--m", "64", "--k", "256"], str(tmp_path / "m.npz"))
    a_q, a_s, a_z, b = matvec_int4_packed.draw_inputs(matvec_int4_packed.parse_args(["--m", "64", "--k", "256"]))
    with np.load(path) as f:
        assert np.array_equal(f["expected"], oref.matvec_cpu_reference_loop(a_q, bf16.bits_of(a_s), a_z, bf16.bits_of(b)))


def test_runner_comparator_semantics_match_reference_restatement(capsys):
    r = HIPRunner()
    e = np.linspace(1, 2, 1000)
    a = e.copy()
    a[:5] += 1.0
    for kw in (dict(rtol=0.1, atol=0.05), dict(rtol=0.1, atol=0.05, max_mismatch_percentage=0.5),
               dict(rtol=0.1, atol=0.05, max_mismatch_percentage=0.49), dict(rtol=0.1, atol=0.05, min_correlation=0.999)):
        assert r._check_outputs([a], [e], **kw) == oref.check_outputs(a, e, **kw), kw
    assert not r._check_outputs([np.ones(10)], [np.ones(10)], rtol=1, atol=1, min_correlation=0.5)   # NaN correlation
    # bf16 outputs are compared as floats, integers exactly
    eb = bf16.from_f32(np.array([1.0, 2.0, 3.0], np.float32))
    ab = bf16.from_f32(np.array([1.0, 2.0, 3.02], np.float32))
    assert r._check_outputs([ab], [eb], rtol=0.1, atol=0.05)
    assert not r._check_outputs([np.array([1, 2, 3])], [np.array([1, 2, 4])])
    capsys.readouterr()


def test_backend_compile_rejects_bad_modules_and_load_needs_gpu():
    b = HIPBackend()
    for bad in (HipModule("matvec_int4", K=100, N=64), HipModule("matvec_int4", K=128, N=40),
                HipModule("matvec_int4", K=128, N=64, gs=64), HipModule("nope", K=128, N=64),
                HipModule("matmul_int4", K=128, N=64, M=0)):
        with pytest.raises(AirBackendError):
            b.compile(bad)
    with pytest.raises(AirBackendError):
        b.compile("not a module")
    art = b.compile(HipModule("dequant_awq", K=128, N=40))
    import torch
    if not torch.cuda.is_available():
        with pytest.raises(AirBackendError):
            b.load(art)


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "w4a16.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(?:int|size_t|const char \*)\s*\*?(\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load_library()
    names = _declared_functions()
    assert "w4a16_gemv_bf16" in names and "awq_dequant_bf16" in names and len(names) >= 12
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/w4a16.h but not exported"
        assert n in _lib.SYMBOLS, f"{n} has no ctypes prototype"
    assert lib.w4a16_abi_version() == 1
    assert lib.w4a16_strerror(0) == b"ok" and b"128" in lib.w4a16_strerror(_lib.ERR_GROUP)


def test_c_abi_rejects_bad_arguments_before_touching_the_gpu():
    lib = _lib.load_library()
    P = 0x10000   # fake, aligned, never dereferenced: validation fails first
    assert lib.awq_dequant_bf16(None, P, P, P, 128, 8, 128, None) == _lib.ERR_NULL
    assert lib.awq_dequant_bf16(P, P, P, None, 128, 8, 128, None) == _lib.ERR_NULL
    assert lib.awq_dequant_bf16(P, P, P, P, 100, 8, 128, None) == _lib.ERR_SHAPE
    assert lib.awq_dequant_bf16(P, P, P, P, 128, 12, 128, None) == _lib.ERR_SHAPE
    assert lib.awq_dequant_bf16(P, P, P, P, 128, 8, 64, None) == _lib.ERR_GROUP
    assert lib.awq_dequant_bf16(P + 4, P, P, P, 128, 8, 128, None) == _lib.ERR_ALIGN
    ws = lib.w4a16_gemm_workspace_bytes(1, 128, 32)
    assert ws > 0 and lib.w4a16_gemm_workspace_bytes(0, 128, 32) == 0
    assert lib.w4a16_gemv_bf16(P, P, P, P, P, 128, 8, 128, P, ws, None) == _lib.ERR_SHAPE      # GEMV needs N % 32 == 0
    assert lib.w4a16_gemv_bf16(P, P, P, P, P, 128, 32, 128, None, ws, None) == _lib.ERR_WORKSPACE
    assert lib.w4a16_gemv_bf16(P, P, P, P, P, 128, 32, 128, P, ws - 1, None) == _lib.ERR_WORKSPACE
    assert lib.w4a16_gemm_bf16(P, P, P, P, P, 0, 128, 32, 128, P, ws, None) == _lib.ERR_SHAPE
    assert lib.w4a16_gemm_bf16(None, P, P, P, P, 4, 128, 32, 128, P, ws, None) == _lib.ERR_NULL
    fws = lib.w4a16_ffn_workspace_bytes(128, 256)
    args = [P] * 10 + [P, None, 128, 256, 128, P, fws, None]
    bad = list(args)
    bad[13] = 200                                                                              # H not a multiple of 128
    assert lib.w4a16_ffn_swiglu_bf16(*bad) == _lib.ERR_SHAPE
    bad = list(args)
    bad[16] = fws - 1
    assert lib.w4a16_ffn_swiglu_bf16(*bad) == _lib.ERR_WORKSPACE
    qws = lib.w4a16_prefill_qkv_workspace_bytes(64, 256)
    assert qws >= 64 * 256 * 2 and lib.w4a16_prefill_qkv_workspace_bytes(64, 8200) == 0
    qargs = [P, P, 1e-5, P, P, P, P, 128, 0, P, 64, 256, 4, 2, 64, 128, P, qws, None]
    bad = list(qargs); bad[14] = 96
    assert lib.w4a16_prefill_rms_qkv_rope_bf16(*bad) == _lib.ERR_SHAPE        # head_dim 64 or 128
    bad = list(qargs); bad[8] = 65
    assert lib.w4a16_prefill_rms_qkv_rope_bf16(*bad) == _lib.ERR_SHAPE        # pos0 + M beyond the table
    bad = list(qargs); bad[17] = qws - 1
    assert lib.w4a16_prefill_rms_qkv_rope_bf16(*bad) == _lib.ERR_WORKSPACE
    bad = list(qargs); bad[6] = None
    assert lib.w4a16_prefill_rms_qkv_rope_bf16(*bad) == _lib.ERR_NULL
    pws = lib.w4a16_prefill_block_workspace_bytes(64, 256, 512)
    assert pws >= 4 * 64 * (256 + 512)
    pargs = [P, P, P, 1e-5] + [P] * 12 + [P, None, None, 64, 256, 512, 128, P, pws, None]
    bad = list(pargs); bad[21] = 500
    assert lib.w4a16_prefill_o_ffn_bf16(*bad) == _lib.ERR_SHAPE
    bad = list(pargs); bad[24] = pws - 1
    assert lib.w4a16_prefill_o_ffn_bf16(*bad) == _lib.ERR_WORKSPACE
    assert lib.rms_norm_rows_bf16(P, P, 1e-5, P, 4, 100, None) == _lib.ERR_SHAPE    # K % 8
    lws = lib.lm_head_workspace_bytes(100)
    assert lws >= 8 * 7 and lib.lm_head_workspace_bytes(0) == 0
    assert lib.lm_head_gemv_bf16(P, None, 0.0, P, None, None, 100, 512, P, lws, None) == _lib.ERR_NULL
    assert lib.lm_head_gemv_bf16(P, None, 0.0, P, P, None, 100, 8200, P, lws, None) == _lib.ERR_SHAPE   # E above 8192
    assert lib.lm_head_gemv_bf16(P, P, -1.0, P, P, None, 100, 512, P, lws, None) == _lib.ERR_SHAPE
    assert lib.lm_head_gemv_bf16(P, None, 0.0, P, P, P + 2, 100, 512, P, lws, None) == _lib.ERR_ALIGN
    assert lib.lm_head_gemv_bf16(P, None, 0.0, P, P, None, 100, 512, P, lws - 1, None) == _lib.ERR_WORKSPACE
    aws = lib.w4a16_attention_workspace_bytes(4, 64)
    bws = lib.w4a16_block_workspace_bytes(256, 512)
    fargs = [P, P, P, P, P, 3, 16, 4, 2, 64, P, aws, P, P, 1e-5] + [P] * 12 + [P, None, 256, 512, 128, P, bws, None]
    bad = list(fargs); bad[4] = None
    assert lib.w4a16_decode_attn_o_gemv_ffn_bf16(*bad) == _lib.ERR_NULL
    bad = list(fargs); bad[29] = 512                                        # E != n_heads * head_dim
    assert lib.w4a16_decode_attn_o_gemv_ffn_bf16(*bad) == _lib.ERR_SHAPE
    bad = list(fargs); bad[5] = 16                                          # pos == max_seq
    assert lib.w4a16_decode_attn_o_gemv_ffn_bf16(*bad) == _lib.ERR_SHAPE
    bad = list(fargs); bad[11] = aws - 1
    assert lib.w4a16_decode_attn_o_gemv_ffn_bf16(*bad) == _lib.ERR_WORKSPACE
    bad = list(fargs); bad[33] = bws - 1
    assert lib.w4a16_decode_attn_o_gemv_ffn_bf16(*bad) == _lib.ERR_WORKSPACE
    bad = list(fargs); bad[12] = None                                       # x_residual
    assert lib.w4a16_decode_attn_o_gemv_ffn_bf16(*bad) == _lib.ERR_NULL
    bad = list(fargs); bad[28] = P + 4                                      # y_sumsq misaligned
    assert lib.w4a16_decode_attn_o_gemv_ffn_bf16(*bad) == _lib.ERR_ALIGN
    gws = lib.w4a16_gemm_workspace_bytes(1, 256, 64)
    assert lib.w4a16_rms_gemv_sumsq_bf16(P, None, 1, P, 1e-5, P, P, P, P, 256, 64, 128, P, gws, None) == _lib.ERR_NULL
    assert lib.w4a16_rms_gemv_sumsq_bf16(P, P, 65, P, 1e-5, P, P, P, P, 256, 64, 128, P, gws, None) == _lib.ERR_SHAPE
    assert lib.w4a16_rms_gemv_sumsq_bf16(P, P, 1, P, 1e-5, P, P, P, P, 256, 64, 128, P, gws - 1, None) == _lib.ERR_WORKSPACE
    assert lib.rope_halfsplit_bf16(P, P, None, 8, 64, None) == _lib.ERR_NULL
    assert lib.rope_halfsplit_bf16(P, P, P, 8, 24, None) == _lib.ERR_SHAPE        # dim % 16
    assert lib.rope_halfsplit_bf16(P, P, P, 0, 64, None) == _lib.ERR_SHAPE
    assert lib.rope_halfsplit_bf16(P, P + 8, P, 8, 64, None) == _lib.ERR_ALIGN
    assert lib.w4a16_workspace_init(None, 1024, None) == _lib.ERR_NULL
    assert lib.w4a16_workspace_init(P, 16, None) == _lib.ERR_WORKSPACE
    assert lib.w4a16_tune(b"no_such_key", 1) == _lib.ERR_TUNE and lib.w4a16_tune(b"gemv_waves", 0) == 0
    # the batched GEMM with caller scratch: scratch only where the split along K is the faster way (long K, enough rows, not
    # the widest matrices), and every argument checked before a launch
    need = lib.w4a16_gemm_stream_scratch_bytes(64, 14336, 4096)
    assert need == 14 * 64 * 4096 * 4
    assert lib.w4a16_gemm_stream_scratch_bytes(64, 4096, 14336) == 0 and lib.w4a16_gemm_stream_scratch_bytes(64, 2048, 4096) == 0
    assert lib.w4a16_gemm_stream_scratch_bytes(16, 14336, 4096) == 0 and lib.w4a16_gemm_stream_scratch_bytes(129, 14336, 4096) == 0
    assert lib.w4a16_gemm_stream_scratch_bytes(64, 14336, 4100) == 0
    big = (P, P, P, 64, 14336, 4096, 128)
    assert lib.w4a16_gemm_stream_scratch_bf16(*big, None, 0, None) == _lib.ERR_WORKSPACE
    assert lib.w4a16_gemm_stream_scratch_bf16(*big, P, need - 1, None) == _lib.ERR_WORKSPACE
    assert lib.w4a16_gemm_stream_scratch_bf16(*big, P + 8, need, None) == _lib.ERR_ALIGN
    assert lib.w4a16_gemm_stream_scratch_bf16(None, P, P, 64, 14336, 4096, 128, P, need, None) == _lib.ERR_NULL
    assert lib.w4a16_gemm_stream_scratch_bf16(P, P, P, 64, 14336, 4096, 64, P, need, None) == _lib.ERR_GROUP
    assert lib.w4a16_gemm_stream_scratch_bf16(P, P, P, 64, 14336, 4100, 128, P, need, None) == _lib.ERR_SHAPE
    assert lib.w4a16_gemm_stream_scratch_bf16(P, P, None, 64, 4096, 14336, 128, None, 0, None) == _lib.ERR_NULL   # (whole-K route)
    assert lib.w4a16_tune(b"gemm_splitk", 3) == _lib.ERR_TUNE and lib.w4a16_tune(b"gemm_splitk", 0) == 0
    # Q4NX order: blocks -> stream order, and the prompt-pass entry points
    assert lib.w4a16_q4nx_blocks_to_stream(None, P, 32, 256, 0, None) == _lib.ERR_NULL
    assert lib.w4a16_q4nx_blocks_to_stream(P, P, 48, 256, 0, None) == _lib.ERR_SHAPE      # whole blocks of 32 rows
    assert lib.w4a16_q4nx_blocks_to_stream(P, P, 32, 128, 0, None) == _lib.ERR_SHAPE      # and of 256 columns
    assert lib.w4a16_q4nx_blocks_to_stream(P, P, 32, 256, 3, None) == _lib.ERR_SHAPE
    assert lib.w4a16_q4nx_blocks_to_stream(P, P + 4, 32, 256, 0, None) == _lib.ERR_ALIGN
    wsq = lib.w4a16_prefill_qkv_workspace_bytes(64, 256)
    assert lib.w4a16_q4nx_prefill_rms_qkv_rope_stream_bf16(P, P, 1e-5, None, P, 80, 0, P, 64, 256, 4, 2, 64, P, wsq, None) == _lib.ERR_NULL
    assert lib.w4a16_q4nx_prefill_rms_qkv_rope_stream_bf16(P, P, 1e-5, P, P, 80, 20, P, 64, 256, 4, 2, 64, P, wsq, None) == _lib.ERR_SHAPE
    assert lib.w4a16_q4nx_prefill_rms_qkv_rope_stream_bf16(P, P, 1e-5, P, P, 80, 0, P, 64, 256, 4, 2, 64, P, wsq - 1, None) == _lib.ERR_WORKSPACE
    wsb = lib.w4a16_prefill_block_workspace_bytes(64, 256, 512)
    blk = [P, P, P, 1e-5, P, P, P, P, P, None, None, 64, 256, 512]
    assert lib.w4a16_q4nx_prefill_o_ffn_stream_bf16(*blk, None, wsb, None) == _lib.ERR_WORKSPACE
    assert lib.w4a16_q4nx_prefill_o_ffn_stream_bf16(*(blk[:4] + [None] + blk[5:]), P, wsb, None) == _lib.ERR_NULL
    assert lib.w4a16_q4nx_prefill_o_ffn_stream_bf16(*(blk[:13] + [500]), P, wsb, None) == _lib.ERR_SHAPE
    with pytest.raises(_lib.W4A16Error):
        _lib.check(_lib.ERR_ALIGN)


def test_kernel_cache_host_contract(tmp_path):
    """What KernelCache decides before it touches the device: module shape rules, registration, the manifest,
    unknown kernels, the shared_alias checks (the reference makes these before any XRT call,
    shared/infra/cache.py:569-603) and the profiler's bookkeeping."""
    from air_hip import cache as kc

    with pytest.raises(AssertionError):
        kc.build_rms_qkv_int4_rope_module(emb_dim=2048, kv_dim=512, n_heads=16, n_kv_heads=8, head_dim=64)
    with pytest.raises(AssertionError):
        kc.build_rms_qkv_int4_rope_module(emb_dim=1024, kv_dim=256, n_heads=16, n_kv_heads=4, head_dim=64)   # k_chunk != emb
    with pytest.raises(AssertionError):
        kc.build_o_gemv_ffn_int4_module(emb_dim=2048, hidden_dim=3072)
    with pytest.raises(AssertionError):
        kc.build_o_gemv_ffn_int4_module(emb_dim=4096, hidden_dim=8192)
    c = kc.KernelCache(cache_dir=tmp_path, profiler=kc.Profiler(enabled=True))
    with pytest.raises(AirBackendError):
        c.compile_and_cache("x", "not a module", {})
    with pytest.raises(AirBackendError):
        c.compile_and_cache("x", kc.DecodeModule("o_gemv_ffn_int4", emb_dim=2048, hidden_dim=8192, gs=64), {})
    c.compile_and_cache("rms_qkv_int4_rope", kc.build_rms_qkv_int4_rope_module(), {"verbose": False})
    c.compile_and_cache("o_gemv_ffn_int4", kc.build_o_gemv_ffn_int4_module(), {})
    c.compile_and_cache("lm_head_gemv", kc.build_lm_head_gemv_module(2048), {})
    assert set(c.profiler.compile_times) == {"rms_qkv_int4_rope", "o_gemv_ffn_int4", "lm_head_gemv"}
    c._save_manifest()
    c2 = kc.KernelCache(cache_dir=tmp_path)
    assert c2.load_manifest() and c2.artifacts == c.artifacts
    assert not kc.KernelCache().load_manifest()

    with pytest.raises(RuntimeError, match="not found in cache"):
        c.load_and_run("attn_gemms", {}, np.zeros(4, np.uint16))
    z = bf16.from_f32(np.zeros(2048))
    args = [z] * 15
    with pytest.raises(ValueError, match="is static"):
        c.load_and_run("o_gemv_ffn_int4", {}, *args, static_input_indices={0, 6}, shared_alias={6: "res"})
    with pytest.raises(ValueError, match="does not exist"):
        c.load_and_run("o_gemv_ffn_int4", {}, *args, shared_alias={15: "res"})
    with pytest.raises(ValueError, match="no pool name"):
        c.load_and_run("o_gemv_ffn_int4", {}, *args, shared_alias={14: ""})
    with pytest.raises(AirBackendError, match="takes 15 arguments"):
        c.load_and_run("o_gemv_ffn_int4", {}, *args[:14])

    prof = kc.Profiler(enabled=True)
    with prof.time_cpu("decode_attention_cpu"):
        pass
    for layer in range(4):
        prof.end_layer(layer % 2, prof.start_layer())
    prof.record_kernel("k", 0.5)
    prof.record_breakdown("k", 1.0, 2.0, 3.0, 4, 5, 6)
    assert len(prof.cpu_times["decode_attention_cpu"]) == 1 and len(prof.per_token_walls_ms(2)) == 2
    assert prof.per_token_walls_ms(3) == [] and prof.kernel_breakdowns["k"][0]["bytes_written"] == 5
    off = kc.Profiler()
    off.record_kernel("k", 1.0)
    assert off.start_layer() is None and off.kernel_times == {} and off.per_token_walls_ms(1) == []


def test_fake_quantize_matches_the_oracle_loop():
    """The vectorised host quantiser against the oracle's scalar restatement, bit for bit, on groups with outliers,
    constant groups and one-sided groups; accepts bf16 bits or floats."""
    rng = np.random.default_rng(9)
    w = (rng.standard_normal((12, 512)) * 10.0 ** rng.uniform(-3, 1, (12, 1))).astype(np.float32)
    w[3, 128:256] = 0.25
    w[4, :128] = np.abs(w[4, :128]) + 1.0
    w[5, 17] = 40.0
    wb = bf16.from_f32(w)
    got = awq.fake_quantize_awq_int4(wb, 128)
    want = oawq.fake_quantize_awq_int4_loop(bf16.to_f32(bf16.bits_of(wb)), 128)
    assert np.array_equal(got[0], want[0]) and np.array_equal(bf16.bits_of(got[1]), want[1]) and np.array_equal(got[2], want[2])
    got_f = awq.fake_quantize_awq_int4(bf16.to_f32(bf16.bits_of(wb)), 128)
    assert all(np.array_equal(np.asarray(a), np.asarray(b)) for a, b in zip(got, got_f))
    assert got[0].shape == (12, 256) and got[1].shape == (4, 12) and got[2].dtype == np.uint8
    with pytest.raises(ValueError):
        awq.fake_quantize_awq_int4(w[:, :100], 128)
