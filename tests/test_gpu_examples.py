"""GPU: the example entry points end to end (PASS! harness), the golden fixtures, full-size
properties, and the host-forced failure path of the split-K reducer."""
import os
import sys

import numpy as np
import pytest
import torch

from helpers import make_awq, make_x
from oracle import awq as oawq, reference as oref
from oracle.bf16 import bf16_bits_to_f32, f32_to_bf16_bits

pytestmark = pytest.mark.gpu
G = os.path.join(os.path.dirname(__file__), "golden")


def dev(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)
    return torch.from_numpy(a).cuda()


def bits(t):
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def test_example_matvec_int4_packed(capsys):
    from air_hip.examples import matvec_int4_packed as ex
    for argv in (["--m", "256", "--k", "256"], ["--m", "2048", "--k", "2048"]):
        print("example matvec", argv, flush=True)
        assert ex.run(ex.parse_args(argv), oref.matvec_cpu_reference) == 0
    assert "PASS!" in capsys.readouterr().out


def test_example_matvec_small_vs_scalar_loop_reference(capsys):
    from air_hip.examples import matvec_int4_packed as ex
    print("example matvec scalar-loop reference", flush=True)
    assert ex.run(ex.parse_args(["--m", "64", "--k", "256"]), oref.matvec_cpu_reference_loop) == 0
    assert "PASS!" in capsys.readouterr().out


def test_example_matvec_add(capsys):
    from air_hip.examples import matvec_int4_packed_add as ex
    print("example matvec add", flush=True)
    assert ex.run(ex.parse_args(["--m", "2048", "--k", "2048"]), oref.matvec_add_cpu_reference) == 0
    assert "PASS!" in capsys.readouterr().out


def test_example_matmul(capsys):
    from air_hip.examples import matmul_int4_packed as ex
    for argv in (["--m", "64", "--k", "128", "--n", "128"], ["--m", "32", "--k", "2048", "--n", "2048"]):
        print("example matmul", argv, flush=True)
        assert ex.run(ex.parse_args(argv), oref.matmul_cpu_reference) == 0
    assert "PASS!" in capsys.readouterr().out


def test_example_swiglu_rms(capsys):
    from air_hip.examples import matvec_int4_swiglu_rms as ex
    print("example swiglu", flush=True)

    def reference(a_q, a_s, a_z, rms_in):
        return oref.swiglu_rms_cpu_reference(a_q, a_s, a_z, rms_in[0], rms_in[1])

    assert ex.run(ex.parse_args(["--m", "4096", "--k", "2048"]), reference) == 0
    assert "PASS!" in capsys.readouterr().out


def test_example_o_gemv_ffn_block(capsys):
    from air_hip.examples import o_gemv_ffn_int4 as ex
    print("example o_gemv_ffn", flush=True)

    def reference(wo, gate, up, wd, attn_out, x_residual, ffn_norm_w):
        dq = lambda t: f32_to_bf16_bits(oref._dequant_l1_f64(t[0], t[1], t[2], t[0].shape[1] * 2).astype(np.float32))
        return oref.o_gemv_ffn_int4_reference(dq(wo), attn_out, x_residual, ffn_norm_w, dq(gate), dq(up), dq(wd))

    assert ex.run(ex.parse_args(["--emb-dim", "1024", "--hidden-dim", "4096"]), reference) == 0
    assert "PASS!" in capsys.readouterr().out


def test_example_dequant_1d_bit_exact(capsys):
    from air_hip.examples import dequant_awq as ex
    print("example dequant", flush=True)
    args = ex.parse_args([])
    assert ex.run(args, oawq.dequant_1d) == 0
    q, s, z = ex.draw_inputs(args)
    got = ex.dequant(q, s, z, args.group_size)
    assert np.array_equal(np.asarray(got), oawq.dequant_1d(q, np.asarray(s), z, 128))
    assert np.array_equal(np.asarray(got), np.load(os.path.join(G, "dequant1d_n1024_seed0.npz"))["out"])
    capsys.readouterr()


@pytest.mark.parametrize("n,gs,herd_n", [(128, 128, 1), (1024, 128, 4), (4096, 64, 8), (1 << 20, 128, 16), (768, 32, 3)])
def test_dequant_1d_on_the_reference_tile_buffer(n, gs, herd_n):
    """The kernel reads the example's [herd_n, tile_bytes] buffer as pack_inputs writes it; random scale bit patterns
    (finite), every zero point, bit-exact against the oracle."""
    from air_hip import awq, bf16, ops
    print(f"dequant 1-D n={n} gs={gs} herd_n={herd_n}", flush=True)
    rng = np.random.default_rng(n + gs)
    q = rng.integers(0, 16, n).astype(np.uint8)
    z = rng.integers(0, 16, n // gs).astype(np.uint8)
    s = rng.integers(0, 65536, n // gs).astype(np.uint16)
    s[(s & 0x7F80) == 0x7F80] = 0x3C00
    packed = awq.pack_inputs_1d(q, bf16.from_bits(s), z, n, gs, herd_n)
    out = ops.awq_dequant_1d(torch.from_numpy(packed.reshape(-1)).cuda(), n, gs, herd_n)
    torch.cuda.synchronize()
    assert np.array_equal(bits(out), oawq.dequant_1d(q, s, z, gs))


def test_kernels_against_golden_fixtures():
    from air_hip import ops
    print("golden fixtures", flush=True)
    f = np.load(os.path.join(G, "gemv_m64_k256_seed42.npz"))
    w = [dev(f["qweight"]), dev(f["qzeros"]), dev(f["scales"])]
    assert np.array_equal(bits(ops.awq_dequant(*w)), f["W_bf16"])
    y = bits(ops.w4a16_gemv(dev(f["B"]), *w)).astype(np.int32)
    assert np.max(np.abs(y - f["D_f64"].astype(np.int32))) <= 1          # one bf16 ulp, no sign flips near zero here
    f = np.load(os.path.join(G, "gemm_m32_k256_n64_seed42.npz"))
    # M = 32: by default the streaming kernel (exact weights), with the limit lowered the tiled
    # prefill kernel (bf16-rounded weights); the fixture holds the expected output of either
    c = bits(ops.w4a16_gemm(dev(f["A"]), dev(f["qweight"]), dev(f["qzeros"]), dev(f["scales"])))
    assert oref.check_outputs(bf16_bits_to_f32(c), bf16_bits_to_f32(f["C_f32"]), rtol=2.0**-7, atol=2e-3)
    ops.tune("gemm_stream_max_m", 16)
    try:
        c = bits(ops.w4a16_gemm(dev(f["A"]), dev(f["qweight"]), dev(f["qzeros"]), dev(f["scales"])))
    finally:
        ops.tune("gemm_stream_max_m", 0)
    assert oref.check_outputs(bf16_bits_to_f32(c), bf16_bits_to_f32(f["C_f64_rounded_w"]), rtol=2.0**-7, atol=2e-3)
    f = np.load(os.path.join(G, "ffn_k256_h128_seed7.npz"))
    trip = lambda n: tuple(dev(a) for a in oawq.l1_to_awq(f[f"{n}_q"], f[f"{n}_s"], f[f"{n}_z"]))
    yy, hh = ops.ffn_swiglu(dev(f["x"]), trip("gate"), trip("up"), trip("down"), return_h=True)
    assert oref.check_outputs(bf16_bits_to_f32(bits(hh)), bf16_bits_to_f32(f["h"]), rtol=0.15, atol=0.5, min_correlation=0.99)
    assert oref.check_outputs(bf16_bits_to_f32(bits(yy)), bf16_bits_to_f32(f["y"]), rtol=0.2, atol=2.0, min_correlation=0.99)
    assert np.mean(bits(hh) != f["h"]) < 0.05


def test_full_size_properties_one_hot_rows_reproduce_the_dequant():
    """Config 1 and config 3 sizes: x = e_k makes every output row a dequantised weight row, so the
    GEMV and the prefill GEMM must reproduce the dequant kernel's rows bit for bit."""
    from air_hip import ops
    print("full-size one-hot property", flush=True)
    K, N = 4096, 11008
    qw, qz, s = make_awq(K, N, seed=11)
    w = [dev(qw), dev(qz), dev(s)]
    dense = ops.awq_dequant(*w)
    for k0 in (0, 127, 128, 2049, 4095):
        x = torch.zeros(K, dtype=torch.bfloat16, device="cuda")
        x[k0] = 1.0
        assert torch.equal(ops.w4a16_gemv(x, *w).view(torch.int16), dense[k0].view(torch.int16)), k0
    K, N, M = 4096, 14336, 2048
    qw, qz, s = make_awq(K, N, seed=12)
    w = [dev(qw), dev(qz), dev(s)]
    dense = ops.awq_dequant(*w)
    rows = torch.randperm(K, device="cuda")[:M]
    x = torch.zeros((M, K), dtype=torch.bfloat16, device="cuda")
    x[torch.arange(M, device="cuda"), rows] = 1.0
    y = ops.w4a16_gemm(x, *w)
    assert torch.equal(y.view(torch.int16), dense[rows].view(torch.int16))
    # scaling x by a power of two scales y exactly (no rounding changes)
    xr = torch.from_numpy(make_x((16, K), seed=5).view(np.int16)).cuda().view(torch.bfloat16)
    y1 = ops.w4a16_gemm(xr, *w)
    y2 = ops.w4a16_gemm(xr * 4, *w)
    assert torch.equal((y1.float() * 4).to(torch.bfloat16).view(torch.int16), y2.view(torch.int16))


def test_reducer_timeout_is_reported_and_workspace_recovers():
    """Fault injection from the host: split-K producers do not publish, so every reducer runs into its
    (tiny) poll bound, gives up and flags the workspace; all waves exit normally."""
    from air_hip import _lib, ops
    print("reducer timeout path", flush=True)
    lib = _lib.load_library()
    K, N = 4096, 1024
    qw, qz, s = make_awq(K, N, seed=21)
    x = dev(make_x((K,), seed=22))
    w = [dev(qw), dev(qz), dev(s)]
    good = ops.w4a16_gemv(x, *w)
    ws = ops.workspace(lib.w4a16_gemm_workspace_bytes(1, K, N), x.device)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.w4a16_workspace_check(ws.data_ptr(), stream) == 0
    try:
        ops.tune("gemv_skip_publish", 1)
        ops.tune("gemv_spin_limit", 8)
        ops.w4a16_gemv(x, *w)
        assert lib.w4a16_workspace_check(ws.data_ptr(), stream) == _lib.ERR_TIMEOUT
        # the host-side check reports it, names the code, and leaves the workspace usable
        with pytest.raises(_lib.W4A16Error) as e:
            ops.check_health()
        assert e.value.code == _lib.ERR_TIMEOUT
        assert lib.w4a16_workspace_check(ws.data_ptr(), stream) == 0
        # checked mode: the call itself raises
        ops.set_checked(True)
        with pytest.raises(_lib.W4A16Error):
            ops.w4a16_gemv(x, *w)
    finally:
        ops.set_checked(False)
        ops.tune("gemv_skip_publish", 0)
        ops.tune("gemv_spin_limit", 0)
    ops.check_health()
    assert torch.equal(ops.w4a16_gemv(x, *w).view(torch.int16), good.view(torch.int16))


def test_backend_runs_the_stream_order_kernels_and_reports_library_errors():
    """HIPBackend re-packs its weight buffers into stream order and runs the whole-K / tiled stream-order kernels: its
    outputs equal the stream-order ops bit for bit; an error code from the library is an AirBackendError."""
    from air_hip import awq, bf16, ops
    from air_hip.backend import AirBackendError, HIPBackend, HipModule
    print("HIPBackend on stream-order kernels", flush=True)
    K, N = 4096, 1024
    qw, qz, s = make_awq(K, N, seed=23)
    x = make_x((K,), seed=24)
    backend = HIPBackend()
    invoker = backend.compile_and_load(HipModule("matvec_int4", K=K, N=N, gs=128))
    args = (awq.pack_buffer(qw, qz, bf16.from_bits(s)), bf16.from_bits(x), np.zeros(N, np.uint16).view(bf16.BF16Array))
    got = np.asarray(invoker(*args)[-1]).view(np.uint16)
    want = bits(ops.w4a16_gemv_stream(dev(x), ops.repack_stream(dev(qw), dev(qz), dev(s))))
    assert np.array_equal(got, want)
    backend.unload()
    xm = make_x((32, K), seed=25)
    invoker = backend.compile_and_load(HipModule("matmul_int4", M=32, K=K, N=N, gs=128))
    got = np.asarray(invoker(bf16.from_bits(xm), args[0], np.zeros((32, N), np.uint16).view(bf16.BF16Array))[-1]).view(np.uint16)
    want = bits(ops.w4a16_gemm_stream(dev(xm), ops.repack_stream(dev(qw), dev(qz), dev(s))))
    assert np.array_equal(got, want)
    with pytest.raises(AirBackendError):
        invoker(bf16.from_bits(xm), args[0])   # no output placeholder
    backend.unload()


@pytest.mark.parametrize("example,argv", [
    # the shapes the reference's own lit tests run (run_packed*_peano.lit, run_packed_npu2_*.lit, run_int4_npu2_peano.lit)
    ("matvec_int4_packed", ["--m", "2048", "--k", "2048"]),
    ("matvec_int4_packed", ["--m", "2048", "--k", "8192"]),
    ("matvec_int4_packed_add", ["--m", "2048", "--k", "2048"]),
    ("matmul_int4_packed", []),                                                # 64 x 128 x 128
    ("matmul_int4_packed", ["--m", "32", "--k", "2048", "--n", "2048"]),
    ("matvec_int4_swiglu_rms", []),                                            # M = 16384 interleaved rows, K = 2048
    # and the tiled kernel
    ("matmul_int4_packed", ["--m", "2048", "--k", "2048", "--n", "2048"]),
    ("o_gemv_ffn_int4", ["--emb-dim", "1024", "--hidden-dim", "4096"]),
    ("dequant_awq", []),
])
def test_examples_run_as_scripts(example, argv, tmp_path, capsys, monkeypatch):
    """`python -m air_hip.examples.<name> <the reference's flags> --expected file.npz` prints PASS! and exits 0, the
    expected output written beforehand by tests/golden/make_expected.py (the reference's examples end in
    exit(runner.run_test(...)), matvec_int4_packed.py:376)."""
    import runpy
    sys.path.insert(0, G)
    try:
        import make_expected
    finally:
        sys.path.remove(G)
    print("script", example, argv, flush=True)
    path = make_expected.write_expected(example, argv, str(tmp_path / "expected.npz"))
    monkeypatch.setattr(sys, "argv", [example + ".py", *argv, "--expected", path])
    with pytest.raises(SystemExit) as e:
        runpy.run_module(f"air_hip.examples.{example}", run_name="__main__")
    assert e.value.code == 0
    assert "PASS!" in capsys.readouterr().out
    # a file computed for other arguments is refused
    import importlib
    from air_hip.examples import _common
    ex = importlib.import_module(f"air_hip.examples.{example}")
    if _common.params_of(ex.parse_args(argv)) != _common.params_of(ex.parse_args([])):
        monkeypatch.setattr(sys, "argv", [example + ".py", "--expected", path])
        with pytest.raises(SystemExit) as e:
            runpy.run_module(f"air_hip.examples.{example}", run_name="__main__")
        assert e.value.code == 2
        capsys.readouterr()


def test_hip_graph_replay_matches_eager():
    from air_hip import ops
    print("graph replay", flush=True)
    K, N = 4096, 11008
    qw, qz, s = make_awq(K, N, seed=31)
    w = [dev(qw), dev(qz), dev(s)]
    xs = [dev(make_x((K,), seed=40 + i)) for i in range(3)]
    x = xs[0].clone()
    st = torch.cuda.Stream()
    with torch.cuda.stream(st):
        y = ops.w4a16_gemv(x, *w)          # warm-up on this stream (allocates its workspace)
        st.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=st):
            ops.w4a16_gemv(x, *w, out=y)
        for xi in xs:
            x.copy_(xi)
            g.replay()
            st.synchronize()
            want = ops.w4a16_gemv(xi, *w)
            st.synchronize()
            assert torch.equal(y.view(torch.int16), want.view(torch.int16))
