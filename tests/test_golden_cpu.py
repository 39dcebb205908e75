"""Oracle against the committed golden fixtures (tests/golden/*.npz, written by make_fixtures.py)."""
import os

import numpy as np

from oracle import awq, reference as ref

G = os.path.join(os.path.dirname(__file__), "golden")


def load(name):
    return np.load(os.path.join(G, name))


def test_gemv_fixture():
    f = load("gemv_m64_k256_seed42.npz")
    assert np.array_equal(ref.matvec_cpu_reference(f["A_q"], f["A_s"], f["A_z"], f["B"]), f["D_f64"])
    assert np.array_equal(ref.matvec_cpu_reference_loop(f["A_q"], f["A_s"], f["A_z"], f["B"]), f["D_loop"])
    qw, qz, s = awq.l1_to_awq(f["A_q"], f["A_s"], f["A_z"])
    assert np.array_equal(qw, f["qweight"]) and np.array_equal(qz, f["qzeros"]) and np.array_equal(s, f["scales"])
    assert np.array_equal(awq.dequant_to_bf16(qw, qz, s, 128), f["W_bf16"])
    # the sequential float32 loop and the float64 sum agree to one bf16 ulp
    a = f["D_loop"].astype(np.int32)
    b = f["D_f64"].astype(np.int32)
    assert np.max(np.abs(a - b)) <= 1


def test_gemm_fixture():
    f = load("gemm_m32_k256_n64_seed42.npz")
    assert np.array_equal(ref.matmul_cpu_reference(f["W_q"], f["W_s"], f["W_z"], f["A"], round_weights=True,
                                                   accumulate="f64"), f["C_f64_rounded_w"])
    got = ref.matmul_cpu_reference(f["W_q"], f["W_s"], f["W_z"], f["A"])
    # float32 BLAS accumulation order may differ between hosts: one bf16 ulp
    assert np.max(np.abs(got.astype(np.int32) - f["C_f32"].astype(np.int32))) <= 1


def test_dequant1d_and_ffn_fixtures():
    f = load("dequant1d_n1024_seed0.npz")
    assert np.array_equal(awq.dequant_1d(f["int4_vals"], f["scales"], f["zeros"], 128), f["out"])
    f = load("ffn_k256_h128_seed7.npz")
    g, u, d = [(f[f"{n}_q"], f[f"{n}_s"], f[f"{n}_z"]) for n in ("gate", "up", "down")]
    h, y = ref.ffn_swiglu_reference(g, u, d, f["x"])
    assert np.array_equal(h, f["h"]) and np.array_equal(y, f["y"])
