"""Writes the small golden fixtures under tests/golden/ from seeded inputs and the CPU oracle.

    python tests/golden/make_fixtures.py

The reference stores no golden vectors for this path (its expected values are computed at
run time by each example's NumPy cpu_reference on seeded inputs), so these are this
repository's own: inputs follow the examples' seeds and draw order
(programming_examples/matrix_vector_multiplication/int4_awq/matvec_int4_packed.py:345-351,
programming_examples/dequant_awq/dequant_awq.py:382-387), expected outputs come from the
oracle after it has been pinned by tests/test_oracle_*.py.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import awq, reference as ref  # noqa: E402
from oracle.bf16 import f32_to_bf16_bits  # noqa: E402


def l1_draw(rows, k, gs):
    q = np.random.randint(0, 16, size=(rows, k), dtype=np.uint8)
    a_q = (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.uint8)
    a_s = f32_to_bf16_bits(np.random.uniform(0.005, 0.02, size=(k // gs, rows)).astype(np.float32))
    a_z = np.random.randint(7, 9, size=(k // gs, rows), dtype=np.uint8)
    return a_q, a_s, a_z


def main():
    gs = 128
    # GEMV, example seed 42, m = 64, k = 256
    np.random.seed(42)
    a_q, a_s, a_z = l1_draw(64, 256, gs)
    b = f32_to_bf16_bits(np.random.randn(256).astype(np.float32))
    qw, qz, s = awq.l1_to_awq(a_q, a_s, a_z)
    np.savez_compressed(os.path.join(HERE, "gemv_m64_k256_seed42.npz"), A_q=a_q, A_s=a_s, A_z=a_z, B=b,
                        qweight=qw, qzeros=qz, scales=s,
                        D_loop=ref.matvec_cpu_reference_loop(a_q, a_s, a_z, b),
                        D_f64=ref.matvec_cpu_reference(a_q, a_s, a_z, b),
                        W_bf16=awq.dequant_to_bf16(qw, qz, s, gs))
    # GEMM, example seed 42, m = 32, k = 256, n = 64
    np.random.seed(42)
    w_q, w_s, w_z = l1_draw(64, 256, gs)
    a = f32_to_bf16_bits(np.random.randn(32, 256).astype(np.float32))
    qw, qz, s = awq.l1_to_awq(w_q, w_s, w_z)
    np.savez_compressed(os.path.join(HERE, "gemm_m32_k256_n64_seed42.npz"), W_q=w_q, W_s=w_s, W_z=w_z, A=a,
                        qweight=qw, qzeros=qz, scales=s,
                        C_f32=ref.matmul_cpu_reference(w_q, w_s, w_z, a),
                        C_f64_rounded_w=ref.matmul_cpu_reference(w_q, w_s, w_z, a, round_weights=True, accumulate="f64"))
    # 1-D dequant, example seed 0, n = 1024
    np.random.seed(0)
    n = 1024
    q = np.random.randint(0, 16, n).astype(np.uint8)
    sc = f32_to_bf16_bits(np.random.uniform(0.01, 0.1, n // gs).astype(np.float32))
    z = np.random.randint(7, 10, n // gs).astype(np.uint8)
    np.savez_compressed(os.path.join(HERE, "dequant1d_n1024_seed0.npz"), int4_vals=q, scales=sc, zeros=z,
                        out=awq.dequant_1d(q, sc, z, gs))
    # SwiGLU front half (no RMSNorm) + down projection, H = 128, K = 256
    np.random.seed(7)
    g = l1_draw(128, 256, gs)
    u = l1_draw(128, 256, gs)
    d = l1_draw(256, 128, gs)
    x = f32_to_bf16_bits(np.random.randn(256).astype(np.float32))
    h, y = ref.ffn_swiglu_reference(g, u, d, x)
    np.savez_compressed(os.path.join(HERE, "ffn_k256_h128_seed7.npz"), x=x, h=h, y=y,
                        **{f"{n_}_{part}": arr for n_, t in (("gate", g), ("up", u), ("down", d))
                           for part, arr in zip(("q", "s", "z"), t)})
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
