"""TEST / BENCHMARK INFRASTRUCTURE ONLY - the reference's NumPy CPU path on AWQ-layout
tensors, vectorised, for timing beside the GPU kernels and for sanity checks.

It restates "unpack -> (q - z) * s in float32 -> x @ W -> bf16":
  unpack / dequant  programming_examples/llms/llama32_1b_int4/awq_pack.py:66-104
  product           programming_examples/matrix_multiplication/int4_awq/matmul_int4_packed.py:104
                    (float32 BLAS), vectorised as
                    programming_examples/decode_ffn_swiglu/matvec_int4_swiglu_rms.py:501-511
  SwiGLU / down     matvec_int4_swiglu_rms.py:512-516,
                    programming_examples/llms/llama32_1b_int4/multi_launch_builder/o_gemv_ffn_int4_fused.py:1078-1094
"""

import numpy as np

from .awq import dequant_to_bf16, dequant_unrounded_f32
from .bf16 import bf16_bits_to_f32, f32_to_bf16_bits
from .reference import silu_tanh_f32


def dequant_numpy(qweight, qzeros, scales_bits, gs=128):
    return dequant_to_bf16(qweight, qzeros, scales_bits, gs)


def gemm_numpy(x_bits, qweight, qzeros, scales_bits, gs=128):
    """bf16 bits of x[M, K] @ W with float32 weights and a float32 BLAS product."""
    w = dequant_unrounded_f32(qweight, qzeros, scales_bits, gs)
    return f32_to_bf16_bits(bf16_bits_to_f32(x_bits) @ w)


def ffn_numpy(x_bits, gate, up, down, gs=128):
    g = bf16_bits_to_f32(gemm_numpy(x_bits, *gate, gs))
    u = bf16_bits_to_f32(gemm_numpy(x_bits, *up, gs))
    h = f32_to_bf16_bits(silu_tanh_f32(g) * u)
    return gemm_numpy(h, *down, gs)
