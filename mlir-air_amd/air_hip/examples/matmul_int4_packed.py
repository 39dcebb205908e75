"""int4-AWQ GEMM: C[M, N] = A[M, K] @ dequant(W)[K, N]
(counterpart of programming_examples/matrix_multiplication/int4_awq/matmul_int4_packed.py)."""

import argparse
import sys

import numpy as np

from .. import awq, bf16
from ..backend import HIPRunner, HipModule
from . import _common
from ._common import draw_l1_weights


def build_module(m, k, n, gs=128, *ignored_tiling, **ignored):
    return HipModule("matmul_int4", M=m, K=k, N=n, gs=gs)


def pack_inputs(W_q, W_s, W_z, M, K, N, GS, N_TILE=16, K_CHUNK=128):
    if W_q.shape != (N, K // 2):
        raise ValueError(f"W_q shape {W_q.shape} vs expected ({N}, {K // 2})")
    return awq.pack_buffer(*awq.awq_from_l1(W_q, W_s, W_z))


def parse_args(argv=None):
    p = argparse.ArgumentParser(prog="matmul_int4_packed.py")
    p.add_argument("--m", type=int, default=64)
    p.add_argument("--k", type=int, default=128)
    p.add_argument("--n", type=int, default=128)
    p.add_argument("--gs", type=int, default=128)
    p.add_argument("-v", "--verbose", action="store_true")
    return _common.add_reference_cli(p).parse_args(argv)


def draw_inputs(args):
    np.random.seed(42)
    W_q, W_s, W_z = draw_l1_weights(args.n, args.k, args.gs)
    A = bf16.from_f32(np.random.randn(args.m, args.k))
    return W_q, W_s, W_z, A


def run(args, cpu_reference):
    module = build_module(args.m, args.k, args.n, args.gs)
    W_q, W_s, W_z, A = draw_inputs(args)
    packed = pack_inputs(W_q, W_s, W_z, args.m, args.k, args.n, args.gs)
    C_ref = bf16.from_bits(cpu_reference(W_q, bf16.bits_of(W_s), W_z, bf16.bits_of(A)))
    return HIPRunner(verbose=args.verbose).run_test(module, inputs=[A, packed], expected_outputs=[C_ref], rtol=0.1,
                                                    atol=0.05, max_mismatch_percentage=0.05, min_correlation=0.999)


def main(argv=None):
    args = parse_args(argv)
    return _common.cli_main(args, build_module(args.m, args.k, args.n, args.gs), run)


if __name__ == "__main__":
    sys.exit(main())
