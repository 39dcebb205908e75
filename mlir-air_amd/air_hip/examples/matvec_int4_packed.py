"""int4-AWQ GEMV: D[M] = dequant(A_q, A_s, A_z)[M, K] @ B[K]
(counterpart of programming_examples/matrix_vector_multiplication/int4_awq/matvec_int4_packed.py)."""

import argparse
import sys

import numpy as np

from .. import awq, bf16
from ..backend import HIPRunner, HipModule
from . import _common
from ._common import draw_l1_weights


def build_module(M, K, GS=128, M_TILE=8, K_CHUNK=2048, N_CORES=8, M_PER_LAUNCH=None):
    """The NPU tiling arguments are accepted for call compatibility and ignored."""
    return HipModule("matvec_int4", K=K, N=M, gs=GS)


def pack_inputs(A_q, A_s, A_z, M, K, GS, M_TILE=8, K_CHUNK=2048, N_CORES=8, M_PER_LAUNCH=None):
    """Kernel-side arrays -> the single packed weight buffer of this backend (AWQ layout)."""
    if A_q.shape != (M, K // 2):
        raise ValueError(f"A_q shape {A_q.shape} vs expected ({M}, {K // 2})")
    return awq.pack_buffer(*awq.awq_from_l1(A_q, A_s, A_z))


def parse_args(argv=None):
    p = argparse.ArgumentParser(prog="matvec_int4_packed.py", description="int4-AWQ GEMV: D = dequant(A) @ B")
    p.add_argument("-v", "--verbose", action="store_true")
    p.add_argument("--m", type=int, default=2048)
    p.add_argument("--k", type=int, default=2048)
    p.add_argument("--gs", type=int, default=128)
    p.add_argument("--m-tile", type=int, default=8, dest="m_tile")
    p.add_argument("--k-chunk", type=int, default=2048, dest="k_chunk")
    p.add_argument("--n-cores", type=int, default=8, dest="n_cores")
    return _common.add_reference_cli(p).parse_args(argv)


def draw_inputs(args):
    np.random.seed(42)
    A_q, A_s, A_z = draw_l1_weights(args.m, args.k, args.gs)
    B = bf16.from_f32(np.random.randn(args.k))
    return A_q, A_s, A_z, B


def run(args, cpu_reference):
    module = build_module(args.m, args.k, GS=args.gs)
    A_q, A_s, A_z, B = draw_inputs(args)
    D_ref = bf16.from_bits(cpu_reference(A_q, bf16.bits_of(A_s), A_z, bf16.bits_of(B)))
    packed = pack_inputs(A_q, A_s, A_z, args.m, args.k, args.gs)
    runner = HIPRunner(verbose=args.verbose)
    return runner.run_test(module, inputs=[packed, B], expected_outputs=[D_ref], rtol=0.1, atol=0.05,
                           min_correlation=0.999)


def main(argv=None):
    args = parse_args(argv)
    return _common.cli_main(args, build_module(args.m, args.k, GS=args.gs), run)


if __name__ == "__main__":
    sys.exit(main())
