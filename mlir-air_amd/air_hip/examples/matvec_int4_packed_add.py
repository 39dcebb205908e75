"""int4-AWQ GEMV with residual: D = dequant(A) @ B + R
(counterpart of .../int4_awq/matvec_int4_packed_add.py)."""

import sys

import numpy as np

from .. import bf16
from ..backend import HIPRunner, HipModule
from . import _common, matvec_int4_packed as base

pack_inputs = base.pack_inputs
parse_args = base.parse_args


def build_module(M, K, GS=128, **ignored):
    return HipModule("matvec_int4_add", K=K, N=M, gs=GS)


def draw_inputs(args):
    A_q, A_s, A_z, B = base.draw_inputs(args)
    R = bf16.from_f32(np.random.randn(args.m))
    return A_q, A_s, A_z, B, R


def run(args, cpu_reference):
    module = build_module(args.m, args.k, GS=args.gs)
    A_q, A_s, A_z, B, R = draw_inputs(args)
    D_ref = bf16.from_bits(cpu_reference(A_q, bf16.bits_of(A_s), A_z, bf16.bits_of(B), bf16.bits_of(R)))
    packed = pack_inputs(A_q, A_s, A_z, args.m, args.k, args.gs)
    return HIPRunner(verbose=args.verbose).run_test(module, inputs=[packed, B, R], expected_outputs=[D_ref],
                                                    rtol=0.1, atol=0.05, min_correlation=0.999)


def main(argv=None):
    args = parse_args(argv)
    return _common.cli_main(args, build_module(args.m, args.k, GS=args.gs), run)


if __name__ == "__main__":
    sys.exit(main())
