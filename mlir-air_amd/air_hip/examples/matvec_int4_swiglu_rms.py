"""Decode FFN front half: RMSNorm -> int4 GEMV on interleaved gate/up rows -> SwiGLU, output M/2
(counterpart of programming_examples/decode_ffn_swiglu/matvec_int4_swiglu_rms.py).

One GPU kernel: every wave normalises the K-slice of x it feeds to the matrix cores, streams the
gate and up matrices and the reducer applies SwiGLU in its epilogue."""

import argparse
import sys

import numpy as np

from .. import awq, bf16
from ..backend import HIPRunner, HipModule
from . import _common
from ._common import draw_l1_weights


def build_module(M, K, GS=128, **ignored):
    if M % 2:
        raise ValueError("M counts interleaved gate/up rows and must be even")
    return HipModule("matvec_int4_swiglu_rms", K=K, N=M // 2, gs=GS)


def pack_inputs(A_q, A_s, A_z, M, K, GS, *ignored):
    """Interleaved kernel-side arrays (row 2i = gate[i], 2i + 1 = up[i]) -> (gate buffer, up buffer)."""
    gate, up = awq.deinterleave_rows(A_q, A_s, A_z)
    return awq.pack_buffer(*awq.awq_from_l1(*gate)), awq.pack_buffer(*awq.awq_from_l1(*up))


def parse_args(argv=None):
    p = argparse.ArgumentParser(prog="matvec_int4_swiglu_rms.py")
    p.add_argument("-v", "--verbose", action="store_true")
    p.add_argument("--m", type=int, default=16384)
    p.add_argument("--k", type=int, default=2048)
    p.add_argument("--gs", type=int, default=128)
    return _common.add_reference_cli(p).parse_args(argv)


def draw_inputs(args):
    np.random.seed(42)
    A_q, A_s, A_z = draw_l1_weights(args.m, args.k, args.gs)
    input_vec = bf16.bits_of(bf16.from_f32(np.random.randn(args.k)))
    norm_weight = bf16.bits_of(bf16.from_f32(np.random.randn(args.k) * 0.1 + 1.0))
    RMS_in = np.stack([input_vec, norm_weight], axis=0).view(bf16.BF16Array)
    return A_q, A_s, A_z, RMS_in


def run(args, cpu_reference):
    module = build_module(args.m, args.k, GS=args.gs)
    A_q, A_s, A_z, RMS_in = draw_inputs(args)
    D_ref = bf16.from_bits(cpu_reference(A_q, bf16.bits_of(A_s), A_z, bf16.bits_of(RMS_in)))
    gate_buf, up_buf = pack_inputs(A_q, A_s, A_z, args.m, args.k, args.gs)
    return HIPRunner(verbose=args.verbose).run_test(module, inputs=[gate_buf, up_buf, RMS_in], expected_outputs=[D_ref],
                                                    rtol=0.15, atol=0.5, min_correlation=0.99)


def main(argv=None):
    args = parse_args(argv)
    return _common.cli_main(args, build_module(args.m, args.k, GS=args.gs), run)


if __name__ == "__main__":
    sys.exit(main())
