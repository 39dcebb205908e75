"""Decode block "O projection + FFN", all three weight matrices int4-AWQ
(counterpart of programming_examples/llms/llama32_1b_int4/multi_launch_builder/o_gemv_ffn_int4_multi.py):

  res1   = dequant(wo) @ attn_out + x_residual
  swiglu = silu(dequant(gate) @ rms_norm(res1)) * (dequant(up) @ rms_norm(res1))
  output = dequant(wdown) @ swiglu + res1

Three kernel launches behind one C-ABI call; res1 and swiglu stay on the device."""

import argparse
import sys

import numpy as np

from .. import awq, bf16
from . import _common
from ..backend import HIPRunner, HipModule


def build_module(emb_dim, hidden_dim, gs=128, **ignored):
    return HipModule("o_gemv_ffn_int4", K=emb_dim, N=hidden_dim, gs=gs)


def gen_int4_weights(M, K, gs, seed):
    """Kernel-side arrays of one matrix with the reference's generator and draw order
    (o_gemv_ffn_int4_multi.py:291-298): nibbles, scales U(0.005, 0.02), zero points in {7, 8}."""
    rng = np.random.default_rng(seed)
    q_unp = rng.integers(0, 16, size=(M, K), dtype=np.uint8)
    a_q = (q_unp[:, 0::2] | (q_unp[:, 1::2] << 4)).astype(np.uint8)
    a_s = bf16.from_f32(rng.uniform(0.005, 0.02, size=(K // gs, M)))
    a_z = rng.integers(7, 9, size=(K // gs, M), dtype=np.uint8)
    return a_q, a_s, a_z


def pack_inputs(A_q, A_s, A_z, *ignored):
    return awq.pack_buffer(*awq.awq_from_l1(A_q, A_s, A_z))


def parse_args(argv=None):
    p = argparse.ArgumentParser(prog="o_gemv_ffn_int4_multi.py")
    p.add_argument("-v", "--verbose", action="store_true")
    p.add_argument("--emb-dim", type=int, default=2048)
    p.add_argument("--hidden-dim", type=int, default=8192)
    p.add_argument("--gs", type=int, default=128)
    return _common.add_reference_cli(p).parse_args(argv)


def draw_inputs(args):
    """Weights from seeds 100 / 150 / 200, vectors from np.random.seed(42) in the reference's
    order (o_gemv_ffn_int4_multi.py:373-389).  Gate/up are drawn as one interleaved matrix."""
    emb, hidden = args.emb_dim, args.hidden_dim
    np.random.seed(42)
    wo = gen_int4_weights(emb, emb, args.gs, 100)
    gu = gen_int4_weights(2 * hidden, emb, args.gs, 150)
    wd = gen_int4_weights(emb, hidden, args.gs, 200)
    attn_out = bf16.from_f32(np.random.randn(emb))
    x_residual = bf16.from_f32(np.random.randn(emb))
    ffn_norm_w = bf16.from_f32(np.random.randn(emb) * 0.1 + 1.0)
    return wo, gu, wd, attn_out, x_residual, ffn_norm_w


def run(args, cpu_reference):
    """`cpu_reference(wo, gate, up, wd, attn_out, x_residual, ffn_norm_w)` takes kernel-side weight
    triples (scales as bf16 bits) and bf16 bit vectors and returns the expected output bits."""
    module = build_module(args.emb_dim, args.hidden_dim, gs=args.gs)
    wo, gu, wd, attn_out, x_residual, ffn_norm_w = draw_inputs(args)
    gate, up = awq.deinterleave_rows(*gu)
    bits = lambda t: (t[0], bf16.bits_of(t[1]), t[2])
    expected = bf16.from_bits(cpu_reference(bits(wo), bits(gate), bits(up), bits(wd), bf16.bits_of(attn_out),
                                            bf16.bits_of(x_residual), bf16.bits_of(ffn_norm_w)))
    inputs = [pack_inputs(*wo), attn_out, x_residual, ffn_norm_w, pack_inputs(*gate), pack_inputs(*up), pack_inputs(*wd)]
    return HIPRunner(verbose=args.verbose).run_test(module, inputs=inputs, expected_outputs=[expected],
                                                    rtol=0.2, atol=2.0, min_correlation=0.99)


def main(argv=None):
    args = parse_args(argv)
    return _common.cli_main(args, build_module(args.emb_dim, args.hidden_dim, gs=args.gs), run)


if __name__ == "__main__":
    sys.exit(main())
