"""Write the expected output of one example run with the CPU oracle:

    python tests/golden/make_expected.py matvec_int4_packed -o expected.npz -- --m 2048 --k 2048
    python -m air_hip.examples.matvec_int4_packed --m 2048 --k 2048 --expected expected.npz   (prints PASS!)

The examples under air_hip/examples draw their inputs from their arguments alone (the reference's seeds and draw
order), so the file holds the output bits and the arguments they belong to.  The reference's examples compute this
inside the script with their own cpu_reference; here the CPU restatements live in oracle/, which only tests may use.
"""
import argparse
import importlib
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
for p in (ROOT, os.path.join(ROOT, "mlir-air_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

from air_hip import awq, bf16  # noqa: E402
from air_hip.examples import _common  # noqa: E402
from oracle import awq as oawq, reference as oref  # noqa: E402
from oracle.bf16 import f32_to_bf16_bits  # noqa: E402

EXAMPLES = ("matvec_int4_packed", "matvec_int4_packed_add", "matmul_int4_packed", "matvec_int4_swiglu_rms",
            "o_gemv_ffn_int4", "dequant_awq")


def expected_bits(example, args):
    """The oracle's output (bf16 bits) for the inputs `example` draws from `args`."""
    ex = importlib.import_module(f"air_hip.examples.{example}")
    b = bf16.bits_of
    if example == "matvec_int4_packed":
        A_q, A_s, A_z, B = ex.draw_inputs(args)
        return oref.matvec_cpu_reference(A_q, b(A_s), A_z, b(B))
    if example == "matvec_int4_packed_add":
        A_q, A_s, A_z, B, R = ex.draw_inputs(args)
        return oref.matvec_add_cpu_reference(A_q, b(A_s), A_z, b(B), b(R))
    if example == "matmul_int4_packed":
        W_q, W_s, W_z, A = ex.draw_inputs(args)
        return oref.matmul_cpu_reference(W_q, b(W_s), W_z, b(A))
    if example == "matvec_int4_swiglu_rms":
        A_q, A_s, A_z, RMS_in = ex.draw_inputs(args)
        rms = b(RMS_in)
        return oref.swiglu_rms_cpu_reference(A_q, b(A_s), A_z, rms[0], rms[1])
    if example == "o_gemv_ffn_int4":
        wo, gu, wd, attn_out, x_residual, ffn_norm_w = ex.draw_inputs(args)
        gate, up = awq.deinterleave_rows(*gu)
        dq = lambda t: f32_to_bf16_bits(oref._dequant_l1_f64(t[0], b(t[1]), t[2], t[0].shape[1] * 2).astype(np.float32))
        return oref.o_gemv_ffn_int4_reference(dq(wo), b(attn_out), b(x_residual), b(ffn_norm_w), dq(gate), dq(up), dq(wd))
    if example == "dequant_awq":
        q, s, z = ex.draw_inputs(args)
        return oawq.dequant_1d(q, b(s), z, args.group_size)
    raise ValueError(f"unknown example {example}")


def write_expected(example, argv, path):
    ex = importlib.import_module(f"air_hip.examples.{example}")
    args = ex.parse_args(list(argv))
    _common.save_expected(path, args, expected_bits(example, args))
    return path


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("example", choices=EXAMPLES)
    ap.add_argument("-o", "--out", required=True)
    argv = sys.argv[1:]
    split = argv.index("--") if "--" in argv else len(argv)   # the example's own arguments follow "--"
    a = ap.parse_args(argv[:split])
    print(write_expected(a.example, argv[split + 1:], a.out))
