"""AWQ int4 -> bf16 dequant of a 1-D vector: out[i] = (q[i] - z[i // gs]) * s[i // gs]
(counterpart of programming_examples/dequant_awq/dequant_awq.py).

`pack_inputs` writes the reference's own tiled buffer ([herd_n, tile_bytes] uint8: per tile Q two elements per byte,
S bf16 per group, Z u8 per group, padded to 4 bytes); the GPU kernel reads that buffer as it is."""

import argparse
import sys

import numpy as np

from .. import awq, bf16
from . import _common
from ..backend import HIPBackend, HIPRunner, HipModule


def packed_tile_bytes(n_tile, group_size):
    return awq.packed_tile_bytes_1d(n_tile, group_size)


def build_module(n, group_size=128, herd_n=4, **ignored):
    if n % herd_n or (n // herd_n) % group_size:
        raise ValueError("N / herd_n must be divisible by group_size")
    return HipModule("dequant_awq_1d", K=n, N=herd_n, gs=group_size)


def pack_inputs(int4_vals, scales, zeros, n, group_size, herd_n=4):
    return awq.pack_inputs_1d(int4_vals, scales, zeros, n, group_size, herd_n)


def parse_args(argv=None):
    p = argparse.ArgumentParser(prog="dequant_awq.py", description="AWQ-style int4 to bf16 dequantization example")
    p.add_argument("-v", "--verbose", action="store_true")
    p.add_argument("--n", type=int, default=1024)
    p.add_argument("--group-size", type=int, default=128)
    p.add_argument("--herd-n", type=int, default=4, dest="herd_n")
    return _common.add_reference_cli(p).parse_args(argv)


def draw_inputs(args):
    np.random.seed(0)
    n_groups = args.n // args.group_size
    int4_vals = np.random.randint(0, 16, args.n).astype(np.uint8)
    scales = bf16.from_f32(np.random.uniform(0.01, 0.1, n_groups))
    zeros = np.random.randint(7, 10, n_groups).astype(np.uint8)
    return int4_vals, scales, zeros


def dequant(int4_vals, scales, zeros, group_size, herd_n=4):
    """Run the 1-D dequant on the GPU and return bf16 [n]."""
    n = len(int4_vals)
    backend = HIPBackend()
    invoker = backend.compile_and_load(build_module(n, group_size, herd_n))
    out = invoker(pack_inputs(int4_vals, scales, zeros, n, group_size, herd_n), np.zeros(n, np.uint16).view(bf16.BF16Array))[-1]
    backend.unload()
    return out


def run(args, cpu_reference):
    int4_vals, scales, zeros = draw_inputs(args)
    ref = bf16.from_bits(cpu_reference(int4_vals, bf16.bits_of(scales), zeros, args.group_size))
    got = dequant(int4_vals, scales, zeros, args.group_size, args.herd_n)
    ok = HIPRunner(verbose=args.verbose)._check_outputs([got], [ref], rtol=1e-1, atol=5e-2)
    print("PASS!" if ok else "failed.")
    return 0 if ok else -1


def main(argv=None):
    args = parse_args(argv)
    return _common.cli_main(args, build_module(args.n, args.group_size, args.herd_n), run)


if __name__ == "__main__":
    sys.exit(main())
