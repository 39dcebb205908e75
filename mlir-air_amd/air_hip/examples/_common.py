import json
import sys

import numpy as np

from .. import bf16

# arguments that do not change the inputs an example draws or the result it expects
_NOT_PARAMS = ("verbose", "expected", "print_module_only", "compile_mode", "output_format")


def add_reference_cli(p):
    """The flags every reference example carries (matvec_int4_packed.py:294-316) plus --expected: this package holds no
    CPU implementation of its operators, so a stand-alone run takes the expected output from a file
    (tests/golden/make_expected.py writes it with the CPU oracle for the same arguments)."""
    p.add_argument("-p", "--print-module-only", action="store_true")
    p.add_argument("--output-format", type=str, choices=["xclbin", "elf"], default="elf", help="accepted and ignored")
    p.add_argument("--compile-mode", type=str, choices=["compile-and-run", "compile-only"], default="compile-and-run",
                   dest="compile_mode")
    p.add_argument("--expected", metavar="FILE.npz", default=None,
                   help="expected output bits and the arguments they were computed for")
    return p


def params_of(args):
    return {k: v for k, v in sorted(vars(args).items()) if k not in _NOT_PARAMS}


def save_expected(path, args, expected_bits):
    np.savez(path, expected=np.asarray(expected_bits, dtype=np.uint16), params=json.dumps(params_of(args)))


def cli_main(args, module, run):
    """The tail of a reference example's __main__ (matvec_int4_packed.py:318-385): print or compile the module, or run
    the test and return run_test's 0 / -1; 2 when no usable --expected file was given."""
    from ..backend import HIPBackend

    if args.print_module_only:
        print(module)
        return 0
    if args.compile_mode == "compile-only":
        backend = HIPBackend(verbose=args.verbose)
        backend.compile(module)
        backend.unload()
        return 0
    if not args.expected:
        print("error: --expected FILE.npz is required to check the result (write it with "
              "tests/golden/make_expected.py for the same arguments)", file=sys.stderr)
        return 2
    with np.load(args.expected) as f:
        expected, params = f["expected"], json.loads(str(f["params"]))
    if params != params_of(args):
        print(f"error: {args.expected} was computed for {params}, this run has {params_of(args)}", file=sys.stderr)
        return 2
    return run(args, lambda *inputs: expected)


def draw_l1_weights(rows, k, gs):
    """The examples' draw order after np.random.seed(...): nibbles, scales, zero points
    (matvec_int4_packed.py:345-350)."""
    q_unp = np.random.randint(0, 16, size=(rows, k), dtype=np.uint8)
    a_q = (q_unp[:, 0::2] | (q_unp[:, 1::2] << 4)).astype(np.uint8)
    n_groups = k // gs
    a_s = bf16.from_f32(np.random.uniform(0.005, 0.02, size=(n_groups, rows)))
    a_z = np.random.randint(7, 9, size=(n_groups, rows), dtype=np.uint8)
    return a_q, a_s, a_z
