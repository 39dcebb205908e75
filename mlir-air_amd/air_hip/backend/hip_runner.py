"""HIPRunner: the examples' test harness, with the reference's tolerance contract
(python/air/backend/xrt_runner.py:165-373 run_test, :394-523 _check_outputs):
np.isclose per element, a mismatch budget of int(total * pct / 100), an optional
Pearson-correlation gate, `PASS!` / `failed.` on stdout and 0 / -1 as the result."""

import numpy as np

from .. import bf16
from .hip import HIPBackend


class HIPRunner:
    def __init__(self, verbose=False, n_perf_iters=0, n_warmup_iters=0, perf_flops=None, report_precision=False,
                 **ignored_reference_kwargs):
        self.verbose = verbose
        self.n_perf_iters = n_perf_iters
        self.n_warmup_iters = n_warmup_iters
        self.perf_flops = perf_flops
        self.report_precision = report_precision
        self.last_latency_us = None

    def run_test(self, module, inputs, expected_outputs=(), rtol=1e-3, atol=1e-8, max_mismatch_percentage=0,
                 min_correlation=None):
        if self.verbose:
            print("Running module: ")
            print(module)
        if not expected_outputs:
            raise AssertionError("expected_outputs must not be empty")
        backend = HIPBackend(verbose=self.verbose, n_perf_iters=self.n_perf_iters, n_warmup_iters=self.n_warmup_iters)
        placeholders = [np.zeros(np.shape(o), np.uint16).view(bf16.BF16Array) if bf16.is_bf16(o)
                        else np.zeros(np.shape(o), np.asarray(o).dtype) for o in expected_outputs]
        invoker = backend.load(backend.compile(module))
        actual = invoker(*(list(inputs) + placeholders))
        self.last_latency_us = backend.last_latency_us
        if self.n_perf_iters > 0 and self.last_latency_us is not None:
            line = f"Latency (us): {self.last_latency_us:.1f}"
            if self.perf_flops is not None:
                line += f" | Throughput: {self.perf_flops / (self.last_latency_us * 1e-6) / 1e9:.6e} GFLOP/s"
            print(line)
        backend.unload()
        actual = list(actual[len(inputs):])
        ok = self._check_outputs(actual, list(expected_outputs), rtol, atol, max_mismatch_percentage, min_correlation)
        print("PASS!" if ok else "failed.")
        return 0 if ok else -1

    def _check_outputs(self, actual_outputs, expected_outputs, rtol=1e-3, atol=1e-8, max_mismatch_percentage=0,
                       min_correlation=None):
        assert len(actual_outputs) == len(expected_outputs), (
            f"Number of actual outputs ({len(actual_outputs)}) does not equal number of expected outputs "
            f"({len(expected_outputs)})")
        for i, (actual, expected) in enumerate(zip(actual_outputs, expected_outputs)):
            floating = bf16.is_bf16(expected) or np.asarray(expected).dtype in (np.float16, np.float32, np.float64)
            if bf16.is_bf16(expected):
                expected = bf16.to_f32(bf16.bits_of(expected)).astype(np.float64)
                actual = bf16.to_f32(bf16.bits_of(actual)).astype(np.float64)
            expected = np.asarray(expected)
            actual = np.reshape(np.asarray(actual), expected.shape)
            if floating:
                if self.report_precision:
                    abs_err = np.abs(actual - expected)
                    print(f"[precision] Output {i} ({abs_err.size} elements): "
                          f"mean_rel_L1={abs_err.mean() / (np.abs(expected).mean() + 1e-30):.3e} | "
                          f"abs_err max={abs_err.max():.3e} | rtol={rtol:.1e} atol={atol:.1e}")
                close = np.isclose(actual, expected, rtol=rtol, atol=atol)
                mismatches = int((~close).sum())
                total = expected.size
                max_ok = int(total * max_mismatch_percentage / 100)
                elementwise_ok = mismatches <= max_ok
                if not elementwise_ok:
                    print(f"ERROR: Output {i} does not meet expected output.")
                    print(f"Shape: {expected.shape}")
                    print(f"Mismatches: {mismatches} / {total} elements"
                          + (f" ({100 * mismatches / total:.2f}%)" if total else " (empty array)"))
                    idx = np.argwhere(~close)[:20]
                    for j in idx:
                        j = tuple(j)
                        print(f"  Index {j}: expected={expected[j]}, actual={actual[j]}, diff={abs(actual[j] - expected[j])}")
                corr_ok = True
                if min_correlation is not None and total > 0:
                    corr = float(np.corrcoef(actual.flatten(), expected.flatten())[0, 1])
                    print(f"Output {i} correlation: {corr:.6f} (threshold: {min_correlation})")
                    if not np.isfinite(corr) or corr < min_correlation:
                        corr_ok = False
                        print(f"ERROR: Output {i} correlation {corr:.6f} below threshold {min_correlation}")
                if not elementwise_ok or not corr_ok:
                    return False
            elif not np.array_equal(actual, expected):
                print(f"ERROR: Output {i} does not meet expected output.")
                return False
        return True
