"""Entry points shaped like the reference's programming examples: the same argument names,
seeds and draw order, `build_module` / `pack_inputs` per example, and `run(args, cpu_reference)`
which hands the expected output to HIPRunner.run_test.  The CPU reference is supplied by the
caller (the tests pass the oracle); nothing here computes on the CPU what the GPU should."""
