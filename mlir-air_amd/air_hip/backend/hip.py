"""HIPBackend: runs a W4A16 module on the MI355X through the C ABI.

Where the reference compiles AIR MLIR with aircc and drives the NPU through XRT
(python/air/backend/xrt.py:345-611, 676-900), a "module" here is a small
description of one operator instance (`HipModule`): the kernels are prebuilt, so
`compile` only validates the description against the kernels' shape rules.

The invoker keeps the reference's calling convention (xrt.py:742-791): it takes
the input arrays followed by output placeholders, copies every array to the
device, runs, and returns a tuple with one array per argument (inputs unchanged,
outputs filled).  bf16 data travels as 16-bit patterns (`air_hip.bf16`).
"""

import dataclasses
import time

import numpy as np

from .. import awq, bf16
from .abc import AirBackend, AirBackendError

OPS = ("dequant_awq", "dequant_awq_1d", "matvec_int4", "matvec_int4_add", "matmul_int4", "matvec_int4_swiglu",
       "matvec_int4_swiglu_rms", "ffn_swiglu_int4", "o_gemv_ffn_int4")
# ops whose N is a hidden size that is also the K of a following projection
_HIDDEN_OPS = ("ffn_swiglu_int4", "o_gemv_ffn_int4")


@dataclasses.dataclass(frozen=True)
class HipModule:
    """One operator instance.  M is the number of activation rows (1 for the GEMVs);
    K is the contraction size, N the number of output features (the examples' `m`)."""

    op: str
    K: int
    N: int
    M: int = 1
    gs: int = 128
    eps: float = 1e-5

    def __str__(self):
        return f"hip.module @{self.op} {{M = {self.M}, K = {self.K}, N = {self.N}, gs = {self.gs}}}"


class HIPBackend(AirBackend):
    """One loaded module per backend object, like XRTBackend (xrt.py:365-368, 700-703)."""

    def __init__(self, verbose=False, n_perf_iters=0, n_warmup_iters=0, **ignored_reference_kwargs):
        self.verbose = verbose
        self.n_perf_iters = n_perf_iters
        self.n_warmup_iters = n_warmup_iters
        self.last_latency_us = None
        self._loaded = None

    # -- compile ---------------------------------------------------------------------
    def compile(self, module):
        if self._loaded is not None:
            raise AirBackendError("Cannot compile while a module is loaded: call unload() first")
        if not isinstance(module, HipModule):
            raise AirBackendError(f"HIPBackend.compile expects a HipModule, got {type(module).__name__}")
        if module.op not in OPS:
            raise AirBackendError(f"unknown op '{module.op}' (known: {', '.join(OPS)})")
        if module.op == "dequant_awq_1d":   # K = n elements, N = herd_n tiles, any even group size that divides a tile
            if module.K <= 0 or module.N <= 0 or module.gs <= 0 or module.gs % 8 or module.K % module.N or (module.K // module.N) % module.gs:
                raise AirBackendError(f"dequant_awq_1d: n = {module.K} must split into {module.N} tiles of whole groups of {module.gs} (a multiple of 8)")
            return module
        if module.gs != awq.GROUP:
            raise AirBackendError(f"group size {module.gs} is not supported (only {awq.GROUP})")
        if module.K <= 0 or module.K % awq.GROUP:
            raise AirBackendError(f"K = {module.K} must be a positive multiple of {awq.GROUP}")
        n_mult = 8 if module.op == "dequant_awq" else 32
        if module.N <= 0 or module.N % n_mult:
            raise AirBackendError(f"N = {module.N} must be a positive multiple of {n_mult}")
        if module.op in _HIDDEN_OPS and module.N % awq.GROUP:
            raise AirBackendError(f"hidden size {module.N} must be a multiple of {awq.GROUP}")
        if module.M <= 0:
            raise AirBackendError(f"M = {module.M} must be positive")
        return module

    # -- load ------------------------------------------------------------------------
    def load(self, artifact):
        if self._loaded is not None:
            raise AirBackendError("A module is already loaded: call unload() first")
        if not isinstance(artifact, HipModule):
            raise AirBackendError("load() expects the artifact returned by compile()")
        import torch

        from .. import _lib, ops

        try:
            _lib.load_library()
        except _lib.LibraryNotBuiltError as e:
            raise AirBackendError(str(e))
        if not torch.cuda.is_available():
            raise AirBackendError("no GPU visible: the HIP backend has no CPU fallback")
        self._loaded = artifact
        mod = artifact

        def to_dev(a):
            a = np.ascontiguousarray(a)
            if bf16.is_bf16(a) or a.dtype == np.uint16:
                return torch.from_numpy(bf16.bits_of(a).view(np.int16)).cuda().view(torch.bfloat16)
            return torch.from_numpy(a).cuda()

        def weights(buf, K, N):
            """The packed weight buffer of one matrix on the device: the dequant op reads the AutoAWQ tensors, every
            product reads the stream-order re-pack (made here, where the reference writes the buffer into its BO:
            staging, outside the timed iterations)."""
            qw, qz, s = awq.unpack_buffer(buf, K, N, mod.gs)
            triple = to_dev(qw), to_dev(qz), to_dev(s)
            return triple if mod.op == "dequant_awq" else ops.repack_stream(*triple, group=mod.gs)

        def run(dev_in):
            if mod.op == "dequant_awq":
                return [ops.awq_dequant(*dev_in[0])]
            if mod.op == "dequant_awq_1d":
                return [ops.awq_dequant_1d(dev_in[0], mod.K, mod.gs, mod.N)]
            if mod.op == "matvec_int4":
                return [ops.w4a16_gemv_stream(dev_in[1], dev_in[0])]
            if mod.op == "matvec_int4_add":
                return [ops.w4a16_gemv_stream(dev_in[1], dev_in[0], residual=dev_in[2])]
            if mod.op == "matmul_int4":
                return [ops.w4a16_gemm_stream(dev_in[0], dev_in[1])]
            if mod.op == "matvec_int4_swiglu":
                return [ops.w4a16_swiglu_stream(dev_in[2], dev_in[0], dev_in[1])]
            if mod.op == "matvec_int4_swiglu_rms":
                return [ops.w4a16_rms_swiglu_stream(dev_in[2][0], dev_in[2][1], dev_in[0], dev_in[1], eps=mod.eps)]
            if mod.op == "ffn_swiglu_int4":
                return [ops.ffn_swiglu_stream(dev_in[3], dev_in[0], dev_in[1], dev_in[2])]
            if mod.op == "o_gemv_ffn_int4":
                wo, attn_out, x_res, norm_w, gate, up, down = dev_in
                return [ops.o_gemv_ffn_stream(attn_out, x_res, norm_w, wo, gate, up, down, eps=mod.eps)]
            raise AirBackendError(f"unknown op {mod.op}")

        def invoker(*args):
            n_out = 1
            inputs, placeholders = list(args[:-n_out]), list(args[-n_out:])
            dev_in = self._stage_inputs(mod, inputs, to_dev, weights)
            try:
                for _ in range(self.n_warmup_iters):
                    run(dev_in)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                iters = max(self.n_perf_iters, 1)
                for _ in range(iters):
                    outs = run(dev_in)
                torch.cuda.synchronize()   # (the stream-order launches keep no state that could time out)
                if self.n_perf_iters > 0:
                    self.last_latency_us = (time.perf_counter() - t0) / iters * 1e6
            except _lib.W4A16Error as e:
                raise AirBackendError(str(e))
            results = list(inputs)
            for o, ph in zip(outs, placeholders):
                host = o.contiguous().view(torch.int16).cpu().numpy().view(np.uint16).view(bf16.BF16Array)
                results.append(host.reshape(np.shape(ph)))
            return tuple(results)

        return invoker

    @staticmethod
    def _stage_inputs(mod, inputs, to_dev, weights):
        def need(n):
            if len(inputs) != n:
                raise AirBackendError(f"{mod.op} takes {n} input array(s) plus one output placeholder, got {len(inputs)}")

        K, N = mod.K, mod.N
        if mod.op == "dequant_awq":
            need(1)
            return [weights(inputs[0], K, N)]
        if mod.op == "dequant_awq_1d":
            need(1)
            tile_bytes = awq.packed_tile_bytes_1d(K // N, mod.gs)[3]
            buf = np.ascontiguousarray(inputs[0], dtype=np.uint8)
            if buf.size != N * tile_bytes:
                raise AirBackendError(f"dequant_awq_1d: packed buffer has {buf.size} bytes, expected {N} tiles of {tile_bytes}")
            return [to_dev(buf.reshape(-1))]
        if mod.op == "matvec_int4":
            need(2)
            return [weights(inputs[0], K, N), to_dev(bf16.bits_of(inputs[1]).reshape(K))]
        if mod.op == "matvec_int4_add":
            need(3)
            return [weights(inputs[0], K, N), to_dev(bf16.bits_of(inputs[1]).reshape(K)),
                    to_dev(bf16.bits_of(inputs[2]).reshape(N))]
        if mod.op == "matmul_int4":
            need(2)
            return [to_dev(bf16.bits_of(inputs[0]).reshape(mod.M, K)), weights(inputs[1], K, N)]
        if mod.op == "matvec_int4_swiglu":
            need(3)
            return [weights(inputs[0], K, N), weights(inputs[1], K, N), to_dev(bf16.bits_of(inputs[2]).reshape(K))]
        if mod.op == "matvec_int4_swiglu_rms":
            need(3)   # gate buffer, up buffer, RMS_in [2, K]: row 0 = x, row 1 = norm weight
            return [weights(inputs[0], K, N), weights(inputs[1], K, N), to_dev(bf16.bits_of(inputs[2]).reshape(2, K))]
        if mod.op == "o_gemv_ffn_int4":
            need(7)   # wo buffer, attn_out, x_residual, ffn_norm_w, gate, up, down buffers; K = emb, N = hidden
            return [weights(inputs[0], K, K), to_dev(bf16.bits_of(inputs[1]).reshape(K)),
                    to_dev(bf16.bits_of(inputs[2]).reshape(K)), to_dev(bf16.bits_of(inputs[3]).reshape(K)),
                    weights(inputs[4], K, N), weights(inputs[5], K, N), weights(inputs[6], N, K)]
        if mod.op == "ffn_swiglu_int4":
            need(4)
            return [weights(inputs[0], K, N), weights(inputs[1], K, N), weights(inputs[2], N, K),
                    to_dev(bf16.bits_of(inputs[3]).reshape(K))]
        raise AirBackendError(f"unknown op {mod.op}")

    def compile_and_load(self, module):
        return self.load(self.compile(module))

    def unload(self):
        self._loaded = None
