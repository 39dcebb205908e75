"""KernelCache and Profiler: the call boundary of the reference's LLM decode path on the GPU.

The reference's decode loop never talks to a backend directly; every device call is
`cache.load_and_run(name, backend_kwargs, *arrays, output_indices=..., static_input_indices=...,
intermediate_indices=..., bo_key=...)` (programming_examples/llms/shared/infra/cache.py:494-737)
on multi-launch ELFs compiled once by `compile_and_cache` (:447-492).  Decode:

  rms_qkv_int4_rope   13 args  (llama32_1b_int4/multi_launch_builder/rms_qkv_int4_rope_multi.py:4-30)
  o_gemv_ffn_int4     15 args  (llama32_1b_int4/multi_launch_builder/o_gemv_ffn_int4_multi.py:14-32)
  lm_head_gemv        1 + 2 P  (shared/builders/lm_head_gemv_multi.py:39-46; call site
                               llama32_1b_int4/llama32_1b_int4_inference.py:459-486)

and the int4 prompt pass (`_run_layer_int4`, llama32_1b_int4/llama32_1b_int4_prefill.py:241-364):

  rms_gemms_rope_int4 13 args  (multi_launch_builder/rms_gemms_rope_int4_multi.py:4-17)
  flash_attn           4 args  (q_roped, k_roped, v, out; causal grouped-query attention)
  o_ffn_int4          15 args  (multi_launch_builder/o_ffn_int4_multi.py:4-17)

This module keeps that interface - names, argument slots, which slots are static / intermediate /
read back, one result per argument with empty arrays for slots that are not read back - so that
`run_decode_block` (llama32_1b_int4/llama32_1b_int4_decode.py:176-313), `run_npu_decode_step` and
`_run_layer_int4` can be pointed at it unchanged.  The packed weight slots take the reference's
buffers (decode: uint8 [tiles, tile_bytes], `matvec_int4_packed.pack_inputs`; prefill: uint8
[N / tile_n, K / 128, tile_bytes], `awq_pack_for_npu`); on the first call of a `bo_key` they are
unpacked, re-packed on the GPU into the stream order the whole-K decode kernels and the tiled prompt-pass
GEMM read (`KernelCache(stream_order=False)`: left as AutoAWQ triples for the checkpoint-layout kernels)
and stay in HBM, the counterpart of the reference's write-once buffer objects.  "Compiling" validates a module description against the
kernels' shape rules; there is nothing to build at run time.

bf16 arrays are `air_hip.bf16.BF16Array` (uint16 bit patterns) or ml_dtypes bfloat16 arrays; results
come back in the dtype of the argument they replace, flat, like the reference's buffer views.
"""

import dataclasses
import json
import collections
import contextlib
import time
from pathlib import Path

import numpy as np

from . import awq, bf16
from .backend.abc import AirBackendError

KERNELS = ("rms_qkv_int4_rope", "o_gemv_ffn_int4", "lm_head_gemv", "rms_gemms_rope_int4", "flash_attn", "o_ffn_int4")


@dataclasses.dataclass(frozen=True)
class DecodeModule:
    """Description of one decode ELF (what the reference's build_*_module returns as MLIR)."""

    kernel: str
    emb_dim: int = 2048
    kv_dim: int = 512
    n_heads: int = 32
    n_kv_heads: int = 8
    head_dim: int = 64
    hidden_dim: int = 8192
    gs: int = 128
    m_tile: int = 8
    k_chunk: int = 2048
    n_cores: int = 8
    n_partitions: int = 8
    n_part: int = 16384
    eps: float = 1e-5
    seq_len: int = 1        # prefill modules: rows per call
    tile_n: int = 16        # prefill modules: output columns per packed weight tile
    tile_k: int = 128       # prefill modules: K chunk of a packed weight tile

    def __str__(self):
        return f"hip.decode_module @{self.kernel} {dataclasses.asdict(self)}"


def build_rms_qkv_int4_rope_module(emb_dim=2048, kv_dim=512, n_heads=32, n_kv_heads=8, head_dim=64, gs=128, m_tile=8,
                                   k_chunk=2048, n_cores=8, **ignored):
    """Same arguments and shape rules as build_rms_qkv_int4_rope_module
    (rms_qkv_int4_rope_multi.py:361-382): Q heads fill the embedding, one K chunk."""
    assert n_heads * head_dim == emb_dim
    assert n_kv_heads * head_dim == kv_dim
    assert k_chunk == emb_dim, "K_CHUNK must equal emb_dim for single-chunk GEMV"
    return DecodeModule("rms_qkv_int4_rope", emb_dim=emb_dim, kv_dim=kv_dim, n_heads=n_heads, n_kv_heads=n_kv_heads,
                        head_dim=head_dim, gs=gs, m_tile=m_tile, k_chunk=k_chunk, n_cores=n_cores)


def build_o_gemv_ffn_int4_module(emb_dim=2048, hidden_dim=8192, gs=128, m_tile=8, k_chunk=2048, n_cores=8):
    """Same arguments and shape rules as build_o_gemv_ffn_int4_module (o_gemv_ffn_int4_multi.py:110-123)."""
    assert emb_dim % k_chunk == 0 and hidden_dim % k_chunk == 0
    assert emb_dim == k_chunk, f"Stage 2 int4 swiglu_rms requires emb_dim ({emb_dim}) == k_chunk ({k_chunk})"
    return DecodeModule("o_gemv_ffn_int4", emb_dim=emb_dim, hidden_dim=hidden_dim, gs=gs, m_tile=m_tile,
                        k_chunk=k_chunk, n_cores=n_cores)


def build_lm_head_gemv_module(emb_dim=2048, n_partitions=8, n_part=16384, **ignored):
    """Same leading arguments as build_lm_head_gemv_module (shared/builders/lm_head_gemv_multi.py:39-46)."""
    return DecodeModule("lm_head_gemv", emb_dim=emb_dim, n_partitions=n_partitions, n_part=n_part)


def build_rms_gemms_rope_int4_module(seq_len=2048, emb_dim=2048, kv_dim=512, n_heads=32, n_kv_heads=8, head_dim=64,
                                     gs=128, tile_m=16, tile_n=16, tile_k_l1=128, **ignored):
    """Same leading arguments as build_rms_gemms_rope_int4_module (rms_gemms_rope_int4_multi.py:196-212)."""
    assert n_heads * head_dim == emb_dim
    assert n_kv_heads * head_dim == kv_dim
    return DecodeModule("rms_gemms_rope_int4", emb_dim=emb_dim, kv_dim=kv_dim, n_heads=n_heads, n_kv_heads=n_kv_heads,
                        head_dim=head_dim, gs=gs, seq_len=seq_len, tile_n=tile_n, tile_k=tile_k_l1)


def build_o_ffn_int4_module(seq_len=2048, emb_dim=2048, hidden_dim=8192, gs=128, tile_m=16, tile_n=16, tile_k_l1=128,
                            **ignored):
    """Same leading arguments as build_o_ffn_int4_module (o_ffn_int4_multi.py:290-298)."""
    return DecodeModule("o_ffn_int4", emb_dim=emb_dim, hidden_dim=hidden_dim, gs=gs, seq_len=seq_len, tile_n=tile_n,
                        tile_k=tile_k_l1)


def build_attn(lk=2048, lkp=64, lq=2048, lqp=256, dk=64, dv=64, num_q_tiles=4, num_cascade_stages=4, num_heads=32,
               num_kv_heads=8, causal=True, **ignored):
    """The flash attention module as the int4 prompt pass builds it (llama32_1b_int4_prefill.py:1219-1233): lq
    queries and lk keys of num_heads / num_kv_heads heads of dk.  Only the causal self-attention of that call
    site is provided: lq == lk, dk == dv, causal."""
    assert lq == lk and dk == dv and causal, "only causal self-attention (lq == lk, dk == dv) is provided"
    return DecodeModule("flash_attn", emb_dim=num_heads * dk, kv_dim=num_kv_heads * dk, n_heads=num_heads,
                        n_kv_heads=num_kv_heads, head_dim=dk, seq_len=lq)


class Profiler:
    """Timing log of the decode loop behind the method names the reference's drivers call
    (shared/infra/cache.py:70-306): record_compile / record_kernel / record_cpu / record_breakdown, start_layer /
    end_layer, time_cpu, report.  One table of samples keyed by (kind, name); a disabled profiler keeps nothing."""

    _BREAKDOWN_FIELDS = ("write_ms", "kernel_ms", "read_ms", "n_written", "bytes_written", "n_readback")

    def __init__(self, enabled=False):
        self.enabled = bool(enabled)
        self._samples = collections.defaultdict(list)   # (kind, name) -> values in recording order
        self.layer_times = []                            # (layer index, seconds)

    def _log(self, kind, name, value):
        if self.enabled:
            self._samples[(kind, name)].append(value)

    def _table(self, kind):
        return {name: vals for (k, name), vals in self._samples.items() if k == kind}

    compile_times = property(lambda self: {n: v[-1] for n, v in self._table("compile").items()})
    kernel_times = property(lambda self: self._table("kernel"))
    cpu_times = property(lambda self: self._table("cpu"))
    kernel_breakdowns = property(lambda self: self._table("breakdown"))

    def record_compile(self, name, duration):
        self._log("compile", name, duration)

    def record_kernel(self, name, duration):
        self._log("kernel", name, duration)

    def record_cpu(self, name, duration):
        self._log("cpu", name, duration)

    def record_breakdown(self, name, *fields):
        self._log("breakdown", name, dict(zip(self._BREAKDOWN_FIELDS, fields)))

    def start_layer(self):
        return time.perf_counter() if self.enabled else None

    def end_layer(self, layer_idx, t0):
        if t0 is not None and self.enabled:
            self.layer_times.append((layer_idx, time.perf_counter() - t0))

    @contextlib.contextmanager
    def time_cpu(self, name):
        """`with profiler.time_cpu("decode_attention_cpu"): ...` logs the block as a host operation."""
        t0 = time.perf_counter()
        try:
            yield self
        finally:
            self._log("cpu", name, time.perf_counter() - t0)

    def per_token_walls_ms(self, n_layers):
        """Wall time of each decoded token: its n_layers consecutive layer samples added up."""
        secs = [t for _, t in self.layer_times]
        if not self.enabled or not secs or len(secs) % n_layers:
            return []
        return [1e3 * sum(secs[i:i + n_layers]) for i in range(0, len(secs), n_layers)]

    def report(self):
        if not self.enabled:
            return
        mean = lambda xs: sum(xs) / len(xs)
        print("Kernel calls (host write + launch + read back):")
        for name, ts in sorted(self.kernel_times.items()):
            print(f"  {name:24s} n={len(ts):5d} avg={1e3 * mean(ts):8.3f} ms total={sum(ts):7.3f} s")
            parts = self.kernel_breakdowns.get(name)
            if parts:
                w, k, r = (mean([b[f] for b in parts]) for f in ("write_ms", "kernel_ms", "read_ms"))
                print(f"  {'':24s} write {w:.3f} ms, kernel {k:.3f} ms, read {r:.3f} ms")
        if self.cpu_times:
            print("Host operations:")
            for name, ts in sorted(self.cpu_times.items()):
                print(f"  {name:24s} n={len(ts):5d} avg={1e3 * mean(ts):8.3f} ms")


def _check_shared_alias(shared_alias, static_input_indices, n_args):
    """Refuse an alias map before anything touches the device (the reference does the same, cache.py:576-603): an
    aliased argument shares one process-wide buffer by pool name, so it cannot also be a per-bo_key static
    argument, must name an existing argument, and needs a usable pool name."""
    static = frozenset(static_input_indices or ())
    problems = []
    for idx, pool in shared_alias.items():
        if not (isinstance(idx, int) and 0 <= idx < n_args):
            problems.append(f"argument {idx!r} does not exist (the call has {n_args} arguments)")
        elif idx in static:
            problems.append(f"argument {idx} is static (kept per bo_key) and cannot join the process-wide pool {pool!r}")
        if not (isinstance(pool, str) and pool):
            problems.append(f"argument {idx!r} has no pool name (got {pool!r})")
    if problems:
        raise ValueError("shared_alias: " + "; ".join(problems))


class KernelCache:
    """Registers decode modules once and runs them with device-resident static arguments."""

    MANIFEST_FILE = "manifest.json"

    def __init__(self, cache_dir=None, verbose=False, profiler=None, stream_order=True):
        self.cache_dir = Path(cache_dir) if cache_dir is not None else None
        if self.cache_dir is not None:
            self.cache_dir.mkdir(parents=True, exist_ok=True)
        self.verbose = verbose
        self.profiler = profiler or Profiler()
        # static weight slots are kept in HBM in stream order (False: as AutoAWQ triples, for the checkpoint-layout kernels)
        self.stream_order = stream_order
        self.artifacts = {}      # name -> DecodeModule
        self._cached_bos = {}    # bo_key -> {arg index or derived name: device tensors}
        self._shared_bos = {}    # (alias, bytes) -> device tensor handed from a producer to a consumer

    def _log(self, msg):
        if self.verbose:
            print(f"  [KernelCache] {msg}")

    # -- registration ----------------------------------------------------------------
    def compile_and_cache(self, name, mlir_module, backend_kwargs=None, output_binary_name="air"):
        t0 = time.time()
        if not isinstance(mlir_module, DecodeModule):
            raise AirBackendError(f"compile_and_cache expects a DecodeModule, got {type(mlir_module).__name__}")
        m = mlir_module
        if m.kernel not in KERNELS:
            raise AirBackendError(f"unknown decode kernel '{m.kernel}' (known: {', '.join(KERNELS)})")
        if m.gs != awq.GROUP:
            raise AirBackendError(f"group size {m.gs} is not supported (only {awq.GROUP})")
        if m.emb_dim <= 0 or m.emb_dim % awq.GROUP:
            raise AirBackendError(f"emb_dim = {m.emb_dim} must be a positive multiple of {awq.GROUP}")
        if m.kernel == "o_gemv_ffn_int4" and (m.hidden_dim <= 0 or m.hidden_dim % awq.GROUP):
            raise AirBackendError(f"hidden_dim = {m.hidden_dim} must be a positive multiple of {awq.GROUP}")
        if m.kernel == "rms_qkv_int4_rope" and (m.head_dim % 16 or (m.emb_dim + 2 * m.kv_dim) % 32):
            raise AirBackendError("head_dim must be a multiple of 16 and emb_dim + 2 kv_dim a multiple of 32")
        if m.kernel in ("rms_gemms_rope_int4", "flash_attn"):
            g = m.n_heads // max(m.n_kv_heads, 1)
            if m.head_dim not in (64, 128) or m.n_heads % m.n_kv_heads or g not in (1, 2, 4, 8):
                raise AirBackendError("head_dim must be 64 or 128 and n_heads / n_kv_heads one of 1, 2, 4, 8")
        if m.kernel in ("rms_gemms_rope_int4", "o_ffn_int4", "flash_attn") and m.seq_len <= 0:
            raise AirBackendError(f"seq_len = {m.seq_len} must be positive")
        if m.kernel == "o_ffn_int4" and (m.hidden_dim <= 0 or m.hidden_dim % awq.GROUP or m.emb_dim > 8192):
            raise AirBackendError("hidden_dim must be a positive multiple of 128 and emb_dim at most 8192")
        self.artifacts[name] = m
        self.profiler.record_compile(name, time.time() - t0)
        self._log(f"registered {name}: {m}")

    def _save_manifest(self):
        if self.cache_dir is None:
            return
        data = {name: dataclasses.asdict(m) for name, m in self.artifacts.items()}
        (self.cache_dir / self.MANIFEST_FILE).write_text(json.dumps(data, indent=1))

    def load_manifest(self):
        """True if a manifest written by _save_manifest was found and loaded (the reference's --run-only path)."""
        if self.cache_dir is None or not (self.cache_dir / self.MANIFEST_FILE).exists():
            return False
        data = json.loads((self.cache_dir / self.MANIFEST_FILE).read_text())
        self.artifacts = {name: DecodeModule(**fields) for name, fields in data.items()}
        return True

    # -- execution -------------------------------------------------------------------
    def load_and_run(self, name, backend_kwargs, *inputs, output_indices=None, static_input_indices=None,
                     intermediate_indices=None, bo_key=None, shared_nonstatic=False, shared_alias=None):
        if name not in self.artifacts:
            raise RuntimeError(f"Kernel '{name}' not found in cache. Available: {list(self.artifacts.keys())}")
        if shared_alias:
            _check_shared_alias(shared_alias, static_input_indices, len(inputs))
        mod = self.artifacts[name]
        n_expected = {"rms_qkv_int4_rope": 13, "o_gemv_ffn_int4": 15, "lm_head_gemv": 1 + 2 * mod.n_partitions,
                      "rms_gemms_rope_int4": 13, "flash_attn": 4, "o_ffn_int4": 15}[mod.kernel]
        if len(inputs) != n_expected:
            raise AirBackendError(f"{name} takes {n_expected} arguments, got {len(inputs)}")

        import torch

        from . import _lib, ops

        try:
            _lib.load_library()
        except _lib.LibraryNotBuiltError as e:
            raise AirBackendError(str(e))
        if not torch.cuda.is_available():
            raise AirBackendError("no GPU visible: the HIP backend has no CPU fallback")

        key = bo_key if bo_key is not None else name
        first_call = key not in self._cached_bos
        slots = self._cached_bos.setdefault(key, {})
        static = set(static_input_indices or [])
        intermediate = set(intermediate_indices or [])
        alias = shared_alias or {}
        readback = {len(inputs) - 1} if output_indices is None else set(output_indices)
        stats = {"n": 0, "bytes": 0}

        def resident(i):
            """Slot i keeps what an earlier call wrote: static and intermediate slots after the first call."""
            return not first_call and (i in static or i in intermediate)

        def vec(i, shape):
            """bf16 argument i on the device; an aliased intermediate slot takes the producer's tensor."""
            a = inputs[i]
            nbytes = int(np.asarray(a).size) * 2
            if i in alias and i in intermediate and (alias[i], nbytes) in self._shared_bos:
                return self._shared_bos[(alias[i], nbytes)].reshape(shape)
            if resident(i) and i in slots:
                return slots[i]
            t = torch.from_numpy(bf16.bits_of(a).view(np.int16).reshape(shape)).cuda().view(torch.bfloat16)
            stats["n"] += 1
            stats["bytes"] += nbytes
            if i in static:
                slots[i] = t
            return t

        def linear(i, M, K):
            """Packed decode buffer i -> kernel-side arrays (A_q [M, K/2], A_s, A_z [K/gs, M])."""
            stats["n"] += 1
            stats["bytes"] += int(np.asarray(inputs[i]).size)
            return awq.unpack_bo_tiles(np.asarray(inputs[i]).view(np.uint8), M, K, mod.gs, mod.m_tile,
                                       min(mod.k_chunk, K), mod.n_cores, M)

        def gemm_linear(i, K, N):
            """Packed prefill buffer i -> kernel-side arrays (W_q [N, K/2], W_s, W_z [K/gs, N])."""
            stats["n"] += 1
            stats["bytes"] += int(np.asarray(inputs[i]).size)
            return awq.unpack_gemm_tiles(np.asarray(inputs[i]).view(np.uint8), K, N, mod.gs, mod.tile_n, mod.tile_k)

        # One layout for every matrix of a call: stream order where the call's kernels take all of them (decode:
        # input lengths in whole groups; prompt pass: whole pairs of groups and 64-column tiles).
        E, H, n_qkv = mod.emb_dim, mod.hidden_dim, mod.emb_dim + 2 * mod.kv_dim
        stream_order = self.stream_order and mod.gs == awq.GROUP and {
            "rms_qkv_int4_rope": E % 128 == 0 and n_qkv % 16 == 0,
            "o_gemv_ffn_int4": E % 128 == 0 and H % 128 == 0,
            "rms_gemms_rope_int4": E % 256 == 0 and n_qkv % 64 == 0,
            "o_ffn_int4": E % 256 == 0 and H % 256 == 0,
        }.get(mod.kernel, False)

        def to_awq_dev(l1):
            """Kernel-side arrays -> the matrix in HBM: in stream order (ops.StreamWeight, the layout the fast
            kernels read) where the call takes it, else the AutoAWQ triple for the checkpoint-layout kernels."""
            qw, qz, sc = awq.awq_from_l1(*l1)
            dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
            triple = dev(qw), dev(qz), dev(bf16.bits_of(sc).view(np.int16)).view(torch.bfloat16)
            return ops.repack_stream(*triple, group=mod.gs) if stream_order else triple

        def weights(tag, indices, build):
            """Device weights derived from packed slots `indices`; kept while all of them are resident."""
            if tag in slots and all(resident(i) for i in indices):
                return slots[tag]
            w = build()
            if all(i in static for i in indices):
                slots[tag] = w
            return w

        t0 = time.time()
        t_write = time.perf_counter()
        try:
            if mod.kernel == "rms_qkv_int4_rope":
                run, outputs = self._stage_rms_qkv(mod, vec, linear, to_awq_dev, weights)
            elif mod.kernel == "o_gemv_ffn_int4":
                run, outputs = self._stage_o_gemv_ffn(mod, vec, linear, to_awq_dev, weights)
            elif mod.kernel == "rms_gemms_rope_int4":
                run, outputs = self._stage_rms_gemms_rope(mod, vec, gemm_linear, to_awq_dev, weights)
            elif mod.kernel == "flash_attn":
                run, outputs = self._stage_flash_attn(mod, vec)
            elif mod.kernel == "o_ffn_int4":
                run, outputs = self._stage_o_ffn(mod, vec, gemm_linear, to_awq_dev, weights)
            else:
                run, outputs = self._stage_lm_head(mod, vec, slots, static, resident, inputs, stats)
            torch.cuda.synchronize()
            t_write_ms = (time.perf_counter() - t_write) * 1e3
            t_kernel = time.perf_counter()
            produced = run(readback)
            ops.check_health()   # synchronises; a reducer that timed out surfaces here
            t_kernel_ms = (time.perf_counter() - t_kernel) * 1e3
        except _lib.W4A16Error as e:
            raise AirBackendError(str(e))
        unknown = sorted(readback - set(outputs))
        if unknown:
            raise AirBackendError(f"{name}: argument slots {unknown} are not outputs of this kernel (outputs: {sorted(outputs)})")

        t_read = time.perf_counter()
        results = []
        for i, a in enumerate(inputs):
            a = np.asarray(a) if not isinstance(a, np.ndarray) else a
            if i not in readback:
                results.append(np.empty(0, dtype=a.dtype))
                continue
            t = produced[i].contiguous()
            if i in alias:
                self._shared_bos[(alias[i], t.numel() * 2)] = t
            host = t.view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1)
            results.append(host.view(bf16.BF16Array) if isinstance(a, bf16.BF16Array) or a.dtype.itemsize != 2
                           else host.view(a.dtype))
        t_read_ms = (time.perf_counter() - t_read) * 1e3
        self.profiler.record_kernel(name, time.time() - t0)
        self.profiler.record_breakdown(name, t_write_ms, t_kernel_ms, t_read_ms, stats["n"], stats["bytes"], len(readback))
        return tuple(results)

    # Each _stage_* uploads what the call needs and returns (run, output slots); run(readback) launches the
    # kernels and returns {slot: device tensor} for the slots asked for.
    @staticmethod
    def _stage_rms_qkv(mod, vec, linear, to_awq_dev, weights):
        from . import ops

        E, KV, nh, nkv, hd = mod.emb_dim, mod.kv_dim, mod.n_heads, mod.n_kv_heads, mod.head_dim
        x = vec(0, (E,))
        norm_w = vec(1, (E,))

        def fused():   # Q | K | V along the output axis: one GEMV instead of three
            parts = [linear(3, E, E), linear(5, KV, E), linear(7, KV, E)]
            a_q = np.concatenate([p[0] for p in parts], axis=0)
            a_s = np.concatenate([bf16.bits_of(p[1]) for p in parts], axis=1)
            a_z = np.concatenate([p[2] for p in parts], axis=1)
            return to_awq_dev((a_q, bf16.from_bits(a_s), a_z))

        wqkv = weights("wqkv", (3, 5, 7), fused)
        lut_q = vec(9, (nh, hd))
        lut_k = vec(10, (nkv, hd))

        def run(readback):
            if isinstance(wqkv, ops.StreamWeight):
                qkv = ops.w4a16_rms_gemv_stream(x, norm_w, wqkv, eps=mod.eps, group=mod.gs)
            else:
                qkv = ops.w4a16_rms_gemv(x, norm_w, *wqkv, eps=mod.eps)
            q, k, v = qkv[:E], qkv[E:E + KV], qkv[E + KV:]
            out = {4: q, 6: k, 8: v}
            if 11 in readback:
                out[11] = ops.rope_halfsplit(q.reshape(nh, hd), lut_q)
            if 12 in readback:
                out[12] = ops.rope_halfsplit(k.reshape(nkv, hd), lut_k)
            if 2 in readback:
                out[2] = ops.rms_norm_rows(x.reshape(1, E), norm_w, eps=mod.eps)
            return out

        return run, (2, 4, 6, 8, 11, 12)

    @staticmethod
    def _stage_o_gemv_ffn(mod, vec, linear, to_awq_dev, weights):
        import torch

        from . import ops

        E, H = mod.emb_dim, mod.hidden_dim
        attn_out = vec(1, (E,))
        x_residual = vec(3, (E,))
        rms_buf = vec(6, (2, E))   # row 0: res1 (written by stage 1), row 1: ffn_norm_w
        wo = weights("wo", (0,), lambda: to_awq_dev(linear(0, E, E)))

        def gate_up():             # rows 2i = gate[i], 2i + 1 = up[i] (llama32_1b_int4_weights.py:173-207)
            gate, up = awq.deinterleave_rows(*linear(7, 2 * H, E))
            return to_awq_dev(gate), to_awq_dev(up)

        wg, wu = weights("wgateup", (7,), gate_up)
        wd = weights("wdown", (12,), lambda: to_awq_dev(linear(12, E, H)))

        def run(readback):
            block = ops.o_gemv_ffn_stream if all(isinstance(w, ops.StreamWeight) for w in (wo, wg, wu, wd)) else ops.o_gemv_ffn
            y, res1, h = block(attn_out, x_residual, rms_buf[1].contiguous(), wo, wg, wu, wd, eps=mod.eps,
                               return_intermediates=True)
            out = {14: y, 11: h}
            if 6 in readback:
                out[6] = torch.stack([res1, rms_buf[1]])
            return out

        return run, (6, 11, 14)

    @staticmethod
    def _stage_rms_gemms_rope(mod, vec, gemm_linear, to_awq_dev, weights):
        import torch

        from . import ops

        M, E, KV, nh, nkv, hd = mod.seq_len, mod.emb_dim, mod.kv_dim, mod.n_heads, mod.n_kv_heads, mod.head_dim
        x = vec(0, (M, E))
        norm_w = vec(1, (E,))

        def fused():
            parts = [gemm_linear(3, E, E), gemm_linear(5, E, KV), gemm_linear(7, E, KV)]
            a_q = np.concatenate([p[0] for p in parts], axis=0)
            a_s = np.concatenate([bf16.bits_of(p[1]) for p in parts], axis=1)
            a_z = np.concatenate([p[2] for p in parts], axis=1)
            return to_awq_dev((a_q, bf16.from_bits(a_s), a_z))

        wqkv = weights("wqkv", (3, 5, 7), fused)
        # slot 9 repeats LUT row m for every Q head of token m ([M, n_heads, head_dim]); the kernel reads the table itself
        lut = vec(9, (M, nh, hd))[:, 0].contiguous()

        def run(readback):
            stream = isinstance(wqkv, ops.StreamWeight)
            rms_qkv_rope = ops.prefill_rms_qkv_rope_stream if stream else ops.prefill_rms_qkv_rope
            qkv = rms_qkv_rope(x, norm_w, wqkv, lut, 0, nh, nkv, hd, eps=mod.eps)
            out = {11: qkv[:, :E], 12: qkv[:, E:E + KV], 8: qkv[:, E + KV:]}
            if readback & {2, 4, 6}:   # the unrotated projections and the normalised input, for diagnosis
                normed = ops.rms_norm_rows(x, norm_w, eps=mod.eps)
                plain = ops.w4a16_gemm_stream(normed, wqkv) if stream else ops.w4a16_gemm(normed, *wqkv)
                out.update({2: normed, 4: plain[:, :E], 6: plain[:, E:E + KV]})
            return out

        return run, (2, 4, 6, 8, 11, 12)

    @staticmethod
    def _stage_flash_attn(mod, vec):
        import torch

        from . import ops

        M, E, KV = mod.seq_len, mod.emb_dim, mod.kv_dim
        q, k, v = vec(0, (M, E)), vec(1, (M, KV)), vec(2, (M, KV))

        def run(readback):
            return {3: ops.prefill_attention(torch.cat([q, k, v], dim=1).contiguous(), mod.n_heads, mod.n_kv_heads, mod.head_dim)}

        return run, (3,)

    @staticmethod
    def _stage_o_ffn(mod, vec, gemm_linear, to_awq_dev, weights):
        from . import ops

        M, E, H = mod.seq_len, mod.emb_dim, mod.hidden_dim
        attn_out = vec(0, (M, E))
        x_residual = vec(3, (M, E))
        norm_w = vec(5, (E,))
        wo = weights("wo", (1,), lambda: to_awq_dev(gemm_linear(1, E, E)))
        wg = weights("wgate", (7,), lambda: to_awq_dev(gemm_linear(7, E, H)))
        wu = weights("wup", (9,), lambda: to_awq_dev(gemm_linear(9, E, H)))
        wd = weights("wdown", (12,), lambda: to_awq_dev(gemm_linear(12, H, E)))

        def run(readback):
            stream = all(isinstance(w, ops.StreamWeight) for w in (wo, wg, wu, wd))
            o_ffn = ops.prefill_o_ffn_stream if stream else ops.prefill_o_ffn
            y, res1, h = o_ffn(attn_out, x_residual, norm_w, wo, wg, wu, wd, eps=mod.eps, return_intermediates=True)
            return {14: y, 4: res1, 11: h}

        return run, (4, 11, 14)

    @staticmethod
    def _stage_lm_head(mod, vec, slots, static, resident, inputs, stats):
        import torch

        from . import ops

        E = mod.emb_dim
        x = vec(0, (E,))
        parts = []
        for p in range(mod.n_partitions):
            i = 1 + 2 * p
            if resident(i) and i in slots:
                parts.append(slots[i])
                continue
            w = torch.from_numpy(bf16.bits_of(inputs[i]).view(np.int16).reshape(mod.n_part, E)).cuda().view(torch.bfloat16)
            stats["n"] += 1
            stats["bytes"] += w.numel() * 2
            if i in static:
                slots[i] = w
            parts.append(w)

        def run(readback):
            return {2 + 2 * p: ops.lm_head(x, parts[p], norm_weight=None, return_argmax=False)
                    for p in range(mod.n_partitions) if 2 + 2 * p in readback}

        return run, tuple(2 + 2 * p for p in range(mod.n_partitions))
