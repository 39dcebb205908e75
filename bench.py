#!/usr/bin/env python3
"""Benchmark of the MI355X W4A16 path.  One JSON line on stdout.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload gemv|probe|gemv_awq|dequant|gemm16|gemm64|gemm64_down|gemm16_awq|prefill|prefill_awq|ffn|ffn_awq|block|block_awq|layer|layer_awq|q4nx_gemv|q4nx_gemm16|q4nx_prefill|lm_head|decode_1b|decode_8b|prefill_block|prefill_block_awq|prefill_1b|prefill_1b_awq|prefill_8b]

Default workload is the decode GEMV (x bf16 [1,4096], W int4 [4096 x 11008], group 128).
A step is one launch of the hot path on synthetic inputs that are already resident in HBM.
To measure HBM rather than the 256 MB Infinity Cache, the steps rotate over enough
independent copies of the weights to exceed it ("cold"); the same-buffer ("hot") rate is
reported beside it.  The timed region is exactly K launches on one stream, bracketed by HIP
events on that stream and by device synchronisation; the launches are queued while a spinning
kernel keeps the GPU busy, so the interval holds the launches and not the host's launch latency.
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "mlir-air_amd"))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
MALL_BYTES = 256 << 20

CONFIGS = {
    # name: (M, K, N, bound, description)
    "dequant": dict(M=0, K=4096, N=4096, cfg=0, desc="AWQ dequant K=4096 N=4096 -> bf16"),
    # the weights re-packed once at load time (untimed, as the reference re-packs them) into stream order
    "gemv": dict(M=1, K=4096, N=11008, cfg=1, desc="decode GEMV W4A16 M=1 K=4096 N=11008 g128, stream-order weights"),
    # read-only pass over the same stream-order arena with the GEMV's launch shape and request pattern (no x, no
    # arithmetic): the floor of any kernel that reads the matrix once; priced with config 1's algorithmic bytes
    "probe": dict(M=1, K=4096, N=11008, cfg=None, desc="read-only probe of the stream-order matrix of config 1 (K=4096 N=11008), GEMV launch shape"),
    # the same product on the AutoAWQ checkpoint layout (split-K kernel with a workspace)
    "gemv_awq": dict(M=1, K=4096, N=11008, cfg=None, desc="decode GEMV W4A16 M=1 K=4096 N=11008 g128, checkpoint-layout weights"),
    "gemm16": dict(M=16, K=4096, N=14336, cfg=2, desc="batched decode GEMM W4A16 M=16 K=4096 N=14336 g128, stream-order weights"),
    # the same product for a batch of 64 (split along K, a launch of four row tiles plus the launch that adds the slices;
    # no BASELINE config)
    "gemm64": dict(M=64, K=4096, N=14336, cfg=None, desc="batched decode GEMM W4A16 M=64 K=4096 N=14336 g128, stream-order weights"),
    "gemm64_down": dict(M=64, K=14336, N=4096, cfg=None, desc="batched decode GEMM W4A16 M=64 K=14336 N=4096 g128 (down projection), stream-order weights, split along K"),
    "gemm16_awq": dict(M=16, K=4096, N=14336, cfg=None, desc="batched decode GEMM W4A16 M=16 K=4096 N=14336 g128, checkpoint-layout weights"),
    "prefill": dict(M=2048, K=4096, N=14336, cfg=3, desc="prefill GEMM W4A16 M=2048 K=4096 N=14336 g128, stream-order weights"),
    "prefill_awq": dict(M=2048, K=4096, N=14336, cfg=None, desc="prefill GEMM W4A16 M=2048 K=4096 N=14336 g128, checkpoint-layout weights"),
    "ffn": dict(M=1, K=4096, N=14336, cfg=4, desc="decode SwiGLU FFN W4A16 K=4096 H=14336 g128, stream-order weights (2 launches)"),
    "ffn_awq": dict(M=1, K=4096, N=14336, cfg=None, desc="decode SwiGLU FFN W4A16 K=4096 H=14336 g128, checkpoint-layout weights (two split-K launches)"),
    "block_awq": dict(M=1, K=4096, N=14336, cfg=None, desc="decode block, checkpoint-layout weights"),
    "layer_awq": dict(M=1, K=4096, N=14336, cfg=None, desc="decode layer, checkpoint-layout weights"),
    # beyond the five headline configs: the O projection + RMSNorm + FFN decode block with residuals (3 launches)
    "block": dict(M=1, K=4096, N=14336, cfg=None, desc="decode block O-proj + RMSNorm + SwiGLU FFN W4A16 E=4096 H=14336 g128"),
    # one whole decode layer: RMSNorm + fused QKV GEMV, then RoPE + KV append + GQA attention over 2048 cached
    # positions (32 heads, 8 KV heads, head_dim 128) and the block above as one call
    "layer": dict(M=1, K=4096, N=14336, cfg=None, desc="decode layer W4A16 E=4096 H=14336 32/8 heads hd=128 pos=2047 g128"),
    # the Q4NX codec (w = q * s + m, 32-column groups) through the same streaming kernel: the gate / up
    # projection shape of Llama-3.1-8B (programming_examples/llms/llama31_8b_q4nx)
    "q4nx_gemv": dict(M=1, K=4096, N=14336, cfg=None, desc="decode GEMV Q4NX M=1 K=4096 N=14336 g32, weights in Q4NX stream order"),
    "q4nx_gemm16": dict(M=16, K=4096, N=14336, cfg=None, desc="batched decode GEMM Q4NX M=16 K=4096 N=14336 g32, weights in Q4NX stream order"),
    "q4nx_prefill": dict(M=2048, K=4096, N=14336, cfg=None, desc="prefill GEMM Q4NX M=2048 K=4096 N=14336 g32, weights in Q4NX stream order"),
    # the tail of a decode step of Llama-3.2-1B: final RMSNorm + bf16 lm_head GEMV + argmax
    "lm_head": dict(M=1, K=2048, N=128256, cfg=None, desc="decode tail RMSNorm + bf16 lm_head GEMV + argmax E=2048 V=128256"),
}
LAYER_HEADS, LAYER_KV, LAYER_HD, LAYER_POS, LAYER_MAXSEQ = 32, 8, 128, 2047, 2048



def measured_traffic(name):
    """HBM bytes per launch of a workload's dominant kernel as measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two
    runs, each scaled by the same counter's reading for a 256 MiB device copy), from profiles/traffic.json: the figure,
    the commit of the kernel it was measured on and the summary under profiles/ that holds the command and the raw
    readings.  None for a workload that has no entry."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            return json.load(f).get(name)
    except OSError:
        return None


def weight_bytes(K, N):
    return K * N // 2 + (K // 128) * (N // 8) * 4 + (K // 128) * N * 2


def q4nx_weight_bytes(K, N):
    return K * N // 2 + 2 * (K // 32) * N * 2


def algorithmic_bytes(name):
    c = CONFIGS[name]
    M, K, N = c["M"], c["K"], c["N"]
    name = name[:-4] if name.endswith("_awq") else name
    if name.startswith("q4nx"):
        return q4nx_weight_bytes(K, N) + M * K * 2 + M * N * 2
    if name == "lm_head":   # weights, x and norm weight in, logits out
        return K * N * 2 + 2 * K * 2 + N * 2
    if name == "dequant":
        return weight_bytes(K, N) + K * N * 2
    if name == "ffn":
        return 3 * weight_bytes(K, N) + K * 2 + K * 2
    if name == "block":   # wo + gate + up + down; attn_out, x_residual, norm weight in, y out
        return weight_bytes(K, K) + 3 * weight_bytes(K, N) + 4 * K * 2
    if name == "layer":   # + fused QKV weights and the K and V caches up to pos
        nqkv = (LAYER_HEADS + 2 * LAYER_KV) * LAYER_HD
        return (weight_bytes(K, nqkv) + 2 * LAYER_KV * (LAYER_POS + 1) * LAYER_HD * 2
                + weight_bytes(K, K) + 3 * weight_bytes(K, N) + 5 * K * 2)
    return weight_bytes(K, N) + M * K * 2 + M * N * 2


def algorithmic_flops(name):
    c = CONFIGS[name]
    name = name[:-4] if name.endswith("_awq") else name
    if name == "ffn":
        return 2 * 3 * c["K"] * c["N"]
    if name in ("block", "layer"):
        return 2 * (3 * c["K"] * c["N"] + c["K"] * c["K"])
    return 2 * max(c["M"], 0) * c["K"] * c["N"]


def make_weights(torch, K, N, seed):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    # uniform random words = uniform uint4 nibbles in every position
    qweight = torch.randint(-2**31, 2**31 - 1, (K, N // 8), dtype=torch.int32, device="cuda", generator=g)
    qzeros = torch.randint(-2**31, 2**31 - 1, (K // 128, N // 8), dtype=torch.int32, device="cuda", generator=g)
    scales = (torch.randn((K // 128, N), device="cuda", generator=g).abs() * 0.02 + 1e-3).to(torch.bfloat16)
    return qweight, qzeros, scales


def make_q4nx_weights(torch, K, N, seed):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    qweight = torch.randint(-2**31, 2**31 - 1, (K, N // 8), dtype=torch.int32, device="cuda", generator=g)
    scales = (torch.randn((K // 32, N), device="cuda", generator=g).abs() * 0.003 + 1e-3).to(torch.bfloat16)
    mins = (-torch.randn((K // 32, N), device="cuda", generator=g).abs() * 0.02 - 0.01).to(torch.bfloat16)
    return qweight, scales, mins


def run_workload(name, steps, warmup, with_cpu_baseline):
    import torch

    from air_hip import _lib

    lib = _lib.load_library()
    c = CONFIGS[name]
    M, K, N = c["M"], c["K"], c["N"]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.Stream()

    q4nx = name.startswith("q4nx")
    lm_head = name == "lm_head"
    stream_order = name in ("gemv", "probe", "gemm16", "gemm64", "gemm64_down", "prefill", "ffn", "block", "layer")     # weights re-packed at load time (untimed)
    kind = name[:-4] if name.endswith("_awq") else name
    per_copy = K * N * 2 if lm_head else q4nx_weight_bytes(K, N) if q4nx else weight_bytes(K, N) * (3 if kind in ("ffn", "block", "layer") else 1) + (weight_bytes(K, K) if kind in ("block", "layer") else 0)
    nqkv = (LAYER_HEADS + 2 * LAYER_KV) * LAYER_HD
    if kind == "layer":
        per_copy += weight_bytes(K, nqkv)
    if kind in ("prefill", "q4nx_prefill"):
        ncopies = 1
    else:
        ncopies = max(2, -(-(MALL_BYTES + MALL_BYTES // 2) // per_copy))
    copies = []
    awq0 = None   # copy 0 in checkpoint layout, for the CPU baseline of a stream-order workload
    for i in range(ncopies):
        if kind == "ffn":
            copies.append((make_weights(torch, K, N, 100 + 3 * i), make_weights(torch, K, N, 101 + 3 * i),
                           make_weights(torch, N, K, 102 + 3 * i)))
        elif kind in ("block", "layer"):
            c4 = (make_weights(torch, K, N, 100 + 5 * i), make_weights(torch, K, N, 101 + 5 * i),
                  make_weights(torch, N, K, 102 + 5 * i), make_weights(torch, K, K, 103 + 5 * i))
            copies.append(c4 + ((make_weights(torch, K, nqkv, 104 + 5 * i),) if kind == "layer" else ()))
        elif q4nx:
            copies.append(make_q4nx_weights(torch, K, N, 100 + i))
            from air_hip import ops
            copies[-1] = (ops.q4nx_repack_stream(*copies[-1]).buf,)   # re-packed at load time (untimed)
        elif lm_head:
            gw = torch.Generator(device="cuda")
            gw.manual_seed(100 + i)
            copies.append(((torch.randn((N, K), device="cuda", generator=gw) * 0.05).to(torch.bfloat16),))
        elif name in ("gemv", "probe"):
            # all copies in one arena, as a loader would place a model's layers
            from air_hip import ops
            w = make_weights(torch, K, N, 100 + i)
            sb = int(lib.w4a16_stream_bytes(K, N))
            if i == 0:
                arena = torch.empty(ncopies * sb, dtype=torch.uint8, device=dev)
            arena[i * sb:(i + 1) * sb].copy_(ops.repack_stream(*w).buf)
            copies.append((arena[i * sb:(i + 1) * sb],) + (w if i == 0 else ()))   # copy 0 keeps its tensors for the CPU baseline
            del w
        else:
            copies.append(make_weights(torch, K, N, 100 + i))
        if stream_order and kind not in ("gemv", "probe"):
            from air_hip import ops
            if i == 0:
                awq0 = copies[0]
            mats = (copies[i],) if kind in ("gemm16", "gemm64", "gemm64_down", "prefill") else copies[i]
            copies[i] = tuple(ops.repack_stream(*m).buf for m in mats)
    gx = torch.Generator(device="cuda")
    gx.manual_seed(7)
    x = torch.randn((max(M, 1), K), device="cuda", generator=gx).to(torch.bfloat16)
    if name == "dequant":
        outs = [torch.empty((K, N), dtype=torch.bfloat16, device=dev) for _ in range(min(ncopies, 8))]
    elif kind in ("ffn", "block", "layer"):
        outs = [torch.empty((K,), dtype=torch.bfloat16, device=dev)]
    else:
        outs = [torch.empty((M, N), dtype=torch.bfloat16, device=dev)]
    if name == "probe":
        probe_out = torch.empty((N,), dtype=torch.int32, device=dev)
    if name in ("gemm16", "gemm64", "gemm64_down", "prefill"):
        gemm_scratch = torch.empty(max(int(lib.w4a16_gemm_stream_scratch_bytes(M, K, N)), 16), dtype=torch.uint8, device=dev)
    if lm_head:
        outs = [torch.empty((N,), dtype=torch.bfloat16, device=dev)]
        best = torch.empty((1,), dtype=torch.int32, device=dev)
        lm_ws = torch.empty(int(lib.lm_head_workspace_bytes(N)), dtype=torch.uint8, device=dev)
    if kind in ("block", "layer", "lm_head"):
        x_residual = torch.randn((K,), device="cuda", generator=gx).to(torch.bfloat16)
        norm_w = (torch.randn((K,), device="cuda", generator=gx) * 0.1 + 1.0).to(torch.bfloat16)
    if kind == "layer":
        kv_shape = (LAYER_KV, LAYER_MAXSEQ, LAYER_HD)
        k_cache = torch.randn(kv_shape, device="cuda", generator=gx).to(torch.bfloat16)
        v_cache = torch.randn(kv_shape, device="cuda", generator=gx).to(torch.bfloat16)
        lut_row = torch.rand((LAYER_HD,), device="cuda", generator=gx).to(torch.bfloat16)
        qkv = torch.empty((nqkv,), dtype=torch.bfloat16, device=dev)
        attn_out = torch.empty((K,), dtype=torch.bfloat16, device=dev)
        attn_ws = torch.empty(int(lib.w4a16_attention_workspace_bytes(LAYER_HEADS, LAYER_HD)), dtype=torch.uint8, device=dev)
        piece = 16 if stream_order else 256
        x_sumsq = (x_residual.float() ** 2).reshape(K // piece, piece).sum(dim=1).contiguous()
        y_sumsq = torch.empty((K // piece,), dtype=torch.float32, device=dev)
    if stream_order and kind in ("ffn", "block", "layer"):
        h_buf = torch.empty((N,), dtype=torch.bfloat16, device=dev)
        bws = torch.empty(int(lib.w4a16_block_stream_workspace_bytes(K, N)), dtype=torch.uint8, device=dev)

    if kind == "ffn":
        ws_bytes = lib.w4a16_ffn_workspace_bytes(K, N)
    elif kind in ("block", "layer"):
        ws_bytes = max(lib.w4a16_block_workspace_bytes(K, N), lib.w4a16_gemm_workspace_bytes(1, K, nqkv))
    else:
        ws_bytes = max(lib.w4a16_gemm_workspace_bytes(max(M, 1), K, N), 16384)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    _lib.check(lib.w4a16_workspace_init(ws.data_ptr(), ws.numel(), stream.cuda_stream))

    def launch(i, st):
        w = copies[i % ncopies]
        if name == "dequant":
            o = outs[i % len(outs)]
            rc = lib.awq_dequant_bf16(w[0].data_ptr(), w[1].data_ptr(), w[2].data_ptr(), o.data_ptr(), K, N, 128, st)
        elif name == "ffn":
            rc = lib.w4a16_ffn_swiglu_stream_bf16(x.data_ptr(), w[0].data_ptr(), w[1].data_ptr(), w[2].data_ptr(),
                                                  outs[0].data_ptr(), h_buf.data_ptr(), K, N, 128, st)
        elif name in ("block", "layer"):
            g, u, d, o = (t.data_ptr() for t in w[:4])
            if name == "layer":
                # the sum of squares of x per 16 columns comes from the block before (here: computed once)
                _lib.check(lib.w4a16_rms_gemv_stream_bf16(x_residual.data_ptr(), x_sumsq.data_ptr(), x_sumsq.numel(),
                                                          norm_w.data_ptr(), 1e-5, w[4].data_ptr(), qkv.data_ptr(), K, nqkv, 128, st))
                _lib.check(lib.w4a16_decode_attn_o_gemv_ffn_stream_bf16(
                    qkv.data_ptr(), lut_row.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), attn_out.data_ptr(), LAYER_POS,
                    LAYER_MAXSEQ, LAYER_HEADS, LAYER_KV, LAYER_HD, attn_ws.data_ptr(), attn_ws.numel(), x_residual.data_ptr(),
                    norm_w.data_ptr(), 1e-5, o, g, u, d, outs[0].data_ptr(), y_sumsq.data_ptr(), K, N, 128, bws.data_ptr(),
                    bws.numel(), st))
                return
            rc = lib.w4a16_o_gemv_ffn_stream_bf16(x.data_ptr(), x_residual.data_ptr(), norm_w.data_ptr(), 1e-5, o, g, u, d,
                                                  outs[0].data_ptr(), None, None, None, K, N, 128, bws.data_ptr(), bws.numel(), st)
        elif name == "ffn_awq":
            g, u, d = w
            rc = lib.w4a16_ffn_swiglu_bf16(x.data_ptr(), g[0].data_ptr(), g[1].data_ptr(), g[2].data_ptr(),
                                           u[0].data_ptr(), u[1].data_ptr(), u[2].data_ptr(),
                                           d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(),
                                           outs[0].data_ptr(), None, K, N, 128, ws.data_ptr(), ws.numel(), st)
        elif name in ("block_awq", "layer_awq"):
            g, u, d, o = w[:4]
            ptrs = [t.data_ptr() for m in (o, g, u, d) for t in m]
            a_in = x
            if name == "layer_awq":
                qw = w[4]
                # the sum of squares of x per 256-column tile comes from the block before (here: computed once)
                _lib.check(lib.w4a16_rms_gemv_sumsq_bf16(x_residual.data_ptr(), x_sumsq.data_ptr(), x_sumsq.numel(),
                                                         norm_w.data_ptr(), 1e-5, qw[0].data_ptr(), qw[1].data_ptr(),
                                                         qw[2].data_ptr(), qkv.data_ptr(), K, nqkv, 128, ws.data_ptr(),
                                                         ws.numel(), st))
                # attention + block as one call (the O projection merges the attention's chunk partials itself)
                _lib.check(lib.w4a16_decode_attn_o_gemv_ffn_bf16(
                    qkv.data_ptr(), lut_row.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), attn_out.data_ptr(), LAYER_POS,
                    LAYER_MAXSEQ, LAYER_HEADS, LAYER_KV, LAYER_HD, attn_ws.data_ptr(), attn_ws.numel(), x_residual.data_ptr(),
                    norm_w.data_ptr(), 1e-5, *ptrs, outs[0].data_ptr(), y_sumsq.data_ptr(), K, N, 128, ws.data_ptr(), ws.numel(), st))
                return
            rc = lib.w4a16_o_gemv_ffn_bf16(a_in.data_ptr(), x_residual.data_ptr(), norm_w.data_ptr(), 1e-5, *ptrs,
                                           outs[0].data_ptr(), None, None, K, N, 128, ws.data_ptr(), ws.numel(), st)
        elif lm_head:
            rc = lib.lm_head_gemv_bf16(x.data_ptr(), norm_w.data_ptr(), 1e-5, w[0].data_ptr(), outs[0].data_ptr(),
                                       best.data_ptr(), N, K, lm_ws.data_ptr(), lm_ws.numel(), st)
        elif name == "gemv":
            rc = lib.w4a16_gemv_stream_bf16(x.data_ptr(), w[0].data_ptr(), outs[0].data_ptr(), K, N, 128, st)
        elif name == "probe":
            rc = lib.w4a16_probe_stream_read(w[0].data_ptr(), probe_out.data_ptr(), K, N, st)
        elif name in ("gemm16", "gemm64", "gemm64_down", "prefill"):
            # (17 .. 128 rows: split along K with plain scratch; other row counts take no scratch)
            rc = lib.w4a16_gemm_stream_scratch_bf16(x.data_ptr(), w[0].data_ptr(), outs[0].data_ptr(), M, K, N, 128,
                                                    gemm_scratch.data_ptr(), gemm_scratch.numel(), st)
        elif name == "q4nx_gemv":
            rc = lib.w4a16_q4nx_gemv_stream_bf16(x.data_ptr(), w[0].data_ptr(), None, outs[0].data_ptr(), K, N, st)
        elif name in ("q4nx_gemm16", "q4nx_prefill"):
            rc = lib.w4a16_q4nx_gemm_stream_bf16(x.data_ptr(), w[0].data_ptr(), None, outs[0].data_ptr(), M, K, N, st)
        else:
            rc = lib.w4a16_gemm_bf16(x.data_ptr(), w[0].data_ptr(), w[1].data_ptr(), w[2].data_ptr(),
                                     outs[0].data_ptr(), M, K, N, 128, ws.data_ptr(), ws.numel(), st)
        _lib.check(rc)

    def spacers(indices):
        """Cold runs walk the weight copies cyclically; between two passes over `indices` the cycle is completed
        with untimed launches, so that the next pass starts on the copy touched longest ago and finds nothing of
        the previous pass in the Infinity Cache (ncopies x per_copy is 1.5 x its size)."""
        if len(set(indices)) > 1:
            for i in range(len(indices) % ncopies, ncopies if len(indices) % ncopies else 0):
                launch(i, stream.cuda_stream)

    def timed_graph(indices):
        """Capture len(indices) launches into one HIP graph; behind a spinning kernel, replay it twice and time the
        second replay (the first is the warm-up that the eager timing gets from its untimed rotation)."""
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(stream):
            with torch.cuda.graph(graph, stream=stream):
                for i in indices:
                    launch(i, stream.cuda_stream)
            graph.replay()          # untimed replay: instantiation / first-touch effects
            spacers(indices)
            stream.synchronize()
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            torch.cuda._sleep(int(2e5) * 16)
            graph.replay()
            spacers(indices)
            e0.record(stream)
            graph.replay()
            e1.record(stream)
            torch.cuda.synchronize()
            wall = time.perf_counter() - t0
        return e0.elapsed_time(e1) * 1e-3, wall

    def timed_eager(indices):
        """The same launches issued one by one behind a spinning kernel: the host queues them while the GPU is
        still busy, so the interval between the events holds the launches and not the host's launch latency."""
        with torch.cuda.stream(stream):
            for i in indices:
                launch(i, stream.cuda_stream)
            spacers(indices)
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            torch.cuda._sleep(int(2e5) * max(16, len(indices) // 2))
            # one untimed rotation over the copies, continuing the cyclic order, right in front of the timed launches:
            # the interval then starts in the steady state of a decode loop (memory and fabric clocks up; after the
            # idle spin the first ~100 us of launches run 5 % slower) and the first event follows a launch of the
            # same kind instead of the spinning kernel
            for i in range(ncopies):
                launch(indices[0] - ncopies + i if len(set(indices)) > 1 else indices[0], stream.cuda_stream)
            e0.record(stream)
            for i in indices:
                launch(i, stream.cuda_stream)
            e1.record(stream)
            torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3

    def timed_overlapped(indices, nstreams=4):
        """The same cold launches dealt round-robin to `nstreams` streams (default priority), so that independent launches
        may overlap on the GPU: not a decode chain (there every launch waits for the one before), but what the kernel
        streams when the per-launch floor is hidden.  Events on the first stream, which the others fork from and join."""
        others = [torch.cuda.Stream() for _ in range(nstreams - 1)]
        sts = [stream] + others
        for n, st in enumerate(others):   # (a stream's first launch sets up its hardware queue: not in the interval)
            launch(n, st.cuda_stream)
        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            spacers(indices)
            torch.cuda.synchronize()
            torch.cuda._sleep(int(2e5) * max(16, len(indices) // 2))
            for i in range(ncopies):
                launch(indices[0] - ncopies + i, stream.cuda_stream)
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record(stream)
        for st in others:
            st.wait_event(e0)
        for n, i in enumerate(indices):
            launch(i, sts[n % nstreams].cuda_stream)
        for st in others:
            ev = torch.cuda.Event()
            ev.record(st)
            stream.wait_event(ev)
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3

    with torch.cuda.stream(stream):
        for i in range(warmup):
            launch(i, stream.cuda_stream)
        stream.synchronize()

    graph_s, cold_wall = timed_graph(list(range(steps)))
    cold_s = timed_eager(list(range(steps)))
    hot_s = timed_eager([0] * steps)

    # one event pair per launch, outside a graph (the reference's harness style,
    # programming_examples/matrix_vector_multiplication/int4_awq/test_packed.cpp:114-150): each figure
    # carries the full eager launch overhead, so these are a distribution, not the throughput claim
    per_launch = []
    with torch.cuda.stream(stream):
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        for i, (a, b) in enumerate(evs):
            a.record(stream)
            launch(i, stream.cuda_stream)
            b.record(stream)
        stream.synchronize()
        per_launch = sorted(a.elapsed_time(b) * 1e3 for a, b in evs)

    n_overlapped = max(steps, 200)   # (the fork and join of the streams cost a few us: spread over enough launches)
    overlapped_s = timed_overlapped(list(range(n_overlapped))) if name == "gemv" else None
    res = {
        "name": name,
        "overlapped_us": overlapped_s / n_overlapped * 1e6 if overlapped_s else None,
        "overlapped_launches": n_overlapped,
        "cold_us": cold_s / steps * 1e6,
        "hot_us": hot_s / steps * 1e6,
        "graph_us": graph_s / steps * 1e6,
        "wall_s": cold_wall,
        "bytes": algorithmic_bytes(name),
        "flops": algorithmic_flops(name),
        "ncopies": ncopies,
        "per_launch_events_us": {"min": per_launch[0], "median": per_launch[len(per_launch) // 2],
                                 "avg": sum(per_launch) / len(per_launch), "max": per_launch[-1]},
    }

    if with_cpu_baseline and kind not in ("block", "layer", "lm_head", "probe") and not name.endswith("_awq") and not q4nx:
        w0 = copies[0][1:] if name == "gemv" else awq0 if awq0 is not None else copies[0]
        res["cpu_baseline"] = cpu_baseline(name, torch, w0, x, outs, launch, stream)
    return res


DECODE_1B_POS0 = 1024
PREFILL_BLOCK = dict(M=2048, E=2048, H=8192)   # the reference example's dimensions (o_ffn_int4_multi.py:291-293)


def run_prefill_block(steps, warmup, stream_order=True):
    """Prefill O projection + residual + RMSNorm + SwiGLU FFN + residual for 2048 tokens at the
    Llama-3.2-1B widths, `steps` calls in one HIP graph: w4a16_prefill_o_ffn_stream_bf16 on stream-order
    weights, or (stream_order=False) w4a16_prefill_o_ffn_bf16 on the checkpoint tensors."""
    import torch

    from air_hip import _lib

    lib = _lib.load_library()
    M, E, H = PREFILL_BLOCK["M"], PREFILL_BLOCK["E"], PREFILL_BLOCK["H"]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.Stream()
    g = torch.Generator(device="cuda")
    g.manual_seed(9)
    ws = [make_weights(torch, K, N, 300 + i) for i, (K, N) in enumerate(((E, E), (E, H), (E, H), (H, E)))]
    ws = [(qw, qz, (sc.float() * 0.1).to(torch.bfloat16)) for qw, qz, sc in ws]
    attn = torch.randn((M, E), device="cuda", generator=g).to(torch.bfloat16)
    xres = torch.randn((M, E), device="cuda", generator=g).to(torch.bfloat16)
    nw = (torch.randn((E,), device="cuda", generator=g) * 0.1 + 1.0).to(torch.bfloat16)
    y = torch.empty((M, E), dtype=torch.bfloat16, device=dev)
    scratch = torch.empty(int(lib.w4a16_prefill_block_workspace_bytes(M, E, H)), dtype=torch.uint8, device=dev)
    ptrs = [t.data_ptr() for w in ws for t in w]
    if stream_order:
        from air_hip import ops
        sws = [ops.repack_stream(*w) for w in ws]
        torch.cuda.synchronize()
        ptrs = [w.buf.data_ptr() for w in sws]
    entry = lib.w4a16_prefill_o_ffn_stream_bf16 if stream_order else lib.w4a16_prefill_o_ffn_bf16

    def launch(st):
        _lib.check(entry(attn.data_ptr(), xres.data_ptr(), nw.data_ptr(), 1e-5, *ptrs, y.data_ptr(),
                         None, None, M, E, H, 128, scratch.data_ptr(), scratch.numel(), st))

    with torch.cuda.stream(stream):
        for _ in range(warmup):
            launch(stream.cuda_stream)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for _ in range(steps):
                launch(stream.cuda_stream)
        graph.replay()
        stream.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record(stream)
        graph.replay()
        e1.record(stream)
        torch.cuda.synchronize()
    sec = e0.elapsed_time(e1) * 1e-3 / steps
    flops = 2 * M * (E * E + 3 * E * H)
    return {"us": sec * 1e6, "flops": flops, "TFLOP/s": flops / sec / 1e12, "finite": bool(torch.isfinite(y.float()).all())}


DECODE_MODELS = {
    # Llama-3.2-1B (programming_examples/llms/llama32_1b/llama32_1b_weights.py:35-47) and Llama-3.1-8B
    "decode_1b": dict(n_layers=16, emb_dim=2048, n_heads=32, head_dim=64, n_kv_heads=8, hidden_dim=8192, vocab_size=128256),
    "decode_8b": dict(n_layers=32, emb_dim=4096, n_heads=32, head_dim=128, n_kv_heads=8, hidden_dim=14336, vocab_size=128256),
}


def run_decode_model(steps, warmup, model="decode_1b", stream_order=True):
    """Greedy decode of a random-weight model in the Llama-3.2-1B shape (16 layers, E=2048, H=8192,
    32/8 heads of 64, vocabulary 128256, tied lm_head) or the Llama-3.1-8B shape, `steps` consecutive
    tokens from position DECODE_1B_POS0 captured as one HIP graph: per token n_layers x (RMSNorm + QKV
    GEMV, attention, O + FFN block) and the tail (final norm, lm_head GEMV, argmax), the token id
    staying on the device."""
    import torch

    from air_hip import decode, weights as wmod

    cfg = wmod.LlamaConfig(**DECODE_MODELS[model])
    E, H, hd = cfg.emb_dim, cfg.hidden_dim, cfg.head_dim
    nqkv = (cfg.n_heads + 2 * cfg.n_kv_heads) * hd
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.Stream()
    g = torch.Generator(device="cuda")
    g.manual_seed(5)

    def lin(K, N, seed):
        qw, qz, sc = make_weights(torch, K, N, seed)
        return qw, qz, (sc.float() * 0.05).to(torch.bfloat16)   # keeps the residual stream O(1) over 16 layers

    def norm_w():
        return (torch.randn((E,), device="cuda", generator=g) * 0.1 + 1.0).to(torch.bfloat16)

    layers = [decode.DecodeLayer(attn_norm=norm_w(), ffn_norm=norm_w(), wqkv=lin(E, nqkv, 10 * i), wo=lin(E, E, 10 * i + 1),
                                 w_gate=lin(E, H, 10 * i + 2), w_up=lin(E, H, 10 * i + 3), w_down=lin(H, E, 10 * i + 4))
              for i in range(cfg.n_layers)]
    if stream_order:
        for l in layers:   # decode reads stream-order weights; the checkpoint-layout tensors are not needed here
            l.with_stream()
    embed = torch.randn((cfg.vocab_size, E), device="cuda", generator=g).to(torch.bfloat16)
    final_norm = norm_w()
    max_seq = 2048
    assert DECODE_1B_POS0 + max(steps, warmup) <= max_seq
    lut = decode.generate_rope_lut(cfg, max_seq)
    cache = [(torch.randn((cfg.n_kv_heads, max_seq, hd), device="cuda", generator=g).to(torch.bfloat16),
              torch.randn((cfg.n_kv_heads, max_seq, hd), device="cuda", generator=g).to(torch.bfloat16))
             for _ in range(cfg.n_layers)]
    first = torch.tensor([1], dtype=torch.int32, device=dev)
    with torch.cuda.stream(stream):
        decode.decode_greedy(first, warmup, layers, embed, final_norm, embed, cfg, cache, DECODE_1B_POS0, lut)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            tokens = decode.decode_greedy(first, steps, layers, embed, final_norm, embed, cfg, cache, DECODE_1B_POS0, lut)
        graph.replay()
        stream.synchronize()
        ref_tokens = tokens.clone()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record(stream)
        graph.replay()
        e1.record(stream)
        torch.cuda.synchronize()
    sec = e0.elapsed_time(e1) * 1e-3
    layer_w = weight_bytes(E, nqkv) + weight_bytes(E, E) + 2 * weight_bytes(E, H) + weight_bytes(H, E)
    kv = 2 * cfg.n_kv_heads * (DECODE_1B_POS0 + steps // 2 + 1) * hd * 2
    per_token = cfg.n_layers * (layer_w + kv + 2 * E * 2) + 2 * cfg.vocab_size * E + 2 * cfg.vocab_size + 3 * E * 2
    return {"us_per_token": sec / steps * 1e6, "tokens_per_s": steps / sec, "bytes_per_token": per_token,
            "replays_agree": bool(torch.equal(ref_tokens, tokens))}


def run_prefill_model(model="decode_1b", M=2048, reps=3, stream_order=True):
    """Prompt pass of M tokens through a random-weight model (air_hip.decode.prefill: per layer RMSNorm + QKV GEMM
    + RoPE, causal attention, O + FFN block; then the decode tail on the last row), captured as one HIP graph.
    stream_order: the layers carry the stream-order re-pack, which the prompt pass then reads (as decode does)."""
    import torch

    from air_hip import decode, weights as wmod

    cfg = wmod.LlamaConfig(**DECODE_MODELS[model])
    E, H, hd = cfg.emb_dim, cfg.hidden_dim, cfg.head_dim
    nqkv = (cfg.n_heads + 2 * cfg.n_kv_heads) * hd
    torch.cuda.set_device(0)
    stream = torch.cuda.Stream()
    g = torch.Generator(device="cuda")
    g.manual_seed(6)

    def lin(K, N, seed):
        qw, qz, sc = make_weights(torch, K, N, seed)
        return qw, qz, (sc.float() * 0.05).to(torch.bfloat16)

    def norm_w():
        return (torch.randn((E,), device="cuda", generator=g) * 0.1 + 1.0).to(torch.bfloat16)

    layers = [decode.DecodeLayer(attn_norm=norm_w(), ffn_norm=norm_w(), wqkv=lin(E, nqkv, 10 * i), wo=lin(E, E, 10 * i + 1),
                                 w_gate=lin(E, H, 10 * i + 2), w_up=lin(E, H, 10 * i + 3), w_down=lin(H, E, 10 * i + 4))
              for i in range(cfg.n_layers)]
    if stream_order:
        for l in layers:
            l.with_stream()
    embed = torch.randn((cfg.vocab_size, E), device="cuda", generator=g).to(torch.bfloat16)
    final_norm = norm_w()
    lut = decode.generate_rope_lut(cfg, M)
    cache = decode.new_kv_cache(cfg, M)
    prompt = torch.randint(0, cfg.vocab_size, (M,), device="cuda", generator=g, dtype=torch.int64)
    with torch.cuda.stream(stream):
        decode.prefill(prompt, layers, embed, final_norm, embed, cfg, cache, lut)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            logits, best = decode.prefill(prompt, layers, embed, final_norm, embed, cfg, cache, lut)
        graph.replay()
        stream.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record(stream)
        for _ in range(reps):
            graph.replay()
        e1.record(stream)
        torch.cuda.synchronize()
    sec = e0.elapsed_time(e1) * 1e-3 / reps
    flops = cfg.n_layers * (2 * M * (E * nqkv + E * E + 3 * E * H) + 2 * M * M * hd * cfg.n_heads) + 2 * E * cfg.vocab_size
    return {"ms": sec * 1e3, "tokens_per_s": M / sec, "flops": flops, "TFLOP/s": flops / sec / 1e12,
            "finite": bool(torch.isfinite(logits).all())}


def cpu_baseline(name, torch, w, x, outs, launch, stream):
    """The reference's NumPy path (restated in oracle/baseline.py) timed on this host's cores,
    on the same inputs as GPU launch 0; also used to sanity-check the GPU result."""
    import numpy as np

    from oracle import baseline
    from oracle.bf16 import bf16_bits_to_f32

    try:
        from threadpoolctl import threadpool_info
        blas_threads = max([p.get("num_threads", 1) for p in threadpool_info() if p.get("user_api") == "blas"] or [1])
    except Exception:
        blas_threads = 1

    def host(t):
        if t.dtype == torch.bfloat16:
            return t.view(torch.int16).cpu().numpy().view(np.uint16)
        return t.cpu().numpy()

    c = CONFIGS[name]
    with torch.cuda.stream(stream):
        launch(0, stream.cuda_stream)
        stream.synchronize()
    got = bf16_bits_to_f32(host(outs[0]))

    if name == "dequant":
        args = tuple(host(t) for t in w)
        fn = lambda: baseline.dequant_numpy(*args)
        sample = "full config 0 (K=4096, N=4096), vectorised NumPy unpack + dequant, median of 3"
    elif name == "ffn":
        g, u, d = (tuple(host(t) for t in m) for m in w)
        xb = host(x)[0]
        fn = lambda: baseline.ffn_numpy(xb, g, u, d)
        sample = "full config 4, vectorised NumPy dequant + float32 BLAS products, median of 3"
    elif name == "prefill":
        # bounded sample: the first 128 rows of x against the full weight matrix
        args = tuple(host(t) for t in w)
        xb = host(x)[:128]
        fn = lambda: baseline.gemm_numpy(xb, *args)
        sample = "rows 0..127 of config 3 (M=128 of 2048) incl. the full dequant, scaled by M; median of 3"
    else:
        args = tuple(host(t) for t in w)
        xb = host(x)
        fn = lambda: baseline.gemm_numpy(xb, *args)
        sample = f"full config {c['cfg']}, vectorised NumPy dequant + float32 BLAS product, median of 3"

    extra = {}
    if name in ("gemv", "gemm16", "prefill", "dequant"):
        wargs = tuple(host(t) for t in w)
        baseline.dequant_numpy(*wargs)                             # warm-up
        t0 = time.perf_counter()
        baseline.dequant_numpy(*wargs)
        extra["dequant_seconds"] = time.perf_counter() - t0      # the unpack + dequant part alone
    if name == "gemv":
        # the reference's own cpu_reference is a scalar double loop (matvec_int4_packed.py:281-286);
        # its C restatement runs at full size on one core
        import ctypes

        import oracle
        from oracle import awq as oawq
        a_q, a_s, a_z = oawq.repack_hf_awq_linear(*wargs, 128)
        a_q, a_s, a_z = (np.ascontiguousarray(t) for t in (a_q, a_s, a_z))
        xb0 = np.ascontiguousarray(host(x)[0])
        out = np.zeros(c["N"], np.uint16)
        clib = oracle.load_c_oracle()
        ptr = lambda a: a.ctypes.data_as(ctypes.c_void_p)
        t0 = time.perf_counter()
        clib.oracle_matvec_loop(ptr(a_q), ptr(a_s), ptr(a_z), ptr(xb0), c["N"], c["K"], 128, ptr(out))
        extra["scalar_loop_c_seconds"] = time.perf_counter() - t0
        extra["scalar_loop_c_max_abs_diff_vs_gpu"] = float(np.max(np.abs(bf16_bits_to_f32(out) - got.reshape(-1))))

    ref = fn()   # warm-up, and the reference output
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    t = sorted(times)[1]
    ref_f = bf16_bits_to_f32(ref)
    n = ref_f.size
    err = float(np.max(np.abs(got.reshape(-1)[:n] - ref_f.reshape(-1))))
    if name == "prefill":
        value = algorithmic_flops(name) * (128 / c["M"]) / t / 1e12
        unit = "TFLOP/s"
    else:
        value = algorithmic_bytes(name) / t / 1e9
        unit = "GB/s"
    return {"value": value, "unit": unit, "cores": int(blas_threads), "kind": "port", "sample": sample,
            "seconds": t, "host_cpus": len(os.sched_getaffinity(0)), "max_abs_diff_vs_gpu": err, **extra}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="gemv", choices=list(CONFIGS) + ["decode_1b", "decode_8b", "prefill_block", "prefill_block_awq", "prefill_1b", "prefill_1b_awq",
                                                             "prefill_8b"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip the short runs of the other configs")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also launch one device copy of 256 MiB (a dispatch of known traffic that calibrates "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--tune", action="append", default=[], metavar="KEY=VALUE",
                    help="set a library tuning key (w4a16_tune) before the run, e.g. --tune gemv_ws_ct=16; repeatable")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py measures the single-GPU W4A16 kernels; --gpus must be 1 "
              "(this build has no multi-GPU path and every box has one GPU)", file=sys.stderr)
        sys.exit(2)

    if a.tune:
        from air_hip import ops
        for kv in a.tune:
            key, _, val = kv.partition("=")
            ops.tune(key, int(val))
    if a.copy_probe:
        import torch
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if a.workload in ("prefill_1b", "prefill_1b_awq", "prefill_8b"):
        model = "decode_8b" if a.workload == "prefill_8b" else "decode_1b"
        r = run_prefill_model(model, 2048, max(1, min(a.steps, 5)), stream_order=not a.workload.endswith("_awq"))
        c = DECODE_MODELS[model]
        shape = (f"{c['n_layers']} layers E={c['emb_dim']} H={c['hidden_dim']} {c['n_heads']}/{c['n_kv_heads']} heads "
                 f"hd={c['head_dim']} V={c['vocab_size']} g128")
        layout = "checkpoint-layout" if a.workload.endswith("_awq") else "stream-order"
        print(json.dumps({
            "metric": f"int4 prefill tokens/s, {'Llama-3.1-8B' if model == 'decode_8b' else 'Llama-3.2-1B'} shape, 2048-token prompt", "value": r["tokens_per_s"], "unit": "tokens/s",
            "n_gpus": 1, "steps": max(1, min(a.steps, 5)), "warmup": 1, "ms_per_step": r["ms"], "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "int4 weights (bf16 lm_head), bf16 activations, fp32 accumulate",
            "data": "synthetic (random weights of the architecture, random prompt)",
            "config": {"workload": f"prompt pass, {shape}, 2048 tokens, causal attention, KV caches filled, {layout} weights",
                       "timing": "one HIP graph of the whole pass, events on the launch stream"},
            "roofline": {"bound": "mfma", "achieved": r["TFLOP/s"], "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": r["TFLOP/s"] / MFMA_BF16_PEAK_TFLOPS, "traffic": None, "algorithmic_per_launch": r["flops"],
                         "avg_launch_us": r["ms"] * 1e3},
            "finite": r["finite"]}))
        return
    if a.workload in ("prefill_block", "prefill_block_awq"):
        steps = min(a.steps, 20)
        r = run_prefill_block(steps, min(a.warmup, 3), stream_order=a.workload == "prefill_block")
        print(json.dumps({
            "metric": "W4A16 prefill O + FFN block TFLOP/s", "value": r["TFLOP/s"], "unit": "TFLOP/s", "n_gpus": 1,
            "steps": steps, "warmup": min(a.warmup, 3), "ms_per_step": r["us"] * 1e-3, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "int4 weights, bf16 activations, fp32 accumulate",
            "data": "synthetic (uniform uint4 q/z, scales (|N(0,1)|*0.02+1e-3)*0.1, activations ~ N(0,1))",
            "config": {"workload": "prefill O-proj + residual + RMSNorm + SwiGLU FFN + residual, M=2048 E=2048 H=8192 g128, "
                                   + ("stream-order weights" if a.workload == "prefill_block" else "checkpoint-layout weights"),
                       "timing": "HIP graph of K calls (5 to 7 launches each), events on the launch stream"},
            "roofline": {"bound": "mfma", "achieved": r["TFLOP/s"], "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": r["TFLOP/s"] / MFMA_BF16_PEAK_TFLOPS, "traffic": None, "algorithmic_per_launch": r["flops"],
                         "avg_launch_us": r["us"]},
            "finite": r["finite"]}))
        return
    if a.workload in DECODE_MODELS:
        steps = min(a.steps, 64)
        r = run_decode_model(steps, min(a.warmup, 8), a.workload)
        m = DECODE_MODELS[a.workload]
        gbs = r["bytes_per_token"] / (r["us_per_token"] * 1e-6) / 1e9
        print(json.dumps({
            "metric": "int4 decode tokens/s, Llama-3.%s shape, batch 1" % ("2-1B" if a.workload == "decode_1b" else "1-8B"), "value": r["tokens_per_s"], "unit": "tokens/s",
            "n_gpus": 1, "steps": steps, "warmup": min(a.warmup, 8), "ms_per_step": r["us_per_token"] * 1e-3,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "int4 weights (bf16 lm_head), bf16 activations, fp32 accumulate",
            "data": "synthetic (random weights of the architecture, random KV cache up to the start position)",
            "config": {"workload": f"greedy decode, {m['n_layers']} layers E={m['emb_dim']} H={m['hidden_dim']} {m['n_heads']}/{m['n_kv_heads']} heads hd={m['head_dim']} V={m['vocab_size']} g128, positions {DECODE_1B_POS0}..{DECODE_1B_POS0 + steps - 1}",
                       "timing": "one HIP graph of all token steps, events on the launch stream"},
            "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                         "traffic": None, "algorithmic_per_launch": r["bytes_per_token"], "avg_launch_us": r["us_per_token"]},
            "replays_agree": r["replays_agree"]}))
        return
    main_res = run_workload(a.workload, a.steps, a.warmup, not a.no_cpu_baseline)
    name = a.workload
    sec = main_res["cold_us"] * 1e-6
    if name in ("prefill", "prefill_awq", "q4nx_prefill"):
        metric, unit = "W4A16 prefill GEMM TFLOP/s", "TFLOP/s"
        value = main_res["flops"] / sec / 1e12
        roof = {"bound": "mfma", "achieved": value, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": value / MFMA_BF16_PEAK_TFLOPS, "traffic": None}
    else:
        metric, unit = "int4 GEMV HBM GB/s at M=1" if name == "gemv" else f"{name} HBM GB/s", "GB/s"
        value = main_res["bytes"] / sec / 1e9
        roof = {"bound": "hbm", "achieved": value, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": value / HBM_PEAK_GBS, "traffic": None}
    t = measured_traffic(name)
    roof["traffic"] = t["bytes"] if t else None
    if t:
        roof["traffic_measured_at"] = {"commit": t["commit"], "profile": t["profile"]}
    roof["kernel"] = {"dequant": "dequant_kernel", "prefill": "gemm_wsp_kernel", "q4nx_prefill": "gemm_wsp_kernel", "q4nx_gemv": "gemv_ws_kernel", "q4nx_gemm16": "gemm_ws_kernel", "prefill_awq": "gemm_kernel", "lm_head": "lm_head_kernel",
                      "gemv": "gemv_ws_kernel", "probe": "probe_ws_kernel", "gemm16": "gemm_ws_kernel", "gemm64": "gemm_ws_rows_kernel", "gemm64_down": "gemm_wsk_kernel", "ffn": "gemv_ws_kernel", "block": "gemv_ws_kernel", "layer": "gemv_ws_kernel"}.get(name, "stream_kernel")
    roof["algorithmic_per_launch"] = main_res["flops"] if name in ("prefill", "prefill_awq", "q4nx_prefill") else main_res["bytes"]
    roof["avg_launch_us"] = main_res["cold_us"]

    out = {
        "metric": metric,
        "value": value,
        "unit": unit,
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": main_res["cold_us"] * 1e-3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16 weights and activations, fp32 accumulate" if name == "lm_head" else "int4 weights, bf16 activations, fp32 accumulate",
        "data": "synthetic (W ~ N(0,1)*0.05 as bf16, x ~ N(0,1))" if name == "lm_head" else "synthetic (uniform uint4 q/z, scales |N(0,1)|*0.02+1e-3, x ~ N(0,1)), random weights",
        "config": {"workload": CONFIGS[name]["desc"], "group": 32 if name.startswith("q4nx") else 128,
                   "weight_copies_rotated": main_res["ncopies"],
                   "timing": "K launches queued on one stream behind a spinning kernel and one untimed rotation over the weight "
                             "copies, HIP events on that stream around the K launches (graph_us_per_step: the same K launches "
                             "replayed as one HIP graph)"},
        "roofline": roof,
        "per_launch_events_us": main_res["per_launch_events_us"],
        "graph_us_per_step": main_res["graph_us"],
        "hot_cache": {"us_per_step": main_res["hot_us"],
                      "value": (main_res["flops"] / 1e12 if name in ("prefill", "prefill_awq", "q4nx_prefill") else main_res["bytes"] / 1e9) / (main_res["hot_us"] * 1e-6),
                      "note": "same buffers every step (Infinity Cache resident for the decode shapes)"},
    }
    if main_res.get("overlapped_us"):
        out["independent_launches_on_4_streams"] = {
            "us_per_step": main_res["overlapped_us"], "launches": main_res["overlapped_launches"],
            "value": main_res["bytes"] / 1e9 / (main_res["overlapped_us"] * 1e-6),
            "note": "cold launches dealt to four streams so that they may overlap: throughput of independent "
                    "GEMVs, not the per-launch figure of a decode chain (value, roofline and ms_per_step above)"}
    if "cpu_baseline" in main_res:
        out["cpu_baseline"] = main_res["cpu_baseline"]

    if not a.no_extra:
        extra = {}
        for other in CONFIGS:
            if other == name:
                continue
            # the other headline configs carry the host baseline as well
            with_cpu = not a.no_cpu_baseline and other in ("dequant", "gemm16", "ffn", "prefill")
            tiled = other.startswith("prefill") or other == "q4nx_prefill"   # the MFMA-bound workloads
            r = run_workload(other, 20 if tiled else 100, 5, with_cpu)
            s = r["cold_us"] * 1e-6
            if tiled:
                extra[other] = {"us": r["cold_us"], "TFLOP/s": r["flops"] / s / 1e12,
                                "frac_mfma_peak": r["flops"] / s / 1e12 / MFMA_BF16_PEAK_TFLOPS}
            else:
                extra[other] = {"us": r["cold_us"], "GB/s": r["bytes"] / s / 1e9,
                                "frac_hbm_peak": r["bytes"] / s / 1e9 / HBM_PEAK_GBS, "hot_us": r["hot_us"]}
            if "cpu_baseline" in r:
                extra[other]["cpu_baseline"] = r["cpu_baseline"]
            if other == "prefill":
                # the compute-bound half of the headline metric, as a block of its own
                tf = r["flops"] / s / 1e12
                out["prefill"] = {
                    "metric": "W4A16 prefill GEMM TFLOP/s", "value": tf, "unit": "TFLOP/s", "steps": 20, "warmup": 5,
                    "ms_per_step": r["cold_us"] * 1e-3, "config": {"workload": CONFIGS["prefill"]["desc"]},
                    "roofline": {"bound": "mfma", "achieved": tf, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                                 "frac": tf / MFMA_BF16_PEAK_TFLOPS, "traffic": (measured_traffic("prefill") or {}).get("bytes"),
                                 "traffic_measured_at": {k: (measured_traffic("prefill") or {}).get(k) for k in ("commit", "profile")},
                                 "kernel": "gemm_wsp_kernel", "algorithmic_per_launch": r["flops"], "avg_launch_us": r["cold_us"]},
                    "graph_us_per_step": r["graph_us"]}
                if "cpu_baseline" in r:
                    out["prefill"]["cpu_baseline"] = r["cpu_baseline"]
        r = run_prefill_block(10, 2)
        extra["prefill_block"] = {"us": r["us"], "TFLOP/s": r["TFLOP/s"], "frac_mfma_peak": r["TFLOP/s"] / MFMA_BF16_PEAK_TFLOPS}
        for name, model in (("prefill_1b", "decode_1b"), ("prefill_8b", "decode_8b")):
            r = run_prefill_model(model, 2048, 2)
            extra[name] = {"ms": r["ms"], "tokens/s": r["tokens_per_s"], "TFLOP/s": r["TFLOP/s"],
                           "frac_mfma_peak": r["TFLOP/s"] / MFMA_BF16_PEAK_TFLOPS}
        for model in DECODE_MODELS:
            r = run_decode_model(32 if model == "decode_1b" else 16, 4, model)
            extra[model] = {"us_per_token": r["us_per_token"], "tokens/s": r["tokens_per_s"],
                            "GB/s": r["bytes_per_token"] / (r["us_per_token"] * 1e-6) / 1e9,
                            "frac_hbm_peak": r["bytes_per_token"] / (r["us_per_token"] * 1e-6) / 1e9 / HBM_PEAK_GBS}
        out["other_workloads"] = extra
    print(json.dumps(out))


if __name__ == "__main__":
    main()
