#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one Q4_K matvec y = W.x with W 14336 x 4096 (the decode-shape weight the headline
metric is quoted on), x fp32, all inputs resident in HBM before the clock starts. Successive
steps walk through enough distinct copies of W (1 GiB in total, four times the 256 MB last-level
cache) that no step finds a useful part of its weights there, so the figure is an HBM figure. The timed region is
bracketed by stream synchronisation and timed with HIP events recorded on the stream the
kernels are launched on.

Prints ONE JSON line. `value` is algorithmic bytes per step (weight bytes + x + y,
33 103 872 B) divided by the time per step. `roofline` restates that against the 8 TB/s HBM
peak; `cpu_baseline` is the reference's own CPU matvec (tf_qmatvec_pool compiled from its
sources, or this repository's C restatement when that library is absent) timed on this host
for a bounded sample; `extra` carries the prefill GEMM (second half of the metric) and the
other benchmark shapes.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from gemm_amd import qlinear
import synth  # noqa: E402

HBM_PEAK_GBPS = 8000.0        # MI355X HBM3E, published
BF16_PEAK_TFLOPS = 2500.0     # MI355X dense bf16 MFMA, published
FP32_PEAK_TFLOPS = 157.3      # MI355X dense fp32 MFMA, published
Q4K = synth.GGML_Q4_K

# HBM bytes moved per Q4_K 14336x4096 matvec launch. Not measured by this script: it is the figure of two
# rocprofv3 --pmc runs of `bench.py --probe gemv` (FETCH_SIZE, then WRITE_SIZE), each scaled by what the
# same counter reads for a device-to-device copy of known size, as recorded with its commands in
# PROFILED_TRAFFIC_SOURCE. It changes only when the kernel's loads change and the profile is taken again;
# tests/test_profiles.py fails when the two files disagree.
PROFILED_TRAFFIC_BYTES = 33297298
PROFILED_TRAFFIC_SOURCE = "profiles/gemv_q4k_14336x4096.md"


def gemv_bytes(type_id, n_rows, n_cols):
    return n_rows * synth.row_bytes(type_id, n_cols) + 4 * n_cols + 4 * n_rows


SPIN_UP_MS = 40.0  # untimed launches of the measured kernel before the warm-up steps of the headline: the shader and
# memory clocks of an idle device take tens of milliseconds of work to settle (a step is 8-9 us)


def time_gemv(type_id, n_rows, n_cols, steps, warmup, min_total_bytes=1 << 30, max_copies=40, spin_up_ms=0.0):
    """-> (ms per step, number of weight copies)"""
    W = synth.make_weights(type_id, n_rows, n_cols, seed=20260 + type_id)
    x = synth.make_activation(n_cols, seed=7)
    copies = max(2, min(max_copies, -(-min_total_bytes // W.nbytes)))
    dWs = [qlinear.DevBuf.from_numpy(W) for _ in range(copies)]
    dx = qlinear.DevBuf.from_numpy(x)
    dy = qlinear.DevBuf(n_rows * 4)
    t_end = time.time() + spin_up_ms * 1e-3
    while time.time() < t_end:
        for i in range(64):
            qlinear.gemv_dev(type_id, dWs[i % copies], dx, dy, n_rows, n_cols)
        qlinear.sync()
    for i in range(warmup):
        qlinear.gemv_dev(type_id, dWs[i % copies], dx, dy, n_rows, n_cols)
    qlinear.sync()
    qlinear.timer_begin()
    for i in range(steps):
        qlinear.gemv_dev(type_id, dWs[i % copies], dx, dy, n_rows, n_cols)
    ms = qlinear.timer_end()  # records the end event on the stream and waits for it
    qlinear.sync()
    for d in dWs:
        d.free()
    return ms / steps, copies


def time_fused(steps):
    """Q4_K, hidden 4096, FFN 14336, 8 KV heads of 128: one launch per fused call shape against the
    separate launches it replaces. -> {name: us}"""
    K, FF = 4096, 14336
    x = qlinear.DevBuf.from_numpy(synth.make_activation(K, seed=3) * np.float32(0.05))
    h = qlinear.DevBuf.from_numpy(synth.make_activation(FF, seed=4))

    def copies(rows, cols, n, seed):
        W = synth.make_weights(Q4K, rows, cols, seed=seed)
        return [qlinear.DevBuf.from_numpy(W) for _ in range(n)]

    def run(fn, n):
        for i in range(n):
            fn(i)
        qlinear.sync()
        qlinear.timer_begin()
        for i in range(steps):
            fn(i % n)
        return round(qlinear.timer_end() / steps * 1e3, 2)

    out = {}
    n = 6
    Wg, Wu = copies(FF, K, n, 51), copies(FF, K, n, 52)
    y1, y2 = qlinear.DevBuf(FF * 4), qlinear.DevBuf(FF * 4)
    out["gate,up: two launches (no activation)"] = run(
        lambda i: (qlinear.gemv_dev(Q4K, Wg[i], x, y1, FF, K), qlinear.gemv_dev(Q4K, Wu[i], x, y2, FF, K)), n)
    out["gate+up+silu: one launch"] = run(lambda i: qlinear.gemv_silu_mul_dev(Q4K, Wg[i], Wu[i], x, y1, FF, K), n)
    for d in Wg + Wu:
        d.free()
    n = 24
    Wq, Wk, Wv = copies(4096, K, n, 53), copies(1024, K, n, 54), copies(1024, K, n, 55)
    q, k, v = qlinear.DevBuf(4096 * 4), qlinear.DevBuf(1024 * 4), qlinear.DevBuf(1024 * 4)
    out["q,k,v: three launches"] = run(
        lambda i: (qlinear.gemv_dev(Q4K, Wq[i], x, q, 4096, K), qlinear.gemv_dev(Q4K, Wk[i], x, k, 1024, K),
                   qlinear.gemv_dev(Q4K, Wv[i], x, v, 1024, K)), n)
    out["q,k,v: one launch"] = run(
        lambda i: qlinear.gemv_multi_dev(Q4K, [Wq[i], Wk[i], Wv[i]], [q, k, v], [4096, 1024, 1024], x, K), n)
    for d in Wq + Wk + Wv:
        d.free()
    n = 12
    Wd = copies(K, FF, n, 56)
    out["down 4096x14336"] = run(lambda i: qlinear.gemv_dev(Q4K, Wd[i], h, q, K, FF), n)
    out["down + residual: one launch"] = run(lambda i: qlinear.gemv_add_dev(Q4K, Wd[i], h, q, K, FF), n)
    for d in Wd + [x, h, y1, y2, q, k, v]:
        d.free()
    return out


def time_decode_step_linear(n_layers=32, steps=5, mix=False):
    """The block-quantized linear operators of one decode step of a Llama-3-8B-shaped model (hidden
    4096, FFN 14336, 32 query / 8 KV heads of 128, vocabulary 128256), all Q4_K except a Q6_K output
    projection (mix=True: V and down projections in Q6_K in the layers where the usual 4-bit K-quant mix puts
    them - the first and last eighth and every third layer between; V then takes a launch of its own),
    each layer with its own weights (3.6 GB in all), as 4 launches per layer + 2:
    Q/K/V in one launch, attention output + residual, gate+up+SiLU, down + residual; then the output
    projection with the greedy pick. Attention, norms and RoPE are outside this library and not run.
    -> dict"""
    K, FF, KV, V = 4096, 14336, 1024, 128256
    Q6K = synth.GGML_Q6_K

    def dev(tid, rows, cols, seed):
        return qlinear.DevBuf.from_numpy(synth.make_weights(tid, rows, cols, seed=seed))

    # one set of host tensors, uploaded once per layer (the values do not matter for timing)
    hq, hk, hv = (synth.make_weights(Q4K, r, K, seed=61 + i) for i, r in enumerate((K, KV, KV)))
    ho, hg, hu = (synth.make_weights(Q4K, r, K, seed=64 + i) for i, r in enumerate((K, FF, FF)))
    hd = synth.make_weights(Q4K, K, FF, seed=67)
    hv6, hd6 = synth.make_weights(Q6K, KV, K, seed=69), synth.make_weights(Q6K, K, FF, seed=70)

    def more_bits(i):
        return mix and (i < n_layers // 8 or i >= 7 * n_layers // 8 or (i - n_layers // 8) % 3 == 2)

    layers = [[qlinear.DevBuf.from_numpy(h) for h in (hq, hk, hv6 if more_bits(i) else hv, ho, hg, hu,
                                                       hd6 if more_bits(i) else hd)] for i in range(n_layers)]
    Wout = dev(Q6K, V, K, 68)
    x = qlinear.DevBuf.from_numpy(synth.make_activation(K, seed=5) * np.float32(0.05))
    q, k, v = qlinear.DevBuf(K * 4), qlinear.DevBuf(KV * 4), qlinear.DevBuf(KV * 4)
    h = qlinear.DevBuf(FF * 4)
    logits, pick = qlinear.DevBuf(V * 4), qlinear.DevBuf(qlinear.ARGMAX_RESULT_BYTES)

    def step(stream=None):
        for i, (Wq, Wk, Wv, Wo, Wg, Wu, Wd) in enumerate(layers):
            if more_bits(i):
                qlinear.gemv_multi_dev(Q4K, [Wq, Wk], [q, k], [K, KV], x, K, stream)
                qlinear.gemv_dev(Q6K, Wv, x, v, KV, K, stream)
            else:
                qlinear.gemv_multi_dev(Q4K, [Wq, Wk, Wv], [q, k, v], [K, KV, KV], x, K, stream)
            qlinear.gemv_add_dev(Q4K, Wo, q, x, K, K, stream)     # attention output (stand-in input: q) + residual
            qlinear.gemv_silu_mul_dev(Q4K, Wg, Wu, x, h, FF, K, stream)
            qlinear.gemv_add_dev(Q6K if more_bits(i) else Q4K, Wd, h, x, K, FF, stream)
        qlinear.gemv_argmax_dev(Q6K, Wout, x, logits, pick, V, K, stream)

    step()
    qlinear.sync()
    t_host = time.time()
    qlinear.timer_begin()
    for _ in range(steps):
        step()
    host_ms = (time.time() - t_host) * 1e3 / steps  # time to enqueue one step from Python
    ms = qlinear.timer_end() / steps
    n_more = sum(more_bits(i) for i in range(n_layers))
    weight_bytes = (n_layers * sum(a.nbytes for a in (hq, hk, hv, ho, hg, hu, hd)) + V * synth.row_bytes(Q6K, K) +
                    n_more * (hv6.nbytes + hd6.nbytes - hv.nbytes - hd.nbytes))
    # the same step captured once into a HIP graph and replayed (the entry points only enqueue kernels)
    hip = ctypes.CDLL("libamdhip64.so")
    stream, graph, gexec = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p()
    graph_ms = None
    if hip.hipStreamCreate(ctypes.byref(stream)) == 0:
        ok = hip.hipStreamBeginCapture(stream, 0) == 0
        if ok:
            step(stream)
            ok = hip.hipStreamEndCapture(stream, ctypes.byref(graph)) == 0
        ok = ok and hip.hipGraphInstantiate(ctypes.byref(gexec), graph, None, None, ctypes.c_size_t(0)) == 0
        if ok:
            hip.hipGraphLaunch(gexec, stream)
            qlinear.sync(stream)
            qlinear.timer_begin(stream)
            for _ in range(steps):
                hip.hipGraphLaunch(gexec, stream)
            graph_ms = qlinear.timer_end(stream) / steps
            hip.hipGraphExecDestroy(gexec)
        if graph:
            hip.hipGraphDestroy(graph)
        hip.hipStreamDestroy(stream)
    for bufs in layers:
        for d in bufs:
            d.free()
    for d in (Wout, x, q, k, v, h, logits, pick):
        d.free()
    return {"ms_per_token": round(ms, 4), "host_enqueue_ms": round(host_ms, 4),
            "ms_per_token_graph_replay": None if graph_ms is None else round(graph_ms, 4),
            "launches": 4 * n_layers + n_more + 3, "layers_with_q6_K_v_and_down": n_more,
            "weight_bytes": weight_bytes,
            "GB/s": round(weight_bytes / (ms * 1e-3) / 1e9, 1),
            "hbm_frac": round(weight_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}


def time_prefill_chunk_linear(n_tok=512, n_layers=32, steps=3):
    """The block-quantized linear operators of one 512-token prefill chunk of the same Llama-3-8B-shaped
    model: seven Q4_K x bf16 GEMMs per layer (Q, K, V, attention output, gate, up, down) through
    qlin_gemm_bf16_any_dev (large-tile kernel for gate and up, small-tile kernel for the 4096- and
    1024-row tensors), each layer with its own weights; inputs are bf16 buffers of the right shapes (attention, norms, the SiLU product and
    the fp32 -> bf16 conversions between the operators are not run). -> dict"""
    K, FF, KV = 4096, 14336, 1024
    shapes = ((K, K), (KV, K), (KV, K), (K, K), (FF, K), (FF, K), (K, FF))
    host = [synth.make_weights(Q4K, r, c, seed=81 + i) for i, (r, c) in enumerate(shapes)]
    layers = [[qlinear.DevBuf.from_numpy(h) for h in host] for _ in range(n_layers)]
    xk = qlinear.DevBuf.from_numpy(synth.to_bf16_bits(synth.make_activation(K, seed=6, tokens=n_tok)))
    xff = qlinear.DevBuf.from_numpy(synth.to_bf16_bits(synth.make_activation(FF, seed=7, tokens=n_tok)))
    out = qlinear.DevBuf(n_tok * FF * 4)
    ws = qlinear.DevBuf(qlinear.gemm_bf16_any_workspace_bytes(FF, K))

    def step():
        for W in layers:
            for i, (r, c) in enumerate(shapes):
                qlinear.gemm_bf16_any_dev(Q4K, W[i], xff if c == FF else xk, out, r, c, n_tok, c, r, ws)

    step()
    qlinear.sync()
    qlinear.timer_begin()
    for _ in range(steps):
        step()
    ms = qlinear.timer_end() / steps
    flops = 2.0 * n_tok * n_layers * sum(r * c for r, c in shapes)
    # Q, K and V of a layer in one launch (qlin_gemm_bf16_multi_dev), gate and up in another, the other two as before
    outs = [qlinear.DevBuf(n_tok * r * 4) for r, _ in shapes[:3]]
    gu = [out, qlinear.DevBuf(n_tok * FF * 4)]

    def step_qkv():
        for W in layers:
            qlinear.gemm_bf16_multi_dev(Q4K, W[:3], xk, outs, [r for r, _ in shapes[:3]], K, n_tok, K,
                                        [r for r, _ in shapes[:3]], ws)
            qlinear.gemm_bf16_any_dev(Q4K, W[3], xk, out, K, K, n_tok, K, K, ws)
            qlinear.gemm_bf16_multi_dev(Q4K, W[4:6], xk, gu, [FF, FF], K, n_tok, K, [FF, FF], ws)
            qlinear.gemm_bf16_any_dev(Q4K, W[6], xff, out, K, FF, n_tok, FF, K, ws)

    step_qkv()
    qlinear.sync()
    qlinear.timer_begin()
    for _ in range(steps):
        step_qkv()
    ms_qkv = qlinear.timer_end() / steps
    for d in outs + gu[1:]:
        d.free()
    # the same chunk for an engine that spends HBM on bf16 copies of its weights (decoded once at load):
    # every GEMM is then the dense library GEMM on the cached copy
    BF16 = synth.GGML_BF16
    cached = []
    for W in layers:
        row = []
        for i, (r, c) in enumerate(shapes):
            b = qlinear.DevBuf(r * c * 2)
            qlinear.dequant_bf16_dev(Q4K, W[i], b, r, c)
            row.append(b)
        cached.append(row)

    def step_cached():
        for Wb in cached:
            for i, (r, c) in enumerate(shapes):
                qlinear.gemm_bf16_any_dev(BF16, Wb[i], xff if c == FF else xk, out, r, c, n_tok, c, r, ws)

    step_cached()
    qlinear.sync()
    qlinear.timer_begin()
    for _ in range(steps):
        step_cached()
    ms_cached = qlinear.timer_end() / steps
    for bufs in layers + cached:
        for d in bufs:
            d.free()
    for d in (xk, xff, out, ws):
        d.free()
    return {"ms_per_chunk": round(ms, 3), "tokens": n_tok, "tokens_per_s": round(n_tok / (ms * 1e-3)),
            "launches": 7 * n_layers, "TFLOP/s": round(flops / (ms * 1e-3) / 1e12, 1),
            "mfma_frac": round(flops / (ms * 1e-3) / 1e12 / BF16_PEAK_TFLOPS, 4),
            "with_q_k_v_in_one_launch_and_gate_up_in_one": {"ms_per_chunk": round(ms_qkv, 3), "tokens_per_s": round(n_tok / (ms_qkv * 1e-3)),
                                         "launches": 4 * n_layers, "TFLOP/s": round(flops / (ms_qkv * 1e-3) / 1e12, 1)},
            "with_cached_bf16_copies_of_the_weights": {
                "ms_per_chunk": round(ms_cached, 3), "tokens_per_s": round(n_tok / (ms_cached * 1e-3)),
                "TFLOP/s": round(flops / (ms_cached * 1e-3) / 1e12, 1),
                "extra_HBM_bytes": 2 * n_layers * sum(r * c for r, c in shapes)}}


def time_gemm(n_tok, n_rows, n_cols, steps, warmup):
    W = synth.make_weights(Q4K, n_rows, n_cols, seed=31)
    Xb = synth.to_bf16_bits(synth.make_activation(n_cols, seed=32, tokens=n_tok))
    dW, dX = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(Xb)
    dY = qlinear.DevBuf(n_tok * n_rows * 4)
    for _ in range(warmup):
        qlinear.gemm_bf16_dev(Q4K, dW, dX, dY, n_rows, n_cols, n_tok, n_cols, n_rows)
    qlinear.sync()
    qlinear.timer_begin()
    for _ in range(steps):
        qlinear.gemm_bf16_dev(Q4K, dW, dX, dY, n_rows, n_cols, n_tok, n_cols, n_rows)
    ms = qlinear.timer_end()
    for d in (dW, dX, dY):
        d.free()
    return ms / steps


def time_host_boundary(n_rows, n_cols, calls=200):
    """qlin_matvec through host pointers: W registered (resident in HBM), x uploaded and y downloaded
    on every call. -> ms per call"""
    lib = qlinear.load()
    W = synth.make_weights(Q4K, n_rows, n_cols, seed=77)
    x = synth.make_activation(n_cols, seed=78)
    y = np.zeros(n_rows, np.float32)
    qlinear.check(lib.qlin_weight_register(W.ctypes.data, W.nbytes))
    for _ in range(5):
        qlinear.check(lib.qlin_matvec(y.ctypes.data, W.ctypes.data, Q4K, n_cols, x.ctypes.data, n_rows))
    t0 = time.perf_counter()
    for _ in range(calls):
        qlinear.check(lib.qlin_matvec(y.ctypes.data, W.ctypes.data, Q4K, n_cols, x.ctypes.data, n_rows))
    dt = (time.perf_counter() - t0) / calls
    qlinear.check(lib.qlin_weight_unregister(W.ctypes.data))
    return dt * 1e3


def time_moe(steps, warmup, n_expert=128, n_embd=2048, n_ff=768, top_k=8, n_tok=64, copies=2, types=None):
    """Grouped MoE expert FFN: -> (ms per step, algorithmic bytes per step, flops per step).
    types = formats of (gate, up, down); default all Q4_K"""
    types = types or (Q4K, Q4K, Q4K)
    sets = []
    for c in range(copies):
        sets.append([qlinear.DevBuf.from_numpy(synth.make_weights(types[i], n_expert * r, k, seed=900 + 3 * c + i))
                     for i, (r, k) in enumerate(((n_ff, n_embd), (n_ff, n_embd), (n_embd, n_ff)))])
    Xb = synth.to_bf16_bits(synth.make_activation(n_embd, seed=41, tokens=n_tok))
    dX = qlinear.DevBuf.from_numpy(Xb)
    dl = qlinear.DevBuf.from_numpy(synth.make_router_logits(n_tok, n_expert, seed=42))
    di, dw = qlinear.DevBuf(n_tok * top_k * 4), qlinear.DevBuf(n_tok * top_k * 4)
    dout = qlinear.DevBuf(n_tok * n_embd * 4)
    dws = qlinear.DevBuf(qlinear.moe_workspace_bytes(n_tok, top_k, n_embd, n_ff, n_expert))
    qlinear.moe_route_dev(dl, n_tok, n_expert, top_k, di, dw)
    qlinear.sync()
    routed = len(np.unique(di.to_numpy(np.int32, (n_tok, top_k))))

    def step(i):
        g, u, d = sets[i % copies]
        qlinear.moe_ffn_types_dev(types, g, u, d, dX, di, dw, dout, n_tok, top_k, n_embd, n_ff, n_expert, dws)

    for i in range(warmup):
        step(i)
    qlinear.sync()
    qlinear.timer_begin()
    for i in range(steps):
        step(i)
    ms = qlinear.timer_end()
    expert_bytes = (n_ff * (synth.row_bytes(types[0], n_embd) + synth.row_bytes(types[1], n_embd)) +
                    n_embd * synth.row_bytes(types[2], n_ff))
    nbytes = routed * expert_bytes + n_tok * n_embd * 2 + n_tok * n_embd * 4 + n_tok * top_k * 8
    flops = 2.0 * n_tok * top_k * 3 * n_ff * n_embd
    for b in [x for st in sets for x in st] + [dX, dl, di, dw, dout, dws]:
        b.free()
    return ms / steps, nbytes, flops, routed


def cpu_baseline(n_rows, n_cols, budget_s=12.0):
    """The reference CPU matvec on this host, all cores the process may use; bounded sample."""
    from oracle import pyoracle  # the only use of the oracle package here: the reported CPU baseline
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = max(1, min(cores, 64))
    W = synth.make_weights(Q4K, n_rows, n_cols, seed=20260 + Q4K)
    x = synth.make_activation(n_cols, seed=7)
    nbytes = gemv_bytes(Q4K, n_rows, n_cols)
    if pyoracle.Reference.available():
        ref, kind = pyoracle.Reference(), "reference"
        run = lambda nt, it: ref.qmatvec_pool_time(Q4K, W, x, n_cols, nt, it)  # noqa: E731
    else:
        orc, kind = pyoracle.Oracle(), "port"
        run = lambda nt, it: orc.gemv_f32_time(Q4K, W, x, n_cols, nt, it)  # noqa: E731
    t1 = run(1, 2)                                    # one thread, to size the sample
    iters1 = max(2, int(budget_s * 0.4 / max(t1, 1e-6)))
    t1 = run(1, iters1)
    tn = run(cores, 3)
    itersn = max(3, int(budget_s * 0.6 / max(tn, 1e-6)))
    tn = run(cores, itersn)
    return {
        "value": round(nbytes / tn / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": kind,
        "sample": "Q4_K 14336x4096 matvec, %d calls on %d threads (%.2f ms/call) after %d calls on 1 thread "
                  "(%.2f ms/call, %.3f GB/s)" % (itersn, cores, tn * 1e3, iters1, t1 * 1e3, nbytes / t1 / 1e9),
    }


def cpu_baselines_other(budget_s=14.0):
    """The reference's CPU path (compiled from its sources) on the other benchmark shapes, bounded
    samples: matvecs on one thread and on all cores, the prefill GEMM entry point on a 128-token
    sample, the MoE block as per-token expert-slice matvecs on a 4-token sample. Empty where the
    compiled reference is absent."""
    from oracle import pyoracle  # reported baseline only
    if not pyoracle.Reference.available():
        return {}
    ref = pyoracle.Reference()
    cores = max(1, min(len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1), 64))
    out = {"cores": cores, "kind": "reference"}
    shapes = [("q8_0", synth.GGML_Q8_0, 4096, 4096), ("q4_K", Q4K, 4096, 4096), ("q4_K", Q4K, 4096, 14336),
              ("q5_K", synth.GGML_Q5_K, 4096, 4096), ("iq4_nl", synth.GGML_IQ4_NL, 14336, 4096),
              ("iq2_xxs", synth.GGML_IQ2_XXS, 4096, 14336), ("iq3_s", synth.GGML_IQ3_S, 4096, 14336),
              ("q6_K", synth.GGML_Q6_K, 151936, 4096)]
    per_shape = budget_s * 0.5 / len(shapes)
    mv = {}
    for tname, tid, r, c in shapes:
        W = synth.make_weights(tid, r, c, seed=20260 + tid)
        x = synth.make_activation(c, seed=7)
        b = gemv_bytes(tid, r, c)
        tn = ref.qmatvec_pool_time(tid, W, x, c, cores, 1)
        tn = ref.qmatvec_pool_time(tid, W, x, c, cores, max(1, int(per_shape * 0.6 / max(tn, 1e-6))))
        rows1 = min(r, 4096)  # one thread: a slice of the rows is enough
        t1 = ref.qmatvec_pool_time(tid, W[:rows1], x, c, 1, 1)
        t1 = ref.qmatvec_pool_time(tid, W[:rows1], x, c, 1, max(1, int(per_shape * 0.4 / max(t1, 1e-6))))
        mv["%s_%dx%d" % (tname, r, c)] = {"ms_all_cores": round(tn * 1e3, 3), "GB/s_all_cores": round(b / tn / 1e9, 2),
                                          "GB/s_1_thread": round(gemv_bytes(tid, rows1, c) / t1 / 1e9, 3)}
    out["matvec"] = mv
    # prefill: tf_gemm_f16_mt_tokenmajor on Q4_K 14336x4096 (per-token fallback for this type), 128 tokens
    n_tok, r, c = 128, 14336, 4096
    W = synth.make_weights(Q4K, r, c, seed=60)
    X = synth.make_activation(c, seed=61, tokens=n_tok)
    t0 = time.time()
    ref.gemm_tokenmajor(Q4K, W, X, c, n_threads=cores)
    dt = time.time() - t0
    out["prefill_q4_K_14336x4096"] = {"sample": "%d tokens through tf_gemm_f16_mt_tokenmajor on %d threads" % (n_tok, cores),
                                      "ms_per_token": round(dt / n_tok * 1e3, 3),
                                      "TFLOP/s": round(2.0 * n_tok * r * c / dt / 1e12, 4)}
    # MoE: per token top-8 experts x (gate, up, down) expert-slice matvecs, one thread (tf_qmatvec_expert)
    n_expert, n_embd, n_ff, top_k, sample_tok = 128, 2048, 768, 8, 4
    g = synth.make_weights(Q4K, n_expert * n_ff, n_embd, seed=31)
    d = synth.make_weights(Q4K, n_expert * n_embd, n_ff, seed=33)
    xt = synth.make_activation(n_embd, seed=41)
    ht = synth.make_activation(n_ff, seed=43)
    t0 = time.time()
    for t in range(sample_tok):
        for k in range(top_k):
            e = (17 * t + 5 * k) % n_expert
            ref.qmatvec_expert(Q4K, g, e, xt, n_ff, n_embd)
            ref.qmatvec_expert(Q4K, g, e, xt, n_ff, n_embd)  # up: same shape and type as gate
            ref.qmatvec_expert(Q4K, d, e, ht, n_embd, n_ff)
    dt = (time.time() - t0) / sample_tok
    out["moe_ffn_128x(768x2048)_top8"] = {"sample": "%d tokens x 8 experts x 3 expert-slice matvecs (tf_qmatvec_expert), 1 thread" % sample_tok,
                                         "ms_per_token": round(dt * 1e3, 3), "ms_for_64_tokens": round(dt * 64 * 1e3, 1)}
    return out


def probe(args):
    """Helper for counter collection (see profiles/): run only the named device work."""
    if args.probe == "copy":
        hip = ctypes.CDLL("libamdhip64.so")
        n = 256 << 20
        a, b = qlinear.DevBuf(n), qlinear.DevBuf(n)
        hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
        for _ in range(4):
            assert hip.hipMemcpy(b.ptr, a.ptr, n, 3) == 0  # hipMemcpyDeviceToDevice
        qlinear.sync()
        print(json.dumps({"probe": "copy", "bytes_each": n, "copies": 4}))
    elif args.probe == "tiny":  # a launch that does next to nothing (reads 4 KB): what a launch costs, with and without a profiler
        buf = qlinear.DevBuf(4096)
        for _ in range(200):
            qlinear.probe_hbm_read(buf)
        qlinear.sync()
        qlinear.timer_begin()
        for _ in range(args.steps):
            qlinear.probe_hbm_read(buf)
        print(json.dumps({"probe": "tiny", "ms_per_step": qlinear.timer_end() / args.steps, "steps": args.steps}))
    elif args.probe == "gemv":
        ms, copies = time_gemv(Q4K, 14336, 4096, args.steps, args.warmup, spin_up_ms=args.spin_up_ms)
        print(json.dumps({"probe": "gemv", "ms_per_step": ms, "copies": copies, "steps": args.steps, "warmup": args.warmup}))
    elif args.probe in ("gemv_q8_0", "gemv_q6_K"):
        tid, r, c = (synth.GGML_Q8_0, 4096, 4096) if args.probe == "gemv_q8_0" else (synth.GGML_Q6_K, 151936, 4096)
        ms, copies = time_gemv(tid, r, c, max(10, args.steps // 8), 3)
        print(json.dumps({"probe": args.probe, "ms_per_step": ms, "copies": copies}))
    elif args.probe == "gemv_any":  # --ptype NAME --prows R --pcols C: that matvec only
        tid = {v: k for k, v in list(synth.TYPE_NAMES.items()) + list(synth.DENSE_TYPES.items())}[args.ptype]
        ms, copies = time_gemv(tid, args.prows, args.pcols, max(10, args.steps // 4), 3)
        print(json.dumps({"probe": "gemv_any %s %dx%d" % (args.ptype, args.prows, args.pcols), "ms_per_step": ms,
                          "copies": copies, "bytes": gemv_bytes(tid, args.prows, args.pcols)}))
    elif args.probe == "gemv_q4_0":
        ms, copies = time_gemv(synth.GGML_Q4_0, 14336, 4096, max(10, args.steps // 4), 3)
        print(json.dumps({"probe": args.probe, "ms_per_step": ms, "copies": copies}))
    elif args.probe == "gemv_silu":  # only the fused gate+up+SiLU launch, 2 x (14336 x 4096) Q4_K
        K, FF, n = 4096, 14336, 6
        x = qlinear.DevBuf.from_numpy(synth.make_activation(K, seed=3) * np.float32(0.05))
        Wg = [qlinear.DevBuf.from_numpy(synth.make_weights(Q4K, FF, K, seed=51)) for _ in range(n)]
        Wu = [qlinear.DevBuf.from_numpy(synth.make_weights(Q4K, FF, K, seed=52)) for _ in range(n)]
        y = qlinear.DevBuf(FF * 4)
        steps = max(20, args.steps // 4)
        for i in range(steps + 5):
            if i == 5:
                qlinear.sync()
                qlinear.timer_begin()
            qlinear.gemv_silu_mul_dev(Q4K, Wg[i % n], Wu[i % n], x, y, FF, K)
        print(json.dumps({"probe": args.probe, "ms_per_step": qlinear.timer_end() / steps}))
    elif args.probe == "dequant":
        W = synth.make_weights(Q4K, 14336, 4096, seed=5)
        dW, dO = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf(14336 * 4096 * 4)
        for _ in range(max(5, args.steps // 20)):
            qlinear.dequant_dev(Q4K, dW, dO, 14336, 4096)
        qlinear.sync()
        print(json.dumps({"probe": args.probe}))
    elif args.probe == "decode_step":
        print(json.dumps({"probe": args.probe, **time_decode_step_linear()}))
    elif args.probe == "moe":
        m, b, fl, routed = time_moe(max(10, args.steps // 20), 3, n_tok=args.ptok)  # --ptok N: that many tokens
        print(json.dumps({"probe": "moe", "tokens": args.ptok, "ms_per_step": m, "bytes": b, "routed": routed}))
    elif args.probe == "gemm":
        ms = time_gemm(512, 14336, 4096, max(3, args.steps // 20), 2)
        print(json.dumps({"probe": "gemm", "ms_per_step": ms}))
    elif args.probe == "gemm_any_q6_K":  # Q6_K, 512 tokens: decoded inside the tile kernel
        ms = time_gemm_any(synth.GGML_Q6_K, 512, 14336, 4096, max(3, args.steps // 20), 2)
        print(json.dumps({"probe": "gemm_any_q6_K", "ms_per_step": ms}))
    elif args.probe == "gemm_any_q8_0":  # Q8_0, 512 tokens: decoded inside the tile kernel
        ms = time_gemm_any(synth.GGML_Q8_0, 512, 14336, 4096, max(3, args.steps // 20), 2)
        print(json.dumps({"probe": "gemm_any_q8_0", "ms_per_step": ms}))
    elif args.probe == "gemm_small_q4_K":  # Q4_K 4096 x 4096 at 512 tokens: the 128-token x 64-row tile kernel
        ms = time_gemm_any(Q4K, 512, 4096, 4096, max(3, args.steps // 20), 2)
        print(json.dumps({"probe": "gemm_small_q4_K", "ms_per_step": ms}))
    elif args.probe == "gemm_small_q4_K_m128":  # Q4_K 14336 x 4096 at 128 tokens: the same kernel, one workgroup per compute unit
        ms = time_gemm_any(Q4K, 128, 14336, 4096, max(3, args.steps // 20), 2)
        print(json.dumps({"probe": "gemm_small_q4_K_m128", "ms_per_step": ms}))
    elif args.probe == "gemm_any_iq4_nl":  # IQ4_NL, 512 tokens: decoded inside the large-tile kernel
        ms = time_gemm_any(synth.GGML_IQ4_NL, 512, 14336, 4096, max(3, args.steps // 20), 2)
        print(json.dumps({"probe": "gemm_any_iq4_nl", "ms_per_step": ms}))
    elif args.probe == "gemm_f32_any_q4_K":  # decode to fp32 + dense fp32 library GEMM, Q4_K, 512 tokens
        ms = time_gemm_f32_any(Q4K, 512, 14336, 4096, max(3, args.steps // 20), 2)
        print(json.dumps({"probe": "gemm_f32_any_q4_K", "ms_per_step": ms}))
    elif args.probe == "gemm_fewtok":  # the few-token kernel at 16 tokens
        ms = time_gemm(16, 14336, 4096, max(3, args.steps // 20), 2)
        print(json.dumps({"probe": "gemm_fewtok", "ms_per_step": ms}))


def time_gemm_any(type_id, n_tok, n_rows, n_cols, steps, warmup):
    """Prefill GEMM for any format (qlin_gemm_bf16_any_dev: decoded inside the tile kernel for the formats that has,
    else decode to bf16 in a workspace + dense library GEMM). -> ms per step"""
    W = synth.make_weights(type_id, n_rows, n_cols, seed=70 + type_id)
    Xb = synth.to_bf16_bits(synth.make_activation(n_cols, seed=71, tokens=n_tok))
    dW, dX = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(Xb)
    dY = qlinear.DevBuf(n_tok * n_rows * 4)
    ws = qlinear.DevBuf(qlinear.gemm_bf16_any_workspace_bytes(n_rows, n_cols))
    for _ in range(warmup):
        qlinear.gemm_bf16_any_dev(type_id, dW, dX, dY, n_rows, n_cols, n_tok, n_cols, n_rows, ws)
    qlinear.sync()
    qlinear.timer_begin()
    for _ in range(steps):
        qlinear.gemm_bf16_any_dev(type_id, dW, dX, dY, n_rows, n_cols, n_tok, n_cols, n_rows, ws)
    ms = qlinear.timer_end() / steps
    for b in (dW, dX, dY, ws):
        b.free()
    return ms


def gemm_route(type_id, n_tok, n_rows, n_cols):
    """what qlin_gemm_bf16_any_dev does with this shape when it is handed a workspace"""
    r = qlinear.load().qlin_probe_gemm_route(type_id, n_rows, n_cols, n_tok, n_cols, 1)
    if r:
        return "decoded inside the product (%s tiles), no workspace" % ("256-token x 128-row" if r == 1 else "128-token x 64-row")
    return "dense library product" if type_id == synth.GGML_BF16 else "decode to bf16 + dense library product"


def time_gemm_two_kernels(type_id, n_tok, n_rows, n_cols, steps, warmup):
    """The route the fused kernel replaces, for comparison: decode the weights to bf16 in a workspace, then the
    dense bf16 product on them. -> ms per step"""
    W = synth.make_weights(type_id, n_rows, n_cols, seed=70 + type_id)
    Xb = synth.to_bf16_bits(synth.make_activation(n_cols, seed=71, tokens=n_tok))
    dW, dX = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(Xb)
    dY = qlinear.DevBuf(n_tok * n_rows * 4)
    ws = qlinear.DevBuf(qlinear.gemm_bf16_any_workspace_bytes(n_rows, n_cols))
    dB = qlinear.DevBuf(n_rows * n_cols * 2)

    def step():
        qlinear.dequant_bf16_dev(type_id, dW, dB, n_rows, n_cols)
        qlinear.gemm_bf16_any_dev(synth.GGML_BF16, dB, dX, dY, n_rows, n_cols, n_tok, n_cols, n_rows, ws)

    for _ in range(warmup):
        step()
    qlinear.sync()
    qlinear.timer_begin()
    for _ in range(steps):
        step()
    ms = qlinear.timer_end() / steps
    for b in (dW, dX, dY, ws, dB):
        b.free()
    return ms


def time_gemm_f32_any(type_id, n_tok, n_rows, n_cols, steps, warmup):
    """Exact prefill GEMM for any format: decode to fp32 in a workspace + the library's dense fp32 GEMM
    (fp32 operands and accumulation). -> ms per step"""
    W = synth.make_weights(type_id, n_rows, n_cols, seed=70 + type_id)
    X = synth.make_activation(n_cols, seed=71, tokens=n_tok)
    dW, dX = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(X)
    dY = qlinear.DevBuf(n_tok * n_rows * 4)
    ws = qlinear.DevBuf(qlinear.gemm_f32_any_workspace_bytes(n_rows, n_cols))
    for _ in range(warmup):
        qlinear.gemm_f32_any_dev(type_id, dW, dX, dY, n_rows, n_cols, n_tok, n_cols, n_rows, ws)
    qlinear.sync()
    qlinear.timer_begin()
    for _ in range(steps):
        qlinear.gemm_f32_any_dev(type_id, dW, dX, dY, n_rows, n_cols, n_tok, n_cols, n_rows, ws)
    ms = qlinear.timer_end() / steps
    for b in (dW, dX, dY, ws):
        b.free()
    return ms


def time_hbm_read_rotating(nbytes=33030144, reps=200, total=1 << 30):
    """A read-only streaming kernel over buffers of the headline's weight size, one launch per buffer, rotating
    through 1 GiB of them like the headline: what one launch of that size can reach on this part, launch and
    drain included. -> GB/s"""
    copies = max(2, -(-total // nbytes))
    bufs = [qlinear.DevBuf(nbytes) for _ in range(copies)]
    for b in bufs:
        qlinear.probe_hbm_read(b)
    qlinear.sync()
    qlinear.timer_begin()
    for i in range(reps):
        qlinear.probe_hbm_read(bufs[i % copies])
    ms = qlinear.timer_end() / reps
    for b in bufs:
        b.free()
    return nbytes / (ms * 1e-3) / 1e9


def time_achievable():
    """What the part sustains on the two priced resources: a register-only loop of the GEMM's matrix
    instruction (with the shader clock it ran at) and a streaming read of 512 MiB / of the headline's
    33 MB, both timed with the same event timer as the kernels."""
    out = {}
    qlinear.probe_mfma_bf16(2000); qlinear.sync()
    best = 0.0
    for _ in range(3):
        qlinear.timer_begin()
        fl = qlinear.probe_mfma_bf16(20000)
        ms = qlinear.timer_end()
        best = max(best, fl / (ms * 1e-3) / 1e12)
    out["mfma_bf16_32x32x16_register_loop_TFLOP/s"] = round(best, 1)
    out["shader_clock_MHz_in_that_loop"] = round(qlinear.probe_clocks(), 0)
    big = qlinear.DevBuf(512 << 20)
    qlinear.probe_hbm_read(big)
    qlinear.sync()
    qlinear.timer_begin()
    for i in range(10):
        qlinear.probe_hbm_read(big)
    out["hbm_read_512MiB_GB/s"] = round((512 << 20) / (qlinear.timer_end() / 10 * 1e-3) / 1e9, 1)
    big.free()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--spin-up-ms", type=float, default=SPIN_UP_MS,
                    help="untimed launches of the headline kernel before its warm-up steps, in ms of wall time")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the GEMM and the other shapes")
    ap.add_argument("--ptype", default="iq2_xxs", help="--probe gemv_any: format name")
    ap.add_argument("--prows", type=int, default=4096)
    ap.add_argument("--pcols", type=int, default=14336)
    ap.add_argument("--ptok", type=int, default=64, help="--probe moe: tokens in the batch")
    ap.add_argument("--probe", choices=["gemv_any", "copy", "tiny", "gemv", "gemv_q8_0", "gemv_q6_K", "gemv_q4_0", "gemv_silu", "dequant", "gemm", "gemm_any_q6_K", "gemm_any_q8_0", "gemm_small_q4_K", "gemm_small_q4_K_m128", "gemm_any_iq4_nl", "gemm_f32_any_q4_K", "gemm_fewtok", "moe", "decode_step"], help="device work only, for rocprofv3 runs")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus %d is not supported (the path shards by "
              "weight rows with no exchange)" % args.gpus, file=sys.stderr)
        return 2
    if args.probe:
        probe(args)
        return 0

    name, n_cu, mem = qlinear.device_info()
    n_rows, n_cols = 14336, 4096
    nbytes = gemv_bytes(Q4K, n_rows, n_cols)
    t0 = time.time()
    ms, copies = time_gemv(Q4K, n_rows, n_cols, args.steps, args.warmup, spin_up_ms=args.spin_up_ms)
    gbps = nbytes / (ms * 1e-3) / 1e9
    floor_gbps = time_hbm_read_rotating()

    extra = {}
    if not args.no_extra:
        shapes = [("q4_K", Q4K, 4096, 4096), ("q4_K", Q4K, 4096, 14336), ("q8_0", synth.GGML_Q8_0, 4096, 4096),
                  ("q5_K", synth.GGML_Q5_K, 4096, 4096), ("iq4_nl", synth.GGML_IQ4_NL, 14336, 4096),
                  ("iq2_xxs", synth.GGML_IQ2_XXS, 4096, 14336), ("iq3_s", synth.GGML_IQ3_S, 4096, 14336),
                  ("q6_K", synth.GGML_Q6_K, 151936, 4096),
                  # down projections whose rows run as column ranges or start off the 16-byte grid
                  ("q6_K", synth.GGML_Q6_K, 4096, 14336), ("q6_K", synth.GGML_Q6_K, 4096, 11008),
                  ("q4_K", Q4K, 8192, 28672), ("q5_K", synth.GGML_Q5_K, 3584, 18944)]
        gemv = {}
        for tname, tid, r, c in shapes:
            st = max(20, args.steps // 8)
            m, _ = time_gemv(tid, r, c, st, 4)
            b = gemv_bytes(tid, r, c)
            gemv["%s_%dx%d" % (tname, r, c)] = {"us": round(m * 1e3, 2), "GB/s": round(b / (m * 1e-3) / 1e9, 1)}
        extra["gemv_other_shapes"] = gemv
        gemm = {}
        for M in (16, 128, 512, 2048):
            m = time_gemm(M, 14336, 4096, max(5, args.steps // 40), 2)
            fl = 2.0 * M * 14336 * 4096
            gemm["M=%d" % M] = {"us": round(m * 1e3, 1), "TFLOP/s": round(fl / (m * 1e-3) / 1e12, 1)}
        extra["q4k_prefill_gemm_14336x4096_bf16"] = gemm
        tf = gemm["M=512"]["TFLOP/s"]
        anyfmt = {}
        for tname, tid, M in (("q6_K", synth.GGML_Q6_K, 512), ("q5_K", synth.GGML_Q5_K, 512), ("q8_0", synth.GGML_Q8_0, 512),
                              ("iq4_nl", synth.GGML_IQ4_NL, 512), ("iq4_xs", synth.GGML_IQ4_XS, 512), ("q4_0", synth.GGML_Q4_0, 512),
                              ("q3_K", synth.GGML_Q3_K, 512), ("q2_K", synth.GGML_Q2_K, 512),
                              ("bf16", synth.GGML_BF16, 512), ("q4_K", Q4K, 1024),
                              ("q5_K", synth.GGML_Q5_K, 1024), ("q4_K", Q4K, 2048), ("q6_K", synth.GGML_Q6_K, 2048)):
            m = time_gemm_any(tid, M, 14336, 4096, max(5, args.steps // 40), 2)
            anyfmt["%s_M=%d" % (tname, M)] = {
                "us": round(m * 1e3, 1), "TFLOP/s": round(2.0 * M * 14336 * 4096 / (m * 1e-3) / 1e12, 1),
                "route": gemm_route(tid, M, 14336, 4096)}
        extra["prefill_gemm_any_format_14336x4096"] = anyfmt
        small = {}
        for tname, tid, M, r, c in (("q4_K", Q4K, 512, 4096, 4096), ("q4_K", Q4K, 512, 6144, 4096), ("q4_K", Q4K, 512, 4096, 14336),
                                    ("q4_K", Q4K, 256, 14336, 4096), ("q6_K", synth.GGML_Q6_K, 128, 14336, 4096),
                                    ("q6_K", synth.GGML_Q6_K, 512, 4096, 14336), ("q8_0", synth.GGML_Q8_0, 512, 4096, 4096)):
            m = time_gemm_any(tid, M, r, c, max(5, args.steps // 40), 2)
            small["%s_M=%d_%dx%d" % (tname, M, r, c)] = {
                "us": round(m * 1e3, 1), "TFLOP/s": round(2.0 * M * r * c / (m * 1e-3) / 1e12, 1), "route": gemm_route(tid, M, r, c)}
        extra["prefill_gemm_other_shapes"] = small
        two = {}
        for tname, tid, M in (("q4_K", Q4K, 512), ("q5_K", synth.GGML_Q5_K, 512), ("q6_K", synth.GGML_Q6_K, 512),
                              ("q8_0", synth.GGML_Q8_0, 512)):
            m = time_gemm_two_kernels(tid, M, 14336, 4096, max(5, args.steps // 40), 2)
            two["%s_M=%d" % (tname, M)] = {"us": round(m * 1e3, 1), "TFLOP/s": round(2.0 * M * 14336 * 4096 / (m * 1e-3) / 1e12, 1)}
        extra["prefill_gemm_14336x4096_decode_to_bf16_plus_library_gemm_for_comparison"] = two
        own = {}
        qlinear.check(qlinear.load().qlin_set_dense_gemm_own(1))
        try:
            for tname, tid, M in (("iq4_nl", synth.GGML_IQ4_NL, 512), ("bf16", synth.GGML_BF16, 512), ("iq4_nl", synth.GGML_IQ4_NL, 2048)):
                m = time_gemm_any(tid, M, 14336, 4096, max(5, args.steps // 40), 2)
                own["%s_M=%d" % (tname, M)] = {"us": round(m * 1e3, 1), "TFLOP/s": round(2.0 * M * 14336 * 4096 / (m * 1e-3) / 1e12, 1)}
        finally:
            qlinear.check(qlinear.load().qlin_set_dense_gemm_own(0))
        extra["prefill_gemm_any_format_14336x4096_decode_to_bf16_plus_own_tile_kernel"] = own
        exact = {}
        for tname, tid, M in (("q4_K", Q4K, 512), ("q6_K", synth.GGML_Q6_K, 512), ("q4_K", Q4K, 64)):
            m = time_gemm_f32_any(tid, M, 14336, 4096, max(3, args.steps // 60), 1)
            tfl = 2.0 * M * 14336 * 4096 / (m * 1e-3) / 1e12
            exact["%s_M=%d" % (tname, M)] = {"us": round(m * 1e3, 1), "TFLOP/s": round(tfl, 1),
                                             "fp32_mfma_frac": round(tfl / FP32_PEAK_TFLOPS, 4)}
        extra["prefill_gemm_exact_fp32_14336x4096_decode_to_fp32_plus_library_gemm"] = exact
        extra["achievable_on_this_gpu"] = time_achievable()
        extra["q4k_prefill_gemm_roofline"] = {"bound": "mfma", "achieved": tf, "peak": BF16_PEAK_TFLOPS,
                                              "unit": "TFLOP/s", "frac": round(tf / BF16_PEAK_TFLOPS, 4),
                                              "traffic": None}

        # every other block format at the headline shape, and the fused call shapes of the decode loop
        other = {}
        for tid, tname in synth.TYPE_NAMES.items():
            if tid == Q4K:
                continue
            m, _ = time_gemv(tid, 14336, 4096, max(20, args.steps // 8), 4)
            b = gemv_bytes(tid, 14336, 4096)
            other[tname] = {"us": round(m * 1e3, 2), "GB/s": round(b / (m * 1e-3) / 1e9, 1)}
        extra["gemv_14336x4096_all_formats"] = other
        extra["q4k_fused_decode_shapes"] = time_fused(max(20, args.steps // 8))

        extra["q4k_llama8b_shaped_decode_step_linear_ops"] = time_decode_step_linear()
        extra["q4k_q6k_mix_llama8b_shaped_decode_step_linear_ops"] = time_decode_step_linear(mix=True)
        extra["q4k_llama8b_shaped_prefill_512tok_linear_ops"] = time_prefill_chunk_linear()

        hb = time_host_boundary(n_rows, n_cols)
        extra["host_pointer_matvec_14336x4096"] = {"us": round(hb * 1e3, 1), "GB/s": round(nbytes / (hb * 1e-3) / 1e9, 1),
                                                  "note": "W registered; x H2D and y D2H every call"}
        m, b, fl, routed = time_moe(max(10, args.steps // 20), 3)
        Q6K = synth.GGML_Q6_K
        Q5K = synth.GGML_Q5_K
        for label, tys in (("q4k_q4k_q6k", (Q4K, Q4K, Q6K)), ("q6k", (Q6K, Q6K, Q6K)), ("q5k_q5k_q6k", (Q5K, Q5K, Q6K)),
                           ("q5k", (Q5K, Q5K, Q5K)), ("q8_0", (synth.GGML_Q8_0,) * 3), ("q3k", (synth.GGML_Q3_K,) * 3),
                           ("q2k", (synth.GGML_Q2_K,) * 3)):
            mm, bb, _, _ = time_moe(max(5, args.steps // 40), 2, types=tys)
            extra["moe_ffn_128x(768x2048)_64tok_top8_%s" % label] = {
                "us": round(mm * 1e3, 1), "bytes": bb, "GB/s": round(bb / (mm * 1e-3) / 1e9, 1),
                "hbm_frac": round(bb / (mm * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}
        # decode: one token (the reference's own MoE block) and a few, each token's eight experts read for it alone
        few = {}
        for nt in (1, 2, 4, 8, 16):
            mm, bb, _, rr = time_moe(max(10, args.steps // 10), 3, n_tok=nt)
            few["%d_tok" % nt] = {"us": round(mm * 1e3, 1), "routed_experts": rr,
                                  "GB/s_of_routed_expert_bytes": round(bb / (mm * 1e-3) / 1e9, 1)}
        extra["q4k_moe_ffn_128x(768x2048)_top8_few_tokens"] = few
        extra["q4k_moe_ffn_128x(768x2048)_64tok_top8"] = {
            "us": round(m * 1e3, 1), "routed_experts": routed, "bytes": b, "GB/s": round(b / (m * 1e-3) / 1e9, 1),
            "hbm_frac": round(b / (m * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4), "TFLOP/s": round(fl / (m * 1e-3) / 1e12, 1)}

    out = {
        "metric": "Q4_K GEMV GB/s (% HBM peak); Q4_K prefill GEMM TFLOP/s at M=512",
        "value": round(gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "Q4_K GEMV 14336x4096, batch 1, x fp32 (the configuration the headline metric is quoted on)",
                   "bytes_per_step": nbytes, "weight_copies_rotated": copies, "device": name.strip(),
                   "compute_units": n_cu,
                   "device_spin_up_ms": args.spin_up_ms,
                   "device_spin_up": "untimed launches of the same kernel ahead of the warm-up steps until the clocks "
                                     "of the idle device have settled; the timed region is the given steps only"},
        "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gbps / HBM_PEAK_GBPS, 4),
                     "launch_floor_frac": round(floor_gbps / HBM_PEAK_GBPS, 4),
                     "launch_floor": "a read-only streaming kernel over the same 33 MB per launch, same rotation: %.1f GB/s; "
                                     "what is left of the peak once a launch of this size has filled and drained the "
                                     "chip" % floor_gbps,
                     "traffic": PROFILED_TRAFFIC_BYTES,
                     "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this kernel, scaled by a copy of "
                                       "known size; not re-measured by this run (" + PROFILED_TRAFFIC_SOURCE + ")"},
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(n_rows, n_cols)
        if extra:
            extra["cpu_reference_other_shapes"] = cpu_baselines_other()
    if extra:
        out["extra"] = extra
    out["wall_s"] = round(time.time() - t0, 1)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
