#!/usr/bin/env python3
"""Benchmark of the speculative-decoding verify step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c4|c1|c5] [--lanes B]

A step is one verify of a 16-token draft block by the 27B-shaped dense target (64 layers, hidden 5120,
64 q / 8 kv heads x 128, SwiGLU 25600, vocabulary 151936, Q4_K weights with Q6_K down-projection and
LM head) over a 32K-token INT8 KV context, greedy acceptance, batch 1: BASELINE.json's headline
configuration. Weights and context are synthetic and resident in HBM before the timed region. One JSON
line goes to stdout; progress goes to stderr.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0   # MI355X published HBM3E bandwidth
# Counters cannot be read from inside the run: the HBM bytes a launch of the dominant kernel moves come from the
# committed summary of two rocprofv3 --pmc runs of this file (FETCH_SIZE, then WRITE_SIZE), each scaled by what the same
# counter reads, in the same run, for plain read and copy kernels of known size (--calibrate-traffic).
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "verify_step_c4_hbm_traffic.md")


def measured_traffic(kernel):
    """(bytes per launch, where it was measured) of `kernel` from the committed traffic summary: its line
    `traffic <kernel>: <bytes> bytes per launch` and the summary's `measured at: <commit, date>` line; (None, None) when
    the summary does not hold the kernel."""
    import re
    try:
        text = open(TRAFFIC_SUMMARY).read()
    except OSError:
        return None, None
    found = re.search(r"^traffic " + re.escape(kernel) + r": (\d+) bytes per launch", text, re.M)
    where = re.search(r"^measured at: (.+)$", text, re.M)
    return (int(found.group(1)) if found else None), (where.group(1).strip() if where else None)


def calibrate_traffic(backend):
    """Plain kernels of known size for the counters' scale, over buffers nothing has read: read_bytes streams 256 MiB
    (its fetch counter against 268,435,456 bytes), copy_bytes moves 256 MiB (fetch and write counters against the
    same), four times each over buffers of their own. Their grids (2051 and 4099 workgroups) tell them from every
    other dispatch of the run."""
    import ctypes
    import splash_amd

    class P(ctypes.Structure):
        _fields_ = [("vectors", ctypes.c_uint64)]
    size = 256 << 20
    sources = [backend.allocate_buffer(size, label="calibration source") for _ in range(8)]
    targets = [backend.allocate_buffer(size, label="calibration target") for _ in range(4)]
    folded = backend.allocate_buffer(1 << 20)
    for b in sources:
        b.fill(0x5A)
    g = splash_amd.CommandGraph()
    for i in range(4):
        g.add("read_bytes", [sources[i], folded], P(size // 16), (2051, 1, 1), (256, 1, 1))
    for i in range(4):
        g.add("copy_bytes", [sources[4 + i], targets[i]], P(size // 16), (4099, 1, 1), (256, 1, 1))
    backend.run(g)
    log(f"traffic calibration: 4 reads and 4 copies of {size} bytes")


WORKLOADS = {
    # hidden, q heads, kv heads, head dim, ffn, vocabulary, layers, context, rows
    "c4": dict(hidden=5120, q_heads=64, kv_heads=8, head_dim=128, ffn=25600, vocabulary=151936, layers=64, context=32768, rows=16,
               name="27B-shaped dense verify step, Q4_K (Q6_K down-proj and lm_head), 16-token draft, 32K INT8 context"),
    "c1": dict(hidden=1024, q_heads=16, kv_heads=8, head_dim=64, ffn=3072, vocabulary=32000, layers=2, context=512, rows=16,
               name="2-layer dense verify step (reference plumbing config), Q4_K, 16-token draft, 512-token INT8 context"),
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def device_copy(backend, source, destination, nbytes):
    """destination <- source on the device (copy_bytes kernel)."""
    import ctypes
    import splash_amd

    class P(ctypes.Structure):
        _fields_ = [("vectors", ctypes.c_uint64)]
    g = splash_amd.CommandGraph()
    g.add("copy_bytes", [source, destination], P(nbytes // 16), (2048, 1, 1), (256, 1, 1))
    backend.run(g)


def build_model(backend, w, lanes, prefill_rows=0):
    """The synthetic model: one layer's tensors are generated and re-tiled on the host, every other
    layer holds its own copy in HBM (distinct addresses, so nothing is served from a cache)."""
    import splash_amd
    from splash_amd import ops, synthetic, verify
    rng = np.random.default_rng(20260101)
    H, D, F, V = w["hidden"], w["head_dim"], w["ffn"], w["vocabulary"]
    QW, KW = w["q_heads"] * D, w["kv_heads"] * D
    context_pages = (w["context"] + ops.PAGE_TOKENS - 1) // ops.PAGE_TOKENS
    physical = context_pages * lanes + 1
    gpu = verify.DenseVerify(backend, H, w["q_heads"], w["kv_heads"], D, F, V, w["layers"], max_lanes=lanes,
                             physical_pages=physical, page_table_entries=context_pages * lanes, prefill_rows=prefill_rows)
    table = rng.permutation(physical)[:context_pages * lanes].astype(np.uint64)
    gpu.buffer(verify.PAGE_TABLE).upload(table)

    def image(fmt, n, k):
        t0 = time.time()
        img = ops.pack_gguf_image(fmt, synthetic.native(rng, fmt, n, k), n, k)
        log(f"  tensor {n}x{k} fmt {fmt}: {img.nbytes / 1e6:.1f} MB in {time.time() - t0:.1f}s")
        return img
    tensors = dict(q=(ops.FMT_Q4K, QW, H), k=(ops.FMT_Q4K, KW, H), v=(ops.FMT_Q4K, KW, H), o=(ops.FMT_Q4K, H, QW),
                   gate=(ops.FMT_Q4K, F, H), up=(ops.FMT_Q4K, F, H), down=(ops.FMT_Q6K, H, F))
    first = {name: backend.from_array(image(*shape), label=name) for name, shape in tensors.items()}
    norm = lambda n: backend.from_array(((1 + 0.05 * rng.standard_normal(n)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16))
    norms = dict(input=norm(H), post=norm(H), q=norm(D), k=norm(D), final=norm(H))
    for layer in range(w["layers"]):
        bufs = first if layer == 0 else {}
        if layer:
            for name in tensors:
                bufs[name] = backend.allocate_buffer(first[name].size_bytes, label=name)
                device_copy(backend, first[name], bufs[name], first[name].size_bytes)
        P = lambda segs, k: ops.Projection([(tensors[n][0], tensors[n][1], bufs[n]) for n in segs], k)
        gpu.set_layer(layer, P(["q", "k", "v"], H), P(["o"], QW), P(["gate"], H), P(["up"], H), P(["down"], F),
                      norms["input"], norms["post"], norms["q"], norms["k"])
        if layer % 16 == 15:
            log(f"  layer {layer + 1}/{w['layers']} resident")
    embedding = backend.from_array(synthetic.native(rng, ops.FMT_Q4K, V, H), label="embedding")
    head = ops.Projection([(ops.FMT_Q6K, V, backend.from_array(image(ops.FMT_Q6K, V, H), label="head"))], H, float32=True)
    gpu.set_head(ops.FMT_Q4K, embedding, norms["final"], head)
    # the INT8 context: one layer's pages from the host, the others copied on the device
    pages = synthetic.kv_pages(rng, w["kv_heads"], D, physical)
    pool0 = gpu.buffer(verify.KV_POOL, 0)
    pool0.upload(pages)
    for layer in range(1, w["layers"]):
        device_copy(backend, pool0, gpu.buffer(verify.KV_POOL, layer), pages.nbytes)
    return gpu


def cpu_baseline(w):
    """The CPU oracle (a port of the reference's test references) timed on this host's cores on a bounded
    sample of the same step: one layer's projections at reduced width and one layer's attention at reduced
    context, scaled to the whole step by algorithmic bytes."""
    from tests import oracle as orc
    from splash_amd import synthetic
    cores = os.cpu_count() or 1
    rng = np.random.default_rng(5)
    rows, H, F = w["rows"], w["hidden"], w["ffn"]
    x = orc.f32_to_bf16(rng.standard_normal((rows, H)).astype(np.float32))
    PASSES = 120
    sample_n = F      # the whole gate projection, and a quarter of the down projection's columns
    t0 = time.time()
    bytes_done = 0
    for fmt, n, k, xin in ((orc.FMT_Q4K, sample_n, H, x), (orc.FMT_Q6K, max(16, H // 4), F, None)):
        nat = synthetic.native(rng, fmt, n, k)
        xi = xin if xin is not None else orc.f32_to_bf16(rng.standard_normal((rows, k)).astype(np.float32))
        t1 = time.time()
        for _ in range(PASSES):
            orc.gemm(fmt, nat, xi, n, want=("chain",), threads=0)
            bytes_done += nat.nbytes
        log(f"  cpu gemm fmt {fmt} {n}x{k} x{PASSES}: {time.time() - t1:.2f}s")
    gemm_seconds = time.time() - t0
    # attention sample: all heads, reduced context
    ctx = min(w["context"], 16384)
    D, KH, QH = w["head_dim"], w["kv_heads"], w["q_heads"]
    pages = (ctx + rows + 255) // 256
    kc = rng.integers(-127, 128, (pages, KH, 256, D)).astype(np.int8)
    vc = rng.integers(-127, 128, (pages, KH, 256, D)).astype(np.int8)
    ks = np.full((pages, KH, 256), 0.03, dtype=np.float32)
    q = orc.f32_to_bf16(rng.standard_normal((rows, QH, D)).astype(np.float32))
    anc = np.array([(2 << r) - 1 for r in range(rows)], dtype=np.uint32)
    t1 = time.time()
    orc.attention(q, kc, ks, vc, ks, np.arange(pages, dtype=np.uint32), anc, ctx, want64=False, threads=0)
    attention_seconds = time.time() - t1
    log(f"  cpu attention ctx {ctx}: {attention_seconds:.2f}s")
    weight_bytes = w["layers"] * ((w["q_heads"] + 2 * KH) * D * H * 0.5625 + H * QH * D * 0.5625 + 2 * F * H * 0.5625 + H * F * 0.8203125) \
        + w["vocabulary"] * H * 0.8203125
    kv_bytes = w["layers"] * w["context"] * KH * (2 * D + 4)
    step_seconds = gemm_seconds * weight_bytes / bytes_done + attention_seconds * (w["context"] / ctx) * w["layers"]
    return {"value": round(step_seconds * 1e3, 1), "unit": "ms", "cores": cores, "kind": "port",
            "sample": f"oracle register-rule GEMM of {sample_n}x{H} Q4_K and {max(16, H // 4)}x{F} Q6_K at {rows} rows ({PASSES} passes each), oracle paged "
                      f"attention of one layer at {ctx}-token context; scaled to the step by weight bytes and context length "
                      f"({gemm_seconds + attention_seconds:.1f}s of CPU work on {cores} threads)"}


def time_c2_ops(backend):
    """BASELINE.json config 2: each projection of the 27B shape alone at M = 1, 4, 8, 16, 32 rows, over a ring of weight
    copies larger than twice the 256 MB memory-side cache so that every pass reads HBM; per-dispatch GPU time (HIP
    events around each dispatch), median over the ring passes after the first. Prints one JSON line."""
    import splash_amd
    from splash_amd import ops, synthetic
    rng = np.random.default_rng(0)
    bf = lambda a: (np.ascontiguousarray(a, np.float32).view(np.uint32) >> 16).astype(np.uint16)
    linear = ops.Linear(backend)
    H, F, Q, KV = 5120, 25600, 8192, 1024
    cases = [("gate_up", ops.FMT_Q4K, [F], H, ops.EPILOGUE_GATE_UP, 2), ("qkv", ops.FMT_Q4K, [Q, KV, KV], H, ops.EPILOGUE_NONE, 1),
             ("o_proj", ops.FMT_Q4K, [H], Q, ops.EPILOGUE_RESIDUAL, 1), ("down", ops.FMT_Q6K, [H], F, ops.EPILOGUE_RESIDUAL, 1)]
    results = []
    for name, fmt, widths, K, epilogue, tensors in cases:
        N = sum(widths)
        weight_bytes = tensors * ops.gguf_image_bytes(fmt, N, K)
        copies = int(np.ceil(2 * 268.4e6 / weight_bytes)) + 1
        images = [rng.integers(0, 256, ops.gguf_image_bytes(fmt, n, K), dtype=np.uint8) for n in widths]
        ring = [ops.Projection([(fmt, n, backend.from_array(im)) for n, im in zip(widths, images)], K) for _ in range(copies)]
        gates = [ops.Projection([(fmt, N, backend.from_array(images[0]))], K) for _ in range(copies)] if tensors == 2 else None
        # the CPU oracle's register-rule projection of the same matrices on this host's cores, whole, at 16 rows
        from tests import oracle as orc
        natives = [synthetic.native(rng, fmt, n, K) for n in widths] * tensors
        x16 = orc.f32_to_bf16(rng.standard_normal((16, K)).astype(np.float32))
        rounds = []
        for _ in range(5):
            t0 = time.time()
            for nat, n in zip(natives, list(widths) * tensors):
                orc.gemm(fmt, nat, x16, n, want=("chain",), threads=0)
            rounds.append(time.time() - t0)
        cpu_us = float(np.median(rounds[1:]) * 1e6)
        log(f"  {name:8s} M=16 on the CPU ({os.cpu_count()} threads): {cpu_us / 1e3:8.2f} ms")
        results.append({"op": name, "device": "cpu", "cores": os.cpu_count(), "kind": "port", "M": 16, "us": round(cpu_us, 1),
                        "GB/s": round(weight_bytes / cpu_us / 1e3, 2)})
        del natives
        for M in (1, 4, 8, 16, 32):
            x = backend.from_array(bf(rng.standard_normal((M, K))))
            out, residual = backend.allocate_buffer(M * N * 4), backend.allocate_buffer(M * N * 2)
            plan = linear.plan(ring[0], M, epilogue)
            scratch = linear.scratch_for(backend, [plan])
            graph = splash_amd.CommandGraph()
            linear.add(graph, ring[0], plan, x, out, scratch, residual=residual, gate=gates[0] if gates else None)   # table pass + first
            passes = 4
            for _ in range(passes):
                for c in range(copies):
                    linear.add(graph, ring[c], plan, x, out, scratch, residual=residual, gate=gates[c] if gates else None, prepared=True)
            backend.set_dispatch_profiling(True)
            _, _, per = backend.run(graph, profiled=True)
            backend.set_dispatch_profiling(False)
            us = float(np.median(np.array(per[2 + copies:]) * 1e6))
            out_bytes = M * N * 2
            algorithmic = weight_bytes + M * K * 2 + out_bytes
            results.append({"op": name, "format": "q4_k" if fmt == ops.FMT_Q4K else "q6_k", "N": N * tensors if tensors == 2 else N, "K": K,
                            "M": M, "splits": plan.splits, "us": round(us, 2), "GB/s": round(algorithmic / us / 1e3, 1),
                            "frac": round(algorithmic / us / 1e3 / HBM_PEAK_GBS, 4)})
            log(f"  {name:8s} M={M:2d} splits={plan.splits:2d} {us:7.2f} us {algorithmic / us / 1e3:7.1f} GB/s")
            del graph, x, out, residual, scratch
        # the column rule (every addition in the reference's order) at its one and two rows: a dispatch a tensor
        for M in (1, 2):
            x = backend.from_array(bf(rng.standard_normal((M, K))))
            out, residual = backend.allocate_buffer(M * N * 4), backend.allocate_buffer(M * N * 2)
            plan = linear.plan(ring[0], M, epilogue, column=True)
            scratch = linear.scratch_for(backend, [plan])
            graph = splash_amd.CommandGraph()
            passes, each = 3, len(widths)
            for _ in range(passes):
                for c in range(copies):
                    linear.add(graph, ring[c], plan, x, out, scratch, residual=residual, gate=gates[c] if gates else None)
            backend.set_dispatch_profiling(True)
            _, _, per = backend.run(graph, profiled=True)
            backend.set_dispatch_profiling(False)
            adds = np.array(per).reshape(passes * copies, each).sum(axis=1)
            us = float(np.median(adds[copies:]) * 1e6)
            algorithmic = weight_bytes + M * K * 2 + M * N * 2
            results.append({"op": name, "rule": "column", "format": "q4_k" if fmt == ops.FMT_Q4K else "q6_k", "N": N * tensors if tensors == 2 else N,
                            "K": K, "M": M, "dispatches": each, "us": round(us, 2), "GB/s": round(algorithmic / us / 1e3, 1),
                            "frac": round(algorithmic / us / 1e3 / HBM_PEAK_GBS, 4)})
            log(f"  {name:8s} M={M:2d} column rule {us:7.2f} us {algorithmic / us / 1e3:7.1f} GB/s ({each} dispatches)")
            del graph, x, out, residual, scratch
        del ring, gates
    print(json.dumps({"metric": "projection us and GB/s by rows (config 2)", "unit": "us", "n_gpus": 1, "data": "synthetic: random images in a ring past the caches",
                      "roofline_peak_gbs": HBM_PEAK_GBS, "results": results}), flush=True)


def time_prefill_ops(backend):
    """The prefill projection (ops.Linear.add_prefill: the staged rule over a chunk of rows, 128 x 128 a workgroup) at the
    27B shape's matrices and chunks of 512, 2048 and 8192 rows: GPU time of a chunk's dispatches (its table passes and its
    projection; HIP events around each dispatch), median of five. The operations counted are the algorithm's, 2 M N K;
    the kernel issues two bf16 MFMAs a product (a half weight is two bf16 parts). Prints one JSON line; the dense MFMA
    peak is bf16's."""
    import splash_amd
    from splash_amd import ops
    rng = np.random.default_rng(0)
    bf = lambda a: (np.ascontiguousarray(a, np.float32).view(np.uint32) >> 16).astype(np.uint16)
    H, F, Q, KV = 5120, 25600, 8192, 1024
    peak = 2500.0
    results = []
    for name, fmt, N, K in (("qkv", ops.FMT_Q4K, Q + 2 * KV, H), ("gate", ops.FMT_Q4K, F, H), ("down", ops.FMT_Q6K, H, F)):
        projection = ops.Projection([(fmt, N, backend.from_array(rng.integers(0, 256, ops.gguf_image_bytes(fmt, N, K), dtype=np.uint8)))], K)
        for M in (512, 2048, 8192):
            x = backend.from_array(bf(rng.standard_normal((M, K))))
            out = backend.allocate_buffer(M * N * 2)
            table = backend.allocate_buffer(ops.Linear.prefill_table_bytes(K, M))
            graph = splash_amd.CommandGraph()
            repeats = 6
            for _ in range(repeats):
                ops.Linear.add_prefill(graph, projection, x, out, table, M)
            per_chunk = len(graph) // repeats
            backend.set_dispatch_profiling(True)
            _, _, per = backend.run(graph, profiled=True)
            backend.set_dispatch_profiling(False)
            chunks = np.array(per).reshape(repeats, per_chunk)[1:] * 1e6
            us, gemm_us = float(np.median(chunks.sum(axis=1))), float(np.median(chunks[:, -1]))
            tflops = 2.0 * M * N * K / us / 1e6
            results.append({"op": name, "format": "q4_k" if fmt == ops.FMT_Q4K else "q6_k", "N": N, "K": K, "M": M, "us": round(us, 1),
                            "projection_us": round(gemm_us, 1), "TFLOP/s": round(tflops, 1), "frac": round(tflops / peak, 4)})
            log(f"  {name:5s} M={M:5d}: {us:9.1f} us a chunk ({gemm_us:9.1f} us the projection) {tflops:7.1f} TFLOP/s")
            del graph, x, out, table
        del projection
    # The chunked prefill attention (ops.PagedAttention.add_chunk_*): a chunk of one sequence at the 27B geometry over a 32K
    # history, the projection pass of every tile and then the tiles' split and merge, eight tiles a dispatch. Operations
    # counted: 4 D per (row, head, visible token), the history and on average half the chunk.
    from splash_amd import synthetic
    QH, KVH, D, history = 64, 8, 128, 32768
    attention = []
    for M in (128, 512, 2048):
        pages = (history + M + ops.PAGE_TOKENS - 1) // ops.PAGE_TOKENS
        raw = synthetic.kv_pages(rng, KVH, D, 8)
        pool = ops.KvPages(backend, KVH, D, pages, rng.permutation(pages).astype(np.uint64))
        pool.upload(np.tile(raw, ((pages + 7) // 8, 1))[:pages])
        plan = ops.AttentionChunkPlan(QH, KVH, D, [(0, M, history, 0)], rotary_pairs=D // 2, normalize=True)
        sizes = plan.workspace_sizes()

        class Workspace:
            queries, query_sums, partials, partial_sums = (backend.allocate_buffer(b) for b in sizes)
        qkv = backend.from_array(bf(rng.standard_normal((M, (QH + 2 * KVH) * D))))
        norm = backend.from_array(bf(np.ones(D)))
        angles = rng.uniform(0, 6.28, (M, D // 2)).astype(np.float32)
        cos, sin = backend.from_array(np.cos(angles)), backend.from_array(np.sin(angles))
        tree = backend.from_array(ops.chain_tree_rows([min(16, M - at) for at in range(0, M, 16)]))
        out = backend.allocate_buffer(M * QH * D * 2)
        graph = splash_amd.CommandGraph()
        repeats = 4
        for _ in range(repeats):
            ops.PagedAttention.add_chunk_projection(graph, plan, qkv, Workspace, pool, query_norm=norm, key_norm=norm, rope_cos=cos, rope_sin=sin)
            ops.PagedAttention.add_chunk_attention(graph, plan, Workspace, tree, pool, out)
        backend.set_dispatch_profiling(True)
        _, _, per = backend.run(graph, profiled=True)
        backend.set_dispatch_profiling(False)
        us = float(np.median(np.array(per).reshape(repeats, -1)[1:].sum(axis=1)) * 1e6)
        flops = 4.0 * D * QH * M * (history + (M + 1) / 2)
        attention.append({"M": M, "history": history, "dispatches": len(graph) // repeats, "us": round(us, 1), "tokens_per_s": round(M / us * 1e6),
                          "TFLOP/s": round(flops / us / 1e6, 1), "frac": round(flops / us / 1e6 / peak, 4)})
        log(f"  chunk attention M={M:5d} over {history}: {us:9.1f} us ({flops / us / 1e6:6.1f} TFLOP/s of the fp16 peak's {peak:.0f})")
        del graph, pool, Workspace, qkv, out
    # GDN::addPrefill at the 35B-A3B shape (16 key / 32 value heads): prepare, scan and gate of a chunk of one lane and layer.
    gdn = ops.GDN(16, 32)
    states = backend.allocate_buffer(gdn.cell_bytes * 2)
    states.upload(np.zeros(gdn.cell_bytes * 2 // 4, np.float32))
    weights = dict(convolution_weights=backend.from_array(bf(rng.standard_normal((gdn.shape.convolution_dimension, 4)) * 0.4)),
                   decay_weights=backend.from_array((-np.exp(rng.uniform(-1, 1, 32))).astype(np.float32)),
                   time_bias=backend.from_array(bf(rng.uniform(-1, 1, 32))), mixer_norm=backend.from_array(bf(np.ones(128))))
    recurrent = []
    for M in (128, 512, 2048):
        work = gdn.prefill_workspace(backend, M)
        packed = backend.from_array(bf(rng.standard_normal((M, gdn.shape.packed_width))))
        graph = splash_amd.CommandGraph()
        repeats = 4
        for _ in range(repeats):
            gdn.add_prefill(graph, dict(packed=packed, states=states, **weights, **work), 0, M, 0, gdn.cell_bytes)
        backend.set_dispatch_profiling(True)
        _, _, per = backend.run(graph, profiled=True)
        backend.set_dispatch_profiling(False)
        parts = np.median(np.array(per).reshape(repeats, 3)[1:], axis=0) * 1e6
        recurrent.append({"M": M, "prepare_us": round(float(parts[0]), 1), "scan_us": round(float(parts[1]), 1), "gate_us": round(float(parts[2]), 1),
                          "us": round(float(parts.sum()), 1), "scan_us_per_token": round(float(parts[1]) / M, 3)})
        log(f"  GDN prefill M={M:5d}: prepare {parts[0]:7.1f} scan {parts[1]:8.1f} gate {parts[2]:6.1f} us ({parts[1] / M:.3f} us a token in the scan)")
        del graph, work, packed
    print(json.dumps({"metric": "prefill projection us and TFLOP/s by rows", "unit": "us", "n_gpus": 1,
                      "data": "synthetic: random images, N(0, 1) rows", "roofline": {"bound": "mfma", "peak": peak, "unit": "TFLOP/s"},
                      "results": results, "chunk_attention": attention, "gdn_prefill": recurrent}), flush=True)


def time_c3_ops(backend):
    """BASELINE.json config 3: block-causal attention of a 16-row chain block (64 query / 8 KV heads of 128) over a paged
    INT8 context of 8K, 32K and 128K tokens (256-token pages, random page table), the split pass and the merge, over a
    ring of KV pools past the caches. Prints one JSON line."""
    import splash_amd
    from splash_amd import ops, synthetic
    rng = np.random.default_rng(0)
    bf = lambda a: (np.ascontiguousarray(a, np.float32).view(np.uint32) >> 16).astype(np.uint16)
    QH, KVH, D, rows = 64, 8, 128, 16
    results = []
    # the contexts BASELINE.json names, and one that ends 16 tokens past a page (the block after a full 32K history)
    for context in (8192, 32768, 32768 + rows, 131072):
        pages = (context + ops.PAGE_TOKENS - 1) // ops.PAGE_TOKENS
        kv_bytes = context * KVH * (2 * D + 4)
        copies = int(np.ceil(2 * 268.4e6 / kv_bytes)) + 1
        raw = synthetic.kv_pages(rng, KVH, D, 8)
        raw = np.tile(raw, ((pages + 7) // 8, 1))[:pages]
        table = rng.permutation(pages).astype(np.uint64)
        pools = []
        for _ in range(copies):
            pool = ops.KvPages(backend, KVH, D, pages, table)
            pool.upload(raw)
            pools.append(pool)
        qkv = backend.from_array(bf(rng.standard_normal((rows, (QH + 2 * KVH) * D))))
        tree = backend.from_array(ops.chain_tree_rows([rows]))
        out = backend.allocate_buffer(rows * QH * D * 2)
        algorithmic = kv_bytes + rows * QH * D * 2 * 2 + pages * 8
        if context % ops.PAGE_TOKENS == 0:
            # the CPU oracle's page loop over the same shape on this host's cores: every head up to 32K, two of the
            # eight KV heads (a quarter of the work, scaled) at 128K
            from tests import oracle as orc
            heads = KVH if context <= 32768 else 2
            kc = rng.integers(-127, 128, (pages, heads, ops.PAGE_TOKENS, D)).astype(np.int8)
            ks = np.full((pages, heads, ops.PAGE_TOKENS), 0.03, dtype=np.float32)
            q = orc.f32_to_bf16(rng.standard_normal((rows, heads * (QH // KVH), D)).astype(np.float32))
            anc = np.array([(2 << r) - 1 for r in range(rows)], dtype=np.uint32)
            t0 = time.time()
            orc.attention(q, kc, ks, kc, ks, np.arange(pages, dtype=np.uint32), anc, context - rows, want64=False, threads=0)
            cpu_us = (time.time() - t0) * 1e6 * KVH / heads
            log(f"  context {context:6d} on the CPU ({os.cpu_count()} threads, {heads} of {KVH} KV heads timed): {cpu_us / 1e3:9.1f} ms")
            results.append({"context": context, "device": "cpu", "cores": os.cpu_count(), "kind": "port", "kv_heads_timed": heads,
                            "us": round(cpu_us, 1), "GB/s": round(algorithmic / cpu_us / 1e3, 3)})
            del kc, ks, q
        for int8_queries in (False, True):
            plan = ops.AttentionPlan(QH, KVH, D, [(0, rows, context - rows, 0)], int8_queries=int8_queries)
            workspace = ops.AttentionWorkspace(backend, plan)
            graph = splash_amd.CommandGraph()
            ops.PagedAttention.add_projection(graph, plan, qkv, workspace, pools[0])
            passes = 4
            for _ in range(passes):
                for pool in pools:
                    ops.PagedAttention.add_attention(graph, plan, workspace, tree, pool, out)
            backend.set_dispatch_profiling(True)
            _, _, per = backend.run(graph, profiled=True)
            backend.set_dispatch_profiling(False)
            pairs = np.array(per[1:]).reshape(-1, 2)[copies:] * 1e6
            split_us, merge_us = float(np.median(pairs[:, 0])), float(np.median(pairs[:, 1]))
            results.append({"context": context, "queries": "int8" if int8_queries else "bf16", "splits": plan.splits,
                            "split_us": round(split_us, 2), "merge_us": round(merge_us, 2),
                            "GB/s": round(algorithmic / (split_us + merge_us) / 1e3, 1),
                            "frac": round(algorithmic / (split_us + merge_us) / 1e3 / HBM_PEAK_GBS, 4),
                            "TFLOP/s": round(4 * rows * QH * D * context / (split_us + merge_us) / 1e6, 1)})
            log(f"  context {context:6d} {'int8' if int8_queries else 'bf16'} queries, splits {plan.splits:2d}: split {split_us:7.2f} us "
                f"merge {merge_us:6.2f} us {algorithmic / (split_us + merge_us) / 1e3:7.1f} GB/s")
            del graph, workspace
        del pools
    print(json.dumps({"metric": "attention us and GB/s by context (config 3)", "unit": "us", "n_gpus": 1,
                      "data": "synthetic: uniform INT8 codes, random page table, ring of pools past the caches",
                      "roofline_peak_gbs": HBM_PEAK_GBS, "results": results}), flush=True)


def time_c5_ops(backend):
    """Per-dispatch GPU time (HIP events around each dispatch) of the Gated DeltaNet step and the MoE layer at the
    35B-A3B shape of BASELINE.json config 5, batch 8 of 16-row blocks; weights and states in rings past the caches.
    Prints one JSON line; not the headline metric (that is the dense step)."""
    import splash_amd
    from splash_amd import ops
    rng = np.random.default_rng(0)
    bf = lambda a: (np.ascontiguousarray(a, np.float32).view(np.uint32) >> 16).astype(np.uint16)
    KH, VH, lanes, rows, copies = 16, 32, 8, 16, 6
    gdn = ops.GDN(KH, VH, layers=copies)
    shape = gdn.shape
    bufs = dict(packed=backend.from_array(bf(rng.standard_normal((lanes * rows, shape.packed_width)))),
                convolution_weights=backend.from_array(bf(rng.standard_normal((shape.convolution_dimension, 4)) * 0.4)),
                states=backend.allocate_buffer(gdn.cell_bytes * 2 * lanes), tape=backend.allocate_buffer(gdn.tape_layer_bytes * copies * 2 * lanes),
                decay_weights=backend.from_array(-np.ones(VH, np.float32)), time_bias=backend.from_array(bf(np.zeros(VH))),
                mixer_norm=backend.from_array(bf(np.ones(128))), hidden=backend.allocate_buffer(lanes * rows * VH * 128 * 2),
                # chain blocks: row r of a block follows row r - 1 (ancestors (2 << r) - 1, parent r - 1, depth r)
                tree_rows=backend.from_array(np.array([[(2 << r) - 1, ((r - 1) & 0xFFFF) | (r << 16)] for _ in range(lanes)
                                                       for r in range(rows)], np.uint32)))

    def lane_list(layer, parity, path):
        return [dict(first_row=l * rows, rows=rows, pending_path=path,
                     pending_tape=((l * 2 + (parity ^ 1)) * copies + layer) * gdn.tape_layer_bytes,
                     step_tape=((l * 2 + parity) * copies + layer) * gdn.tape_layer_bytes,
                     current_cell=(l * 2 + parity) * gdn.cell_bytes, next_cell=(l * 2 + (parity ^ 1)) * gdn.cell_bytes) for l in range(lanes)]
    graph = splash_amd.CommandGraph()
    for layer in range(copies):
        gdn.add_decode(graph, bufs, layer, lane_list(layer, 0, 0))
    for _ in range(3):
        for layer in range(copies):
            gdn.add_decode(graph, bufs, layer, lane_list(layer, 1, 0xFFFF))   # folds 16 pending rows, runs 16
    backend.set_dispatch_profiling(True)
    _, _, per = backend.run(graph, profiled=True)
    gdn_us = float(np.median(np.array(per[copies:]) * 1e6))
    state_bytes = lanes * VH * 128 * 128 * 4 * 2
    H, F, E, K, R = 2048, 768, 128, 8, 128
    image = lambda n, k: backend.from_array(rng.integers(0, 256, ops.gguf_image_bytes(ops.FMT_Q4K, n, k) * E, dtype=np.uint8))
    sets = [(image(F, H), image(F, H), image(H, F)) for _ in range(3)]
    moe = ops.MoE(backend, H, F, E, K, R)
    x, res = backend.from_array(bf(rng.standard_normal((R, H)))), backend.from_array(bf(rng.standard_normal((R, H))))
    scores, out = backend.from_array(rng.standard_normal((R, E)).astype(np.float32)), backend.allocate_buffer(R * H * 2)
    graph = splash_amd.CommandGraph()
    for _ in range(4):
        for s in sets:
            moe.add_routing(graph, scores)
            moe.add_routed(graph, x, res, out, *s)
    _, _, per = backend.run(graph, profiled=True)
    backend.set_dispatch_profiling(False)
    med = np.median(np.array(per).reshape(-1, 6)[3:] * 1e6, axis=0)
    names = ["moe_route_select", "moe_group_routes", "moe_gather_table", "gguf_moe_decode_q4k_gt", "gguf_moe_decode_q4k_a", "moe_combine"]
    weights = E * 3 * F * H * 0.5625
    print(json.dumps({
        "ops": "c5", "n_gpus": 1, "data": "synthetic",
        "gdn_decode": {"workload": "32 value heads x 8 lanes, 16 pending + 16 rows", "us": round(gdn_us, 1),
                       "state_bytes": state_bytes, "achieved_gbs": round(state_bytes / gdn_us / 1e3, 1)},
        "moe_layer": {"workload": "hidden 2048, 128 experts top-8, FFN 768, 128 rows", "us": {n: round(float(m), 1) for n, m in zip(names, med)},
                      "total_us": round(float(med.sum()), 1), "expert_weight_bytes": int(weights),
                      "expert_gbs": round(weights / float(med[3] + med[4]) / 1e3, 1)}}), flush=True)


def time_state_codec(backend):
    """The cached form of a lane's recurrent layers at the 35B-A3B shape (36 GDN layers of 32 value heads x 128 x 128 fp32,
    75.5 MB a lane): quantize and dequantize over a ring of lanes' states past the caches, per-dispatch GPU time (HIP
    events around each dispatch). Algorithmic bytes a value: 4 read + 1 + 2/32 written, and the reverse. Prints one JSON
    line; not the headline metric."""
    import splash_amd
    from splash_amd import ops
    rng = np.random.default_rng(0)
    layers, rows, columns, copies = 36, 32 * 128, 128, 8
    shape = ops.StateCodec.shape(layers, rows, columns)
    state_bytes, codes_bytes = layers * rows * columns * 4, layers * ops.StateCodec.layer_bytes(rows, columns)
    base = rng.standard_normal(state_bytes // 4).astype(np.float32)
    states = [backend.from_array(base) for _ in range(copies)]
    codes = [backend.allocate_buffer(codes_bytes) for _ in range(copies)]
    graph = splash_amd.CommandGraph()
    for _ in range(4):
        for c in range(copies):
            ops.StateCodec.add_quantize(graph, states[c], codes[c], shape)
        for c in range(copies):
            ops.StateCodec.add_dequantize(graph, codes[c], states[c], shape)
    backend.set_dispatch_profiling(True)
    _, _, per = backend.run(graph, profiled=True)
    backend.set_dispatch_profiling(False)
    per = np.array(per).reshape(4, 2, copies)[1:] * 1e6
    moved = state_bytes + codes_bytes
    result = {"ops": "state", "n_gpus": 1, "data": "synthetic", "workload": "36 layers x 4096 rows x 128 fp32 values a lane",
              "bytes": moved}
    for name, us in (("state_quantize", float(np.median(per[:, 0]))), ("state_dequantize", float(np.median(per[:, 1])))):
        result[name] = {"us": round(us, 1), "achieved_gbs": round(moved / us / 1e3, 1), "frac": round(moved / us / 1e3 / HBM_PEAK_GBS, 4)}
        log(f"  {name:16s} {us:7.1f} us {moved / us / 1e3:7.1f} GB/s")
    print(json.dumps(result), flush=True)


def time_draft_candidates(backend):
    """The draft selector's candidates and edge scores at the headline vocabulary (151936 columns) for 1 and 8 lanes:
    per-dispatch GPU time (HIP events around each dispatch) over a ring of logits past the caches. Algorithmic bytes of the
    top-16 kernel: the 7 proposal rows a lane of fp32 logits, read once. Prints one JSON line; not the headline metric."""
    import splash_amd
    from splash_amd import ops
    rng = np.random.default_rng(0)
    vocabulary, copies = 151936, 8
    result = {"ops": "draft", "n_gpus": 1, "data": "synthetic", "workload": "7 proposal rows a lane of 151936 fp32 logits, rank-256 codebooks"}
    before, after = (backend.from_array((rng.standard_normal((vocabulary, 256)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16))
                     for _ in range(2))
    for lanes in (1, 8):
        logits = [backend.from_array(rng.standard_normal((lanes * 8, vocabulary)).astype(np.float32)) for _ in range(copies)]
        hidden = backend.from_array((rng.standard_normal((lanes * 8, 256)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16))
        scratch = backend.allocate_buffer(ops.DraftSelector.candidate_scratch_bytes(lanes, vocabulary))
        out = [backend.allocate_buffer(lanes * 7 * 16 * 4), backend.allocate_buffer(lanes * 7 * 16 * 4), backend.allocate_buffer(lanes * 7 * 256 * 4)]
        graph = splash_amd.CommandGraph()
        for _ in range(4):
            for c in range(copies):
                ops.DraftSelector.add_candidates(graph, logits[c], hidden, scratch, *out, before, after, vocabulary, vocabulary, vocabulary,
                                                 [1] * lanes)
        backend.set_dispatch_profiling(True)
        _, _, per = backend.run(graph, profiled=True)
        backend.set_dispatch_profiling(False)
        per = np.array(per).reshape(4, copies, 2)[1:] * 1e6
        moved = lanes * 7 * vocabulary * 4
        top, edges = float(np.median(per[:, :, 0])), float(np.median(per[:, :, 1]))
        result[f"lanes_{lanes}"] = {"top16_us": round(top, 1), "top16_gbs": round(moved / top / 1e3, 1),
                                    "top16_frac": round(moved / top / 1e3 / HBM_PEAK_GBS, 4), "edges_us": round(edges, 1)}
        log(f"  {lanes} lane(s): top16 {top:6.1f} us {moved / top / 1e3:7.1f} GB/s, edges {edges:6.1f} us")
        del logits, graph
    # The draft model's forward pass (model::DFlashDraft) at a 27B target's widths: hidden 5120, the target's head of 151936
    # tokens (Q6_K, fp32 logits), five layers of intermediate 13824 (a draft's config states its own layers and
    # intermediate size; these stand in), every lane past its window of 2048 positions. One command a step, replayed.
    from splash_amd import synthetic, verify
    H, F, L = 5120, 13824, 5
    bf = lambda a: (np.ascontiguousarray(a, np.float32).view(np.uint32) >> 16).astype(np.uint16)
    image = lambda fmt, n, k: backend.from_array(ops.pack_gguf_image(fmt, synthetic.native(rng, fmt, n, k), n, k))
    P = lambda n, k, fmt=ops.FMT_Q4K, f32=False: ops.Projection([(fmt, n, image(fmt, n, k))], k, f32)
    norm = lambda n: backend.from_array(bf(1 + 0.05 * rng.standard_normal(n)))
    draft = verify.DFlashDraft(backend, L, H, vocabulary, F, 5, max_lanes=8)
    for layer in range(L):
        draft.set_layer(layer, attention_dynamic=P(H // 4, H), qkv=P(6144, H), output=P(H, 4096), mlp_dynamic=P(H // 4, H), gate=P(F, H), up=P(F, H),
                        down=P(H, F), input_norm=norm(H), attention_convolution=backend.from_array(bf(rng.standard_normal((4, H)) * 0.5)),
                        query_norm=norm(128), key_norm=norm(128), post_attention_norm=norm(H),
                        mlp_convolution=backend.from_array(bf(rng.standard_normal((4, H)) * 0.5)))
    draft.set_model(P(H, 5 * H), norm(H), norm(H), P(256, H), norm(H), P(vocabulary, H, ops.FMT_Q6K, True))
    draft.buffer(verify.DFLASH_RINGS).upload(bf(rng.standard_normal(8 * L * 2 * ops.DRAFT_RING_BYTES // 2) * 0.5))
    angles = rng.uniform(0, 6.28, (8 * 16, 64))
    draft.buffer(verify.DFLASH_ROPE_COS).upload(np.cos(angles).astype(np.float32))
    draft.buffer(verify.DFLASH_ROPE_SIN).upload(np.sin(angles).astype(np.float32))
    weights = L * (2 * ops.gguf_image_bytes(ops.FMT_Q4K, H // 4, H) + ops.gguf_image_bytes(ops.FMT_Q4K, 6144, H) + ops.gguf_image_bytes(ops.FMT_Q4K, H, 4096)
                   + 3 * ops.gguf_image_bytes(ops.FMT_Q4K, F, H)) + ops.gguf_image_bytes(ops.FMT_Q6K, vocabulary, H) + ops.gguf_image_bytes(ops.FMT_Q4K, 256, H)
    for lanes in (1, 8):
        draft.buffer(verify.DFLASH_HIDDEN, 0).upload(bf(rng.standard_normal((lanes * 8, H))))
        graph = draft.encode_decode([40000 + 100 * l for l in range(lanes)])
        kernels = graph.kernels()
        command = backend.record(graph)
        for _ in range(3):
            command.submit().wait()
        step = float(np.median([command.submit().wait()[0] for _ in range(10)])) * 1e6
        backend.set_dispatch_profiling(True)
        _, _, per = backend.run(graph, profiled=True)
        backend.set_dispatch_profiling(False)
        by = {}
        for name, seconds in zip(kernels, per):
            by.setdefault(name, []).append(seconds * 1e6)
        split, merge = float(np.median(by["draft_attention_split"])), float(np.median(by["draft_attention_merge"]))
        ring = lanes * 2 * ops.DRAFT_RING_BYTES
        result[f"draft_step_lanes_{lanes}"] = {"us": round(step, 1), "dispatches": len(kernels), "weights_gb": round(weights / 1e9, 3),
                                               "weights_gbs": round(weights / step / 1e3, 1), "frac": round(weights / step / 1e3 / HBM_PEAK_GBS, 4),
                                               "attention_split_us": round(split, 1), "attention_merge_us": round(merge, 1),
                                               "attention_ring_gbs": round(ring / split / 1e3, 1)}
        log(f"  draft step, {lanes} lane(s): {step:8.1f} us ({len(kernels)} dispatches, {weights / 1e9:.2f} GB of weights: {weights / step / 1e3:6.1f} GB/s); "
            f"attention split {split:5.1f} us + merge {merge:4.1f} us over {ring / 1e6:.0f} MB of rings")
    print(json.dumps(result), flush=True)


C5 = dict(hidden=2048, vocabulary=151936, layers=48, q_heads=32, kv_heads=4, head_dim=128, gdn_key_heads=16, gdn_value_heads=32,
          experts=128, top_k=8, expert_ffn=768, context=16384, rows=16, lanes=8,
          name="35B-A3B-shaped hybrid MoE verify step: 36 GDN + 12 attention layers, 128 experts top-8 (Q4_K), 16-token draft, "
               "16K INT8 context, batch 8")


def bench_c5(backend, args):
    """BASELINE.json config 5 at full size: a step of 8 lanes x 16 rows that folds the 16 rows each lane accepted of the
    step before (the worst case of the rollback protocol) and runs 16 new ones. Not the headline metric."""
    import splash_amd
    from splash_amd import ops, synthetic, verify
    w = C5
    lanes_n = args.lanes if args.lanes > 1 else w["lanes"]
    rng = np.random.default_rng(20260105)
    H, D, F, V, E = w["hidden"], w["head_dim"], w["expert_ffn"], w["vocabulary"], w["experts"]
    context_pages = (w["context"] + ops.PAGE_TOKENS - 1) // ops.PAGE_TOKENS
    physical = context_pages * lanes_n + 1
    t0 = time.time()
    gpu = verify.HybridVerify(backend, H, V, w["layers"], w["q_heads"], w["kv_heads"], D, w["gdn_key_heads"], w["gdn_value_heads"], E,
                              w["top_k"], F, max_lanes=lanes_n, physical_pages=physical, page_table_entries=context_pages * lanes_n)
    gpu.buffer(verify.PAGE_TABLE).upload(rng.permutation(physical)[:context_pages * lanes_n].astype(np.uint64))
    packed, QKV, QW, GW = gpu.dims.gdn_packed_width, (w["q_heads"] + 2 * w["kv_heads"]) * D, w["q_heads"] * D, w["gdn_value_heads"] * 128
    image = lambda fmt, n, k: ops.pack_gguf_image(fmt, synthetic.native(rng, fmt, n, k), n, k)
    experts = lambda n, k: np.concatenate([image(ops.FMT_Q4K, n, k) for _ in range(8)] * (E // 8))   # eight distinct experts, tiled
    tensors = dict(gdn_in=image(ops.FMT_Q4K, packed, H), gdn_out=image(ops.FMT_Q4K, H, GW), qkv=image(ops.FMT_Q4K, QKV, H),
                   o=image(ops.FMT_Q4K, H, QW), router=image(ops.FMT_Q6K, E, H), gate=experts(F, H), up=experts(F, H), down=experts(H, F))
    first = {name: backend.from_array(t, label=name) for name, t in tensors.items()}
    bf = lambda a: (np.ascontiguousarray(a, np.float32).view(np.uint32) >> 16).astype(np.uint16)
    norm = lambda n: backend.from_array(bf(1 + 0.05 * rng.standard_normal(n)))
    shared = dict(input_norm=norm(H), post_norm=norm(H))
    conv_dim = (2 * w["gdn_key_heads"] + w["gdn_value_heads"]) * 128
    gdn_small = dict(convolution_weights=backend.from_array(bf(rng.standard_normal((conv_dim, 4)) * 0.4)),
                     decay_weights=backend.from_array((-np.exp(rng.uniform(-1, 1, w["gdn_value_heads"]))).astype(np.float32)),
                     time_bias=backend.from_array(bf(rng.uniform(-1, 1, w["gdn_value_heads"]))), mixer_norm=norm(128))
    attention_small = dict(query_norm=norm(D), key_norm=norm(D))

    for layer in range(w["layers"]):
        attends = gpu.attends(layer)
        names = ("qkv", "o") if attends else ("gdn_in", "gdn_out")
        fresh = lambda name: first[name] if layer == (3 if attends else 0) or (name in ("gate", "up", "down", "router") and layer == 0) else None
        buf = {}
        for name in names + ("router", "gate", "up", "down"):
            buf[name] = fresh(name)
            if buf[name] is None:
                buf[name] = backend.allocate_buffer(first[name].size_bytes, label=name)
                device_copy(backend, first[name], buf[name], first[name].size_bytes)
        widths = dict(qkv=(QKV, H), o=(H, QW), gdn_in=(packed, H), gdn_out=(H, GW))
        P = lambda name: ops.Projection([(ops.FMT_Q4K, widths[name][0], buf[name])], widths[name][1])
        gpu.set_layer(layer, P(names[0]), P(names[1]), router=ops.Projection([(ops.FMT_Q6K, E, buf["router"])], H, float32=True),
                      gate_images=buf["gate"], up_images=buf["up"], down_images=buf["down"], **shared,
                      **(attention_small if attends else gdn_small))
        if layer % 12 == 11:
            log(f"  layer {layer + 1}/{w['layers']} resident")
    gpu.set_head(ops.FMT_Q4K, backend.from_array(synthetic.native(rng, ops.FMT_Q4K, V, H), label="embedding"), norm(H),
                 ops.Projection([(ops.FMT_Q6K, V, backend.from_array(image(ops.FMT_Q6K, V, H), label="head"))], H, float32=True))
    pages = synthetic.kv_pages(rng, w["kv_heads"], D, physical)
    pool0 = gpu.buffer(verify.KV_POOL, 0)
    pool0.upload(pages)
    for layer in range(1, w["layers"] // 4):
        device_copy(backend, pool0, gpu.buffer(verify.KV_POOL, layer), pages.nbytes)
    log(f"model resident in {time.time() - t0:.1f}s; allocated {backend.memory_stats().allocated_bytes / 1e9:.2f} GB")
    rows = w["rows"] * lanes_n
    lane = lambda i, parity, path: verify.HybridLane(w["rows"], w["context"] - w["rows"], table_first=i * context_pages,
                                                     pending_path=path, parity=parity)
    gpu.set_block([lane(i, 1, 0) for i in range(lanes_n)], rng.integers(0, V, rows).astype(np.uint32))
    backend.run(gpu.encode([lane(i, 1, 0) for i in range(lanes_n)], commit=False))      # the step before: fills the tapes
    lanes = [lane(i, 0, 0xFFFF) for i in range(lanes_n)]
    graph = gpu.encode(lanes, commit=True)
    kernels = graph.kernels()
    step_bytes = gpu.step_bytes(lanes)
    log(f"step: {len(kernels)} dispatches, {step_bytes / 1e9:.3f} GB algorithmic")
    command = backend.record(graph)
    for _ in range(args.warmup):
        command.submit().wait()
    gpu_seconds = 0.0
    wall0 = time.time()
    for _ in range(args.steps):
        gpu_seconds += command.submit().wait()[0]
    wall_ms = (time.time() - wall0) / args.steps * 1e3
    ms = gpu_seconds / args.steps * 1e3
    selected, retained, accepted, mask = gpu.results(lanes)
    log(f"{ms:.3f} ms/step on the GPU clock, {wall_ms:.3f} ms/step wall; retained {retained.tolist()}")
    backend.set_dispatch_profiling(True)
    _, _, per = backend.run(graph, profiled=True)
    backend.set_dispatch_profiling(False)
    by_kernel = {}
    for name, seconds in zip(kernels, per):
        by_kernel.setdefault(name, []).append(seconds)
    totals = sorted(((sum(v), k) for k, v in by_kernel.items()), reverse=True)
    for total, name in totals[:14]:
        log(f"  {name:36s} x{len(by_kernel[name]):4d}  avg {total / len(by_kernel[name]) * 1e6:8.2f} us  total {total * 1e3:7.3f} ms")
    print(json.dumps({
        "metric": "verify-step ms (config 5: hybrid MoE, batch 8)", "value": round(ms, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 x int4/int6 codes -> fp32 (MFMA); fp32 recurrent state; int8 KV", "data": "synthetic",
        "config": {"workload": w["name"], "lanes": lanes_n, "rows_per_lane": w["rows"], "context_tokens": w["context"],
                   "layers": w["layers"], "dispatches": len(kernels), "acceptance": "greedy", "pending_rows_folded": 16},
        "step_hbm": {"algorithmic_gb": round(step_bytes / 1e9, 3), "achieved_gbs": round(step_bytes / (ms * 1e-3) / 1e9, 1),
                     "frac_of_peak": round(step_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "wall_ms_per_step": round(wall_ms, 4)},
        "kernels_ms": {name: round(total * 1e3, 3) for total, name in totals[:14]}, "cpu_baseline": None}), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c4", choices=sorted(WORKLOADS) + ["c5"])
    ap.add_argument("--lanes", type=int, default=1)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--chain", action="store_true",
                    help="one dispatch for a layer's four projections after its attention instead of a dispatch each")
    ap.add_argument("--fused-prepare", action="store_true",
                    help="a layer's q|k|v projection prepares its attention block itself: one dispatch instead of the "
                         "projection and the prepare kernel")
    ap.add_argument("--prompt-chunk", type=int, default=0,
                    help="instead of the verify step: a chunk of this many prompt tokens (up to 2048) of one sequence "
                         "through every layer, no head (DenseVerify.encode_prefill)")
    ap.add_argument("--staged-prefill", action="store_true",
                    help="with --prompt-chunk above a step's rows: the chunk's projections through the prefill tile (the staged "
                         "rule, as the reference's prompt chunks run) instead of windows of the step's kernels")
    ap.add_argument("--calibrate-traffic", action="store_true",
                    help="after the steps, run plain read and copy kernels of known size: the scale of the FETCH_SIZE / "
                         "WRITE_SIZE counters of a rocprofv3 --pmc run of this command")
    ap.add_argument("--temperature", type=float, default=0.0,
                    help="above 0: rejection-sampling acceptance at this temperature against a full-vocabulary draft "
                         "distribution softmax(N(0, 2)) instead of greedy acceptance")
    ap.add_argument("--direct-launch", action="store_true",
                    help="launch the step's dispatches one by one on the command stream instead of replaying a recorded HIP graph")
    ap.add_argument("--penalties", action="store_true",
                    help="every lane takes sampling penalties (repetition 1.1, presence 0.1, frequency 0.1) over a history of "
                         "4096 tokens: the step then rewrites its logits rows before it selects and counts what it keeps")
    ap.add_argument("--ops", choices=["c2", "c3", "c5", "state", "draft", "prefill"],
                    help="instead of the dense step: c2 the projections alone by rows, c3 attention alone by context, "
                         "c5 the GDN step and the MoE layer of config 5, state the recurrent layers' cached form")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py measures one GPU: this build runs the verify step on a single MI355X (no collectives); use --gpus 1")
        sys.exit(2)
    import splash_amd
    from splash_amd import ops, verify
    backend = splash_amd.Backend(0)
    if args.ops:
        {"c2": time_c2_ops, "c3": time_c3_ops, "c5": time_c5_ops, "state": time_state_codec, "draft": time_draft_candidates,
         "prefill": time_prefill_ops}[args.ops](backend)
        return
    if args.workload == "c5":
        bench_c5(backend, args)
        return
    w = WORKLOADS[args.workload]
    info = backend.device_info()
    log(f"device {info.name.decode()} {info.arch.decode()} CUs {info.compute_units}")
    if args.prompt_chunk > 2048:
        raise SystemExit("a prompt chunk holds up to 2048 tokens")
    t0 = time.time()
    gpu = build_model(backend, w, args.lanes, prefill_rows=args.prompt_chunk)
    log(f"model resident in {time.time() - t0:.1f}s; allocated {backend.memory_stats().allocated_bytes / 1e9:.2f} GB")
    context_pages = (w["context"] + ops.PAGE_TOKENS - 1) // ops.PAGE_TOKENS
    lanes = [verify.Lane(w["rows"], w["context"] - w["rows"], table_first=i * context_pages, temperature=args.temperature)
             for i in range(args.lanes)]
    rows = w["rows"] * args.lanes
    rng = np.random.default_rng(1)
    gpu.set_block(lanes, rng.integers(0, w["vocabulary"], rows).astype(np.uint32), uniforms=rng.random((rows, 2), dtype=np.float32))
    if args.chain:
        gpu.set_chained(True)
    if args.fused_prepare:
        gpu.set_fused_prepare(True)
    if args.prompt_chunk:
        # a prompt chunk that ends the context: every layer, no head
        tokens = args.prompt_chunk
        if args.staged_prefill:
            gpu.set_staged_prefill(True)
        gpu.set_prefill_block(rng.integers(0, w["vocabulary"], tokens).astype(np.uint32))
        command = backend.record(gpu.encode_prefill(0, w["context"] - tokens, tokens))
        for _ in range(args.warmup):
            command.submit().wait()
        seconds = sum(command.submit().wait()[0] for _ in range(args.steps)) / args.steps
        log(f"prompt chunk of {tokens} tokens: {seconds * 1e3:.3f} ms, {tokens / seconds:.0f} tokens/s")
        print(json.dumps({"metric": "prompt chunk ms (every layer of the 27B shape, no head)", "value": round(seconds * 1e3, 4),
                          "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "tokens": tokens,
                          "tokens_per_s": round(tokens / seconds, 1), "higher_is_better": False, "data": "synthetic",
                          "projections": "prefill tile, staged rule" if args.staged_prefill else "the step's kernels, register rule",
                          "config": {"workload": w["name"] if "name" in w else args.workload, "context_tokens": w["context"]}}), flush=True)
        return
    if args.penalties:
        from splash_amd import ops as _ops
        table = gpu.buffer(verify.PENALTY_WORDS)
        for i in range(args.lanes):
            history = rng.integers(0, w["vocabulary"], 4096).astype(np.uint32)
            table.upload(_ops.Sampling.rebuild_penalty_words(w["vocabulary"], history, 2048), offset_bytes=i * w["vocabulary"] * 4)
            gpu.set_penalties(i, 1.1, 0.1, 0.1)
    graph = gpu.encode(lanes, commit=True)
    if args.temperature > 0:
        # the draft model's distributions of the block's rows: softmax of N(0, 2) logits over the whole vocabulary
        draft = np.exp(rng.normal(0.0, 2.0, (rows, w["vocabulary"])).astype(np.float32))
        draft /= draft.sum(axis=1, keepdims=True)
        gpu.buffer(verify.DRAFT_PROBABILITIES).upload(draft.astype(np.float32))
    kernels = graph.kernels()
    step_bytes = gpu.step_bytes(lanes)
    log(f"step: {len(kernels)} dispatches, {step_bytes / 1e9:.3f} GB algorithmic")
    command = backend.record(graph)
    for _ in range(args.warmup):
        command.submit().wait()
    # K steps, one HIP graph launch each, back to back on the command stream; each ticket's GPU time
    # is the step's first kernel start to its last kernel end.
    wall0 = time.time()
    gpu_seconds = 0.0
    for _ in range(args.steps):
        gpu_seconds += (backend.run(graph) if args.direct_launch else command.submit().wait())[0]
    wall = time.time() - wall0
    ms = gpu_seconds / args.steps * 1e3
    wall_ms = wall / args.steps * 1e3
    selected, retained, accepted, mask = gpu.results(lanes)
    log(f"{ms:.3f} ms/step on the GPU clock, {wall_ms:.3f} ms/step wall; retained {retained.tolist()} accepted {accepted.tolist()}")
    # The dominant kernel, measured live: one more step with an event pair around every dispatch on the command stream.
    backend.set_dispatch_profiling(True)
    _, _, per = backend.run(graph, profiled=True)
    backend.set_dispatch_profiling(False)
    by_kernel = {}
    for name, seconds in zip(kernels, per):
        by_kernel.setdefault(name, []).append(seconds)
    totals = sorted(((sum(v), k) for k, v in by_kernel.items()), reverse=True)
    for total, name in totals[:8]:
        log(f"  {name:36s} x{len(by_kernel[name]):3d}  avg {total / len(by_kernel[name]) * 1e6:8.2f} us  total {total * 1e3:7.3f} ms")
    dominant = totals[0][1]
    H, F = w["hidden"], w["ffn"]
    QW, QKV = w["q_heads"] * w["head_dim"], (w["q_heads"] + 2 * w["kv_heads"]) * w["head_dim"]
    Q4, Q6 = 0.5625, 0.8203125                                   # bytes a weight: 144 / 256 and 210 / 256
    context_bytes = args.lanes * w["context"] * w["kv_heads"] * (2 * w["head_dim"] + 4)

    def algorithmic(kernel):
        """Algorithmic HBM bytes of one launch of a step's kernel: every operand once (weights, the bf16 rows in and out,
        the residual rows, the table a residual projection leaves for the next one); None for a kernel this does not price."""
        if kernel.startswith("gguf_decode_chain"):
            # a layer's chained dispatch: output (Q4_K), gate and up (Q4_K), down (Q6_K) and the next layer's q|k|v (Q4_K)
            return (H * QW + 2 * F * H + QKV * H) * Q4 + H * F * Q6 + rows * 2 * (QW + 3 * H + 2 * F + QKV)
        if kernel.endswith("_g") or kernel.endswith("_gt"):
            return 2 * F * H * Q4 + rows * H * 2 + rows * F * 2   # gate and up once + bf16 rows in and out
        if kernel.startswith("gguf_decode_q6k") and kernel.endswith("_rn"):
            return H * F * Q6 + rows * F * 2 + 3 * rows * H * 2 + rows * H * 2 // 2   # down: weights, rows in, residual in/out, next table
        if kernel.startswith("gguf_decode_q4k") and kernel.endswith("_rn"):
            return H * QW * Q4 + rows * QW * 2 + 3 * rows * H * 2 + rows * H * 2 // 2  # output projection, likewise
        if kernel.startswith("gguf_decode_q4k") and kernel.endswith("_a"):
            return QKV * H * Q4 + rows * H * 2 + rows * QKV * 2   # fused q|k|v
        if kernel.startswith("gguf_decode_q6k") and kernel.endswith("_a_f32"):
            return w["vocabulary"] * H * Q6 + rows * H * 2 + rows * w["vocabulary"] * 4   # LM head, fp32 logits
        if kernel.startswith("attention_q8") and "_split" in kernel:
            return context_bytes + rows * QW * 2 + rows * QW * 2  # the lanes' KV once, queries in, rows out (partials are not algorithmic)
        return None

    def roofline_of(kernel):
        launches = by_kernel[kernel][:-1] if kernel.startswith("gguf_decode_chain") else by_kernel[kernel]
        avg = sum(launches) / len(launches)
        size = algorithmic(kernel)
        traffic, traffic_at = measured_traffic(kernel) if args.workload == "c4" and args.lanes == 1 else (None, None)
        return {"bound": "hbm", "kernel": kernel, "achieved": round(size / avg / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(size / avg / 1e9 / HBM_PEAK_GBS, 4), "traffic": traffic, "traffic_measured_at": traffic_at,
                "launches": len(launches), "avg_us": round(avg * 1e6, 2), "total_ms": round(sum(launches) * 1e3, 3),
                "algorithmic_bytes": int(size)}
    # The roofline line is the kernel with the most time in this run (among those priced above); the gate/up pass, the
    # largest mover of bytes, is reported beside it when it is another one.
    priced = [k for _, k in totals if algorithmic(k) is not None]
    gate_up = [k for k in priced if k.startswith("gguf_decode_chain") or k.endswith("_g") or k.endswith("_gt")][0]
    roofline = roofline_of(priced[0])
    roofline["largest_total"] = dominant
    if args.calibrate_traffic:
        calibrate_traffic(backend)
    result = {
        "metric": "verify-step ms + % HBM roofline, 27B-shape Q4_K, 16-tok draft, 32K ctx" if args.workload == "c4" else "verify-step ms (config 1)",
        "value": round(ms, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16 x int4/int6 codes -> fp32 (MFMA); int8 KV",
        "data": "synthetic: native Q4_K/Q6_K blocks with uniform codes and model-like scales (every layer a copy in its own HBM), "
                "uniform INT8 KV codes, uniform-random draft tokens, random page table",
        "config": {"workload": w["name"], "lanes": args.lanes, "rows_per_lane": w["rows"], "context_tokens": w["context"],
                   "layers": w["layers"], "dispatches": len(kernels),
                   "acceptance": (f"rejection sampling, T = {args.temperature}" if args.temperature > 0 else "greedy") +
                                 (", sampling penalties" if args.penalties else "")},
        "step_hbm": {"algorithmic_gb": round(step_bytes / 1e9, 3), "achieved_gbs": round(step_bytes / (ms * 1e-3) / 1e9, 1),
                     "frac_of_peak": round(step_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "wall_ms_per_step": round(wall_ms, 4)},
        "roofline": roofline,
        "kernels": [roofline_of(k) for k in priced[:7]],
    }
    if gate_up != priced[0]:
        result["roofline_gate_up"] = roofline_of(gate_up)
    if not args.no_cpu_baseline:
        log("cpu baseline (oracle on the host cores)...")
        result["cpu_baseline"] = cpu_baseline(w)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
