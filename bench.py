"""Benchmark of the BF16N hot path on one MI355X.

A step is one fused decode+GEMV over the output projection (248320 x 2048 BF16 weights N(0, 0.02), HUFPAIR, one BF16
activation vector N(0, 1), FP32 accumulation, FP32 output) with the encoded weights resident in HBM.  Two copies of the
weights at different addresses are used in turn so that the 256 MB last-level cache does not serve the stream.
Reported: compressed bytes per second (metric), the roofline of the GEMV kernel on algorithmic bytes, the BF16 GEMV of
the stock BLAS on the uncompressed tensor, a kernel that only reads as many bytes, the other configurations of the path
(batch 4, the small 4-bit-code matrices, the MoE decode layer as one HIP graph, the batched MoE prefill, the 40-layer
decode step next to the same step on uncompressed BF16 weights) and the CPU restatement (oracle) of decode+GEMV on
bounded samples.  All tensors come from the counter-based generator of orin_qwen_lossless_amd/synth.py.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--rows R] [--no-cpu] [--no-configs] [--suite]
"""
from __future__ import annotations

import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
SETTLE_MS = 40.0       # untimed load before the timed region of the headline kernel (see time_blocks)
MIN_TIMED_MS = 50.0    # the block of `steps` launches is repeated until at least this long has been timed
TRAFFIC_PROFILE = os.path.join("profiles", "k_w64_mmv_lm_head_248320x2048_hbm_traffic_pmc.txt")


def measured_traffic(rows: int, K: int):
    """HBM bytes per launch of the headline kernel from hardware counters (not measurable in-process): the line
    `traffic_bytes_per_launch[<rows>x<K>] = N` of the committed counter summary, or None."""
    try:
        text = open(os.path.join(ROOT, TRAFFIC_PROFILE)).read()
    except OSError:
        return None
    m = re.search(r"traffic_bytes_per_launch\[%dx%d\]\s*=\s*(\d+)" % (rows, K), text)
    return int(m.group(1)) if m else None


def time_kernel(fn, steps: int, warmup: int, settle_ms: float = 0.0):
    """Per-launch durations (ms) of `steps` calls from HIP events recorded around every call on the launch stream
    (torch's current stream, which is the one the library launches on), after `warmup` untimed calls and, for
    settle_ms, further untimed calls: the events are created first, so that nothing idles the GPU between the untimed
    calls and the timed ones."""
    import torch

    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for i in range(warmup):
        fn(i)
    if settle_ms > 0:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        i = warmup
        while (time.perf_counter() - t0) * 1e3 < settle_ms:
            for _ in range(16):
                fn(i)
                i += 1
            torch.cuda.synchronize()
        for i in range(4):
            fn(i)  # the queue is not empty when the first timed call arrives
    for i in range(steps):
        ev[i][0].record()
        fn(i)
        ev[i][1].record()
    torch.cuda.synchronize()
    return [a.elapsed_time(b) for a, b in ev]


def time_blocks(fn, steps: int, warmup: int, settle_ms: float, min_ms: float):
    """Blocks of `steps` back-to-back launches (synchronised on both sides), repeated until min_ms have been timed (three
    blocks at least); returns the per-block wall times and the per-block times between two HIP events recorded on the
    launch stream around the block, in ms.  The first 15 ms of load after idle
    run up to 15 % slow on this part (clocks settle): after the warm-up the kernel keeps running, untimed, until
    settle_ms have passed, so that a short block measures the same state as a long one."""
    import torch

    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    i = warmup
    while (time.perf_counter() - t0) * 1e3 < settle_ms:
        for _ in range(16):
            fn(i)
            i += 1
        torch.cuda.synchronize()
    blocks, events, total = [], [], 0.0
    while len(blocks) < 3 or total < min_ms:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for j in range(steps):
            fn(j)
        e1.record()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) * 1e3
        blocks.append(dt)
        events.append(e0.elapsed_time(e1))
        total += dt
    return blocks, events


def med_us(fn, steps: int = 50, warmup: int = 5) -> float:
    import numpy as np

    return float(np.median(time_kernel(fn, steps, warmup))) * 1e3


def graph_us(fn, n: int = 16, reps: int = 30) -> float:
    """Per-call time of a short operation: n calls captured into one HIP graph (alternating weight copies through the
    call index), the graph replayed `reps` times between HIP events; host launch overhead stays out of the figure."""
    import torch

    fn(0)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for i in range(n):
            fn(i)
    return med_us(lambda i: graph.replay(), reps, 3) / n


def encode_to_device(ops, w_dev, n_matrices: int = 1, copies: int = 1, engine: str = "mi355x", matrix_core_order: bool = False,
                     mode: str = "hybrid"):
    """Encode a [rows, K] BF16 device tensor under the mi355x policy (n_matrices stacked experts; matrix_core_order: the
    policy's dense_frag_order option) and upload `copies` copies; returns (list of weights, compressed bytes,
    description)."""
    import numpy as np
    import torch

    rows, K = w_dev.shape
    fmt, R, cm, _, w64 = ops.choose(rows // n_matrices, K, n_matrices, engine=engine, mode=mode, expert=n_matrices > 1,
                                    dense_frag_order=matrix_core_order)
    wbits = w_dev.cpu().view(torch.int16).numpy().view(np.uint16)
    plane, aux, fmt_out, _ = ops.encode_bits(wbits, fmt, R, cm, wave64=w64)
    ta = torch.from_numpy(aux)
    meta = ops.parse_header(ta)
    ws = [ops.upload(torch.from_numpy(plane), ta, meta, "cuda") for _ in range(copies)]
    desc = f"{ops.FORMAT_NAMES[fmt_out]} R={R}{' chunk-major' if cm else ''}{' wave64' if w64 else ''}{' tiles 32x256' if R == 32 else ''}"
    return ws, plane.size + aux.size, desc


def read_probe_gbs(nbytes: int) -> dict:
    """A kernel that only reads (libbf16n_probe.so, built from csrc/bench_probe.hip next to the product library: the
    yardstick of the reference's bench/micro/bwprobe.cu) over as many bytes as the compressed matrix, two buffers in
    turn: GB/s per access pattern (median of 30 launches each).  pattern 0 / 1: a contiguous range per wavefront,
    non-temporal / plain loads; 2 / 3: grid-stride."""
    import ctypes as C

    import torch

    path = os.path.join(ROOT, "orin_qwen_lossless_amd", "libbf16n_probe.so")
    if not os.path.exists(path):
        raise OSError(f"{path} is missing: build it with `python -m orin_qwen_lossless_amd.build`")
    probe = C.CDLL(path).bf16n_probe_read
    probe.restype, probe.argtypes = C.c_int, [C.c_void_p, C.c_uint64, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    bufs = [torch.randint(0, 255, (nbytes // 1024 * 1024,), dtype=torch.uint8, device="cuda") for _ in range(2)]
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")

    def read(buf, pattern, wpc):
        if probe(buf.data_ptr(), buf.numel(), pattern, wpc, sink.data_ptr(), torch.cuda.current_stream().cuda_stream) != 0:
            raise RuntimeError("bf16n_probe_read failed")

    out = {}
    for pattern, name in ((0, "wavefront_ranges_nontemporal"), (1, "wavefront_ranges_plain"), (2, "grid_stride_nontemporal"), (3, "grid_stride_plain")):
        for wpc in (8, 16):
            t = med_us(lambda i: read(bufs[i & 1], pattern, wpc), 30, 5)
            out[f"{name}_{wpc}_waves_per_cu"] = round(bufs[0].numel() / t / 1e3, 1)
    return out


# ---------------------------------------------------------------- CPU baseline (the oracle as the thing timed)

def cpu_baseline(wbits, K: int, xf, sample_rows: int, budget_s: float):
    """The oracle's decode+GEMV (reference layout, R = 16) on the first sample_rows rows of the workload, all host
    threads available to this process (capped at 16); and the CPU reference configuration, one 2048 x 2048 pair-coded
    matrix, on one thread and on all."""
    import numpy as np

    from oracle import pyoracle as O
    from orin_qwen_lossless_amd import ops, synth

    threads = max(1, min(16, len(os.sched_getaffinity(0))))

    def run(plane, aux, x, nrows, nthreads, seconds):
        O.decode_gemv(plane, aux, x, 0, nrows, nthreads)  # warm-up
        reps, total, best = 0, 0.0, None
        while total < seconds and reps < 5000:
            t0 = time.perf_counter()
            O.decode_gemv(plane, aux, x, 0, nrows, nthreads)
            dt = time.perf_counter() - t0
            total += dt
            reps += 1
            best = dt if best is None else min(best, dt)
        return total / reps, best, reps

    sub = np.ascontiguousarray(wbits[:sample_rows])
    plane, aux, _, _ = ops.encode_bits(sub, 3, 16, False)
    nbytes = plane.size + aux.size
    mean, best, reps = run(plane, aux, xf, sample_rows, threads, budget_s * 0.6)
    out = {"value": round(nbytes / mean / 1e9, 4), "unit": "GB/s", "cores": threads, "kind": "port",
           "sample": f"first {sample_rows} of the workload's rows ({sample_rows}x{K}, HUFPAIR R=16 reference layout, "
                     f"{nbytes} compressed bytes), mean of {reps} runs ({mean * 1e3:.1f} ms each, best {best * 1e3:.1f} ms)"}
    # the CPU reference configuration: 2048 x 2048, pair code, reference layout (R = 4, what its policy gives the shape)
    w1 = synth.weights(2048, 2048, 11)
    x1 = synth.bf16_bits_to_f32(synth.activations(1, 2048, 12)[0])
    p1, a1, _, _ = ops.encode_bits(w1, 3, 4, False)
    assert np.array_equal(O.decode(p1, a1), w1), "round trip of the 2048 x 2048 matrix"
    b1 = p1.size + a1.size
    cfg1 = {"workload": "2048x2048 BF16 N(0,0.02), HUFPAIR R=4 reference layout, round trip verified, decode+GEMV FP32",
            "compressed_bytes": int(b1)}
    for nt in sorted({1, threads}):
        m1, best1, r1 = run(p1, a1, x1, 2048, nt, budget_s * 0.2)
        cfg1[f"threads_{nt}"] = {"us": round(m1 * 1e6, 1), "GBps": round(b1 / m1 / 1e9, 3), "runs": r1}
    out["config1_2048x2048"] = cfg1
    return out


# ---------------------------------------------------------------- the other configurations of the path

def decode_step_config(ops, gen, head, head_tiles, head_bf16, K: int, batches=(1, 4, 16), n_layers: int = 40, n_sets: int = 40,
                       n_sets_4bit: int = 8) -> dict:
    """The 40-layer decode step as one HIP graph on BF16N weights and on uncompressed BF16 weights with stock kernels
    (orin_qwen_lossless_amd/decode_step.py), output projection included.  n_sets distinct weight sets are used in turn
    (40: every layer has weights of its own, nothing a step reads is read twice; a step's 3.4 GB also pass through the
    256 MB last-level cache between two replays).  Batches above one token are verify steps: their output projection
    is the one the policy gives a caller who states so (dense_frag_order: matrix-core tiles)."""
    import numpy as np
    import torch

    from orin_qwen_lossless_amd import decode_step as D, synth

    t0 = time.perf_counter()
    sets, raw, nbytes = D.make_layer_sets(ops, gen, n_sets, True)
    setup_s = time.perf_counter() - t0
    res = {"layers": n_layers, "weight_sets": n_sets, "weight_sets_setup_s": round(setup_s, 1),
           "bf16_comparator": "the same graph on uncompressed BF16 weights with stock kernels (torch linear / bmm = hipBLASLt), the same glue "
                              "and top-k launches.  bf16_us: the experts a token selects are gathered by index_select and multiplied "
                              "as a batch (what a graph can capture when the routing is decided on the device).  bf16_static_ids_us: "
                              "the expert matrices are read in place, one GEMV launch per expert and matrix, with expert ids fixed "
                              "on the host at capture (a captured graph cannot do that with device-side routing: a lower bound for "
                              "stock kernels).  speedup_vs_bf16 is against the faster of the two"}
    for T in batches:
        xin = [synth.activations_torch(T, K, 300 + i, "cuda") for i in range(4)]
        hbuf = xin[0].clone()
        entry = {}
        hd = head if T == 1 else head_tiles
        head_bytes = hd.plane.numel() + hd.aux.numel()
        static_ids = [[(7 * t + 31 * j) % D.E for j in range(D.TOPK)] for t in range(T)] if T <= 4 else None
        steps = [("bf16n", D.Bf16nStep(ops, sets, hd, n_layers, T)), ("bf16", D.Bf16Step(ops, raw, head_bf16, n_layers, T))]
        if static_ids is not None:
            steps.append(("bf16_static", D.Bf16Step(ops, raw, head_bf16, n_layers, T, static_ids=static_ids)))
        for name, step in steps:
            graph, out = D.capture(step, hbuf)
            eager = step(hbuf).clone()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager), "graph replay differs from the eager step"

            def replay(i):
                hbuf.copy_(xin[i & 3])
                graph.replay()

            entry[name] = float(np.median(time_kernel(replay, 12, 3))) * 1e3
            del graph
        touched = n_layers * D.layer_bytes(nbytes, T) + head_bytes
        expected = n_layers * D.layer_bytes(nbytes, T, expected=True) + head_bytes  # (the rates below: on these)
        bf16_bytes = 2 * (n_layers * (sum(r * k for n_, (r, k, m) in D.SHAPES.items() if m == 1)
                                      + (min(T * D.TOPK, D.E) + 1) * 3 * D.N_MID * K) + head_bf16.numel())
        t = entry["bf16n"]
        best_bf16 = min(v for k_, v in entry.items() if k_ != "bf16n")
        gemv_path = T * (D.TOPK + 1) <= max(ops.MOE_GEMV_MIN_PAIRS, ops.MOE_GEMV_PAIRS_PER_EXPERT[0] * D.EA)
        res[f"batch{T}"] = {"us": round(t, 1), "launches_per_layer": D.launches_per_layer(ops, T, gemv_path),
                            "output_projection": "16-row units" if T == 1 else "matrix-core tiles (dense_frag_order)",
                            "compressed_bytes_touched_upper_bound": int(touched),
                            "compressed_bytes_touched_expected": int(expected), "GBps": round(expected / t / 1e3, 1),
                            "frac_of_hbm_peak": round(expected / t / 1e3 / HBM_PEAK_GBS, 4), "tokens_per_s": round(T / t * 1e6, 1),
                            "bf16_us": round(entry["bf16"], 1),
                            "bf16_static_ids_us": round(entry["bf16_static"], 1) if "bf16_static" in entry else None,
                            "speedup_vs_bf16": round(best_bf16 / t, 2),
                            "bf16_bytes_touched": int(bf16_bytes), "bf16_us_at_hbm_peak": round(bf16_bytes / HBM_PEAK_GBS / 1e3, 1),
                            "eager_equals_graph": True}
    # the same step with the expert stacks in the 4-bit code (the policy's nibble mode for them): no decode chain
    # in the routed GEMVs, 7 % more expert bytes
    sets4, _, nbytes4 = D.make_layer_sets(ops, gen, n_sets_4bit, False, expert_mode="nibble")
    res["experts_4bit_code"] = {"expert_bytes_vs_tiles": round(nbytes4["gate"] / nbytes["gate"], 4), "weight_sets": n_sets_4bit}
    for T in (1, 4):
        xin = [synth.activations_torch(T, K, 300 + i, "cuda") for i in range(4)]
        hbuf = xin[0].clone()
        hd = head if T == 1 else head_tiles
        graph, _ = D.capture(D.Bf16nStep(ops, sets4, hd, n_layers, T), hbuf)

        def replay4(i):
            hbuf.copy_(xin[i & 3])
            graph.replay()

        t = float(np.median(time_kernel(replay4, 12, 3))) * 1e3
        expected = n_layers * D.layer_bytes(nbytes4, T, expected=True) + hd.plane.numel() + hd.aux.numel()
        res["experts_4bit_code"][f"batch{T}"] = {"us": round(t, 1), "vs_policy_layout": round(res[f"batch{T}"]["us"] / t, 3),
                                                   "compressed_bytes_touched_expected": int(expected),
                                                   "frac_of_hbm_peak": round(expected / t / 1e3 / HBM_PEAK_GBS, 4)}
        del graph
    res["layer_sets_4bit"] = sets4[:1]
    del sets4
    res["layer_sets"] = sets
    res["nbytes"] = nbytes
    return res


def configs(ops, w_head, head_copies, comp_bytes: int, K: int, n_sets: int = 40) -> dict:
    """The other configurations, compact: batch 4 on the output projection, the two small matrices, the MoE decode
    layer as one HIP graph, the batched prefill at 2048 and 8192 tokens, the 40-layer decode step at batch 1 and 4."""
    import numpy as np
    import torch

    from orin_qwen_lossless_amd import decode_step as D, synth

    out = {}
    seed = [1000]

    def gen(rows, k):
        seed[0] += 1
        return synth.weights_torch(rows, k, seed[0], "cuda")

    rows = w_head.shape[0]
    x4 = synth.activations_torch(4, K, 21, "cuda")
    x1 = synth.activations_torch(1, K, 2, "cuda")
    t4 = graph_us(lambda i: ops.mmv(x4, head_copies[i & 1]), 8)
    k4 = ops.last_kernel()
    t1 = graph_us(lambda i: ops.mmv(x1, head_copies[i & 1]), 8)
    algo4 = comp_bytes + 4 * K * 2 + 4 * rows * 4
    # the layout the policy gives the same matrix when the caller states that it verifies several tokens per step
    # (dense_frag_order: 32 x 256 tiles in matrix-core operand order; one decode of the matrix serves up to 32 tokens)
    tiles, tile_bytes, tile_desc = encode_to_device(ops, w_head, copies=2, matrix_core_order=True)
    tt4 = graph_us(lambda i: ops.mmv(x4, tiles[i & 1]), 8)
    kt4 = ops.last_kernel()
    tt1 = graph_us(lambda i: ops.mmv(x1, tiles[i & 1]), 8)
    talgo4 = tile_bytes + 4 * K * 2 + 4 * rows * 4
    out["lm_head_batch4"] = {"timing": "8 launches per HIP graph replay, two weight copies in turn",
                             "units_of_16_rows": {"us": round(t4, 2), "batch1_us": round(t1, 2), "vs_batch1": round(t4 / t1, 3), "kernel": k4,
                                                  "GBps": round(algo4 / t4 / 1e3, 1), "frac_of_hbm_peak": round(algo4 / t4 / 1e3 / HBM_PEAK_GBS, 4)},
                             "matrix_core_tiles": {"layout": tile_desc, "compressed_bytes": tile_bytes, "us": round(tt4, 2), "batch1_us": round(tt1, 2),
                                                   "vs_batch1": round(tt4 / tt1, 3), "vs_batch1_of_16_row_units": round(tt4 / t1, 3), "kernel": kt4,
                                                   "GBps": round(talgo4 / tt4 / 1e3, 1),
                                                   "frac_of_hbm_peak": round(talgo4 / tt4 / 1e3 / HBM_PEAK_GBS, 4)},
                             "us": round(min(t4, tt4), 2), "policy": "dense_frag_order (the caller verifies several tokens per step) selects the tiles"}
    for r, k in ((512, 2048), (2048, 512)):
        ws, nb, desc = encode_to_device(ops, gen(r, k), copies=2)
        xx = synth.activations_torch(1, k, 22, "cuda")
        t = graph_us(lambda i: ops.mmv(xx, ws[i & 1]))
        out[f"gemv_{r}x{k}"] = {"layout": desc, "us": round(t, 2), "GBps": round(nb / t / 1e3, 1), "timing": "16 launches per HIP graph replay"}
    # decode step (builds the layer sets that the MoE layer and the prefill configurations reuse)
    step = decode_step_config(ops, gen, head_copies[0], tiles[0], w_head, K, n_sets=n_sets)
    del tiles
    sets, nbytes, sets4 = step.pop("layer_sets"), step.pop("nbytes"), step.pop("layer_sets_4bit")
    out["decode_step"] = step
    # MoE decode layer, batch 1: router GEMV, top-8 on the device, 8 routed + the shared expert, weighted sum + norm
    st = D.Bf16nStep(ops, sets, None, 1, 1)
    xs = [synth.activations_torch(1, K, 400 + i, "cuda") for i in range(8)]
    xbuf, hres = xs[0].clone(), synth.activations_torch(1, K, 399, "cuda")
    layer_i = [0]

    def moe_layer():
        ys, wts, ids = st.experts(sets[layer_i[0] % len(sets)], xbuf)
        return ops.add_rmsnorm(hres, ys=ys, topk_weights=wts)

    graph, _ = D.capture(moe_layer)

    def replay(i):
        xbuf.copy_(xs[i & 7])  # other tokens pick other experts: the routed experts are not cache-resident
        graph.replay()

    t_layer = med_us(replay, 64, 8)
    del graph
    # the same layer eight times in one graph (eight tokens, the weight sets in turn): without the replay's own launch
    routing8 = [D.routing_buffers(1, "cuda") for _ in range(8)]

    def eight_layers():
        outs = []
        for j in range(8):
            st.routing = routing8[j]
            ys, wts, ids = st.experts(sets[j % len(sets)], xs[j])
            outs.append(ops.add_rmsnorm(hres, ys=ys, topk_weights=wts))
        return outs

    graph8, _ = D.capture(eight_layers)
    t_steady = med_us(lambda i: graph8.replay(), 32, 4) / 8
    del graph8
    touched = nbytes["router"] + (nbytes["gate"] + nbytes["up"] + nbytes["down"]) * (D.TOPK + 1) // D.EA
    fused_topk = ops.topk_in_gemv_supported(sets[0]["gate"], sets[0]["up"], D.E, D.TOPK)
    out["moe_layer_batch1_graph"] = {"us": round(t_layer, 2), "us_per_layer_of_8_in_one_graph": round(t_steady, 2),
                                     "launches": 4 if fused_topk else 5,  # router, (top-8,) gate/up, down, weighted sum + norm
                                     "compressed_bytes_touched": int(touched),
                                     "GBps": round(touched / t_layer / 1e3, 1), "frac_of_hbm_peak": round(touched / t_layer / 1e3 / HBM_PEAK_GBS, 4),
                                     "experts": "256 routed (top-8, softmax weights renormalised) + 1 shared, 32x256 tiles"}
    # batched prefill: routing lists, fused gate/up + SwiGLU (BF16 out), down; experts as in the decode step
    w = sets[0]
    for T in (2048, 8192):
        xp = synth.activations_torch(T, K, 500 + T, "cuda")
        _, ids = ops.router_topk(synth.normal_torch(T * D.E, 600 + T, "cuda").view(T, D.E), D.TOPK)

        def prefill(i):
            src1, dst, bounds = ops.mm_ids_route(ids, D.EA, False)
            a = ops.moe_mm_ids(xp, ids, w["gate"], D.EA, up=w["up"], out_dtype=torch.bfloat16, routes=(src1, dst, bounds))
            return ops.moe_mm_ids(a, ids, w["down"], D.EA, routes=(dst, dst, bounds))

        t = med_us(prefill, 10, 2)
        flops = 2.0 * T * D.TOPK * 3 * D.N_MID * K
        wbytes = (nbytes["gate"] + nbytes["up"] + nbytes["down"]) * D.E // D.EA
        out[f"moe_prefill_T{T}"] = {"us": round(t, 1), "TFLOPs": round(flops / t / 1e6, 1),
                                    "frac_of_bf16_mfma_peak": round(flops / t / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4),
                                    "weight_decode_GBps": round(wbytes / t / 1e3, 1), "tokens_per_s": round(T / t * 1e6, 0)}
        w, keep = sets4[0], w  # the same with the expert stacks in the 4-bit code
        t4 = med_us(prefill, 10, 2)
        w = keep
        out[f"moe_prefill_T{T}"]["experts_4bit_code"] = {"us": round(t4, 1), "frac_of_bf16_mfma_peak": round(flops / t4 / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)}
    return out


def suite(ops, w_head, head_copies, K: int) -> dict:
    """A wider sweep, on request: the output projection at other batch sizes in both of its layouts."""
    from orin_qwen_lossless_amd import synth

    batches = {}
    tiles, tbytes, tdesc = encode_to_device(ops, w_head, copies=2, matrix_core_order=True)
    for T in (1, 2, 4, 8, 16, 32, 128):
        xT = synth.activations_torch(T, K, 700 + T, "cuda")
        base = graph_us(lambda i: ops.mmv(xT, head_copies[i & 1]), 4, 10) if T <= 8 else med_us(lambda i: ops.linear(xT, head_copies[i & 1]), 10, 2)
        batches[str(T)] = {"units_of_16_rows_us": round(base, 1),
                           "path": "gemv" if T <= 8 else "gemv, two launches" if T <= ops.gemv_max_tokens(head_copies[0]) else "dequant + BF16 GEMM",
                           "tiles_us": round(graph_us(lambda i: ops.mmv(xT, tiles[i & 1]), 4, 10), 1)}
    return {"lm_head_batches": {"tiles": tdesc, "tiles_bytes": tbytes, "by_batch": batches}}


def prefill_only(T: int, steps: int, mode: str = "hybrid", two_phase_mib: int = 0) -> None:
    """Only the batched MoE kernels of one 35B-A3B-shaped layer (256 experts x (gate, up 512 x 2048; down 2048 x 512),
    top-8, experts in the mi355x policy's layout) on T tokens: routing lists once, then fused gate/up + SwiGLU (BF16)
    and down, `steps` times.  For profiling these kernels alone; prints its own JSON line."""
    import torch

    from orin_qwen_lossless_amd import ops, synth

    torch.cuda.set_device(0)
    ops.init()
    E, topk, N, K = 256, 8, 512, 2048
    (gate,), gb, gdesc = encode_to_device(ops, synth.weights_torch(E * N, K, 31, "cuda"), n_matrices=E, mode=mode)
    (up,), ub, _ = encode_to_device(ops, synth.weights_torch(E * N, K, 32, "cuda"), n_matrices=E, mode=mode)
    (down,), db, ddesc = encode_to_device(ops, synth.weights_torch(E * K, N, 33, "cuda"), n_matrices=E, mode=mode)
    x = synth.activations_torch(T, K, 34, "cuda")
    _, ids = ops.router_topk(synth.normal_torch(T * E, 35, "cuda").view(T, E), topk)
    src1, dst, bounds = ops.mm_ids_route(ids, E, False)
    scratch = None
    if two_phase_mib > 0:  # the two-phase form (expand a group of experts into scratch, multiply from there) for every call
        ops.MM_IDS_TWO_PHASE_PAIRS_PER_EXPERT = 1
        scratch = torch.empty(two_phase_mib << 20, dtype=torch.uint8, device="cuda")

    def gate_up(i):
        return ops.moe_mm_ids(x, ids, gate, E, up=up, out_dtype=torch.bfloat16, routes=(src1, dst, bounds), scratch=scratch)

    a = gate_up(0)
    t_gu = med_us(gate_up, steps, 2)
    t_dn = med_us(lambda i: ops.moe_mm_ids(a, ids, down, E, routes=(dst, dst, bounds), scratch=scratch), steps, 2)
    flops_gu, flops_dn = 2.0 * T * topk * 2 * N * K, 2.0 * T * topk * K * N
    print(json.dumps({"workload": f"MoE prefill, {T} tokens, top-{topk} of {E} experts", "gate_up": gdesc, "down": ddesc,
                      "form": f"two phases through {two_phase_mib} MiB of scratch" if two_phase_mib else "fused decode + matrix cores",
                      "gate_up_us": round(t_gu, 1), "down_us": round(t_dn, 1), "gate_up_bytes": gb + ub, "down_bytes": db,
                      "gate_up_TFLOPs": round(flops_gu / t_gu / 1e6, 1), "down_TFLOPs": round(flops_dn / t_dn / 1e6, 1),
                      "frac_of_bf16_mfma_peak": round((flops_gu + flops_dn) / (t_gu + t_dn) / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)}))


def decode_only(T: int, steps: int, n_sets: int = 40, expert_mode: str = "hybrid") -> None:
    """Only the 40-layer decode step on BF16N weights at batch T, `steps` graph replays (for profiling); prints its own
    JSON line."""
    import numpy as np
    import torch

    from orin_qwen_lossless_amd import decode_step as D, ops, synth

    torch.cuda.set_device(0)
    ops.init()
    K = D.K_MODEL
    seed = [2000]

    def gen(rows, k):
        seed[0] += 1
        return synth.weights_torch(rows, k, seed[0], "cuda")

    sets, _, nbytes = D.make_layer_sets(ops, gen, n_sets, False, expert_mode=expert_mode)
    (head,), hb, _ = encode_to_device(ops, gen(248320, K), matrix_core_order=T > 1)
    xin = [synth.activations_torch(T, K, 300 + i, "cuda") for i in range(4)]
    hbuf = xin[0].clone()
    graph, _ = D.capture(D.Bf16nStep(ops, sets, head, 40, T), hbuf)

    def replay(i):
        hbuf.copy_(xin[i & 3])
        graph.replay()

    t = float(np.median(time_kernel(replay, steps, 3))) * 1e3
    touched = 40 * D.layer_bytes(nbytes, T) + hb
    print(json.dumps({"workload": f"40-layer decode step + output projection, batch {T}, one HIP graph", "us": round(t, 1),
                      "compressed_bytes_touched_upper_bound": int(touched), "GBps": round(touched / t / 1e3, 1)}))


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--rows", type=int, default=248320)
    ap.add_argument("--K", type=int, default=2048)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-rows", type=int, default=16384)
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU work of the baseline leg, about")
    ap.add_argument("--no-configs", action="store_true", help="only the headline kernel: skip the other configurations")
    ap.add_argument("--weight-sets", type=int, default=40, help="distinct weight sets of the 40-layer decode step (40: one per layer)")
    ap.add_argument("--suite", action="store_true", help="also sweep the output projection over batch sizes in both layouts")
    ap.add_argument("--prefill", type=int, default=0, metavar="T",
                    help="run only the batched MoE kernels of one layer on T tokens (for profiling) and exit")
    ap.add_argument("--two-phase-mib", type=int, default=0, metavar="M",
                    help="with --prefill: the two-phase form of the batched product (bf16n_mm_ids_scratch) through M MiB of scratch")
    ap.add_argument("--experts-4bit", action="store_true", help="with --prefill / --decode-step: the expert stacks in the 4-bit code (policy mode nibble)")
    ap.add_argument("--decode-step", type=int, default=0, metavar="T",
                    help="run only the 40-layer decode step at batch T (for profiling) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU (the path has no collective); run with --gpus 1")
    if args.prefill > 0:
        prefill_only(args.prefill, min(args.steps, 20), "nibble" if args.experts_4bit else "hybrid", args.two_phase_mib)
        return
    if args.decode_step > 0:
        decode_only(args.decode_step, min(args.steps, 20), args.weight_sets, "nibble" if args.experts_4bit else "hybrid")
        return

    import numpy as np
    import torch

    from orin_qwen_lossless_amd import ops, synth

    torch.cuda.set_device(0)
    ops.init()
    rows, K = args.rows, args.K
    t0 = time.perf_counter()
    w_dev = synth.weights_torch(rows, K, 1, "cuda")
    wbits = w_dev.cpu().view(torch.int16).numpy().view(np.uint16)
    fmt, R, cm, _, w64 = ops.choose(rows, K, engine="mi355x")
    t1 = time.perf_counter()
    plane, aux, fmt_out, _ = ops.encode_bits(wbits, fmt, R, cm, wave64=w64)
    t_enc = time.perf_counter() - t1
    ta = torch.from_numpy(aux)
    meta = ops.parse_header(ta)
    copies = [ops.upload(torch.from_numpy(plane), ta, meta, "cuda") for _ in range(2)]
    assert ops.roundtrip_equal(copies[0], w_dev), "GPU decode is not bit-exact"  # the load-time verify, before timing
    x = synth.activations_torch(1, K, 2, "cuda")
    y = ops.mmv(x, copies[0])
    ref = (w_dev.float() @ x[0].float())
    err = float(((y[0] - ref).abs() / (w_dev.float().abs() @ x[0].float().abs())).max())
    assert err < 1e-5, f"GEMV error {err}"

    comp_bytes = plane.size + aux.size
    algo_bytes = comp_bytes + K * 2 + rows * 4  # weights (plane + aux incl. table, unit bases, padding) + x + y
    step = lambda i: ops.mmv(x, copies[i & 1])  # noqa: E731
    step(0)
    kernel_name = ops.last_kernel()  # what the library's dispatch launched for this call
    blocks, block_events = time_blocks(step, args.steps, args.warmup, SETTLE_MS, MIN_TIMED_MS)
    ms = float(np.median(blocks)) / args.steps
    # the kernel's average launch duration over the timed region: HIP events on the launch stream around each block
    # (events around every single launch, the second pass, add their own dispatch gap to each: reported beside it)
    kern_ms = float(np.median(block_events)) / args.steps
    durs = time_kernel(step, args.steps, args.warmup, SETTLE_MS)
    # stock BF16 GEMV on the uncompressed tensor (the "vs BF16" column), same timing
    w2 = [w_dev, w_dev.clone()]
    xt = x[0].contiguous()
    blas_blocks, _ = time_blocks(lambda i: torch.mv(w2[i & 1], xt), args.steps, args.warmup, SETTLE_MS, MIN_TIMED_MS)
    blas_us = float(np.median(blas_blocks)) / args.steps * 1e3
    blas_single_us = med_us(lambda i: torch.mv(w2[i & 1], xt), min(args.steps, 100), 10)
    del w2
    probe = read_probe_gbs(comp_bytes)
    stream_gbs = max(probe.values())
    traffic = measured_traffic(rows, K)

    out = {
        "metric": "fused decode+GEMV HBM GB/s (% peak, compressed bytes); us/decode step vs BF16",
        "value": round(comp_bytes / (ms * 1e-3) / 1e9, 2),
        "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"output projection {rows}x{K} BF16 N(0,0.02), {ops.FORMAT_NAMES[fmt_out]} R={R} "
                               f"{'wave64' if w64 else 'reference'} layout, fused decode+GEMV, batch 1 BF16 activations "
                               "N(0,1), FP32 accumulate/out; 2 weight copies alternated; the timed steps are separate launches, "
                               f"in blocks of {args.steps} repeated until {MIN_TIMED_MS:.0f} ms are timed (median block of {len(blocks)}); "
                               f"after the {args.warmup} warm-up steps the kernel keeps running untimed until {SETTLE_MS:.0f} ms have passed (clocks settle)",
                   "rows": rows, "K": K, "batch": 1, "compressed_bytes": comp_bytes, "bits_per_weight": round(8 * comp_bytes / (rows * K), 4),
                   "ratio_of_bf16": round(comp_bytes / (2 * rows * K), 4), "generator": "synth.py: splitmix64 counters + Box-Muller, seeds 1 (weights) and 2 (activations)"},
        "roofline": {"bound": "hbm", "achieved": round(algo_bytes / (kern_ms * 1e-3) / 1e9, 2), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(algo_bytes / (kern_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "traffic": traffic, "traffic_source": TRAFFIC_PROFILE if traffic is not None else None,
                     "kernel": kernel_name, "algorithmic_bytes": algo_bytes, "avg_launch_us": round(kern_ms * 1e3, 3),
                     "timing": f"HIP events around each block of {args.steps} back-to-back launches, median block / {args.steps}",
                     "single_launch_event_us": {"mean": round(float(np.mean(durs)) * 1e3, 2), "median": round(float(np.median(durs)) * 1e3, 2)}},
        "extra": {"pct_of_hbm_peak_compressed": round(100 * comp_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 2),
                  "us_per_matrix": round(ms * 1e3, 2), "block_us_per_step_min_max": [round(min(blocks) / args.steps * 1e3, 2), round(max(blocks) / args.steps * 1e3, 2)],
                  "blas_bf16_gemv_us": round(blas_us, 2), "speedup_vs_blas_bf16": round(blas_us / (ms * 1e3), 3),
                  "blas_timing": "the same blocks of back-to-back launches after the same settle time as the headline kernel (median block); "
                                 "blas_bf16_gemv_single_launch_event_us: events around single launches, as single_launch_event_us",
                  "blas_bf16_gemv_single_launch_event_us": round(blas_single_us, 2),
                  "plain_stream_read_GBps": round(stream_gbs, 1), "read_probe_GBps": probe,
                  "kernel_vs_plain_stream_read": round(algo_bytes / (kern_ms * 1e-3) / 1e9 / stream_gbs, 3), "tokens_per_s_lm_head_only": round(1e3 / ms, 1),
                  "host_encode_s": round(t_enc, 2), "max_err_over_sum_abs": err},
    }
    if not args.no_configs:
        out["extra"]["configs"] = configs(ops, w_dev, copies, comp_bytes, K, args.weight_sets)
    if args.suite:
        out["extra"]["suite"] = suite(ops, w_dev, copies, K)
    out["extra"]["gpu_s"] = round(time.perf_counter() - t0, 1)
    if not args.no_cpu:
        xf = x[0].float().cpu().numpy()
        out["cpu_baseline"] = cpu_baseline(wbits, K, xf, min(args.cpu_rows, rows // 16 * 16), args.cpu_seconds)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
