"""Benchmark of the BF16N hot path on one MI355X.

A step is one fused decode+GEMV over the output projection (248320 x 2048 BF16 weights N(0, 0.02), HUFPAIR, one BF16
activation vector N(0, 1), FP32 accumulation, FP32 output) with the encoded weights resident in HBM.  Two copies of the
weights at different addresses are used in turn so that the 256 MB last-level cache does not serve the stream.
Reported: compressed bytes per second (metric), the roofline of the GEMV kernel on algorithmic bytes, the BF16 GEMV of
the stock BLAS on the uncompressed tensor, and the CPU restatement (oracle) of decode+GEMV on a bounded sample.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--rows R] [--no-cpu]
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
SETTLE_MS = 40.0  # untimed load before the timed region of the headline kernel (see time_kernel)
# HBM bytes per GEMV launch from hardware counters (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000 KiB, each factor calibrated
# on a copy of known size in the same profiler run), for the workloads that were profiled; not measurable in-process.
MEASURED_TRAFFIC = {(248320, 2048): 711_400_000}


def gen_weights(rows: int, K: int, seed: int):
    """N(0, 0.02) -> BF16 (RNE) on the GPU, returned as a CPU bf16 tensor and kept on the device for the BLAS baseline."""
    import torch

    g = torch.Generator(device="cuda").manual_seed(seed)
    w = torch.empty((rows, K), dtype=torch.bfloat16, device="cuda")
    step = 1 << 15
    for r0 in range(0, rows, step):
        n = min(step, rows - r0)
        w[r0: r0 + n] = (torch.randn((n, K), generator=g, device="cuda") * 0.02).to(torch.bfloat16)
    return w


def time_kernel(fn, steps: int, warmup: int, graph: bool = False, settle_ms: float = 0.0):
    """Wall time of `steps` back-to-back launches (synchronised on both sides), then per-launch durations (ms) of a
    second pass from HIP events recorded around every launch on the launch stream (torch's current stream, which is the
    one the library launches on).  graph: the `steps` launches of the wall-time pass are captured into one HIP graph
    first and the timed region is its replay (the launchers only enqueue kernels), which keeps host launch overhead and
    inter-launch gaps out of the job time."""
    import torch

    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    if settle_ms > 0:
        # the first 15 ms of load after idle run up to 15 % slow on this part (clocks settle): keep launching, untimed,
        # until that long has passed, so that a short timed region measures the same state as a long one
        t0 = time.perf_counter()
        i = warmup
        while (time.perf_counter() - t0) * 1e3 < settle_ms:
            for _ in range(16):
                fn(i)
                i += 1
            torch.cuda.synchronize()
    if graph:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(steps):
                fn(i)
        g.replay()  # untimed: the first replay uploads the graph
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        g.replay()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        del g
    else:
        t0 = time.perf_counter()
        for i in range(steps):
            fn(i)
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for i in range(steps):
        ev[i][0].record()
        fn(i)
        ev[i][1].record()
    torch.cuda.synchronize()
    return [a.elapsed_time(b) for a, b in ev], wall


def cpu_baseline(wbits, K: int, xf, sample_rows: int):
    """The oracle's decode+GEMV (reference layout, R = 16) on the first sample_rows rows, all host threads available
    to this process (capped at 16)."""
    import numpy as np

    from oracle import pyoracle as O
    from orin_qwen_lossless_amd import ops

    threads = max(1, min(16, len(os.sched_getaffinity(0))))
    sub = np.ascontiguousarray(wbits[:sample_rows])
    plane, aux, _, _ = ops.encode_bits(sub, 3, 16, False)
    nbytes = plane.size + aux.size
    O.decode_gemv(plane, aux, xf, 0, sample_rows, threads)  # warm-up
    reps, t_total, best = 0, 0.0, None
    while t_total < 12.0 and reps < 5000:
        t0 = time.perf_counter()
        O.decode_gemv(plane, aux, xf, 0, sample_rows, threads)
        dt = time.perf_counter() - t0
        t_total += dt
        reps += 1
        best = dt if best is None else min(best, dt)
    med = t_total / reps
    return {"value": round(nbytes / med / 1e9, 4), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"first {sample_rows} of the workload's rows ({sample_rows}x{K}, HUFPAIR R=16 reference layout, "
                      f"{nbytes} compressed bytes), mean of {reps} runs ({med * 1e3:.1f} ms each, best {best * 1e3:.1f} ms)"}


def encode_to_device(ops, w_dev, n_matrices: int = 1, copies: int = 1, engine: str = "mi355x", matrix_core_order: bool = False):
    """Encode a [rows, K] BF16 device tensor under the mi355x policy (n_matrices stacked experts; matrix_core_order: the
    policy's dense_frag_order option) and upload `copies` copies; returns (list of weights, compressed bytes,
    description)."""
    import numpy as np
    import torch

    rows, K = w_dev.shape
    fmt, R, cm, _, w64 = ops.choose(rows // n_matrices, K, n_matrices, engine=engine, expert=n_matrices > 1,
                                    dense_frag_order=matrix_core_order)
    wbits = w_dev.cpu().view(torch.int16).numpy().view(np.uint16)
    plane, aux, fmt_out, _ = ops.encode_bits(wbits, fmt, R, cm, wave64=w64)
    ta = torch.from_numpy(aux)
    meta = ops.parse_header(ta)
    ws = [ops.upload(torch.from_numpy(plane), ta, meta, "cuda") for _ in range(copies)]
    desc = f"{ops.FORMAT_NAMES[fmt_out]} R={R}{' chunk-major' if cm else ''}{' wave64' if w64 else ''}{' tiles 32x256' if R == 32 else ''}"
    return ws, plane.size + aux.size, desc


def med_us(fn, steps: int = 50, warmup: int = 5) -> float:
    import numpy as np

    d, _ = time_kernel(fn, steps, warmup)
    return float(np.median(d)) * 1e3


def graph_us(fn, n: int = 16, reps: int = 30) -> float:
    """Per-call time of a short operation: n calls captured into one HIP graph (alternating weight copies through the
    call index), the graph replayed `reps` times between HIP events; host launch overhead stays out of the figure."""
    import numpy as np
    import torch

    fn(0)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for i in range(n):
            fn(i)
    d, _ = time_kernel(lambda i: graph.replay(), reps, 3)
    return float(np.median(d)) * 1e3 / n


def decode_step(ops, head, randw, randx, K: int, n_layers: int = 40, n_sets: int = 4, head_tiles=None) -> dict:
    """One decode step of the 35B-A3B shape as a single HIP graph: n_layers x (qkv 5120 x K, o K x 4096, router, top-8 of
    256 experts, fused gate/up, down, combine, shared expert) + the output projection.  n_sets distinct weight sets are
    used in turn and every layer's input is the previous layer's output (re-normalised), so that layers sharing a
    weight set route to different experts; attention itself is not part of this path."""
    import numpy as np
    import torch

    E, topk, N = 256, 8, 512
    sets, nbytes = [], {}
    for _ in range(n_sets):
        d = {}
        for name, (rows, k, nm) in {"qkv": (5120, K, 1), "o": (K, 4096, 1), "router": (E, K, 1), "gate": (E * N, K, E),
                                    "up": (E * N, K, E), "down": (E * K, N, E), "sh_gate_up": (2 * N, K, 1),
                                    "sh_down": (K, N, 1)}.items():
            ws, nb, _ = encode_to_device(ops, randw(rows, k), n_matrices=nm)
            d[name] = ws[0]
            nbytes[name] = nb
        sets.append(d)
    touched = n_layers * (nbytes["qkv"] + nbytes["o"] + nbytes["router"] + nbytes["sh_gate_up"] + nbytes["sh_down"]
                          + (nbytes["gate"] + nbytes["up"] + nbytes["down"]) * topk // E)
    res = {"layers": n_layers, "weight_sets": n_sets}
    for T, hd, tag in ((1, head, ""), (4, head, ""), (16, head, ""), (16, head_tiles, "_head_as_tiles")):
        if hd is None:
            continue
        xin = [randx(T, K) for _ in range(4)]
        xbuf = xin[0].clone()

        def step():
            # the glue between the products is two residual adds and two norms per layer (without the norms the SwiGLU
            # squares the activations layer after layer); the engine's attention is outside this path
            h = xbuf
            for layer in range(n_layers):
                w = sets[layer % n_sets]
                q = ops.linear(h, w["qkv"])
                h = torch.nn.functional.rms_norm(h + ops.linear(q[:, :4096], w["o"]), (K,))
                wts, ids = ops.router_topk(ops.mmv(h, w["router"]), topk)
                y = ops.moe_experts(h, w["gate"], w["up"], w["down"], wts, ids, E)
                sh = ops.mmv(ops.mmv_glu(h, w["sh_gate_up"]), w["sh_down"], out_dtype=torch.bfloat16)
                h = torch.nn.functional.rms_norm(h + y + sh, (K,))
            return ops.linear(h, hd)

        step()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()

        def replay(i):
            xbuf.copy_(xin[i & 3])
            graph.replay()

        d, _ = time_kernel(replay, 12, 3)
        t = float(np.median(d)) * 1e3
        # experts touched: at most T * top-k distinct ones per layer
        tb = touched + (n_layers * (nbytes["gate"] + nbytes["up"] + nbytes["down"]) * topk // E) * (min(T, E // topk) - 1) + hd.plane.numel() + hd.aux.numel()
        res[f"batch{T}{tag}"] = {"graph_us": round(t, 1), "compressed_bytes_touched_upper_bound": int(tb),
                            "GBps": round(tb / t / 1e3, 1), "tokens_per_s": round(T / t * 1e6, 1)}
        del graph
    return res


def suite(ops, w_head, head_copies, x1, K: int) -> dict:
    """The other configurations of the path, each timed with HIP events (median of 50 launches): batch 4 on the output
    projection, the small NIBBLE matrices, one MoE layer at batch 1 as a captured HIP graph, and the batched prefill."""
    import numpy as np
    import torch

    out = {}
    g = torch.Generator(device="cuda").manual_seed(3)

    def randw(rows, k):
        return (torch.randn((rows, k), generator=g, device="cuda") * 0.02).to(torch.bfloat16)

    def randx(*shape):
        return torch.randn(shape, generator=g, device="cuda").to(torch.bfloat16)

    # batch 4 on the output projection (one decode shared by the four columns)
    x4 = randx(4, K)
    t4 = med_us(lambda i: ops.mmv(x4, head_copies[i & 1]))
    out["lm_head_batch4_us"] = round(t4, 2)
    # the output projection at other batch sizes: groups of up to eight columns per decode in the layout above, then
    # dequant + a stock GEMM; and the same matrix as 32 x 256 tiles (the policy's matrix-core order for dense matrices),
    # where BF16 activations go through the matrix cores at any batch size
    batches = {}
    tiles, tbytes, tdesc = encode_to_device(ops, w_head, copies=2, matrix_core_order=True)
    for T in (1, 2, 4, 8, 16, 32, 128):
        xT = randx(T, K)
        base = graph_us(lambda i: ops.mmv(xT, head_copies[i & 1]), 4, 10) if T <= 8 else med_us(lambda i: ops.linear(xT, head_copies[i & 1]), 10, 2)
        batches[str(T)] = {"units_of_16_rows_us": round(base, 1), "path": "gemv" if T <= 8 else "dequant + BF16 GEMM",
                           "tiles_us": round(graph_us(lambda i: ops.mmv(xT, tiles[i & 1]), 4, 10), 1)}
    out["lm_head_batches"] = {"tiles": tdesc, "tiles_bytes": tbytes, "by_batch": batches}
    head_tiles = tiles[0]
    del tiles
    # small NIBBLE matrices
    for rows, k in ((512, 2048), (2048, 512)):
        ws, nbytes, desc = encode_to_device(ops, randw(rows, k), copies=2)
        xx = randx(1, k)
        t = graph_us(lambda i: ops.mmv(xx, ws[i & 1]))
        out[f"gemv_{rows}x{k}"] = {"layout": desc, "us": round(t, 2), "GBps": round(nbytes / t / 1e3, 1),
                                   "timing": "16 launches per HIP graph replay"}
    # one MoE layer of the 35B-A3B shape: router 256x2048, 256 experts x (gate 512x2048, up 512x2048, down 2048x512),
    # top-8 of 256 computed on the device (softmax, renormalised top-k weights)
    E, topk, N = 256, 8, 512
    router, rb, rdesc = encode_to_device(ops, randw(E, K))
    wg, wu = randw(E * N, K), randw(E * N, K)
    down, db, ddesc = encode_to_device(ops, randw(E * K, N), n_matrices=E)
    router, down = router[0], down[0]
    xs = [randx(1, K) for _ in range(8)]
    xbuf = xs[0].clone()
    pairs = {}
    for engine in ("mi355x", "llama"):  # gate / up: this build's wave64 units, and the reference's chunk-major units
        gate, gb, gdesc = encode_to_device(ops, wg, n_matrices=E, engine=engine)
        up, ub, _ = encode_to_device(ops, wu, n_matrices=E, engine=engine)
        gate, up = gate[0], up[0]
        pairs[engine] = (gate, up, gdesc)

        def layer():
            wts, ids = ops.router_topk(ops.mmv(xbuf, router), topk)
            return ops.moe_experts(xbuf, gate, up, down, wts, ids, E)

        layer()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            layer()

        def replay(i):
            xbuf.copy_(xs[i & 7])  # other tokens pick other experts: the 8 routed experts are not cache-resident
            graph.replay()

        t_layer = med_us(replay, 64, 8)
        touched = rb + (gb + ub + db) * topk // E
        out[f"moe_layer_batch1_gate_up_{engine}"] = {
            "layouts": {"router": rdesc, "gate_up": gdesc, "down": ddesc}, "graph_us": round(t_layer, 2),
            "compressed_bytes_touched": int(touched), "GBps": round(touched / t_layer / 1e3, 1),
            "routing": "softmax over 256 logits, top-8 (ties: lower index), weights renormalised to sum 1"}
        del graph
    # prefill: fused gate/up + SwiGLU (BF16 out), then down, over routing lists computed on the device
    for T in (2048, 8192):
        xp = randx(T, K)
        lg = torch.randn((T, E), generator=g, device="cuda")
        wts, ids = ops.router_topk(lg, topk)
        for engine, (gate, up, gdesc) in pairs.items():

            def prefill(i):  # as ops.moe_experts does it: one routing pass, fused gate/up + SwiGLU (BF16), down
                src1, dst, bounds = ops.mm_ids_route(ids, E, False)
                a = ops.moe_mm_ids(xp, ids, gate, E, up=up, out_dtype=torch.bfloat16, routes=(src1, dst, bounds))
                return ops.moe_mm_ids(a, ids, down, E, routes=(dst, dst, bounds))

            t = med_us(prefill, 10, 2)
            t_gu = med_us(lambda i: ops.moe_mm_ids(xp, ids, gate, E, up=up, out_dtype=torch.bfloat16), 10, 2)
            flops = 2.0 * T * topk * (2 * N * K + K * N)
            out[f"moe_prefill_T{T}_gate_up_{engine}"] = {
                "gate_up": gdesc, "us": round(t, 1), "gate_up_us": round(t_gu, 1), "TFLOPs": round(flops / t / 1e6, 2),
                "frac_of_bf16_mfma_peak": round(flops / t / 1e6 / 2500.0, 4), "tokens_per_s": round(T / t * 1e6, 0)}
    out["decode_step"] = decode_step(ops, head_copies[0], randw, randx, K, head_tiles=head_tiles)
    return out


def prefill_only(T: int, steps: int) -> None:
    """Only the batched MoE kernels of one 35B-A3B-shaped layer (256 experts x (gate, up 512 x 2048; down 2048 x 512),
    top-8, experts in the mi355x policy's layout) on T tokens: routing lists once, then fused gate/up + SwiGLU (BF16)
    and down, `steps` times.  For profiling these kernels alone; prints its own JSON line."""
    import numpy as np
    import torch

    from orin_qwen_lossless_amd import ops

    torch.cuda.set_device(0)
    ops.init()
    E, topk, N, K = 256, 8, 512, 2048
    g = torch.Generator(device="cuda").manual_seed(3)

    def randw(rows, k):
        return (torch.randn((rows, k), generator=g, device="cuda") * 0.02).to(torch.bfloat16)

    (gate,), _, gdesc = encode_to_device(ops, randw(E * N, K), n_matrices=E)
    (up,), _, _ = encode_to_device(ops, randw(E * N, K), n_matrices=E)
    (down,), _, ddesc = encode_to_device(ops, randw(E * K, N), n_matrices=E)
    x = torch.randn((T, K), generator=g, device="cuda").to(torch.bfloat16)
    _, ids = ops.router_topk(torch.randn((T, E), generator=g, device="cuda"), topk)
    src1, dst, bounds = ops.mm_ids_route(ids, E, False)

    def gate_up(i):
        return ops.moe_mm_ids(x, ids, gate, E, up=up, out_dtype=torch.bfloat16, routes=(src1, dst, bounds))

    a = gate_up(0)
    t_gu = med_us(gate_up, steps, 2)
    t_dn = med_us(lambda i: ops.moe_mm_ids(a, ids, down, E, routes=(dst, dst, bounds)), steps, 2)
    flops_gu, flops_dn = 2.0 * T * topk * 2 * N * K, 2.0 * T * topk * K * N
    print(json.dumps({"workload": f"MoE prefill, {T} tokens, top-{topk} of {E} experts", "gate_up": gdesc, "down": ddesc,
                      "gate_up_us": round(t_gu, 1), "down_us": round(t_dn, 1),
                      "gate_up_TFLOPs": round(flops_gu / t_gu / 1e6, 1), "down_TFLOPs": round(flops_dn / t_dn / 1e6, 1),
                      "frac_of_bf16_mfma_peak": round((flops_gu + flops_dn) / (t_gu + t_dn) / 1e6 / 2500.0, 4)}))


def head_tiles_only(T: int, steps: int, rows: int, K: int) -> None:
    """Only the output projection in the policy's matrix-core order (32 x 256 tiles) at batch T: bf16n_mmv with BF16
    activations, which runs on the matrix cores, `steps` times on two alternated copies.  For profiling this kernel
    alone; prints its own JSON line."""
    import torch

    from orin_qwen_lossless_amd import ops

    torch.cuda.set_device(0)
    ops.init()
    w = gen_weights(rows, K, 1)
    tiles, nbytes, desc = encode_to_device(ops, w, copies=2, matrix_core_order=True)
    g = torch.Generator(device="cuda").manual_seed(2)
    x = torch.randn((T, K), generator=g, device="cuda").to(torch.bfloat16)
    y = ops.mmv(x, tiles[0])
    err = float(((y.double() - x.double() @ w.double().t()).abs() / (x.double().abs() @ w.double().abs().t())).max())
    t = med_us(lambda i: ops.mmv(x, tiles[i & 1]), steps, 5)
    algo = nbytes + T * K * 2 + T * rows * 4
    print(json.dumps({"workload": f"output projection {rows}x{K}, {desc}, batch {T} BF16 activations, FP32 out", "us": round(t, 2),
                      "compressed_bytes": nbytes, "algorithmic_bytes": algo, "GBps": round(algo / t / 1e3, 1),
                      "frac_of_hbm_peak": round(algo / t / 1e3 / HBM_PEAK_GBS, 4), "max_err_over_sum_abs": err}))


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--rows", type=int, default=248320)
    ap.add_argument("--K", type=int, default=2048)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-rows", type=int, default=16384)
    ap.add_argument("--graph", action="store_true", help="time the steps as one HIP graph replay instead of separate launches")
    ap.add_argument("--suite", action="store_true", help="also time batch 4, the NIBBLE matrices, a MoE layer and the prefill")
    ap.add_argument("--prefill", type=int, default=0, metavar="T",
                    help="run only the batched MoE kernels of one layer on T tokens (for profiling) and exit")
    ap.add_argument("--head-tiles", type=int, default=0, metavar="T",
                    help="run only the output projection as 32 x 256 tiles at batch T (for profiling) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU (the path has no collective); run with --gpus 1")
    if args.prefill > 0:
        prefill_only(args.prefill, min(args.steps, 20))
        return
    if args.head_tiles > 0:
        head_tiles_only(args.head_tiles, min(args.steps, 50), args.rows, args.K)
        return

    import numpy as np
    import torch

    from orin_qwen_lossless_amd import ops

    torch.cuda.set_device(0)
    ops.init()
    rows, K = args.rows, args.K
    t0 = time.perf_counter()
    w_dev = gen_weights(rows, K, seed=1)
    w_cpu = w_dev.cpu()
    wbits = w_cpu.view(torch.int16).numpy().view(np.uint16)
    fmt, R, cm, _, w64 = ops.choose(rows, K, engine="mi355x")
    t1 = time.perf_counter()
    plane, aux, fmt_out, _ = ops.encode_bits(wbits, fmt, R, cm, wave64=w64)
    t_enc = time.perf_counter() - t1
    ta = torch.from_numpy(aux)
    meta = ops.parse_header(ta)
    copies = [ops.upload(torch.from_numpy(plane), ta, meta, "cuda") for _ in range(2)]
    assert ops.roundtrip_equal(copies[0], w_dev), "GPU decode is not bit-exact"  # the load-time verify, before timing
    g = torch.Generator(device="cuda").manual_seed(2)
    x = torch.randn((1, K), generator=g, device="cuda").to(torch.bfloat16)
    y = ops.mmv(x, copies[0])
    ref = (w_dev.float() @ x[0].float())
    err = float(((y[0] - ref).abs() / (w_dev.float().abs() @ x[0].float().abs())).max())
    assert err < 1e-5, f"GEMV error {err}"

    comp_bytes = plane.size + aux.size
    algo_bytes = comp_bytes + K * 2 + rows * 4  # weights (plane + aux incl. table, unit bases, padding) + x + y
    # the steps are launched one by one: at 135 us per step the launches keep ahead of the GPU, and a HIP graph replay of
    # the same steps measured slower (138 us per step at 200 steps, a fixed cost of about half a millisecond per replay)
    use_graph = args.graph
    durs, wall = time_kernel(lambda i: ops.mmv(x, copies[i & 1]), args.steps, args.warmup, graph=use_graph, settle_ms=SETTLE_MS)
    ms = wall * 1e3 / args.steps
    kern_ms = float(np.mean(durs))
    # stock BF16 GEMV on the uncompressed tensor (the "vs BF16" column), same timing loop
    w2 = [w_dev, w_dev.clone()]
    xt = x[0].contiguous()
    bd, _ = time_kernel(lambda i: torch.mv(w2[i & 1], xt), min(args.steps, 100), 10)
    blas_us = float(np.median(bd)) * 1e3
    # a plain streaming read of as many bytes as the compressed matrix (stock reduction over an FP64 view, two
    # buffers alternated): what the memory system gives a kernel that does nothing but read
    nread = comp_bytes // 8 * 8
    bufs = [torch.randint(0, 255, (nread,), dtype=torch.uint8, device="cuda") for _ in range(2)]
    sd, _ = time_kernel(lambda i: bufs[i & 1].view(torch.float64).sum(), 30, 5)
    stream_gbs = nread / (float(np.median(sd)) * 1e-3) / 1e9
    del bufs

    out = {
        "metric": "fused decode+GEMV HBM GB/s (% peak, compressed bytes); us/decode step vs BF16",
        "value": round(comp_bytes / (ms * 1e-3) / 1e9, 2),
        "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"output projection {rows}x{K} BF16 N(0,0.02), {ops.FORMAT_NAMES[fmt_out]} R={R} "
                               f"{'wave64' if w64 else 'reference'} layout, fused decode+GEMV, batch 1 BF16 activations "
                               "N(0,1), FP32 accumulate/out; 2 weight copies alternated; the timed steps are "
                               + ("one HIP graph replay" if use_graph else "separate launches")
                               + f"; after the {args.warmup} warm-up steps the kernel keeps running untimed until {SETTLE_MS:.0f} ms have passed (clocks settle)",
                   "rows": rows, "K": K, "batch": 1, "compressed_bytes": comp_bytes, "bits_per_weight": round(8 * comp_bytes / (rows * K), 4),
                   "ratio_of_bf16": round(comp_bytes / (2 * rows * K), 4)},
        "roofline": {"bound": "hbm", "achieved": round(algo_bytes / (kern_ms * 1e-3) / 1e9, 2), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(algo_bytes / (kern_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "traffic": MEASURED_TRAFFIC.get((rows, K)),
                     "kernel": "k_w64_mmv<bf16_t, 4, 1, 2>", "algorithmic_bytes": algo_bytes, "avg_launch_us": round(kern_ms * 1e3, 2),
                     "median_launch_us": round(float(np.median(durs)) * 1e3, 2)},
        "extra": {"pct_of_hbm_peak_compressed": round(100 * comp_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 2),
                  "us_per_matrix": round(ms * 1e3, 2), "blas_bf16_gemv_us": round(blas_us, 2),
                  "speedup_vs_blas_bf16": round(blas_us / (ms * 1e3), 3),
                  "plain_stream_read_GBps": round(stream_gbs, 1), "kernel_vs_plain_stream_read": round(algo_bytes / (kern_ms * 1e-3) / 1e9 / stream_gbs, 3), "tokens_per_s_lm_head_only": round(1e3 / ms, 1),
                  "host_encode_s": round(t_enc, 2), "max_err_over_sum_abs": err, "setup_s": round(time.perf_counter() - t0, 1)},
    }
    if args.suite:
        out["extra"]["suite"] = suite(ops, w_dev, copies, x, K)
    if not args.no_cpu:
        xf = x[0].float().cpu().numpy()
        out["cpu_baseline"] = cpu_baseline(wbits, K, xf, min(args.cpu_rows, rows // 16 * 16))
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
