"""One decode step of a 35B-A3B-shaped MoE transformer as a sequence of launches over the operator layer, and the same
step on uncompressed BF16 weights with stock GEMV / GEMM kernels: the measurement harness for the decode configurations
(MoE decode layer; full decode-step weight stream).  The engines own this composition in the reference (llama.cpp's
graph, vLLM's model code around vllm_bf16n/linear.py:*, moe.py:62-67); attention itself is not on the BF16N path and is
replaced by a slice of the qkv output.

Per layer (pre-norm, residual stream h in BF16):
    x1 = rmsnorm(h)                         | comes out of the previous layer's glue launch
    q  = qkv x1;  o = W_o q[:, :4096]       | 5120 x 2048 and 2048 x 4096
    x2 = rmsnorm(h2), h2 = h + o            | one glue launch (add_rmsnorm)
    ids, wts = top-8(softmax(router x2))    | 256 x 2048, on the device
    ys_k = down_k(silu(gate_k x2) * (up_k x2)) for the 8 routed experts and the shared one
    h' = h2 + sum_k wts_k ys_k, x1' = rmsnorm(h')             | one glue launch (weighted sum, residual, norm)
256 experts x (gate 512 x 2048, up 512 x 2048, down 2048 x 512) and one shared expert of the same shape.  The shared
expert is stacked behind the routed ones as expert 256 and runs as a ninth slot of every token with weight 1: its two
products ride in the routed experts' launches instead of two launches of their own (run on a second stream beside the
routed ones they cost more than in line: the fork and join of the graph outweighed them).  7 launches per layer while
the experts run as GEMV columns (the gate / up launch selects them itself), 8 with the batched kernels up to 8 tokens
(selection and routing lists in one launch), 9 beyond."""
from __future__ import annotations

import numpy as np
import torch

E, TOPK, N_MID, K_MODEL, QKV_ROWS, ATT = 256, 8, 512, 2048, 5120, 4096
EA = E + 1  # the routed experts and the shared one behind them
SHAPES = {"qkv": (QKV_ROWS, K_MODEL, 1), "o": (K_MODEL, ATT, 1), "router": (E, K_MODEL, 1), "gate": (EA * N_MID, K_MODEL, EA),
          "up": (EA * N_MID, K_MODEL, EA), "down": (EA * K_MODEL, N_MID, EA)}


def encode_policy(ops, w_dev: torch.Tensor, n_matrices: int = 1, mode: str = "hybrid"):
    """[rows, K] BF16 device tensor -> (Weight in the layout of the mi355x policy, compressed bytes).  mode: the policy's
    (hybrid, huffman or nibble: the 4-bit code for everything)."""
    rows, k = w_dev.shape
    fmt, R, cm, _, w64 = ops.choose(rows // n_matrices, k, n_matrices, engine="mi355x", mode=mode, expert=n_matrices > 1)
    bits = w_dev.cpu().view(torch.int16).numpy().view(np.uint16)
    plane, aux, _, _ = ops.encode_bits(bits, fmt, R, cm, wave64=w64)
    ta = torch.from_numpy(aux)
    return ops.upload(torch.from_numpy(plane), ta, ops.parse_header(ta), w_dev.device), plane.size + aux.size


def make_layer_sets(ops, gen_weights, n_sets: int, keep_bf16: bool, expert_mode: str = "hybrid"):
    """n_sets weight sets of one layer.  gen_weights(rows, K) -> BF16 device tensor.  Returns (encoded sets, BF16 sets or
    None, compressed bytes by matrix name of one set).  expert_mode "nibble": the expert stacks in the 4-bit code (7 %
    more bytes than the policy's tiles, no decode chain: the form for decode at one or two tokens)."""
    enc_sets, raw_sets, nbytes = [], [] if keep_bf16 else None, {}
    for _ in range(n_sets):
        enc, raw = {}, {}
        for name, (rows, k, nm) in SHAPES.items():
            w = gen_weights(rows, k)
            enc[name], nbytes[name] = encode_policy(ops, w, nm, expert_mode if nm > 1 else "hybrid")
            if keep_bf16:
                raw[name] = w
        enc_sets.append(enc)
        if keep_bf16:
            raw_sets.append(raw)
    return enc_sets, raw_sets, nbytes


def layer_bytes(nbytes: dict, tokens: int, expected: bool = False) -> int:
    """Compressed bytes one layer touches for `tokens` tokens: the upper bound (every token picks other experts), or the
    expectation for uniform routing (tokens share experts: 102 distinct ones of 256 for 16 tokens' 128 picks)."""
    routed = E * (1.0 - (1.0 - TOPK / E) ** tokens) if expected else min(tokens * TOPK, E)
    experts = routed + 1  # + the shared expert
    dense = sum(nbytes[k] for k in ("qkv", "o", "router"))
    return dense + int((nbytes["gate"] + nbytes["up"] + nbytes["down"]) * experts) // EA


def launches_per_layer(ops, tokens: int, gemv_path: bool) -> int:
    """Kernel launches of one layer of Bf16nStep: qkv, o, glue, router, (top-k,) gate / up, down, glue."""
    if gemv_path:
        return 7 if getattr(ops, "TOPK_IN_EXPERT_GEMV", False) else 8
    return 8 if tokens <= ops.TOPK_ROUTE_ONE_LAUNCH_TOKENS else 9


def routing_buffers(n_tok: int, device) -> tuple[torch.Tensor, torch.Tensor]:
    """(weights f32, ids int32) [n_tok, 9]: columns 0..7 are written by the router's top-k in every step, column 8
    names the shared expert with weight 1."""
    wts = torch.ones((n_tok, TOPK + 1), dtype=torch.float32, device=device)
    ids = torch.full((n_tok, TOPK + 1), E, dtype=torch.int32, device=device)
    return wts, ids


class Bf16nStep:
    """The step on BF16N weights: launches through the operator layer only."""

    def __init__(self, ops, sets, head, n_layers: int, n_tok: int):
        self.ops, self.sets, self.head, self.n_layers = ops, sets, head, n_layers
        self.routing = routing_buffers(n_tok, sets[0]["qkv"].plane.device)

    def experts(self, w, x2):
        """(ys [T, 9, K] FP32 per-slot outputs, wts [T, 9], ids [T, 9])."""
        ops = self.ops
        logits, routes = ops.mmv(x2, w["router"]), None
        batched = ops.moe_experts_batched(x2.shape[0], TOPK + 1, w["gate"], w["up"], w["down"], EA)
        if not batched and ops.topk_in_gemv_supported(w["gate"], w["up"], E, TOPK):
            # the gate / up GEMV selects the experts itself: no top-k launch
            wts, ids = self.routing
            hidden = ops.mmv_glu2_topk(x2, w["gate"], w["up"], logits, TOPK, N_MID, self.routing)
            return ops.mmv(hidden, w["down"], ids, K_MODEL), wts, ids
        if batched:
            wts, ids, routes = ops.router_topk_routes(logits, TOPK, EA, out=self.routing)  # one launch up to 16 tokens
        else:
            wts, ids = ops.router_topk(logits, TOPK, out=self.routing)
        return ops.moe_experts_rows(x2, w["gate"], w["up"], w["down"], ids, EA, routes), wts, ids

    def layer(self, w, h, x1):
        ops = self.ops
        q = ops.linear(x1, w["qkv"])
        o = ops.linear(q[:, :ATT], w["o"])
        x2, h2 = ops.add_rmsnorm(h, o, want_sum=True)
        ys, wts, _ = self.experts(w, x2)
        return ops.add_rmsnorm(h2, ys=ys, topk_weights=wts, want_sum=True)  # (x1', h')

    def __call__(self, h):
        x1 = self.ops.add_rmsnorm(h)
        for i in range(self.n_layers):
            x1, h = self.layer(self.sets[i % len(self.sets)], h, x1)
        return self.ops.linear(x1, self.head) if self.head is not None else x1


class Bf16Step:
    """The same step on uncompressed BF16 weights with stock kernels (torch: hipBLASLt GEMV / GEMM), the same glue
    launches and the same device-side routing.  Experts: the nine selected matrices of a token are gathered by id
    (index_select) and multiplied as a batch — the form a graph can capture when the routing is decided on the device.
    With static_ids (a host list of experts per token, fixed at capture) the products read the expert matrices in
    place instead, which a captured graph with device-side routing cannot do: a lower bound for stock kernels."""

    def __init__(self, ops, raw_sets, head_w, n_layers: int, n_tok: int, static_ids=None):
        self.ops, self.n_layers, self.head_w, self.static_ids = ops, n_layers, head_w, static_ids
        self.sets = [dict(w, gate3=w["gate"].view(EA, N_MID, K_MODEL), up3=w["up"].view(EA, N_MID, K_MODEL),
                          down3=w["down"].view(EA, K_MODEL, N_MID)) for w in raw_sets]
        self.routing = routing_buffers(n_tok, raw_sets[0]["qkv"].device)

    def experts(self, w, x2):
        F = torch.nn.functional
        T = x2.shape[0]
        wts, ids = self.ops.router_topk(F.linear(x2, w["router"]).float(), TOPK, out=self.routing)
        if self.static_ids is not None:
            rows = []
            for t in range(T):
                for e in list(self.static_ids[t]) + [E]:
                    hid = F.silu(F.linear(x2[t: t + 1], w["gate3"][e]).float()) * F.linear(x2[t: t + 1], w["up3"][e]).float()
                    rows.append(F.linear(hid.to(torch.bfloat16), w["down3"][e]).float())
            return torch.cat(rows).view(T, TOPK + 1, K_MODEL), wts, ids
        flat = ids.reshape(-1).long()
        g = torch.index_select(w["gate3"], 0, flat)                     # [T * 9, 512, 2048]
        u = torch.index_select(w["up3"], 0, flat)
        d = torch.index_select(w["down3"], 0, flat)                     # [T * 9, 2048, 512]
        xr = x2.repeat_interleave(TOPK + 1, 0).unsqueeze(-1)            # [T * 9, 2048, 1]
        hid = F.silu(torch.bmm(g, xr).float()) * torch.bmm(u, xr).float()
        return torch.bmm(d, hid.to(torch.bfloat16)).float().view(T, TOPK + 1, K_MODEL), wts, ids

    def layer(self, w, h, x1):
        F, ops = torch.nn.functional, self.ops
        q = F.linear(x1, w["qkv"])
        o = F.linear(q[:, :ATT], w["o"])
        x2, h2 = ops.add_rmsnorm(h, o, want_sum=True)
        ys, wts, _ = self.experts(w, x2)
        return ops.add_rmsnorm(h2, ys=ys, topk_weights=wts, want_sum=True)

    def __call__(self, h):
        x1 = self.ops.add_rmsnorm(h)
        for i in range(self.n_layers):
            x1, h = self.layer(self.sets[i % len(self.sets)], h, x1)
        return torch.nn.functional.linear(x1, self.head_w) if self.head_w is not None else x1


def capture(fn, *args):
    """Warm up on a side stream (nothing initialises lazily under capture), then capture fn(*args) into one HIP graph."""
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        fn(*args)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        out = fn(*args)
    return g, out
