#!/usr/bin/env python3
"""Headline benchmark of the codebook linear hot path on one MI355X.

A "step" is one batch-1 pass over the 7 block linears of one Qwen2.5-7B-shaped layer
(q/o 3584x3584, k/v 512x3584, gate/up 18944x3584, down 3584x18944; d = 8, K = 65,536 fp16
codebook per matrix, uint16 tags = 2 bits per weight, fp16 row scales, bf16 activations), run as
the serving path runs it: 4 launches (q|k|v stacked, o, gate|up stacked, down) through the C ABI.
Steps rotate over enough distinct layers (>= 4x the 256 MB last-level cache) that tags stream from
HBM.  K steps are captured in one HIP graph; the graph is replayed several times, each replay timed
with HIP events on the launch stream, and the median replay counts.

The batch-1 kernels read a load-time regrouping of the tags by codebook slice (about 2.9 bytes per
tag in HBM instead of the file's 2), built by the library when a layer is loaded; value still counts
the packed file's bytes, which is what the metric is quoted on.

value = packed (algorithmic) bytes of a layer / time per layer, in GB/s.  The same JSON line
carries us_per_layer, the roofline of the dominant kernel (gate|up launch, HIP events around graph
replays of that launch alone), the M = 2048 prefill GEMM in TFLOP/s (cfg4), the small-batch crossover
of the d = 4 / 12-bit format (cfg3), the 27B-class layer with 16 column orders at batch 1 and at 2048
rows (cfg5), the 8-bit block-32 output head (152,064 x 3,584) at decode batch sizes 1 to 64, the layer
with its three elementwise neighbours (add + RMS norm twice, SiLU * up) as separate launches and fused
into the consuming products, and the CPU baseline (the reference's CPU route, oracle port, on the host
cores).  Synthetic tensors come from one CPU generator (seed 0) consumed in a fixed order: per layer
and matrix tags, table, row scales, row orders; activations last.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_PEAK_TFLOPS = 2500.0      # MI355X dense fp16 / bf16
# HBM bytes one gate|up launch of stream_kernel moves: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of
# `bench.py --roofline-only --copy-probe`, scaled by the same counters' reading of a 256 MiB copy; the figures and
# the commands are in the file named here.  It is a property of the kernel as profiled, not measured by this run.
GATE_UP_TRAFFIC = {"bytes": 59_540_000, "source": "profiles/stream_kernel_gate_up_7b_bs1.md"}

SHAPES_7B = {"q": (3584, 3584), "k": (512, 3584), "v": (512, 3584), "o": (3584, 3584),
             "gate": (18944, 3584), "up": (18944, 3584), "down": (3584, 18944)}
SHAPES_27B = {"q": (5120, 5120), "k": (1024, 5120), "v": (1024, 5120), "o": (5120, 5120), "gate": (17408, 5120),
              "up": (17408, 5120), "down": (5120, 17408)}
LAUNCHES = (("q", "k", "v"), ("o",), ("gate", "up"), ("down",))
REPS = 5


def launch_bytes(shapes, names, d, bits, G=1, M=1, B=1):
    """Algorithmic bytes of one launch: tags + table + row scales (+ row orders and their index) of its pieces, each
    counted once, + x + y."""
    n = 0
    C = shapes[names[0]][1]
    for nm in names:
        R, C = shapes[nm]
        n += R * ((C // d) * bits // 32) * 4 + G * (1 << bits) * d * 2 + R * 2 + B * R * 2
        if G > 1:
            n += R
        if M > 1:
            n += R + M * C * 2
    return n + B * C * 2


def skewed_tags(torch, gen, R, n, bits, how):
    """Tags whose codeword popularity follows a Zipf law (weight 1 / rank): "zipf" scatters the popular codewords over
    the whole codebook (what k-means labels look like), "zipf-sorted" makes codeword 0 the most popular one, so the
    first slice of 4096 codewords holds most of the tags (the worst case for a slice stream)."""
    K = 1 << bits
    w = 1.0 / torch.arange(1, K + 1, dtype=torch.float64)
    cdf = torch.cumsum(w / w.sum(), 0)
    rank = torch.searchsorted(cdf, torch.rand(R, n, generator=gen, dtype=torch.float64)).clamp_(max=K - 1)
    return rank if how == "zipf-sorted" else torch.randperm(K, generator=gen)[rank]


def make_layer(torch, dev, gen, shapes, d, bits, G=1, M=1, tags="uniform", stream="later"):
    """One layer of PackedLinear pieces with synthetic contents drawn from the CPU generator `gen` (per matrix: tags,
    table, row scales, codebook ids, row orders); the pieces of each launch get their load-time tag streams cut for
    that launch (as PackedShards does at load)."""
    from quantexperiments_amd.kernels import PackedLinear, prepare_stack
    from quantexperiments_amd.masks import seeded_perms
    from quantexperiments_amd.packed import pack_bits
    out = {}
    for i, (nm, (R, C)) in enumerate(shapes.items()):
        W = (C // d) * bits // 32
        if tags == "uniform":
            words = torch.randint(-2 ** 31, 2 ** 31, (R, W), dtype=torch.int64, generator=gen).to(torch.int32)
        else:
            words = pack_bits(skewed_tags(torch, gen, R, C // d, bits, tags), bits)
        table = torch.randn(G << bits, d, generator=gen).to(torch.float16)
        rs = (torch.randn(R, generator=gen) * 0.005 + 0.02).abs().to(torch.float16)
        rb = torch.randint(0, G, (R,), generator=gen).to(torch.uint8) if G > 1 else None
        rm = torch.randint(0, M, (R,), generator=gen).to(torch.uint8) if M > 1 else None
        perms = seeded_perms(C, M, gen)
        t = lambda a: None if a is None else a.to(dev)
        out[nm] = PackedLinear(t(words), t(table), t(rs), t(rb), t(rm), perms.to(dev), 1 << bits, d, stream=stream)
    for l in LAUNCHES:
        prepare_stack([out[n] for n in l])
    return out


def timed_graph(torch, fn, reps=REPS):
    """ms per replay of a HIP graph of fn(): median of `reps` replays, each between two events on torch's current
    stream (the stream the graph's kernels are launched on); one untimed replay first."""
    fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    g.replay()
    torch.cuda.synchronize()
    ts = []
    for _ in range(reps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        g.replay()
        b.record()
        torch.cuda.synchronize()
        ts.append(a.elapsed_time(b))
    del g
    return sorted(ts)[len(ts) // 2]


def cpu_baseline(torch, layer, x, d, bits, shapes):
    """The reference's CPU route (unpack, gather, scale, fp32 matmul, bf16) on the host cores: one full layer per
    repetition, median of REPS repetitions after one warm-up."""
    from oracle import sq_oracle as O
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    host = {nm: (p.words.cpu(), p.table.cpu(), p.row_scale.cpu()) for nm, p in layer.items()}
    xs = {C: x[C].cpu() for C in x}

    def one_layer():
        dec = mm = 0.0
        t0 = time.perf_counter()
        for nm, (w, t, rs) in host.items():
            _, a, b = O.torch_cpu_layer(w, t, rs, None, None, bits, xs[shapes[nm][1]])
            dec += a
            mm += b
        return time.perf_counter() - t0, dec, mm

    one_layer()
    runs = sorted(one_layer() for _ in range(REPS))
    total, dec, mm = runs[len(runs) // 2]
    nbytes = sum(launch_bytes(shapes, l, d, bits) for l in LAUNCHES)
    return {"value": nbytes / total / 1e9, "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"one full 7B-shaped layer (7 matrices, bs=1) per repetition, median of {REPS} after one warm-up; "
                      "torch gather + scale + fp32 matmul + bf16 round",
            "us_per_layer": total * 1e6, "decode_s": dec, "matmul_s": mm}


def prefill(torch, dev, layers, shapes, names=("gate", "down"), T=2048, dense=True, calls=20):
    """T-row prefill GEMM of single matrices: ms per product and TFLOP/s, from HIP-graph replays of `calls` products
    that rotate over the same matrix of up to 7 distinct layers (median of REPS replays); with `dense`, also the time
    of a dense bf16 GEMM of the same shape in PyTorch, timed the same way."""
    from quantexperiments_amd.kernels import linear_gemm
    res = {}
    for nm in names:
        R, C = shapes[nm]
        mats = [L[nm] for L in layers[:7]]
        x = torch.randn(T, C, device=dev).to(torch.bfloat16)
        y = torch.empty(T, R, device=dev, dtype=torch.bfloat16)
        ms = timed_graph(torch, lambda: [linear_gemm([mats[i % len(mats)]], x, y) for i in range(calls)]) / calls
        res[nm] = {"ms": ms, "tflops": 2.0 * T * R * C / (ms * 1e-3) / 1e12, "products_per_replay": calls, "matrices_rotated": len(mats)}
        if dense:
            # for scale: the same product on a dense bf16 copy of the weights through PyTorch (the vendor GEMM library),
            # timed the same way; it reads 4x the bytes and decodes nothing
            w = (torch.randn(R, C, device=dev) * 0.02).to(torch.bfloat16)
            lib = timed_graph(torch, lambda: [torch.matmul(x, w.t(), out=y) for _ in range(calls)]) / calls
            res[nm].update(library_dense_ms=lib, library_dense_tflops=2.0 * T * R * C / (lib * 1e-3) / 1e12, speed_vs_library_dense=lib / ms)
            del w
    return res


def layer_times(torch, dev, layers, shapes, B, fn, gen, rounds=None):
    """us per layer and per launch of fn(pieces, x, y).  Per layer: one HIP graph of whole layers (the 4 launches of
    every layer in turn, `rounds` times over `layers`), so that the weights walked between two uses of a matrix exceed
    the last-level cache and a replay holds about a hundred calls; per launch: a graph of that launch alone over the
    same layers and rounds.  `rounds` defaults to what makes 24 calls of every launch."""
    if rounds is None:
        rounds = max(1, -(-24 // len(layers)))
    xs = {C: torch.randn(B, C, generator=gen).to(torch.bfloat16).to(dev) for C in sorted({c for _, c in shapes.values()})}
    ys = {l: torch.empty(B, sum(shapes[n][0] for n in l), device=dev, dtype=torch.bfloat16) for l in LAUNCHES}

    def run(launches):
        for _ in range(rounds):
            for L in layers:
                for l in launches:
                    fn([L[n] for n in l], xs[shapes[l[0]][1]], ys[l])
    per = {"|".join(l): timed_graph(torch, lambda: run((l,))) * 1e3 / (len(layers) * rounds) for l in LAUNCHES}
    tot = timed_graph(torch, lambda: run(LAUNCHES)) * 1e3 / (len(layers) * rounds)
    return tot, per


def small_batch_crossover(torch, dev, gen, n_layers):
    """cfg3: the 7B shapes in the d = 4, K = 4096, 12-bit format (3 bits per weight) from 1 to 256 activation rows, on
    the two routes PackedShards.forward can take: "direct" = the library's own choice (sq_linear_small up to 32 rows;
    sq_linear_gemm above: passes of 32 rows through the decode-time kernel up to 224 rows, then decode + 256 x 256
    tile GEMM) and "dequant" = decode to fp16 + dense GEMM (the reference's large-M route).  Per M: both times, the
    faster route and its fractions of the HBM roofline (packed bytes + x + y) and of the MFMA roofline (2 M R C).
    crossover_M = the first M at which the MFMA fraction exceeds the HBM fraction: where the product stops being
    bandwidth-bound on paper; route_change_M = the first M at which the dequant route is the faster one."""
    from quantexperiments_amd.kernels import linear_gemm, linear_small
    from quantexperiments_amd.vllm_ext.core import PackedShards
    d, bits = 4, 12
    layers = [make_layer(torch, dev, gen, SHAPES_7B, d, bits) for _ in range(n_layers)]
    shards = {l: PackedShards([layers[0][n] for n in l], large="dequant") for l in LAUNCHES}
    flops1 = 2.0 * sum(R * C for R, C in SHAPES_7B.values())
    res, cross, change = {}, None, None
    for M in (1, 2, 4, 8, 16, 32, 48, 64, 96, 128, 192, 256):
        nbytes = sum(launch_bytes(SHAPES_7B, l, d, bits, B=M) for l in LAUNCHES)
        direct, per = layer_times(torch, dev, layers if M <= 32 else layers[:2], SHAPES_7B, M, linear_small if M <= 32 else linear_gemm, gen,
                                  rounds=None if M <= 32 else 4)
        r = {"direct_us_per_layer": direct, "per_launch_us": per}
        best, route = direct, "direct"
        if M > 1:
            x = {C: torch.randn(M, C, generator=gen).to(torch.bfloat16).to(dev) for C in (3584, 18944)}
            r["dequant_us_per_layer"] = timed_graph(torch, lambda: [shards[l]._large(x[SHAPES_7B[l[0]][1]]) for l in LAUNCHES]) * 1e3
            if r["dequant_us_per_layer"] < best:
                best, route = r["dequant_us_per_layer"], "dequant"
        r.update(faster=route, us_per_layer=best, GBps=nbytes / best / 1e3, frac_hbm=nbytes / best / 1e3 / HBM_PEAK_GBS,
                 tflops=flops1 * M / best / 1e6, frac_mfma=flops1 * M / best / 1e6 / MFMA_PEAK_TFLOPS)
        if cross is None and r["frac_mfma"] > r["frac_hbm"]:
            cross = M
        if change is None and route == "dequant":
            change = M
        res[f"M{M}"] = r
    return {"workload": "cfg3: 7B shapes, d=4, K=4096, 12-bit tags (3 bpw), bf16 rows", "layers_rotated": n_layers,
            "flops_per_row": flops1, "rows": res, "crossover_M": cross, "route_change_M": change,
            "note": "direct = sq_linear_small (M <= 32) / sq_linear_gemm (passes of 32 rows up to 224, then decode + tile GEMM); "
                    "dequant = sq_dequant to fp16 + sq_gemm_dense; crossover_M = first M whose MFMA fraction exceeds its HBM "
                    "fraction; route_change_M = first M at which the dequant route is faster (null: never up to 256)"}


def masked_27b(torch, dev, gen, n_layers):
    """cfg5: the 27B-class layer, d = 8, K = 65,536, 16 column orders per matrix, at batch 1 (HBM roofline) and at
    2048 rows (MFMA roofline)."""
    from quantexperiments_amd.kernels import linear_gemm, linear_small
    d, bits, M = 8, 16, 16
    layers = [make_layer(torch, dev, gen, SHAPES_27B, d, bits, 1, M) for _ in range(n_layers)]
    nbytes = sum(launch_bytes(SHAPES_27B, l, d, bits, 1, M) for l in LAUNCHES)
    flops1 = 2.0 * sum(R * C for R, C in SHAPES_27B.values())
    us1, per1 = layer_times(torch, dev, layers, SHAPES_27B, 1, linear_small, gen)
    us2k, per2k = layer_times(torch, dev, layers[:2], SHAPES_27B, 2048, linear_gemm, gen, rounds=5)
    return {"workload": "cfg5: 27B-class layer (hidden 5120, intermediate 17408), d=8, K=65536, 16 column orders, 4-bit order index per row",
            "layers_rotated": n_layers, "bytes_per_layer": nbytes,
            "bs1": {"us_per_layer": us1, "per_launch_us": per1, "GBps_packed": nbytes / us1 / 1e3, "frac_hbm": nbytes / us1 / 1e3 / HBM_PEAK_GBS},
            "M2048": {"us_per_layer": us2k, "per_launch_us": per2k, "tflops": flops1 * 2048 / us2k / 1e6,
                      "frac_mfma": flops1 * 2048 / us2k / 1e6 / MFMA_PEAK_TFLOPS}}


def lm_head(torch, dev, rows=(1, 4, 8, 16, 32, 64)):
    """The 7B model's 8-bit block-32 output head (152,064 x 3,584 int8 + fp16 block scales = 579 MB, more than
    twice the last-level cache): microseconds and weight bytes per second for a few decode batch sizes."""
    from quantexperiments_amd.kernels import q8_linear
    V, C = 152064, 3584
    g = torch.Generator(device=dev).manual_seed(1)
    q = torch.randint(-127, 128, (V, C), dtype=torch.int8, device=dev, generator=g)
    sc = (torch.rand(V, C // 32, device=dev, generator=g) * 0.002 + 0.0005).to(torch.float16)
    nbytes = q.numel() + sc.numel() * 2
    res = {"shape": [V, C], "bytes": nbytes, "peak": HBM_PEAK_GBS, "unit": "GB/s"}
    for B in rows:
        x = torch.randn(B, C, device=dev, generator=g).to(torch.bfloat16)
        y = torch.empty(B, V, device=dev, dtype=torch.bfloat16)
        q8_linear(q, sc, x, y)                   # grows the workspace outside capture
        ms = timed_graph(torch, lambda: [q8_linear(q, sc, x, y) for _ in range(20)], reps=3) / 20
        gbs = nbytes / (ms * 1e-3) / 1e9
        res[f"B{B}"] = {"us": ms * 1e3, "achieved": gbs, "frac": gbs / HBM_PEAK_GBS}
    return res


def neighbours(torch, dev, layers, x, y):
    """One decoder layer with the three elementwise neighbours of its products (add + RMS norm before q|k|v and
    before gate|up, SiLU * up before down), as separate launches and fused (add + norm into the product that consumes
    it, SiLU * up into the gate|up product that feeds it: four launches per layer); and the two stand-alone kernels by
    themselves.  Microseconds per layer / per launch inside a HIP graph."""
    from quantexperiments_amd.kernels import addnorm, linear_small, linear_small_from, linear_small_silu, silu_mul
    L, I = LAUNCHES, SHAPES_7B["gate"][0]
    h = [torch.randn(1, 3584, device=dev), torch.empty(1, 3584, device=dev)]
    w = torch.ones(3584, device=dev, dtype=torch.bfloat16)
    x1 = torch.empty(1, 3584, device=dev, dtype=torch.bfloat16)
    act = torch.empty(1, I, device=dev, dtype=torch.bfloat16)
    gate, up = y[L[2]][:, :I], y[L[2]][:, I:]

    def separate():
        for Ly in layers:
            addnorm(h[1], y[L[3]], w, 1e-6, x1, h_out=h[0])
            linear_small([Ly[n] for n in L[0]], x1, y[L[0]])
            linear_small([Ly[n] for n in L[1]], x[3584], y[L[1]])          # (attention sits between q|k|v and o)
            addnorm(h[0], y[L[1]], w, 1e-6, x1, h_out=h[1])
            linear_small([Ly[n] for n in L[2]], x1, y[L[2]])
            silu_mul(gate, up, act)
            linear_small([Ly[n] for n in L[3]], act, y[L[3]])

    def fused():
        for Ly in layers:
            linear_small_from([Ly[n] for n in L[0]], y[L[0]], x1, h_in=h[1], add=y[L[3]], w=w, eps=1e-6, h_out=h[0])
            linear_small([Ly[n] for n in L[1]], x[3584], y[L[1]])
            linear_small_silu([Ly[n] for n in L[2]], None, act, x_out=x1, h_in=h[0], add=y[L[1]], w=w, eps=1e-6, h_out=h[1])
            linear_small([Ly[n] for n in L[3]], act, y[L[3]])

    res = {}
    for name, fn, per in (("layer_separate_us", separate, len(layers)), ("layer_fused_us", fused, len(layers)),
                          ("addnorm_us", lambda: [addnorm(h[0], y[L[1]], w, 1e-6, x1, h_out=h[1]) for _ in range(28)], 28),
                          ("silu_mul_us", lambda: [silu_mul(gate, up, act) for _ in range(28)], 28)):
        res[name] = timed_graph(torch, fn, reps=3) * 1e3 / per
    return res


def copy_probe(torch, dev):
    """Three 256 MiB device-to-device copies: a kernel of known HBM traffic to scale profiler counters by."""
    src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    return {"bytes_read": 256 << 20, "bytes_written": 256 << 20, "launches": 3}


def resident_bytes(layer):
    """Bytes one layer keeps in HBM, by kind, and per weight."""
    kinds = {"tags": 0, "tables": 0, "row_scales": 0, "row_orders": 0, "tag_stream": 0}
    weights = 0
    for p in layer.values():
        weights += p.R * p.C
        size = lambda t: 0 if t is None else t.numel() * t.element_size()
        kinds["tags"] += size(p.words)
        kinds["tables"] += size(p.table)
        kinds["row_scales"] += size(p.row_scale) + size(p.row_book)
        kinds["row_orders"] += size(p.row_mask) + size(p.perms) + size(p.row_order)
        kinds["tag_stream"] += size(p.stream)
    total = sum(kinds.values())
    return {**kinds, "total": total, "bits_per_weight": 8.0 * total / weights}


def sweep(torch, dev, spec: str, rows: str, n_layers: int, tags: str = "uniform", stream=True):
    """Other formats and shapes than the headline's, one layer (4 launches) per activation-row count:
    spec = "<7b|27b>,d,bits,G,M", e.g. "7b,4,12,1,1" (cfg3), "27b,8,16,1,16" (cfg5), "27b,4,12,4,1" (the shipped 27B
    format).  Up to 32 rows through sq_linear_small, above through sq_linear_gemm; n_layers distinct layers rotated
    in one HIP graph, HIP events around the replay, median of 5."""
    from quantexperiments_amd.kernels import linear_small, linear_gemm
    model, d, bits, G, M = spec.split(",")
    d, bits, G, M = int(d), int(bits), int(G), int(M)
    shapes = SHAPES_7B if model == "7b" else SHAPES_27B
    gen = torch.Generator().manual_seed(0)
    layers = [make_layer(torch, dev, gen, shapes, d, bits, G, M, tags, "later" if stream else False) for _ in range(n_layers)]
    nbytes = sum(launch_bytes(shapes, l, d, bits, G, M) for l in LAUNCHES)
    res = {}
    for B in [int(b) for b in rows.split(",")]:
        tot, per = layer_times(torch, dev, layers, shapes, B, linear_small if B <= 32 else linear_gemm, gen)
        res[f"B{B}"] = {"us_per_layer": tot, "GBps_packed": nbytes / tot / 1e3,
                        "tflops": 2.0 * B * sum(R * C for R, C in shapes.values()) / tot / 1e6, "per_launch_us": per}
    return {"sweep": spec, "tags": tags, "load_time_layouts": bool(stream), "layers_rotated": n_layers, "rows": res,
            "resident": resident_bytes(layers[0])}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=280)
    ap.add_argument("--warmup", type=int, default=28)
    ap.add_argument("--layers", type=int, default=28, help="distinct layers the steps rotate over")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--prefill-calls", type=int, default=20, help="prefill products per timed graph replay (1: short profiler runs)")
    ap.add_argument("--roofline-only", action="store_true",
                    help="run only the dominant launch (gate|up) and print only its roofline object: the command "
                         "the rocprofv3 summaries under profiles/ are made with")
    ap.add_argument("--no-head", action="store_true", help="skip the 8-bit lm_head GEMV")
    ap.add_argument("--no-neighbours", action="store_true", help="skip the layer with its elementwise neighbours")
    ap.add_argument("--no-configs", action="store_true", help="skip the cfg3 (small-batch crossover) and cfg5 (27B, column orders) objects")
    ap.add_argument("--head-only", action="store_true",
                    help="run only the 8-bit lm_head GEMV and print only its object (the command its rocprofv3 "
                         "summary under profiles/ is made with)")
    ap.add_argument("--sweep", default="", metavar="MODEL,d,bits,G,M",
                    help="time one layer of another format / shape set instead of the headline workload and print only "
                         "that object, e.g. 7b,4,12,1,1 (cfg3), 27b,8,16,1,16 (cfg5); see --rows")
    ap.add_argument("--rows", default="1", help="activation-row counts for --sweep, comma separated")
    ap.add_argument("--tags", default="uniform", choices=("uniform", "zipf", "zipf-sorted"),
                    help="tag distribution of --sweep: uniform, or Zipf codeword popularity scattered over / sorted into the codebook")
    ap.add_argument("--no-stream", action="store_true",
                    help="--sweep without the load-time layouts (slice streams, tile-major copies): every row count then runs "
                         "on the kernels that read the packed file's own layout")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run three 256 MiB device copies (a kernel of known traffic to scale rocprofv3 counters by)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures the one-GPU hot path; multi-GPU runs are not part of this build (use --gpus 1)")

    import torch
    from quantexperiments_amd.kernels import linear_small
    if not torch.cuda.is_available():
        sys.exit("bench.py needs an MI355X (no CPU fallback)")
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    if args.head_only:
        print(json.dumps({"lm_head": lm_head(torch, dev)}))
        return
    if args.sweep:
        print(json.dumps(sweep(torch, dev, args.sweep, args.rows, min(args.layers, 4 if args.sweep.startswith("27b") else 16), args.tags,
                               not args.no_stream)))
        return
    D, BITS = 8, 16
    gen = torch.Generator().manual_seed(0)
    layers = [make_layer(torch, dev, gen, SHAPES_7B, D, BITS) for _ in range(args.layers)]
    x = {C: torch.randn(1, C, generator=gen).to(torch.bfloat16).to(dev) for C in (3584, 18944)}
    y = {l: torch.empty(1, sum(SHAPES_7B[n][0] for n in l), device=dev, dtype=torch.bfloat16) for l in LAUNCHES}

    def step(i):
        L = layers[i % len(layers)]
        for l in LAUNCHES:
            linear_small([L[n] for n in l], x[SHAPES_7B[l[0]][1]], y[l])

    gu = LAUNCHES[2]
    gu_bytes = launch_bytes(SHAPES_7B, gu, D, BITS)

    rounds = max(1, -(-96 // len(layers)))       # a graph of one launch holds about a hundred calls, like a graph of layers

    def gate_up_all():
        for _ in range(rounds):
            for L in layers:
                linear_small([L[n] for n in gu], x[3584], y[gu])

    def roofline():
        dur_us = timed_graph(torch, gate_up_all) * 1e3 / (len(layers) * rounds)
        achieved = gu_bytes / (dur_us * 1e-6) / 1e9
        return {"bound": "hbm", "kernel": "sq::stream_kernel (gate|up launch, 2 x 18944x3584)",
                "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                "bytes_per_launch": gu_bytes, "us_per_launch": dur_us, "traffic": GATE_UP_TRAFFIC["bytes"],
                "traffic_source": GATE_UP_TRAFFIC["source"],
                "stream_bytes_per_launch": sum(layers[0][n].stream.numel() for n in gu)}

    if args.roofline_only:
        out = {"roofline": roofline()}
        if args.copy_probe:
            out["copy_probe"] = copy_probe(torch, dev)
        print(json.dumps(out))
        return

    step(0)                                      # grows the shared workspace, which must not happen under capture
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for i in range(args.steps):
            step(i)
    g.replay()                                   # graph upload / first-launch costs stay outside the timed region
    torch.cuda.synchronize()
    replays = []
    for _ in range(REPS):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        g.replay()                               # exactly --steps layer steps
        e1.record()
        torch.cuda.synchronize()
        replays.append(e0.elapsed_time(e1))
    del g
    ms_per_step = sorted(replays)[len(replays) // 2] / args.steps
    layer_bytes = sum(launch_bytes(SHAPES_7B, l, D, BITS) for l in LAUNCHES)
    tag_bytes = sum(R * (C // D) * BITS // 8 for R, C in SHAPES_7B.values())
    value = layer_bytes / (ms_per_step * 1e-3) / 1e9

    per_launch = {}
    for l in LAUNCHES:
        def one(l=l):
            for _ in range(rounds):
                for L in layers:
                    linear_small([L[n] for n in l], x[SHAPES_7B[l[0]][1]], y[l])
        nb = launch_bytes(SHAPES_7B, l, D, BITS)
        us = timed_graph(torch, one) * 1e3 / (len(layers) * rounds)
        per_launch["|".join(l)] = {"us": us, "bytes": nb, "frac_hbm": nb / us / 1e3 / HBM_PEAK_GBS}

    out = {
        "metric": "codebook GEMV HBM GB/s + us/layer @7B bs=1; prefill GEMM TFLOP/s @M=2048",
        "value": value, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16xf16->f32 (bf16 activations in/out)", "data": "synthetic (CPU generator, seed 0)",
        "config": {"workload": "cfg2: one Qwen2.5-7B-shaped layer, 7 block linears, bs=1, d=8, K=65536, uint16 tags "
                               "(2 bpw), fp16 row scales, bf16 x/y; 4 launches per layer (q|k|v, o, gate|up, down)",
                   "layers_rotated": len(layers), "bytes_per_layer": layer_bytes, "tag_bytes_per_layer": tag_bytes,
                   "timing": f"HIP events around one graph replay of --steps layer steps, median of {REPS} replays",
                   "replay_ms": replays},
        "us_per_layer": ms_per_step * 1e3,
        "frac_hbm": value / HBM_PEAK_GBS,
        "tag_only_GBps": tag_bytes / (ms_per_step * 1e-3) / 1e9,
        "per_launch": per_launch,
        "resident": resident_bytes(layers[0]),
        "roofline": roofline(),
    }
    if args.copy_probe:
        out["copy_probe"] = copy_probe(torch, dev)
    if not args.no_prefill:
        pf = prefill(torch, dev, layers, SHAPES_7B, calls=max(1, args.prefill_calls))
        out["prefill"] = {"M": 2048, "gate_18944x3584": pf["gate"], "down_3584x18944": pf["down"],
                          "peak_tflops": MFMA_PEAK_TFLOPS,
                          "frac_of_peak": min(pf["gate"]["tflops"], pf["down"]["tflops"]) / MFMA_PEAK_TFLOPS}
    if not args.no_neighbours:
        out["layer_with_neighbours"] = neighbours(torch, dev, layers, x, y)
    cpu_layer = layers[0] if not args.no_cpu else None
    del layers[1:]                               # the rotated layers are no longer used
    if not args.no_configs:
        out["cfg3_small_batch"] = small_batch_crossover(torch, dev, gen, 8)
        out["cfg5_masked_27b"] = masked_27b(torch, dev, gen, 4)
    if not args.no_head:
        out["lm_head_q8"] = lm_head(torch, dev)
    if cpu_layer is not None:
        out["cpu_baseline"] = cpu_baseline(torch, cpu_layer, x, D, BITS, SHAPES_7B)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
