#!/usr/bin/env python3
"""Benchmark of the low-bit linear hot path on one MI355X.

A "step" is one pass of the hot path over one batch of synthetic input: the
Llama-2-7B decode linear sweep of BASELINE.json configs[1] - 32 layers x
(q, k, v, o [4096x4096], gate, up [11008x4096], down [4096x11008]) in sym_int4,
fp16 activations at M = 1, every linear a separate launch.  The 224 launches of
a sweep are captured once in a HIP graph and replayed, so that Python launch
cost is not billed as bandwidth.  The seven linears of a layer are chained on
one stream; --parallel-branches instead captures q|k|v and gate|up as parallel
graph branches (measured slower on MI355X: cross-queue dependencies cost more
than the overlap gains).  Weights (3.64 GB) are resident
in HBM before the timed region and exceed the 256 MB Infinity Cache, so every
sweep streams them from HBM.

Prints ONE JSON line: metric / value / unit, the roofline and cpu_baseline objects, and one timed leg per
other configuration under "extra".
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "ipex-llm_amd"))

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E peak
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X published dense fp16/bf16 MFMA peak

SYM_INT4 = 2
LLAMA2_7B = [("q", 4096, 4096), ("k", 4096, 4096), ("v", 4096, 4096), ("o", 4096, 4096),
             ("gate", 11008, 4096), ("up", 11008, 4096), ("down", 4096, 11008)]
N_LAYERS = 32


def blob_bytes(n, k):
    return n * k // 32 * 18


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--m", type=int, default=1, help="rows of x (decode batch)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip the M=4/8 and single-shape figures")
    ap.add_argument("--parallel-branches", action="store_true",
                    help="capture q|k|v and gate|up as parallel graph branches instead of one chain")
    ap.add_argument("--roofline-only", action="store_true",
                    help="run only the serialized [11008 x 4096] GEMV loop the roofline object is measured on")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run only the prefill GEMM (M=2048 on [11008 x 4096], sym_int4, fp16) and print its rate")
    ap.add_argument("--batch-only", action="store_true",
                    help="run only the batch-sized product (M=32, 64, 128 on [11008 x 4096], sym_int4, fp16)")
    ap.add_argument("--quantize-only", action="store_true",
                    help="run only the block quantizer (fp32 [11008 x 4096] -> sym_int4, tiled) and print its rate")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (no sharding, no collectives); --gpus must be 1",
              file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the low-bit kernels have no CPU implementation", file=sys.stderr)
        sys.exit(3)
    import ipex_llm.ggml.model.llama.llama_cpp as ggml

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev)
    gen.manual_seed(1002)

    def stream():
        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    if args.quantize_only:
        n, k = 11008, 4096
        ws = [torch.randn((n, k), generator=gen, device=dev, dtype=torch.float32) * 0.02 for _ in range(4)]
        bs = [torch.empty(blob_bytes(n, k), dtype=torch.uint8, device=dev) for _ in range(4)]

        def quant():
            for w, b in zip(ws, bs):
                ggml.lowbit_quantize(w.data_ptr(), b.data_ptr(), SYM_INT4, n, k, ggml.LAYOUT_TILED, stream())
        for _ in range(max(1, args.warmup)):
            quant()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            quant()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / (args.steps * 4)
        byts = 4 * n * k + blob_bytes(n, k)
        print(json.dumps({"quantize": {"kernel": "quantize_tiled_kernel<sym_int4> on fp32 [11008 x 4096]",
                                       "bound": "hbm", "bytes_per_launch": byts, "avg_launch_us": round(us, 2),
                                       "achieved": round(byts / us / 1e3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                       "frac": round(byts / us / 1e3 / HBM_PEAK_GBS, 4)}}))
        return

    # ---- synthetic weights: N(0, 0.02) with 0.1 % outliers at +-0.5, quantized on the GPU
    layers = []
    for _ in range(4 if args.prefill_only else N_LAYERS):
        mods = []
        for name, n, k in LLAMA2_7B:
            w = torch.randn((n, k), generator=gen, device=dev, dtype=torch.float32) * 0.02
            mask = torch.rand((n, k), generator=gen, device=dev) < 0.001
            sign = torch.where(torch.rand((n, k), generator=gen, device=dev) < 0.5, 0.5, -0.5)
            w = torch.where(mask, sign, w)
            blob = torch.empty(blob_bytes(n, k), dtype=torch.uint8, device=dev)
            ggml.lowbit_quantize(w.data_ptr(), blob.data_ptr(), SYM_INT4, n, k, ggml.LAYOUT_TILED, stream())
            mods.append((name, n, k, blob))
            del w, mask, sign
        layers.append(mods)
    torch.cuda.synchronize()

    def make_io(m):
        xs = {k: torch.randn((m, k), generator=gen, device=dev, dtype=torch.float32).half()
              for k in (4096, 11008)}
        ys = {name: torch.empty((m, n), dtype=torch.float16, device=dev) for name, n, _ in LLAMA2_7B}
        return xs, ys

    side = [torch.cuda.Stream(), torch.cuda.Stream()]

    def sweep(m, xs, ys):
        def run(mod):
            name, n, k, blob = mod
            ggml.lowbit_forward(xs[k].data_ptr(), blob.data_ptr(), ys[name].data_ptr(), SYM_INT4,
                                ggml.LAYOUT_TILED, ggml.DT_F16, m, n, k, stream())

        def branches(group):
            # first member on the current stream, the others on side streams, then join
            cur = torch.cuda.current_stream()
            for s_, mod in zip(side, group[1:]):
                s_.wait_stream(cur)
                with torch.cuda.stream(s_):
                    run(mod)
            run(group[0])
            for s_, _ in zip(side, group[1:]):
                cur.wait_stream(s_)

        for mods in layers:
            if not args.parallel_branches:
                for mod in mods:
                    run(mod)
            else:
                branches(mods[0:3])      # q, k, v
                run(mods[3])             # o
                branches(mods[4:6])      # gate, up
                run(mods[6])             # down

    def capture(fn):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()                                   # eager warm-up on the capture stream
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fn()
        return g

    def time_graph(g, steps, warmup):
        for _ in range(warmup):
            g.replay()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps         # ms per replay

    launches = N_LAYERS * len(LLAMA2_7B)
    w_bytes = sum(blob_bytes(n, k) for _, n, k in LLAMA2_7B) * N_LAYERS

    def sweep_bytes(m):
        io = sum(m * k * 2 + m * n * 2 for _, n, k in LLAMA2_7B) * N_LAYERS
        return w_bytes + io

    xs, ys = make_io(args.m)

    def prefill_leg(m=2048):
        """One [11008 x 4096] linear at M rows over 8 distinct weights per graph replay."""
        gu8 = [b for mods in layers for (name, n, k, b) in mods if name in ("gate", "up")][:8]
        xp = torch.randn((m, 4096), generator=gen, device=dev, dtype=torch.float32).half()
        yp = torch.empty((m, 11008), dtype=torch.float16, device=dev)

        def prefill():
            st = stream()
            for b in gu8:
                ggml.lowbit_forward(xp.data_ptr(), b.data_ptr(), yp.data_ptr(), SYM_INT4, ggml.LAYOUT_TILED,
                                    ggml.DT_F16, m, 11008, 4096, st)
        g4 = capture(prefill)
        ms4 = time_graph(g4, 10, 10) / len(gu8)           # clocks settle after some tens of launches
        flop = 2.0 * m * 11008 * 4096
        return {"kernel": "gemm_mfma_kernel<sym_int4,f16> on [11008 x 4096], M=%d" % m, "bound": "mfma",
                "flop_per_launch": flop, "ms": round(ms4, 4), "achieved": round(flop / (ms4 * 1e-3) / 1e12, 1),
                "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(flop / (ms4 * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS, 4)}

    if args.prefill_only:
        print(json.dumps({"prefill": prefill_leg()}))
        return

    def batch_leg(m):
        """One [11008 x 4096] linear at a serving batch of M rows, cycling over the 64 distinct gate / up
        weights (1.6 GB, far beyond the Infinity Cache) per graph replay, with the workspace the library
        asks for (HBM-bound: the weights are read once)."""
        gu8 = [b for mods in layers for (name, n, k, b) in mods if name in ("gate", "up")]
        xp = torch.randn((m, 4096), generator=gen, device=dev, dtype=torch.float32).half()
        yp = torch.empty((m, 11008), dtype=torch.float16, device=dev)
        ws_bytes = max(16, ggml.lowbit_workspace_bytes(m, 11008, 4096))
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)

        def batch():
            st = stream()
            for b in gu8:
                ggml.lowbit_forward_ws(xp.data_ptr(), b.data_ptr(), yp.data_ptr(), SYM_INT4, ggml.LAYOUT_TILED,
                                       ggml.DT_F16, m, 11008, 4096, ws.data_ptr(), ws_bytes, st)
        gb = capture(batch)
        msb = time_graph(gb, 5, 3) / len(gu8)
        hb = blob_bytes(11008, 4096) + m * 4096 * 2 + m * 11008 * 2
        return {"kernel": "gemm_ring_kernel<sym_int4,f16> + reduction on [11008 x 4096], M=%d" % m, "bound": "hbm",
                "bytes_per_launch": hb, "ms": round(msb, 4), "achieved": round(hb / (msb * 1e-3) / 1e9, 1),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(hb / (msb * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                "TFLOP/s": round(2.0 * m * 11008 * 4096 / (msb * 1e-3) / 1e12, 1)}

    if args.batch_only:
        print(json.dumps({"batch": {"M%d" % m: batch_leg(m) for m in (32, 64, 128)}}))
        return

    # ---- roofline leg: the metric's single shape (N=11008, K=4096) as a serialized chain of
    # launches cycling over the 64 distinct gate/up weights (1.6 GB, far beyond the Infinity Cache)
    gu = [b for mods in layers for (name, n, k, b) in mods if name in ("gate", "up")]

    def headline():
        st = stream()
        for b in gu:
            ggml.lowbit_forward(xs[4096].data_ptr(), b.data_ptr(), ys["gate"].data_ptr(), SYM_INT4,
                                ggml.LAYOUT_TILED, ggml.DT_F16, args.m, 11008, 4096, st)
    g3 = capture(headline)
    ms3 = time_graph(g3, max(5, args.steps), max(3, args.warmup))
    hb = blob_bytes(11008, 4096) + args.m * 4096 * 2 + args.m * 11008 * 2
    us = ms3 * 1e3 / len(gu)
    roofline = {"bound": "hbm", "kernel": "gemv_mfma_kernel<sym_int4,f16> on [11008 x 4096], M=%d" % args.m,
                "achieved": round(hb / (us * 1e-6) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(hb / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                # HBM bytes per launch from rocprofv3 FETCH_SIZE / WRITE_SIZE counters of this very loop
                # (profiles/gemv_sym_int4_f16_N11008_K4096_M1.md); valid for M = 1 only
                "traffic": 25496723 if args.m == 1 else None,
                "bytes_per_launch": hb, "avg_launch_us": round(us, 3),
                "how": "HIP events around graph replays of 64 chained launches over 64 distinct weights"}
    if args.roofline_only:
        print(json.dumps({"roofline": roofline}))
        return

    g = capture(lambda: sweep(args.m, xs, ys))
    ms = time_graph(g, args.steps, args.warmup)
    total = sweep_bytes(args.m)
    gbs = total / (ms * 1e-3) / 1e9

    out = {
        "metric": "sym_int4 decode GEMV GB/s",
        "value": round(gbs, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "Llama-2-7B decode linear sweep (BASELINE configs[1]): 32 layers x 7 "
                               "linears, sym_int4, fp16 x, one launch per linear, HIP-graph replay, " +
                               ("7 chained launches per layer" if not args.parallel_branches else
                                "q|k|v and gate|up as parallel graph branches"),
                   "M": args.m, "launches_per_step": launches, "weight_bytes_per_step": w_bytes,
                   "algorithmic_bytes_per_step": total},
        "pct_hbm_peak": round(100.0 * gbs / HBM_PEAK_GBS, 2),
    }
    out["roofline"] = roofline

    if not args.no_extra:
        extra = {}
        for m in (4, 8):
            if m == args.m:
                continue
            xs2, ys2 = make_io(m)
            g2 = capture(lambda: sweep(m, xs2, ys2))
            ms2 = time_graph(g2, max(5, args.steps // 2), 3)
            extra[f"sweep_M{m}"] = {"ms_per_step": round(ms2, 4),
                                    "GB/s": round(sweep_bytes(m) / (ms2 * 1e-3) / 1e9, 1)}
            del g2
        # same sweep with q|k|v stored as one [12288 x 4096] weight and gate|up as one [22016 x 4096]
        # (what the reference does by default: merged qkv_proj, fused gate/up): 4 launches per layer
        merged = []
        for mods in layers[:N_LAYERS]:
            d = {name: blob for name, _, _, blob in mods}
            # tile rows are contiguous in the tiled layout, so concatenating blobs concatenates rows
            merged.append([("qkv", 12288, 4096, torch.cat([d["q"], d["k"], d["v"]])), ("o", 4096, 4096, d["o"]),
                           ("gateup", 22016, 4096, torch.cat([d["gate"], d["up"]])),
                           ("down", 4096, 11008, d["down"])])
        ym = {"qkv": torch.empty((args.m, 12288), dtype=torch.float16, device=dev), "o": ys["o"],
              "gateup": torch.empty((args.m, 22016), dtype=torch.float16, device=dev), "down": ys["down"]}

        def sweep_merged():
            st = stream()
            for mods in merged:
                for name, n, k, blob in mods:
                    ggml.lowbit_forward(xs[k].data_ptr(), blob.data_ptr(), ym[name].data_ptr(), SYM_INT4,
                                        ggml.LAYOUT_TILED, ggml.DT_F16, args.m, n, k, st)
        g5 = capture(sweep_merged)
        ms5 = time_graph(g5, max(5, args.steps // 2), 3)
        extra["sweep_merged_qkv_gateup"] = {"ms_per_step": round(ms5, 4), "launches_per_step": 4 * N_LAYERS,
                                            "GB/s": round(sweep_bytes(args.m) / (ms5 * 1e-3) / 1e9, 1)}
        del merged, g5
        # same sweep with the gate and up projections fused into one launch that also applies
        # SiLU(gate) * up (xe_linear.mlp_forward_xpu): 6 launches per layer
        if args.m <= 4:
            yg = torch.empty((args.m, 11008), dtype=torch.float16, device=dev)

            def sweep_fused():
                st = stream()
                for mods in layers:
                    d = {name: (n, k, blob) for name, n, k, blob in mods}
                    for name in ("q", "k", "v", "o"):
                        n, k, blob = d[name]
                        ggml.lowbit_forward(xs[k].data_ptr(), blob.data_ptr(), ys[name].data_ptr(), SYM_INT4,
                                            ggml.LAYOUT_TILED, ggml.DT_F16, args.m, n, k, st)
                    ggml.lowbit_mlp_forward(xs[4096].data_ptr(), d["gate"][2].data_ptr(), d["up"][2].data_ptr(),
                                            yg.data_ptr(), SYM_INT4, ggml.DT_F16, args.m, 11008, 4096, 0, st)
                    n, k, blob = d["down"]
                    ggml.lowbit_forward(xs[k].data_ptr(), blob.data_ptr(), ys["down"].data_ptr(), SYM_INT4,
                                        ggml.LAYOUT_TILED, ggml.DT_F16, args.m, n, k, st)
            g6 = capture(sweep_fused)
            ms6 = time_graph(g6, max(5, args.steps // 2), 3)
            extra["sweep_fused_gate_up"] = {"ms_per_step": round(ms6, 4), "launches_per_step": 6 * N_LAYERS,
                                            "GB/s": round(sweep_bytes(args.m) / (ms6 * 1e-3) / 1e9, 1)}
            del g6
        extra["prefill_M2048_N11008_K4096"] = prefill_leg(2048)
        extra.update(other_configs(ggml, torch, gen, dev, layers[0], capture, time_graph, stream))
        out["extra"] = extra

    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(layers[0], args.m, ggml, torch)

    print(json.dumps(out))


QT = {"sym_int4": 2, "asym_int4": 3, "sym_int8": 8, "nf4": 10, "fp8_e4m3": 15}
QT_BYTES = {2: (18, 32), 3: (20, 32), 8: (34, 32), 10: (34, 64), 15: (132, 128)}


def other_configs(ggml, torch, gen, dev, layer0, capture, time_graph, stream):
    """The parity-test configurations of BASELINE.json timed once each (not the headline):
    configs[2] prefill, configs[3] Llama-3-70B shapes in nf4 / sym_int8, configs[4] Mixtral experts (prefill and decode)."""
    res = {}

    def new_weight(n, k, qtype, std):
        w = torch.randn((n, k), generator=gen, device=dev, dtype=torch.float32) * std
        tb, qk = QT_BYTES[qtype]
        blob = torch.empty(n * k // qk * tb, dtype=torch.uint8, device=dev)
        ggml.lowbit_quantize(w.data_ptr(), blob.data_ptr(), qtype, n, k, ggml.LAYOUT_TILED, stream())
        torch.cuda.synchronize()
        return blob

    def time_set(mods, qtype, dt, tdt, m, reps):
        xs = {k: torch.randn((m, k), generator=gen, device=dev, dtype=torch.float32).to(tdt)
              for k in {k for _, k, _ in mods}}
        ys = {n: torch.empty((m, n), dtype=tdt, device=dev) for n, _, _ in mods}

        # caller-owned workspace: lets the GEMM split K where the output tiles alone do not fill the GPU
        ws_bytes = max(16, max(ggml.lowbit_workspace_bytes(m, n, k) for n, k, _ in mods))
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)

        def run():
            st = stream()
            for n, k, blob in mods:
                ggml.lowbit_forward_ws(xs[k].data_ptr(), blob.data_ptr(), ys[n].data_ptr(), qtype, ggml.LAYOUT_TILED,
                                       dt, m, n, k, ws.data_ptr(), ws_bytes, st)
        g = capture(run)
        ms = time_graph(g, reps, 2)
        flop = sum(2.0 * m * n * k for n, k, _ in mods)
        byts = sum(b.numel() + 2 * m * (n + k) for n, k, b in mods)
        return {"ms": round(ms, 4), "TFLOP/s": round(flop / ms / 1e9, 1), "GB/s": round(byts / ms / 1e6, 1)}

    # configs[2]: one layer's 7 linears at M = 512 / 2048, sym_int4 and asym_int4, fp16
    sym = [(n, k, b) for _, n, k, b in layer0]
    asym = [(n, k, new_weight(n, k, QT["asym_int4"], 0.02)) for n, k, _ in sym]
    for name, mods in (("sym_int4", sym), ("asym_int4", asym)):
        for m in (512, 2048):
            res[f"prefill_layer_{name}_M{m}"] = time_set(mods, QT[name], ggml.DT_F16, torch.float16, m, 5)
    # the same layer at serving batch sizes (one decode token per sequence)
    for m in (32, 64, 128):
        res[f"batched_decode_layer_sym_int4_M{m}"] = time_set(sym, QT["sym_int4"], ggml.DT_F16, torch.float16, m, 10)
    del asym
    # configs[3]: Llama-3-70B linear set (q, k, v, gate, up, down), bf16
    shapes70 = [(8192, 8192), (1024, 8192), (1024, 8192), (28672, 8192), (28672, 8192), (8192, 28672)]
    for name in ("nf4", "sym_int8"):
        mods = [(n, k, new_weight(n, k, QT[name], 0.015)) for n, k in shapes70]
        for m in (1, 16, 1024):
            res[f"llama3_70b_{name}_M{m}"] = time_set(mods, QT[name], ggml.DT_BF16, torch.bfloat16, m,
                                                      5 if m > 16 else 20)
        del mods
    # configs[4]: Mixtral 8x7B expert FFN, fp8_e4m3, 512 tokens, top-2, bf16: three grouped launches
    import torch.nn.functional as F
    n_exp, hid, ffn, tokens = 8, 4096, 14336, 512
    qt = QT["fp8_e4m3"]
    blobs = {p: [new_weight(n, k, qt, 0.02) for _ in range(n_exp)]
             for p, (n, k) in (("w1", (ffn, hid)), ("w3", (ffn, hid)), ("w2", (hid, ffn)))}
    ptrs = {p: torch.tensor([b.data_ptr() for b in bl], dtype=torch.int64, device=dev) for p, bl in blobs.items()}
    logits = torch.randn((tokens, n_exp), generator=gen, device=dev)
    hidden = torch.randn((tokens, hid), generator=gen, device=dev).bfloat16()
    prob, experts = torch.topk(F.softmax(logits, dim=-1), 2, dim=-1)
    flat = experts.reshape(-1)
    order = torch.argsort(flat, stable=True)
    offsets = torch.zeros(n_exp + 1, dtype=torch.int32, device=dev)
    offsets[1:] = torch.cumsum(torch.bincount(flat, minlength=n_exp), 0).to(torch.int32)
    rows = tokens * 2
    xs = hidden[order // 2].contiguous()
    h1 = torch.empty((rows, ffn), dtype=torch.bfloat16, device=dev)
    h3 = torch.empty((rows, ffn), dtype=torch.bfloat16, device=dev)
    yo = torch.empty((rows, hid), dtype=torch.bfloat16, device=dev)

    def moe():
        st = stream()
        ggml.lowbit_grouped_forward(xs.data_ptr(), ptrs["w1"].data_ptr(), h1.data_ptr(), offsets.data_ptr(), n_exp,
                                    rows, qt, ggml.DT_BF16, ffn, hid, st)
        ggml.lowbit_grouped_forward(xs.data_ptr(), ptrs["w3"].data_ptr(), h3.data_ptr(), offsets.data_ptr(), n_exp,
                                    rows, qt, ggml.DT_BF16, ffn, hid, st)
        ggml.lowbit_grouped_forward(h1.data_ptr(), ptrs["w2"].data_ptr(), yo.data_ptr(), offsets.data_ptr(), n_exp,
                                    rows, qt, ggml.DT_BF16, hid, ffn, st)
    g = capture(moe)
    ms = time_graph(g, 10, 2)
    flop = 2.0 * rows * 3 * ffn * hid
    wb = sum(b.numel() for bl in blobs.values() for b in bl)
    res["mixtral_moe_fp8_512tok_top2"] = {"ms": round(ms, 4), "TFLOP/s": round(flop / ms / 1e9, 1),
                                          "weight_GB/s": round(wb / ms / 1e6, 1),
                                          "rows_per_expert": [int(v) for v in (offsets[1:] - offsets[:-1]).tolist()]}
    # the same experts at decode: one token through its top-2 experts in two launches (xe_linear.moe_forward_vec);
    # 16 different expert pairs per graph replay, so that the weights come from HBM
    pairs = [(i % n_exp, (i * 3 + 1) % n_exp) for i in range(16)]
    ids = [torch.tensor(p, dtype=torch.int32, device=dev) for p in pairs]
    rw = torch.tensor([0.6, 0.4], dtype=torch.float32, device=dev)
    x1 = torch.randn((1, hid), generator=gen, device=dev).bfloat16()
    work = torch.empty((2, ffn), dtype=torch.bfloat16, device=dev)
    y1 = torch.empty((1, hid), dtype=torch.bfloat16, device=dev)

    def moe_decode():
        st = stream()
        for t in ids:
            ggml.lowbit_moe_forward(x1.data_ptr(), t.data_ptr(), rw.data_ptr(), 2, n_exp, ptrs["w1"].data_ptr(),
                                    ptrs["w3"].data_ptr(), ptrs["w2"].data_ptr(), work.data_ptr(), y1.data_ptr(), qt,
                                    ggml.DT_BF16, hid, ffn, 0, st)
    g = capture(moe_decode)
    ms = time_graph(g, 10, 2) / len(ids)
    tok_bytes = 2 * 3 * blobs["w1"][0].numel()
    res["mixtral_moe_fp8_decode_top2"] = {"ms": round(ms, 4), "weight_GB/s": round(tok_bytes / ms / 1e6, 1),
                                          "launches_per_token": 2}
    return res


def cpu_baseline(mods, m, ggml, torch):
    """The reference's CPU low-bit matmul (restated in oracle/) on the host cores, on a bounded
    sample: the 7 linears of ONE layer, repeated for about 10 s."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import numpy as np
    import lowbit_oracle as orc
    threads = orc.max_threads()
    blobs = []
    for name, n, k, blob in mods:
        g = torch.empty_like(blob)
        ggml.lowbit_relayout(blob.data_ptr(), g.data_ptr(), SYM_INT4, n, k, ggml.LAYOUT_TILED,
                             ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        blobs.append((n, k, g.cpu().numpy()))
    torch.cuda.synchronize()
    rng = np.random.default_rng(7)
    xs = {k: rng.standard_normal((m, k)).astype(np.float32) for k in (4096, 11008)}
    nbytes = sum(b.size + m * k * 2 + m * n * 2 for n, k, b in blobs)

    def one_pass():
        for n, k, b in blobs:
            orc.mul_mat_q(b, xs[k], (n, k), SYM_INT4)
    one_pass()
    t0 = time.perf_counter()
    passes = 0
    while True:
        one_pass()
        passes += 1
        dt = time.perf_counter() - t0
        if dt > 10.0:
            break
    return {"value": round(nbytes * passes / dt / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"1 of 32 layers (7 linears, {nbytes} algorithmic bytes) x {passes} passes, "
                      f"oracle ggml-style Q8_0-activation matmul, OpenMP"}


if __name__ == "__main__":
    main()
