#!/usr/bin/env python3
"""Benchmark of the low-bit linear hot path on one MI355X.

A "step" is one pass of the hot path over one batch of synthetic input: the
Llama-2-7B decode linear sweep of BASELINE.json configs[1] - 32 layers x
(q, k, v, o [4096x4096], gate, up [11008x4096], down [4096x11008]) in sym_int4,
fp16 activations at M = 1, every linear a separate launch.  The 224 launches of
a sweep are captured once in a HIP graph and replayed, so that Python launch
cost is not billed as bandwidth.  Weights (3.64 GB) are resident in HBM before
the timed region and exceed the 256 MB Infinity Cache, so every sweep streams
them from HBM.

Prints ONE JSON line: metric / value / unit, the `roofline` object of the
metric's single shape ([11008 x 4096], M = 1), `cpu_baseline` (the oracle's
ggml-style matmul on the host cores), and under `extra` one timed leg per other
configuration of BASELINE.json, each with bound / achieved / peak / frac from
the algorithmic bytes or FLOP of that configuration.
"""
import argparse
import ctypes
import json
import os
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "ipex-llm_amd"))

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E peak
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X published dense fp16 / bf16 MFMA peak

QT = {"sym_int4": 2, "asym_int4": 3, "sym_int8": 8, "nf4": 10, "fp8_e4m3": 15}
QT_BYTES = {2: (18, 32), 3: (20, 32), 8: (34, 32), 10: (34, 64), 15: (132, 128)}
SYM_INT4 = 2
LLAMA2_7B = [("q", 4096, 4096), ("k", 4096, 4096), ("v", 4096, 4096), ("o", 4096, 4096),
             ("gate", 11008, 4096), ("up", 11008, 4096), ("down", 4096, 11008)]
N_LAYERS = 32
# HBM bytes per launch of the metric's GEMV from rocprofv3 counters (FETCH_SIZE x 1.9993 + WRITE_SIZE)
GEMV_TRAFFIC = {"bytes": 25492716, "source": "profiles/gemv_sym_int4_f16_N11008_K4096_M1.md (counter run, not this run)"}


def blob_bytes(n, k, qtype=SYM_INT4):
    tb, qk = QT_BYTES[qtype]
    return n * k // qk * tb


def hbm(byts, ms, **more):
    gbs = byts / (ms * 1e-3) / 1e9
    return dict(bound="hbm", bytes=int(byts), ms=round(ms, 4), achieved=round(gbs, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                frac=round(gbs / HBM_PEAK_GBS, 4), **more)


def mfma(flop, ms, **more):
    tf = flop / (ms * 1e-3) / 1e12
    return dict(bound="mfma", flop=flop, ms=round(ms, 4), achieved=round(tf, 1), peak=MFMA_F16_PEAK_TFLOPS,
                unit="TFLOP/s", frac=round(tf / MFMA_F16_PEAK_TFLOPS, 4), **more)


def device_info(torch, ggml):
    """The `rocminfo` facts the figures rest on, from the HIP runtime, plus the clocks the driver reports now."""
    info = ggml.lowbit_device_info()
    info["hbm_bytes"] = torch.cuda.get_device_properties(0).total_memory
    info["peaks_used"] = {"hbm_GB/s": HBM_PEAK_GBS, "mfma_f16_bf16_dense_TFLOP/s": MFMA_F16_PEAK_TFLOPS}
    try:       # a child process; "sclk clock level: N: (2400Mhz)" style lines
        out = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=20).stdout
        now = {}
        for line in out.splitlines():
            for key in ("sclk", "mclk", "fclk"):
                if key + " clock level" in line and "(" in line:
                    now[key] = line.split("(")[-1].split(")")[0]
        if now:
            info["clocks_now"] = now
    except Exception:  # noqa: BLE001
        pass
    return info


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--m", type=int, default=1, help="rows of x (decode batch)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip the legs of the other configurations")
    ap.add_argument("--roofline-only", action="store_true",
                    help="run only the serialized [11008 x 4096] GEMV loop the roofline object is measured on")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run only the prefill GEMM (M=2048 on [11008 x 4096], sym_int4, fp16) and print its rate")
    ap.add_argument("--batch-only", action="store_true",
                    help="run only the batch-sized product (M=32, 64, 128 on [11008 x 4096], sym_int4, fp16)")
    ap.add_argument("--quantize-only", action="store_true",
                    help="run only the block quantizer (fp32 [11008 x 4096] -> sym_int4, tiled) and print its rate")
    ap.add_argument("--floor-only", action="store_true",
                    help="run the serialized [11008 x 4096] GEMV loop next to what launches that only READ the same bytes "
                         "cost in the same chain (libstream_floor.so: an empty kernel, twelve read patterns)")
    ap.add_argument("--llama3-70b-only", action="store_true",
                    help="run only the Llama-3-70B linear set (nf4 and sym_int8, bf16, M = 1, 16, 1024)")
    ap.add_argument("--mlp-only", action="store_true",
                    help="only the gated MLP at prefill: gate and up as two launches plus the activation, and as one fused launch")
    ap.add_argument("--choice-only", action="store_true",
                    help="only the check of the kernel choice: lowbit_forward_ws against every kernel it chooses from, "
                         "timed on the same inputs (--choice-full: the 40 shapes the estimates were fitted on)")
    ap.add_argument("--choice-full", action="store_true")
    ap.add_argument("--moe-only", action="store_true",
                    help="run only the Mixtral expert FFN legs (fp8_e4m3, 512 tokens top-2, and one token)")
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
        """ms per replay, HIP events on the stream the replays run on (torch's current stream)."""
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
        return e0.elapsed_time(e1) / steps

    def new_weight(n, k, qtype, std, outliers=False):
        w = torch.randn((n, k), generator=gen, device=dev, dtype=torch.float32) * std
        if outliers:                                  # 0.1 % of the entries at +-0.5
            mask = torch.rand((n, k), generator=gen, device=dev) < 0.001
            sign = torch.where(torch.rand((n, k), generator=gen, device=dev) < 0.5, 0.5, -0.5)
            w = torch.where(mask, sign, w)
        blob = torch.empty(blob_bytes(n, k, qtype), dtype=torch.uint8, device=dev)
        ggml.lowbit_quantize(w.data_ptr(), blob.data_ptr(), qtype, n, k, ggml.LAYOUT_TILED, stream())
        torch.cuda.synchronize()
        return blob

    # ------------------------------------------------------------------ quantizer leg
    def quantize_leg(steps, warmup):
        n, k = 11008, 4096
        ws = [torch.randn((n, k), generator=gen, device=dev, dtype=torch.float32) * 0.02 for _ in range(4)]
        bs = [torch.empty(blob_bytes(n, k), dtype=torch.uint8, device=dev) for _ in range(4)]

        def quant():
            for w, b in zip(ws, bs):
                ggml.lowbit_quantize(w.data_ptr(), b.data_ptr(), SYM_INT4, n, k, ggml.LAYOUT_TILED, stream())
        for _ in range(max(1, warmup)):
            quant()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            quant()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / (steps * 4)
        return hbm(4 * n * k + blob_bytes(n, k), ms, kernel="quantize_tiled_kernel<sym_int4> on fp32 [11008 x 4096]")

    if args.quantize_only:
        print(json.dumps({"quantize": quantize_leg(args.steps, args.warmup)}))
        return

    # ------------------------------------------------------------------ Mixtral legs (configs[4])
    def moe_legs():
        import torch.nn.functional as F
        res = {}
        n_exp, hid, ffn, tokens = 8, 4096, 14336, 512
        qt = QT["fp8_e4m3"]
        blobs = {p: [new_weight(n, k, qt, 0.02) for _ in range(n_exp)]
                 for p, (n, k) in (("w1", (ffn, hid)), ("w3", (ffn, hid)), ("w2", (hid, ffn)))}
        ptrs = {p: torch.tensor([b.data_ptr() for b in bl], dtype=torch.int64, device=dev) for p, bl in blobs.items()}
        logits = torch.randn((tokens, n_exp), generator=gen, device=dev)
        hidden = torch.randn((tokens, hid), generator=gen, device=dev).bfloat16()
        _, experts = torch.topk(F.softmax(logits, dim=-1), 2, dim=-1)
        flat = experts.reshape(-1)
        order = torch.argsort(flat, stable=True)
        offsets = torch.zeros(n_exp + 1, dtype=torch.int32, device=dev)
        offsets[1:] = torch.cumsum(torch.bincount(flat, minlength=n_exp), 0).to(torch.int32)
        rows = tokens * 2
        xs = hidden[order // 2].contiguous()
        h1 = torch.empty((rows, ffn), dtype=torch.bfloat16, device=dev)
        h3 = torch.empty((rows, ffn), dtype=torch.bfloat16, device=dev)
        yo = torch.empty((rows, hid), dtype=torch.bfloat16, device=dev)

        ws_bytes = ggml.lowbit_grouped_workspace_bytes(n_exp, rows, hid, ffn)
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)

        # as moe_ffn_grouped runs it: the fused gate/up launch (SiLU in the epilogue), then the down projection
        # with its K-split workspace
        def moe():
            st = stream()
            ggml.lowbit_grouped_mlp_forward(xs.data_ptr(), ptrs["w1"].data_ptr(), ptrs["w3"].data_ptr(), h1.data_ptr(),
                                            offsets.data_ptr(), n_exp, rows, qt, ggml.DT_BF16, ffn, hid, 0, st)
            ggml.lowbit_grouped_forward_ws(h1.data_ptr(), ptrs["w2"].data_ptr(), yo.data_ptr(), offsets.data_ptr(), n_exp,
                                           rows, qt, ggml.DT_BF16, hid, ffn, ws.data_ptr(), ws_bytes, st)

        # the three products as separate grouped launches (the activation and the product of the two halves are
        # then torch's and not in the timed region)
        def moe_unfused():
            st = stream()
            for p, xin, out, n, k in (("w1", xs, h1, ffn, hid), ("w3", xs, h3, ffn, hid), ("w2", h1, yo, hid, ffn)):
                ggml.lowbit_grouped_forward_ws(xin.data_ptr(), ptrs[p].data_ptr(), out.data_ptr(), offsets.data_ptr(), n_exp,
                                               rows, qt, ggml.DT_BF16, n, k, ws.data_ptr(), ws_bytes, st)
        ms = time_graph(capture(moe), 10, 2)
        flop = 2.0 * rows * 3 * ffn * hid
        wb = sum(b.numel() for bl in blobs.values() for b in bl)
        leg = mfma(flop, ms, kernel="gemm_mfma_kernel<fp8_e4m3,bf16> grouped, 256-row tiles: fused gate/up + SiLU, then down with 2 K splits "
                                    "(+ grouped_splitk_reduce_kernel); 8 experts, 512 tokens top-2")
        leg["hbm_floor"] = hbm(wb, ms)
        leg["rows_per_expert"] = [int(v) for v in (offsets[1:] - offsets[:-1]).tolist()]
        leg["three_separate_launches_ms"] = round(time_graph(capture(moe_unfused), 10, 2), 4)
        # what launches that only READ the gate and up weights, in the pattern the grouped GEMM walks them, take
        # (libstream_floor.so; the fused gate/up launch reads the same bytes and multiplies)
        floor_path = os.path.join(ROOT, "ipex-llm_amd", "ipex_llm", "libs", "libstream_floor.so")
        if os.path.exists(floor_path):
            floor = ctypes.CDLL(floor_path)
            floor.stream_floor_read_tiles.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                      ctypes.c_void_p, ctypes.c_void_p]
            sink = torch.zeros(4, dtype=torch.int32, device=dev)
            both = torch.cat([ptrs["w1"], ptrs["w3"]])

            def read_gate_up():
                assert floor.stream_floor_read_tiles(both.data_ptr(), 2 * n_exp, ffn // 16, hid // 128, 2112,
                                                     sink.data_ptr(), stream()) == 0
            leg["gate_up_weights_read_only_ms"] = round(time_graph(capture(read_gate_up), 10, 2), 4)
        res["mixtral_moe_fp8_512tok_top2"] = leg
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
        ms = time_graph(capture(moe_decode), 10, 2) / len(ids)
        tok_bytes = 2 * 3 * blobs["w1"][0].numel() + 2 * (hid + 2 * ffn + 2 * ffn + hid)
        res["mixtral_moe_fp8_decode_top2"] = hbm(tok_bytes, ms, kernel="gemv_mfma_kernel<fp8_e4m3,bf16> expert modes, 2 launches per token")
        return res

    def choice_check(full):
        """lowbit_forward_ws against every kernel it chooses from - GEMV passes, the ring kernel, narrow tiles, the
        GEMM at 1 .. 16 K splits - on the same inputs, each launch on weights it has not just read (several copies
        per graph replay).  Reports how far the pick lies above the fastest alternative."""
        F16, BF16 = (torch.float16, ggml.DT_F16), (torch.bfloat16, ggml.DT_BF16)
        if full:
            cases = ([(2, F16, sh) for sh in ((11008, 4096), (4096, 4096), (4096, 11008), (12288, 4096), (22016, 4096), (1024, 8192),
                                             (8192, 8192), (28672, 8192), (8192, 28672), (2048, 2048), (5632, 2048), (2048, 5632),
                                             (14336, 4096), (4096, 14336))]
                     + [(2, BF16, sh) for sh in ((11008, 4096), (4096, 4096), (8192, 8192))]
                     + [(3, F16, sh) for sh in ((11008, 4096), (4096, 4096), (2048, 2048))]
                     + [(8, BF16, sh) for sh in ((8192, 8192), (1024, 8192), (28672, 8192), (8192, 28672), (10240, 8192))]
                     + [(8, F16, sh) for sh in ((5632, 2048), (4096, 4096), (11008, 4096))]
                     + [(15, BF16, sh) for sh in ((14336, 4096), (4096, 14336), (4096, 4096), (6144, 4096))]
                     + [(10, BF16, sh) for sh in ((28672, 8192), (8192, 8192), (1024, 8192), (8192, 28672), (10240, 8192), (4096, 4096),
                                                  (11008, 4096), (4096, 11008))])
            ms = (17, 24, 32, 40, 48, 64, 96, 128, 160, 192, 256, 320, 384, 512, 640, 768, 1024, 1536, 2048)
        else:
            cases = [(2, F16, (11008, 4096)), (2, F16, (4096, 4096)), (2, F16, (4096, 11008)), (2, BF16, (4096, 4096)),
                     (8, BF16, (8192, 8192)), (10, BF16, (8192, 8192)), (15, BF16, (14336, 4096)), (8, F16, (5632, 2048))]
            ms = (24, 48, 96, 160, 256, 384, 512, 768, 1024, 2048)
        ws_all = 2 << 30
        ws = torch.empty(ws_all, dtype=torch.uint8, device=dev)
        names = {ggml.PLAN_GEMV: "gemv", ggml.PLAN_RING: "ring", ggml.PLAN_GEMM: "gemm", ggml.PLAN_GEMM_SPLIT: "split",
                 ggml.PLAN_GEMM_NARROW: "narrow"}
        points = []
        for qt, (tdt, dt), (n, k) in cases:
            copies = max(2, min(8, int(400e6 / blob_bytes(n, k, qt))))
            blobs = [new_weight(n, k, qt, 0.02) for _ in range(copies)]
            for m in ms:
                x = torch.randn((m, k), generator=gen, device=dev).to(tdt)
                y = torch.empty((m, n), dtype=tdt, device=dev)
                a = (qt, ggml.LAYOUT_TILED, dt, m, n, k)

                def timed(call):
                    def run():
                        st = stream()
                        for b in blobs:
                            call(b, st)
                    g = capture(run)
                    return min(time_graph(g, 4, 2 if i == 0 else 0) for i in range(3)) / copies * 1e3
                need = max(16, ggml.lowbit_workspace_bytes(m, n, k))
                alt = {}
                t_pick = timed(lambda b, st: ggml.lowbit_forward_ws(x.data_ptr(), b.data_ptr(), y.data_ptr(), *a, ws.data_ptr(), need, st))
                if m <= 128:
                    alt["gemv"] = timed(lambda b, st: ggml.lowbit_gemv(x.data_ptr(), b.data_ptr(), y.data_ptr(), *a, 0, st))
                if m <= 256 or qt == 10:
                    alt["ring"] = timed(lambda b, st: ggml.lowbit_gemm_ring(x.data_ptr(), b.data_ptr(), y.data_ptr(), *a, ws.data_ptr(),
                                                                            ws_all, 0, st))
                alt["narrow"] = timed(lambda b, st: ggml.lowbit_gemm_narrow(x.data_ptr(), b.data_ptr(), y.data_ptr(), *a, st))
                for splits in (1, 2, 3, 4, 5, 6, 8, 10, 12, 16):
                    tiles = ((m + 127) // 128) * ((n + 255) // 256)
                    if splits * 2 > k // 128 or splits * tiles * 128 * 256 * 4 > ws_all:
                        break
                    alt[f"s{splits}"] = timed(lambda b, st: ggml.lowbit_gemm_ws(x.data_ptr(), b.data_ptr(), y.data_ptr(), *a, ws.data_ptr(),
                                                                              ws_all, splits, st))
                best = min(alt, key=alt.get)
                points.append({"qtype": qt, "act": "f16" if dt == ggml.DT_F16 else "bf16", "N": n, "K": k, "M": m,
                               "pick": names[ggml.lowbit_forward_plan(qt, ggml.LAYOUT_TILED, m, n, k, True, need)],
                               "pick_us": round(t_pick, 1), "best": best, "best_us": round(alt[best], 1),
                               "above_best": round(t_pick / alt[best], 3)})
            del blobs
        ratios = sorted(p["above_best"] for p in points)
        return {"kernel_choice": {"points": len(points), "mean_above_best": round(sum(ratios) / len(ratios), 4),
                                  "median": ratios[len(ratios) // 2], "more_than_10_percent_above": sum(r > 1.1 for r in ratios),
                                  "worst": sorted(points, key=lambda p: -p["above_best"])[:8],
                                  "sum_of_picks_ms": round(sum(p["pick_us"] for p in points) / 1e3, 3),
                                  "sum_of_bests_ms": round(sum(p["best_us"] for p in points) / 1e3, 3)}}

    if args.choice_only or args.choice_full:
        print(json.dumps(choice_check(args.choice_full)))
        return

    def mlp_legs():
        """The gate and up projections of a Llama-2-7B MLP ([11008 x 4096] each) on a prefill batch, fp16 and bf16:
        as the reference's modules run them - two products, then SiLU and the product as elementwise kernels (torch's:
        they are not this library's, and are timed here because the fused launch replaces them) - and as one
        lowbit_mlp_forward launch.  Six weight pairs per graph replay, so that the weights come from HBM."""
        import torch.nn.functional as F
        res = {}
        n, k = 11008, 4096
        pairs = [(new_weight(n, k, SYM_INT4, 0.02, outliers=True), new_weight(n, k, SYM_INT4, 0.02, outliers=True)) for _ in range(6)]
        for tdt, dt, tag in ((torch.float16, ggml.DT_F16, "f16"), (torch.bfloat16, ggml.DT_BF16, "bf16")):
            for m in (512, 2048):
                x = torch.randn((m, k), generator=gen, device=dev).to(tdt)
                g, u, h = (torch.empty((m, n), dtype=tdt, device=dev) for _ in range(3))
                ws_bytes = max(16, ggml.lowbit_workspace_bytes(m, n, k))
                ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)

                def two():
                    st = stream()
                    for a, b in pairs:
                        for blob, y in ((a, g), (b, u)):
                            ggml.lowbit_forward_ws(x.data_ptr(), blob.data_ptr(), y.data_ptr(), SYM_INT4, ggml.LAYOUT_TILED, dt, m, n, k,
                                                   ws.data_ptr(), ws_bytes, st)
                        torch.mul(F.silu(g), u, out=h)

                def fused():
                    st = stream()
                    for a, b in pairs:
                        ggml.lowbit_mlp_forward(x.data_ptr(), a.data_ptr(), b.data_ptr(), h.data_ptr(), SYM_INT4, dt, m, n, k, 0, st)
                ms2 = time_graph(capture(two), 10, 2) / len(pairs)
                ms1 = time_graph(capture(fused), 10, 2) / len(pairs)
                leg = mfma(2 * 2.0 * m * n * k, ms1, kernel="gemm_mfma_kernel<sym_int4> fused gate/up form, one table-free group")
                leg["two_launches_plus_activation_ms"] = round(ms2, 4)
                res[f"prefill_mlp_gate_up_sym_int4_{tag}_M{m}"] = leg
        return res

    if args.mlp_only:
        print(json.dumps(mlp_legs()))
        return

    if args.moe_only:
        print(json.dumps(moe_legs()))
        return

    if args.llama3_70b_only:
        print(json.dumps(other_configs(ggml, torch, gen, dev, None, capture, time_graph, stream, new_weight, only_70b=True)))
        return

    # ---- synthetic weights: N(0, 0.02) with 0.1 % outliers at +-0.5, quantized on the GPU
    layers = []
    for _ in range(4 if args.prefill_only else N_LAYERS):
        layers.append([(name, n, k, new_weight(n, k, SYM_INT4, 0.02, outliers=True)) for name, n, k in LLAMA2_7B])

    def make_io(m):
        xs = {k: torch.randn((m, k), generator=gen, device=dev, dtype=torch.float32).half()
              for k in (4096, 11008)}
        ys = {name: torch.empty((m, n), dtype=torch.float16, device=dev) for name, n, _ in LLAMA2_7B}
        return xs, ys

    def sweep(m, xs, ys):
        st = stream()
        for mods in layers:
            for name, n, k, blob in mods:
                ggml.lowbit_forward(xs[k].data_ptr(), blob.data_ptr(), ys[name].data_ptr(), SYM_INT4,
                                    ggml.LAYOUT_TILED, ggml.DT_F16, m, n, k, st)

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
        ms4 = time_graph(capture(prefill), 10, 10) / len(gu8)     # clocks settle after some tens of launches
        leg = mfma(2.0 * m * 11008 * 4096, ms4, kernel="gemm_mfma_kernel<sym_int4,f16> on [11008 x 4096], M=%d" % m)
        if m == 2048:
            # The same kernel on the first 8192 rows of the same weights (the tiled layout keeps 16 rows of the
            # weight together): 256 tiles of 256 x 256, one per CU, where [11008 x 4096] has 344 tiles' worth of work.
            # Its time, times 344 / 256, is what dealing the tiles out evenly could reach at best.
            def filled():
                st = stream()
                for b in gu8:
                    ggml.lowbit_forward(xp.data_ptr(), b.data_ptr(), yp.data_ptr(), SYM_INT4, ggml.LAYOUT_TILED,
                                        ggml.DT_F16, m, 8192, 4096, st)
            ms_f = time_graph(capture(filled), 10, 10) / len(gu8)
            leg["filled_launch_N8192"] = {"ms": round(ms_f, 4), "frac": round(2.0 * m * 8192 * 4096 / (ms_f * 1e-3) / 2.5e15, 4),
                                          "tiles": "256 of 256 x 256 on 256 CUs",
                                          "even_deal_bound_ms": round(ms_f * 344 / 256, 4)}
        return leg

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
        msb = time_graph(capture(batch), 5, 3) / len(gu8)
        leg = hbm(blob_bytes(11008, 4096) + m * 4096 * 2 + m * 11008 * 2, msb,
                  kernel="gemm_ring_kernel<sym_int4,f16> on [11008 x 4096], M=%d" % m)
        leg["TFLOP/s"] = round(2.0 * m * 11008 * 4096 / (msb * 1e-3) / 1e12, 1)
        return leg

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
    ms3 = time_graph(capture(headline), max(5, args.steps), max(3, args.warmup))
    hb = blob_bytes(11008, 4096) + args.m * 4096 * 2 + args.m * 11008 * 2
    us = ms3 * 1e3 / len(gu)
    roofline = {"bound": "hbm", "kernel": "gemv_mfma_kernel<sym_int4,f16> on [11008 x 4096], M=%d" % args.m,
                "achieved": round(hb / (us * 1e-6) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(hb / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                "traffic": GEMV_TRAFFIC["bytes"] if args.m == 1 else None, "traffic_source": GEMV_TRAFFIC["source"],
                "bytes_per_launch": hb, "avg_launch_us": round(us, 3),
                "how": "HIP events around graph replays of 64 chained launches over 64 distinct weights"}
    if args.roofline_only:
        print(json.dumps({"roofline": roofline}))
        return
    if args.floor_only:
        # The same chain - one launch per distinct weight, 64 per graph replay, HIP events around the replays - with
        # launches that do nothing, and with launches that read the weight's bytes (rounded down to 16) and nothing else.
        floor = ctypes.CDLL(os.path.join(ROOT, "ipex-llm_amd", "ipex_llm", "libs", "libstream_floor.so"))
        floor.stream_floor_pattern_name.restype = ctypes.c_char_p
        floor.stream_floor_read.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
        floor.stream_floor_empty.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        sink = torch.zeros(4, dtype=torch.int32, device=dev)
        nbytes = hb // 16 * 16

        def chain(launch):
            def run():
                st = stream()
                for b in gu:
                    assert launch(b, st) == 0
            return time_graph(capture(run), max(5, args.steps), max(3, args.warmup)) * 1e3 / len(gu)
        res = {"gemv_us": round(us, 3), "bytes": hb,
               "empty_launch_us": round(chain(lambda b, st: floor.stream_floor_empty(sink.data_ptr(), st)), 3), "reads_us": {}}
        for p in range(floor.stream_floor_patterns()):
            res["reads_us"][floor.stream_floor_pattern_name(p).decode()] = round(
                chain(lambda b, st: floor.stream_floor_read(b.data_ptr(), nbytes, p, sink.data_ptr(), st)), 3)
        best = min(res["reads_us"].values())
        res["fastest_read_us"], res["slowest_read_us"] = best, max(res["reads_us"].values())
        res["fastest_read_frac_of_hbm_peak"] = round(nbytes / (best * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)
        res["gemv_frac_of_hbm_peak"] = roofline["frac"]
        print(json.dumps({"floor": res}))
        return

    ms = time_graph(capture(lambda: sweep(args.m, xs, ys)), args.steps, args.warmup)
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
                               "linears, sym_int4, fp16 x, one launch per linear, HIP-graph replay, "
                               "7 chained launches per layer",
                   "M": args.m, "launches_per_step": launches, "weight_bytes_per_step": w_bytes,
                   "algorithmic_bytes_per_step": total, "device": device_info(torch, ggml)},
        "pct_hbm_peak": round(100.0 * gbs / HBM_PEAK_GBS, 2),
    }
    out["roofline"] = roofline

    if not args.no_extra:
        extra = {}
        # configs[0]: one [4096 x 4096] linear, M = 1, over the 128 distinct q/k/v/o weights
        qkvo = [b for mods in layers for (name, n, k, b) in mods if n == 4096 and k == 4096]

        def cfg0():
            st = stream()
            for b in qkvo:
                ggml.lowbit_forward(xs[4096].data_ptr(), b.data_ptr(), ys["q"].data_ptr(), SYM_INT4, ggml.LAYOUT_TILED,
                                    ggml.DT_F16, 1, 4096, 4096, st)
        if args.m == 1:
            ms0 = time_graph(capture(cfg0), 10, 3) / len(qkvo)
            extra["single_N4096_K4096_M1"] = hbm(blob_bytes(4096, 4096) + 2 * 4096 * 2, ms0,
                                                 kernel="gemv_mfma_kernel<sym_int4,f16> on [4096 x 4096], M=1 (BASELINE configs[0])")
        for m in (4, 8):
            if m == args.m:
                continue
            xs2, ys2 = make_io(m)
            ms2 = time_graph(capture(lambda: sweep(m, xs2, ys2)), max(5, args.steps // 2), 3)
            extra[f"sweep_M{m}"] = hbm(sweep_bytes(m), ms2, launches_per_step=launches)
        # The same sweep as the reference runs it by default: q|k|v stored as one [12288 x 4096] weight
        # (_optimize_pre merges them) and gate|up either concatenated or fused with the activation
        # (xe_linear.mlp_forward_xpu).  Tile rows are contiguous in the tiled layout, so concatenating blobs
        # concatenates rows.
        merged = []
        for mods in layers:
            d = {name: blob for name, _, _, blob in mods}
            merged.append({"qkv": torch.cat([d["q"], d["k"], d["v"]]), "o": d["o"], "gate": d["gate"], "up": d["up"],
                           "gateup": torch.cat([d["gate"], d["up"]]), "down": d["down"]})
        ym = {"qkv": torch.empty((args.m, 12288), dtype=torch.float16, device=dev),
              "gateup": torch.empty((args.m, 22016), dtype=torch.float16, device=dev),
              "act": torch.empty((args.m, 11008), dtype=torch.float16, device=dev)}

        def fwd(x, blob, y, n, k, st):
            ggml.lowbit_forward(x.data_ptr(), blob.data_ptr(), y.data_ptr(), SYM_INT4, ggml.LAYOUT_TILED, ggml.DT_F16,
                                args.m, n, k, st)

        def sweep_merged():
            st = stream()
            for d in merged:
                fwd(xs[4096], d["qkv"], ym["qkv"], 12288, 4096, st)
                fwd(xs[4096], d["o"], ys["o"], 4096, 4096, st)
                fwd(xs[4096], d["gateup"], ym["gateup"], 22016, 4096, st)
                fwd(xs[11008], d["down"], ys["down"], 4096, 11008, st)
        ms5 = time_graph(capture(sweep_merged), max(5, args.steps // 2), 3)
        extra["sweep_merged_qkv_gateup"] = hbm(sweep_bytes(args.m), ms5, launches_per_step=4 * N_LAYERS)
        if args.m <= 16:
            def mlp(d, st):
                ggml.lowbit_mlp_forward(xs[4096].data_ptr(), d["gate"].data_ptr(), d["up"].data_ptr(), ym["act"].data_ptr(),
                                        SYM_INT4, ggml.DT_F16, args.m, 11008, 4096, 0, st)

            def sweep_fused():
                st = stream()
                for mods, d in zip(layers, merged):
                    for name, n, k, blob in mods[:4]:
                        fwd(xs[k], blob, ys[name], n, k, st)
                    mlp(d, st)
                    fwd(xs[11008], d["down"], ys["down"], 4096, 11008, st)
            ms6 = time_graph(capture(sweep_fused), max(5, args.steps // 2), 3)
            extra["sweep_fused_gate_up"] = hbm(sweep_bytes(args.m), ms6, launches_per_step=6 * N_LAYERS)

            def sweep_merged_fused():
                st = stream()
                for d in merged:
                    fwd(xs[4096], d["qkv"], ym["qkv"], 12288, 4096, st)
                    fwd(xs[4096], d["o"], ys["o"], 4096, 4096, st)
                    mlp(d, st)
                    fwd(xs[11008], d["down"], ys["down"], 4096, 11008, st)
            ms7 = time_graph(capture(sweep_merged_fused), max(5, args.steps // 2), 3)
            extra["sweep_merged_qkv_fused_mlp"] = hbm(sweep_bytes(args.m), ms7, launches_per_step=4 * N_LAYERS,
                                                      note="what a converted Llama runs per token: qkv_proj, o_proj, "
                                                           "mlp_forward_xpu, down_proj")
        # the same four launches per layer at M = 4 / 8 (lowbit_mlp_forward fuses gate and up at up to 16 rows)
        for m in (4, 8):
            if m == args.m:
                continue
            xs2, ys2 = make_io(m)
            yq = torch.empty((m, 12288), dtype=torch.float16, device=dev)
            ya = torch.empty((m, 11008), dtype=torch.float16, device=dev)

            def sweep_m_merged_fused():
                st = stream()
                for d in merged:
                    for x, blob, y, n, k in ((xs2[4096], d["qkv"], yq, 12288, 4096), (xs2[4096], d["o"], ys2["o"], 4096, 4096)):
                        ggml.lowbit_forward(x.data_ptr(), blob.data_ptr(), y.data_ptr(), SYM_INT4, ggml.LAYOUT_TILED, ggml.DT_F16,
                                            m, n, k, st)
                    ggml.lowbit_mlp_forward(xs2[4096].data_ptr(), d["gate"].data_ptr(), d["up"].data_ptr(), ya.data_ptr(),
                                            SYM_INT4, ggml.DT_F16, m, 11008, 4096, 0, st)
                    ggml.lowbit_forward(xs2[11008].data_ptr(), d["down"].data_ptr(), ys2["down"].data_ptr(), SYM_INT4,
                                        ggml.LAYOUT_TILED, ggml.DT_F16, m, 4096, 11008, st)
            ms8 = time_graph(capture(sweep_m_merged_fused), max(5, args.steps // 2), 3)
            extra[f"sweep_M{m}_merged_qkv_fused_mlp"] = hbm(sweep_bytes(m), ms8, launches_per_step=4 * N_LAYERS)
        del merged
        extra["prefill_M2048_N11008_K4096"] = prefill_leg(2048)
        extra["quantize_sym_int4_N11008_K4096"] = quantize_leg(5, 2)
        extra.update(other_configs(ggml, torch, gen, dev, layers[0], capture, time_graph, stream, new_weight))
        extra.update(mlp_legs())
        extra.update(moe_legs())
        out["extra"] = extra

    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(layers[0], args.m, ggml, torch)

    print(json.dumps(out))


def other_configs(ggml, torch, gen, dev, layer0, capture, time_graph, stream, new_weight, only_70b=False):
    """The parity-test configurations of BASELINE.json timed once each (not the headline): configs[2] prefill
    and configs[3] Llama-3-70B shapes in nf4 / sym_int8."""
    res = {}

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
        ms = time_graph(capture(run), reps, 2)
        flop = sum(2.0 * m * n * k for n, k, _ in mods)
        byts = sum(b.numel() + 2 * m * (n + k) for n, k, b in mods)
        return ms, flop, byts

    def leg(mods, qtype, dt, tdt, m, reps, compute_bound):
        ms, flop, byts = time_set(mods, qtype, dt, tdt, m, reps)
        out = mfma(flop, ms) if compute_bound else hbm(byts, ms)
        out["TFLOP/s" if not compute_bound else "GB/s"] = round((flop / ms / 1e9) if not compute_bound else (byts / ms / 1e6), 1)
        out["launches"] = len(mods)
        return out

    def fused_mlp_leg(mods, qtype, dt, tdt, m, reps, compute_bound=True):
        """mods = [qkv, o, gate, up, down]: gate and up go out as one lowbit_mlp_forward launch (SiLU and the product in
        its epilogue; the FLOP counted are the linears' alone, as in the other legs)."""
        (nq, kq, bq), (no, ko, bo), (ng, kg, bg), (_, _, bu), (nd, kd, bd) = mods
        x = torch.randn((m, kq), generator=gen, device=dev, dtype=torch.float32).to(tdt)
        ys = [torch.empty((m, n), dtype=tdt, device=dev) for n in (nq, no, ng, nd)]
        ws_bytes = max(16, max(ggml.lowbit_workspace_bytes(m, n, k) for n, k, _ in mods))
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)

        def run():
            st = stream()
            for (n, k, blob), xin, y in (((nq, kq, bq), x, ys[0]), ((no, ko, bo), x, ys[1])):
                ggml.lowbit_forward_ws(xin.data_ptr(), blob.data_ptr(), y.data_ptr(), qtype, ggml.LAYOUT_TILED, dt, m, n, k,
                                       ws.data_ptr(), ws_bytes, st)
            ggml.lowbit_mlp_forward(x.data_ptr(), bg.data_ptr(), bu.data_ptr(), ys[2].data_ptr(), qtype, dt, m, ng, kg, 0, st)
            ggml.lowbit_forward_ws(ys[2].data_ptr(), bd.data_ptr(), ys[3].data_ptr(), qtype, ggml.LAYOUT_TILED, dt, m, nd, kd,
                                   ws.data_ptr(), ws_bytes, st)
        ms = time_graph(capture(run), reps, 2)
        out = mfma(sum(2.0 * m * n * k for n, k, _ in mods), ms) if compute_bound else \
            hbm(sum(b.numel() + 2 * m * (n + k) for n, k, b in mods), ms)
        out["launches"] = 4
        return out

    def merged_qkv(mods):
        """The first three weights (q, k, v: same K) as one: the tile rows of a merged weight follow each other in
        the tiled layout, so the blobs concatenate."""
        (nq, k, bq), (nk, _, bk), (nv, _, bv) = mods[:3]
        return [(nq + nk + nv, k, torch.cat([bq, bk, bv]))] + list(mods[3:])

    if not only_70b:
        # configs[2]: one layer's 7 linears at M = 512 / 2048, sym_int4 and asym_int4, fp16
        sym = [(n, k, b) for _, n, k, b in layer0]
        asym = [(n, k, new_weight(n, k, QT["asym_int4"], 0.02, outliers=True)) for n, k, _ in sym]
        for name, mods in (("sym_int4", sym), ("asym_int4", asym)):
            for m in (512, 2048):
                res[f"prefill_layer_{name}_M{m}"] = leg(mods, QT[name], ggml.DT_F16, torch.float16, m, 5, True)
        # as a converted model runs the layer: q | k | v are one weight of [12288 x 4096] (merge_qkv), five launches;
        # and with gate and up in the fused launch that also applies the activation (lowbit_mlp_forward), four
        for m in (512, 2048):
            res[f"prefill_layer_sym_int4_M{m}_merged_qkv"] = leg(merged_qkv(sym), QT["sym_int4"], ggml.DT_F16,
                                                                 torch.float16, m, 5, True)
            res[f"prefill_layer_sym_int4_M{m}_merged_qkv_fused_mlp"] = fused_mlp_leg(merged_qkv(sym), QT["sym_int4"], ggml.DT_F16,
                                                                                 torch.float16, m, 5)
        # the same layer at serving batch sizes (one decode token per sequence)
        for m in (32, 64, 128):
            res[f"batched_decode_layer_sym_int4_M{m}"] = leg(sym, QT["sym_int4"], ggml.DT_F16, torch.float16, m, 10, False)
            res[f"batched_decode_layer_sym_int4_M{m}_merged_qkv_fused_mlp"] = fused_mlp_leg(merged_qkv(sym), QT["sym_int4"], ggml.DT_F16,
                                                                                        torch.float16, m, 10, False)
        del asym
    # configs[3]: Llama-3-70B linear set (q, k, v, gate, up, down), bf16
    shapes70 = [(8192, 8192), (1024, 8192), (1024, 8192), (28672, 8192), (28672, 8192), (8192, 28672)]
    for name in ("nf4", "sym_int8"):
        mods = [(n, k, new_weight(n, k, QT[name], 0.015)) for n, k in shapes70]
        for m in (1, 16, 1024):
            res[f"llama3_70b_{name}_M{m}"] = leg(mods, QT[name], ggml.DT_BF16, torch.bfloat16, m, 5 if m > 16 else 20, m > 16)
        # q | k | v as one weight of [10240 x 8192], four launches
        mq = merged_qkv(mods)
        for m in (1, 16, 1024):
            res[f"llama3_70b_{name}_M{m}_merged_qkv"] = leg(mq, QT[name], ggml.DT_BF16, torch.bfloat16, m,
                                                            5 if m > 16 else 20, m > 16)
        del mods, mq
    return res


def cpu_baseline(mods, m, ggml, torch):
    """The reference's CPU low-bit matmul (restated in oracle/; the reference's own kernel is a closed binary) on
    the host cores of the GPU box.  Headline entry: the 7 linears of ONE of the 32 layers of the benchmarked
    sweep, repeated for about 10 s.  `more`: the other configurations, a few seconds each."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import numpy as np
    import lowbit_oracle as orc
    isa = orc.use_fast_build()
    threads = orc.max_threads()
    try:
        model = [ln.split(":", 1)[1].strip() for ln in open("/proc/cpuinfo") if ln.startswith("model name")][0]
    except Exception:  # noqa: BLE001
        model = "unknown"
    rng = np.random.default_rng(7)

    def host_blob(n, k, blob, qtype):
        g = torch.empty_like(blob)
        ggml.lowbit_relayout(blob.data_ptr(), g.data_ptr(), qtype, n, k, ggml.LAYOUT_TILED,
                             ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        return g.cpu().numpy()

    def timed(fn, budget_s):
        fn()
        t0 = time.perf_counter()
        passes = 0
        while True:
            fn()
            passes += 1
            dt = time.perf_counter() - t0
            if dt > budget_s:
                return passes, dt

    def l3_note(working_set_bytes):
        """Whether a repeated pass over `working_set_bytes` stays in the host's last-level caches (then the rate is
        a cache rate, not a DRAM rate): the sum of the distinct L3 instances the visible cores report."""
        total = 0
        try:
            seen = set()
            for cpu in sorted(os.listdir("/sys/devices/system/cpu")):
                base = f"/sys/devices/system/cpu/{cpu}/cache/index3"
                if not os.path.isdir(base):
                    continue
                shared = open(base + "/shared_cpu_list").read().strip()
                if shared in seen:
                    continue
                seen.add(shared)
                size = open(base + "/size").read().strip()
                total += int(size[:-1]) * (1 << 10 if size.endswith("K") else 1 << 20 if size.endswith("M") else 1)
        except Exception:  # noqa: BLE001
            total = 0
        if not total:
            return f"working set {working_set_bytes >> 20} MiB, host L3 size unknown"
        fits = "fits" if working_set_bytes <= total else "does not fit"
        return f"working set {working_set_bytes >> 20} MiB {fits} the host's {total >> 20} MiB of L3 (repeated passes)"

    blobs = [(n, k, host_blob(n, k, blob, SYM_INT4)) for name, n, k, blob in mods]
    xs = {k: rng.standard_normal((m, k)).astype(np.float32) for k in (4096, 11008)}
    nbytes = sum(b.size + m * k * 2 + m * n * 2 for n, k, b in blobs)

    def one_pass():
        for n, k, b in blobs:
            orc.mul_mat_q(b, xs[k], (n, k), SYM_INT4)
    passes, dt = timed(one_pass, 10.0)
    out = {"value": round(nbytes * passes / dt / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
           "cpu": model, "isa": isa,
           "sample": f"1 of 32 layers (7 linears, {nbytes} algorithmic bytes) x {passes} passes, "
                     f"oracle ggml-style Q8_0-activation matmul, OpenMP; {l3_note(sum(b.size for _, _, b in blobs))}"}
    more = {}
    # configs[0]: [4096 x 4096], M = 1
    n, k, b = blobs[0]
    x1 = rng.standard_normal((1, k)).astype(np.float32)
    p, t = timed(lambda: orc.mul_mat_q(b, x1, (n, k), SYM_INT4), 2.0)
    more["single_N4096_K4096_M1"] = {"GB/s": round((b.size + 2 * (n + k)) * p / t / 1e9, 2),
                                     "sample": f"{p} calls; {l3_note(b.size)}"}
    # configs[1] at M = 4 / 8: the same layer
    for mm in (4, 8):
        xm = {kk: rng.standard_normal((mm, kk)).astype(np.float32) for kk in (4096, 11008)}
        p, t = timed(lambda: [orc.mul_mat_q(bb, xm[kk], (nn, kk), SYM_INT4) for nn, kk, bb in blobs], 3.0)
        byts = sum(bb.size + mm * kk * 2 + mm * nn * 2 for nn, kk, bb in blobs)
        more[f"layer_M{mm}"] = {"GB/s": round(byts * p / t / 1e9, 2), "sample": f"1 of 32 layers x {p} passes"}
    # configs[2]: one layer at M = 512 (x 32 would be the sweep)
    x512 = {kk: rng.standard_normal((512, kk)).astype(np.float32) for kk in (4096, 11008)}
    t0 = time.perf_counter()
    for nn, kk, bb in blobs:
        orc.mul_mat_q(bb, x512[kk], (nn, kk), SYM_INT4)
    t = time.perf_counter() - t0
    more["prefill_layer_sym_int4_M512"] = {"TFLOP/s": round(sum(2.0 * 512 * nn * kk for nn, kk, _ in blobs) / t / 1e12, 4),
                                           "sample": "1 of 32 layers, one pass"}
    # configs[3], sym_int8 (nf4 has no CPU matmul in the reference: low_bit_linear.py:689-692 raises): [8192 x 8192], M = 1
    w8 = (rng.standard_normal((8192, 8192)) * 0.015).astype(np.float32)
    b8 = orc.quantize(w8, QT["sym_int8"])
    x8 = rng.standard_normal((1, 8192)).astype(np.float32)
    p, t = timed(lambda: orc.mul_mat_q(b8, x8, (8192, 8192), QT["sym_int8"]), 2.0)
    more["llama3_70b_q_proj_sym_int8_M1"] = {"GB/s": round((b8.size + 4 * 8192) * p / t / 1e9, 2),
                                             "sample": f"{p} calls; {l3_note(b8.size)}"}
    # the block quantizer (ggml_quantize_tensor): GB/s of fp32 input + blob output
    p, t = timed(lambda: orc.quantize(w8, SYM_INT4), 2.0)
    more["quantize_sym_int4_8192x8192"] = {"GB/s": round((w8.nbytes + blob_bytes(8192, 8192)) * p / t / 1e9, 2),
                                           "sample": f"{p} calls"}
    out["more"] = more
    return out


if __name__ == "__main__":
    main()
