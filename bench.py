#!/usr/bin/env python3
"""Benchmark of the block-float hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--legs all|primary|none]
    python bench.py --summarise trace KERNEL_TRACE.csv | pmc COUNTERS.csv [KERNEL] | traffic FETCH.csv WRITE.csv

A "step" is one pass of the primary workload over one batch of synthetic input with everything resident in HBM:
by default the Falcon-7B decode MLP (bf16 [32,4544] x BFP8_B [4544,18176], then [32,18176] x BFP8_B [18176,4544]).
Each step uses the next of several distinct copies of the weights (footprint > 512 MiB), so the 256 MiB
Infinity Cache cannot serve the weight stream.  One JSON line is printed; `legs` carries the other workloads
(pack / unpack GB/s, Mistral decode GEMMs, prefill GEMM, BERT-like bmm), each with its own roofline fraction.

Times come from HIP events recorded on the stream the kernels are launched on (torch's current stream).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "tt-metal_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
ROTATE_BYTES = 512 << 20
# HBM bytes per launch come from hardware counters (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE, on this same command
# with --counter-calibration).  Counters cannot be read from inside this process: `bench.py --summarise traffic FETCH.csv
# WRITE.csv` turns the two counter files into the summary below, and every run reads roofline.traffic from it (null for a
# leg the summary does not list).
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "bench_all_workloads_hbm_traffic.md")
WORKLOAD_NAMES = {
    "decode_falcon": "decode_falcon: bf16 [32,4544] x BFP8_B [4544,18176], then [32,18176] x BFP8_B [18176,4544] (Falcon-7B decode MLP)",
    "decode_mistral": "decode_mistral: M=32 bf16 x fused QKV / O (BFP8_B) and gate / up / down (BFP4_B) of a Mistral-7B layer",
    "prefill": "prefill: bf16 [2048,4096] x BFP8_B [4096,14336], and bmm [12,384,1024] x [12,1024,1024] BFP8_B",
    "pack_bfp4_4k": "pack_bfp4_4k: fused tilize+pack and unpack+untilize of fp32 [1,1,4096,4096] (stress mixture) to BFP4_B",
    "pack_bfp8_1k": "pack_bfp8_1k: fused tilize+pack and unpack+untilize of fp32 [1,1,1024,1024] ~ N(0,1) to BFP8_B",
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="decode_falcon",
                    choices=["decode_falcon", "decode_mistral", "prefill", "pack_bfp4_4k", "pack_bfp8_1k"])
    ap.add_argument("--legs", default="all", choices=["all", "primary", "none"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--row-major", action="store_true", help="GEMM activations and output dense row-major instead of TILE layout")
    ap.add_argument("--counter-calibration", action="store_true",
                    help="first launch a plain elementwise copy of 256 MiB three times, so that a hardware-counter run "
                         "(FETCH_SIZE / WRITE_SIZE) can be scaled by what the same counter reads for a known transfer")
    ap.add_argument("--summarise", nargs="+", metavar=("KIND", "FILE"),
                    help="no benchmark: print a summary of rocprofv3 output of this command (trace FILE | pmc FILE [KERNEL] | traffic FETCH WRITE)")
    return ap.parse_args()


def main():
    args = parse_args()
    if args.summarise:
        from ttmi import counters

        kind, files = args.summarise[0], args.summarise[1:]
        if kind == "trace" and len(files) == 1:
            print(counters.summarise_trace(files[0]))
        elif kind == "pmc" and len(files) in (1, 2):
            print(counters.summarise_pmc(files[0], files[1] if len(files) == 2 else None))
        elif kind == "traffic" and len(files) == 2:
            print(counters.traffic_lines(files[0], files[1]))
        else:
            sys.exit("bench.py --summarise trace FILE | pmc FILE [KERNEL] | traffic FETCH_FILE WRITE_FILE")
        return
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (no collectives, no sharding); --gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    from ttmi import capi, workloads

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the block-float path has no CPU fallback", file=sys.stderr)
        sys.exit(3)
    torch.cuda.set_device(0)
    capi.lib()
    FMT = {"bfp8_b": capi.BFLOAT8_B, "bfp4_b": capi.BFLOAT4_B}

    def dev(a):
        return torch.from_numpy(np.ascontiguousarray(a)).cuda()

    def bf16_dev(bits):
        return dev(bits.view(np.int16)).view(torch.bfloat16)

    def time_loop(fn, steps, warmup):
        """fn(i) launches step i.  Returns average milliseconds per step over `steps` timed steps."""
        for i in range(warmup):
            fn(i)
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for i in range(steps):
            fn(warmup + i)
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) / steps

    def copies_for(nbytes):
        return max(2, -(-ROTATE_BYTES // nbytes))

    def hbm_roofline(nbytes, ms):
        gbs = nbytes / (ms * 1e-3) / 1e9
        return {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None}

    def mfma_roofline(flops, ms):
        tf = flops / (ms * 1e-3) / 1e12
        return {"bound": "mfma", "achieved": round(tf, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None}

    # ------------------------------------------------------------------------------------------------
    # GEMM workloads
    # ------------------------------------------------------------------------------------------------
    def gemm_leg(spec, steps, warmup, seed):
        name, m, k, n, fmt, batch = spec
        b = batch or 1
        w = workloads.weights_f32(k, n, seed, batch=batch)
        words = capi.pack_tensor(FMT[fmt], dev(w))
        del w
        a_shape_batch = batch
        a = bf16_dev(workloads.activations_bf16(m, k, seed + 1, batch=a_shape_batch))
        nbytes = workloads.gemm_bytes(m, k, n, fmt, batch)
        flops = workloads.gemm_flops(m, k, n, batch)
        hbm_bound = m <= 64
        ncopies = copies_for(words.numel() * 4) if hbm_bound else 2
        wcopies = [words] + [words.clone() for _ in range(ncopies - 1)]
        acopies = [a] + [a.clone() for _ in range(ncopies - 1)]
        # pre-built argument lists: the timed loop is nothing but C-ABI calls on torch's current stream
        L = capi.lib()
        stream = torch.cuda.current_stream().cuda_stream
        c = torch.empty((b, m, n), dtype=torch.bfloat16, device="cuda")
        # operands in TILE layout, as ttnn.matmul requires of its inputs and returns its output
        # (ttnn/cpp/ttnn/operations/matmul.hpp:39-42); --row-major times dense row-major activations and output instead
        layout = capi.ROW_MAJOR if args.row_major else capi.TILE
        if layout == capi.TILE:
            acopies = [capi.tilize(t) for t in acopies]
        calls = [(acopies[j].data_ptr(), layout, wcopies[j].data_ptr(), FMT[fmt], b, b, m, k, n, None, capi.ACT_NONE,
                  c.data_ptr(), layout, capi.BFLOAT16, None, 0, stream) for j in range(ncopies)]

        def run(i):
            capi.check(L.ttmi_matmul_bfp(*calls[i % ncopies]))

        ms = time_loop(run, steps, warmup)
        roof = hbm_roofline(nbytes, ms) if hbm_bound else mfma_roofline(flops, ms)
        vendor_ms = None
        if not hbm_bound:
            # for scale only: the vendor library's plain bf16 GEMM (torch.matmul -> hipBLASLt / rocBLAS) on the same M, K, N with
            # dense bf16 weights already in memory, i.e. without any block-float work; the better of B as [K,N] and as [N,K]^T
            dense = torch.randn((b, k, n), dtype=torch.bfloat16, device="cuda")
            dense_t = dense.transpose(1, 2).contiguous()
            a_dense = torch.randn((b, m, k), dtype=torch.bfloat16, device="cuda")
            vendor_ms = min(time_loop(lambda i: torch.matmul(a_dense, dense), steps, 2),
                            time_loop(lambda i: torch.matmul(a_dense, dense_t.transpose(1, 2)), steps, 2))
            del dense, dense_t, a_dense
        leg = {"workload": name, "shape": [b, m, k, n], "weights": fmt, "ms": round(ms, 5),
               "tflops": round(flops / (ms * 1e-3) / 1e12, 2), "gbs": round(nbytes / (ms * 1e-3) / 1e9, 1),
               "algorithmic_bytes": nbytes, "flops": flops, "weight_copies_rotated": ncopies,
               "layout": "row_major" if args.row_major else "tile", "roofline": roof}
        if vendor_ms is not None:
            leg["vendor_bf16_gemm_ms"] = round(vendor_ms, 5)
            leg["vendor_bf16_gemm_frac"] = round(flops / (vendor_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)
        return leg, (run, wcopies, acopies, c)

    def block_leg(name, steps, warmup, seed):
        """A whole decode MLP block as tt-metal's model code issues it (M = 32, operands in TILE layout), every launch
        through the C ABI: Falcon-7B dense_h_to_4h with fused GELU -> dense_4h_to_h (models/demos/falcon7b/tt/falcon_mlp.py:56-80),
        Mistral-7B silu(x w1) * (x w3) -> w2 (models/demos/mistral7b/tt/mistral_mlp.py:43-82)."""
        L = capi.lib()
        stream = torch.cuda.current_stream().cuda_stream
        m = 32
        if name.startswith("falcon_mlp_block"):
            gemms = [("w1", 4544, 18176, "bfp8_b", capi.ACT_GELU), ("w2", 18176, 4544, "bfp8_b", capi.ACT_NONE)]
        else:
            gemms = [("w1", 4096, 14336, "bfp4_b", capi.ACT_SILU), ("w3", 4096, 14336, "bfp4_b", capi.ACT_NONE),
                     ("w2", 14336, 4096, "bfp4_b", capi.ACT_NONE)]
        packed = {g[0]: capi.pack_tensor(FMT[g[3]], dev(workloads.weights_f32(g[1], g[2], seed + i))) for i, g in enumerate(gemms)}
        per_block = sum(t.numel() * 4 for t in packed.values())
        ncopies = copies_for(per_block)
        copies = [{k: (v if j == 0 else v.clone()) for k, v in packed.items()} for j in range(ncopies)]
        x = capi.tilize(bf16_dev(workloads.activations_bf16(m, gemms[0][1], seed + 7)))
        hidden = gemms[0][2]
        h1 = torch.empty(m * hidden, dtype=torch.bfloat16, device="cuda")
        h3 = torch.empty(m * hidden, dtype=torch.bfloat16, device="cuda")
        out = torch.empty(m * gemms[-1][2], dtype=torch.bfloat16, device="cuda")

        def mm(a, w, k, n, fmt, act, c):
            return (a.data_ptr(), capi.TILE, w.data_ptr(), FMT[fmt], 1, 1, m, k, n, None, act, c.data_ptr(), capi.TILE, capi.BFLOAT16, None, 0, stream)

        plans = []
        for cp in copies:
            if name.startswith("falcon_mlp_block"):
                plans.append([("mm", mm(x, cp["w1"], 4544, 18176, "bfp8_b", capi.ACT_GELU, h1)),
                              ("mm", mm(h1, cp["w2"], 18176, 4544, "bfp8_b", capi.ACT_NONE, out))])
            else:
                plans.append([("mm", mm(x, cp["w1"], 4096, 14336, "bfp4_b", capi.ACT_SILU, h1)),
                              ("mm", mm(x, cp["w3"], 4096, 14336, "bfp4_b", capi.ACT_NONE, h3)),
                              ("el", (capi.OP_MUL, h1.data_ptr(), h3.data_ptr(), 0.0, h1.data_ptr(), h1.numel(), stream)),
                              ("mm", mm(h1, cp["w2"], 14336, 4096, "bfp4_b", capi.ACT_NONE, out))])

        if name == "falcon_mlp_block_bfp8_act":
            # the same block with a BFLOAT8_B intermediate, as Falcon-40B's BFLOAT8_B configuration issues it
            # (models/demos/falcon40b/tt/falcon_mlp.py:97-135, output_dtype of dense_h_to_4h): packed in the epilogue of the
            # first GEMM, expanded inside the second (ttmi_matmul_bfp_ab) - two launches, no bf16 copy of the intermediate
            h8 = torch.empty(m * hidden // 1024 * 1088 // 4, dtype=torch.int32, device="cuda")
            plans = [[("mm", (x.data_ptr(), capi.TILE, cp["w1"].data_ptr(), FMT["bfp8_b"], 1, 1, m, 4544, 18176, None, capi.ACT_GELU, h8.data_ptr(),
                              capi.TILE, capi.BFLOAT8_B, None, 0, stream)),
                      ("ab", (h8.data_ptr(), capi.BFLOAT8_B, cp["w2"].data_ptr(), FMT["bfp8_b"], 1, 1, m, 18176, 4544, None, capi.ACT_NONE, out.data_ptr(),
                              capi.TILE, capi.BFLOAT16, None, 0, stream))] for cp in copies]

        if name == "mistral_mlp_block_fused":
            # the same block with silu(x w1) * (x w3) as ONE launch (ttmi_matmul_bfp_gated), then w2: two launches instead of four
            plans = [[("gated", (x.data_ptr(), capi.TILE, cp["w1"].data_ptr(), cp["w3"].data_ptr(), FMT["bfp4_b"], 1, 1, m, 4096, 14336, None,
                                 capi.ACT_SILU, h1.data_ptr(), capi.TILE, capi.BFLOAT16, None, 0, stream)),
                      ("mm", mm(h1, cp["w2"], 14336, 4096, "bfp4_b", capi.ACT_NONE, out))] for cp in copies]

        def run(i):
            for kind, call in plans[i % ncopies]:
                capi.check(L.ttmi_matmul_bfp(*call) if kind == "mm" else L.ttmi_matmul_bfp_gated(*call) if kind == "gated" else
                           L.ttmi_matmul_bfp_ab(*call) if kind == "ab" else L.ttmi_eltwise_bf16(*call))

        ms = time_loop(run, steps, warmup)
        nbytes = sum(workloads.gemm_bytes(m, g[1], g[2], g[3], None) for g in gemms) + (3 * m * hidden * 2 if len(gemms) == 3 else 0)
        if name == "falcon_mlp_block_bfp8_act":    # the intermediate is written and read as packed tiles
            nbytes -= 2 * (m * hidden * 2 - m * hidden // 1024 * 1088)
        if name == "mistral_mlp_block_fused":      # x once, no [32, 14336] intermediates but the one that feeds w2
            nbytes = sum((g[1] // 32) * (g[2] // 32) * 576 for g in gemms) + m * 4096 * 2 + 2 * m * hidden * 2 + m * 4096 * 2
        flops = sum(workloads.gemm_flops(m, g[1], g[2], None) for g in gemms)
        leg = {"workload": name, "launches": len(plans[0]), "ms": round(ms, 5), "tflops": round(flops / (ms * 1e-3) / 1e12, 2),
               "gbs": round(nbytes / (ms * 1e-3) / 1e9, 1), "algorithmic_bytes": nbytes, "flops": flops,
               "weight_copies_rotated": ncopies, "layout": "tile", "roofline": hbm_roofline(nbytes, ms)}
        del copies, packed
        return leg

    def codec_leg(name, x_np, fmt, steps, warmup):
        x = dev(x_np)
        nbytes_in = x.numel() * 4
        words = capi.pack_tensor(fmt, x)
        nbytes = nbytes_in + words.numel() * 4
        ncopies = copies_for(nbytes_in)
        xs = [x] + [x.clone() for _ in range(ncopies - 1)]
        ws = [words] + [words.clone() for _ in range(ncopies - 1)]
        L = capi.lib()
        stream = torch.cuda.current_stream().cuda_stream
        batch, h, w = capi._bhw(x)
        out_words = torch.empty_like(words)
        out_x = torch.empty_like(x)
        pack_calls = [(fmt, t.data_ptr(), capi.FLOAT32, batch, h, w, w, h * w, out_words.data_ptr(), stream) for t in xs]
        unpack_calls = [(fmt, t.data_ptr(), batch, h, w, out_x.data_ptr(), capi.FLOAT32, stream) for t in ws]

        ms_p = time_loop(lambda i: capi.check(L.ttmi_pack_rowmajor_as_bfp_tiles(*pack_calls[i % ncopies])), steps, warmup)
        ms_u = time_loop(lambda i: capi.check(L.ttmi_unpack_bfp_tiles_as_rowmajor(*unpack_calls[i % ncopies])), steps, warmup)

        def graph_ms(entry, calls):
            """The same launches (one per rotating buffer) captured once into a HIP graph and replayed: what the kernels take
            when no host call stands between them (a launch from Python costs 5 to 9 us here, more than a small kernel)."""
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            on_side = [c[:-1] + (side.cuda_stream,) for c in calls]
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for c in on_side:
                    capi.check(entry(*c))
            reps = max(2, -(-steps // len(on_side)))
            graph.replay()
            torch.cuda.synchronize()
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            for _ in range(reps):
                graph.replay()
            stop.record()
            torch.cuda.synchronize()
            return start.elapsed_time(stop) / (reps * len(on_side))

        ms_p_graph = graph_ms(L.ttmi_pack_rowmajor_as_bfp_tiles, pack_calls)
        ms_u_graph = graph_ms(L.ttmi_unpack_bfp_tiles_as_rowmajor, unpack_calls)
        # same loop on one buffer: the working set sits in the Infinity Cache ("hot")
        ms_p_hot = time_loop(lambda i: capi.check(L.ttmi_pack_rowmajor_as_bfp_tiles(*pack_calls[0])), steps, warmup)
        legs = []
        runs = (lambda i: capi.check(L.ttmi_pack_rowmajor_as_bfp_tiles(*pack_calls[i % ncopies])),
                lambda i: capi.check(L.ttmi_unpack_bfp_tiles_as_rowmajor(*unpack_calls[i % ncopies])))
        keep = (xs, ws, out_words, out_x)
        for op, ms_stream, ms_graph, hot in (("pack", ms_p, ms_p_graph, ms_p_hot), ("unpack", ms_u, ms_u_graph, None)):
            ms = min(ms_stream, ms_graph)
            leg = {"workload": f"{name}_{op}", "shape": list(x.shape), "ms": round(ms, 5), "gbs": round(nbytes / (ms * 1e-3) / 1e9, 1),
                   "algorithmic_bytes": nbytes, "buffers_rotated": ncopies, "roofline": hbm_roofline(nbytes, ms),
                   "ms_stream_launches": round(ms_stream, 5), "ms_hip_graph": round(ms_graph, 5)}
            if hot is not None:
                leg["gbs_cache_resident"] = round(nbytes / (hot * 1e-3) / 1e9, 1)
            legs.append(leg)
        return legs, (runs, keep)

    def measured_ceilings():
        """What this box delivers to kernels that do no arithmetic, with kernels the box already has and the same rotation over
        more than the Infinity Cache holds: a read-only pass (torch.sum), a copy (torch.mul(src, 1.0, out=dst)) and an empty
        launch, timed as every leg is.  A roofline fraction can then be read against 8 TB/s and against what the part gives."""
        n = 128 << 20                                   # 512 MiB of fp32 per buffer
        bufs = [torch.ones(n, dtype=torch.float32, device="cuda") for _ in range(3)]
        out = torch.empty(n, dtype=torch.float32, device="cuda")
        ms_read = time_loop(lambda i: torch.sum(bufs[i % 3]), 12, 3)
        ms_copy = time_loop(lambda i: torch.mul(bufs[i % 3], 1.0, out=out), 12, 3)
        # the decode GEMM's own size: 88 MB read per launch, rotated the same way
        k = 22 << 20
        ms_read_88mb = time_loop(lambda i: torch.sum(bufs[i % 3][(i % 5) * k:(i % 5 + 1) * k]), 30, 5)
        del bufs, out
        torch.cuda.empty_cache()
        tiny = torch.zeros(64, dtype=torch.float32, device="cuda")
        ms_launch = time_loop(lambda i: tiny.add_(1.0), 200, 20)
        return {"measured_read_gbs": round(n * 4 / (ms_read * 1e-3) / 1e9, 1), "measured_copy_gbs": round(2 * n * 4 / (ms_copy * 1e-3) / 1e9, 1),
                "measured_read_88mb_us": round(ms_read_88mb * 1e3, 2), "measured_read_88mb_gbs": round(k * 4 / (ms_read_88mb * 1e-3) / 1e9, 1),
                "launch_floor_us": round(ms_launch * 1e3, 2),
                "how": "torch.sum over 512 MiB (3 buffers rotated), torch.mul(src, 1.0, out=dst) over 512 MiB + 512 MiB, torch.sum over 88 MB slices, "
                       "a 64-element add_ back to back; HIP events on the launching stream"}

    if args.counter_calibration:
        src = torch.ones(64 << 20, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.mul(src, 1.0, out=dst)   # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    t0 = time.time()
    legs = []
    primary = None
    primary_state = None
    steps, warmup = args.steps, args.warmup

    def note(msg):
        print(f"[bench {time.time() - t0:6.1f}s] {msg}", file=sys.stderr, flush=True)

    gemm_sets = {"decode_falcon": workloads.DECODE_FALCON, "decode_mistral": workloads.DECODE_MISTRAL, "prefill": workloads.PREFILL}
    order = [args.workload] + ([w for w in ("decode_falcon", "decode_mistral", "prefill", "pack_bfp4_4k", "pack_bfp8_1k")
                               if w != args.workload] if args.legs == "all" else [])
    results = {}
    primary_runs, primary_keep = [], []
    for wl in order:
        note(f"workload {wl}")
        is_primary = wl == args.workload
        sub_steps = steps if is_primary else max(10, min(steps, 30))
        if wl in gemm_sets:
            sub = []
            for idx, spec in enumerate(gemm_sets[wl]):
                big = spec[1] > 64
                leg, state = gemm_leg(spec, max(5, sub_steps // 5) if big and not is_primary else sub_steps, 2 if big else warmup, 1234 + 10 * idx)
                sub.append(leg)
                if is_primary:
                    primary_runs.append(state[0])
                    primary_keep.append(state)
                del state
                torch.cuda.empty_cache()
            if not is_primary or args.legs != "none":
                block = {"decode_falcon": "falcon_mlp_block", "decode_mistral": "mistral_mlp_block"}.get(wl)
                if block and not args.row_major:
                    sub.append(block_leg(block, sub_steps, warmup, 4321))
                    torch.cuda.empty_cache()
                    if wl == "decode_mistral":
                        sub.append(block_leg("mistral_mlp_block_fused", sub_steps, warmup, 4321))
                        torch.cuda.empty_cache()
                    if wl == "decode_falcon":
                        sub.append(block_leg("falcon_mlp_block_bfp8_act", sub_steps, warmup, 4321))
                        torch.cuda.empty_cache()
            results[wl] = sub
        else:
            fmt = capi.BFLOAT4_B if wl == "pack_bfp4_4k" else capi.BFLOAT8_B
            x = workloads.stress_mixture() if wl == "pack_bfp4_4k" else workloads.roundtrip_1k()
            results[wl], state = codec_leg(wl, x, fmt, sub_steps, warmup)
            if is_primary:
                primary_runs.extend(state[0])
                primary_keep.append(state)
            del state
            torch.cuda.empty_cache()
        if is_primary:
            # THE timed region of the bench contract: W warm-up steps, then exactly K steps, one step = every part of
            # the workload once, back to back on one stream, device synchronised on both sides
            def step(i):
                for run in primary_runs:
                    run(i)

            total_ms = time_loop(step, steps, warmup)
            primary_keep.clear()
            primary_runs = []
            torch.cuda.empty_cache()

    prim = [l for l in results[args.workload] if "launches" not in l]     # the whole-block legs are reported, not summed
    if args.workload in gemm_sets:
        total_flops = sum(l["flops"] for l in prim)
        value, unit = total_flops / (total_ms * 1e-3) / 1e12, "TFLOP/s"
        dtype = "bf16"
    else:
        total_bytes = sum(l["algorithmic_bytes"] for l in prim)
        value, unit = total_bytes / (total_ms * 1e-3) / 1e9, "GB/s"
        dtype = "u32"
    metric = "bfp8_b-weight matmul TFLOP/s + % roofline (M=32, M=2048); pack/unpack GB/s"
    dominant = max(prim, key=lambda l: l["ms"])

    # ------------------------------------------------------------------------------------------------
    # CPU baseline: the oracle (a port of the reference's host path) timed on this host, bounded sample
    # ------------------------------------------------------------------------------------------------
    cpu = None
    if not args.no_cpu_baseline:
        note("cpu baseline")
        from concurrent.futures import ThreadPoolExecutor

        from oracle import bfp_oracle as oracle

        oracle.build()
        host_threads = torch.get_num_threads()

        def pack_all_cores(fmt_code, x2d):
            """The oracle's from_torch sequence on bands of 32-row multiples, one band per host thread (ctypes drops the GIL)."""
            rows = x2d.shape[0]
            band = max(32, (rows // host_threads) // 32 * 32)
            bands = [x2d[r:r + band] for r in range(0, rows, band)]
            t = time.time()
            with ThreadPoolExecutor(host_threads) as pool:
                list(pool.map(lambda b: oracle.from_torch_bfp_tiles(fmt_code, np.ascontiguousarray(b)), bands))
            return time.time() - t
        if args.workload in gemm_sets:
            name, m, k, n, fmt, batch = gemm_sets[args.workload][0]
            n_s = min(n, 2048)
            w = workloads.weights_f32(k, n_s, 999)
            t = time.time()
            words = oracle.from_torch_bfp_tiles(FMT[fmt], w)
            t_pack = time.time() - t
            t = time.time()
            w_un = oracle.to_torch_bfp_tiles(FMT[fmt], words, (k, n_s))
            t_unpack = time.time() - t
            a = torch.from_numpy(workloads.bf16_bits_to_f32(workloads.activations_bf16(m, k, 998)))
            wt = torch.from_numpy(w_un)
            threads = torch.get_num_threads()
            torch.matmul(a, wt)
            reps, t = 0, time.time()
            while time.time() - t < 8.0:
                torch.matmul(a, wt)
                reps += 1
            t_mm = (time.time() - t) / reps
            # single-thread gold loop (tests/tt_metal/tt_metal/test_gold_impls.hpp:237-290) on a slice
            n_g = 256
            t = time.time()
            oracle.gold_bmm(oracle.bf16_truncate(a.numpy()), oracle.bf16_truncate(w_un[:, :n_g]), 1, m, k, n_g)
            t_gold = time.time() - t
            cpu = {"value": round(2.0 * m * k * n_s / t_mm / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
                   "sample": f"torch.matmul fp32 [{m},{k}]x[{k},{n_s}] on oracle-unpacked {fmt} weights ({n_s} of {n} columns, {reps} reps); "
                             f"oracle from_torch sequence on that slice, 1 thread",
                   "gold_bmm_1thread_tflops": round(2.0 * m * k * n_g / t_gold / 1e12, 5),
                   "from_torch_pack_melem_s_1thread": round(k * n_s / t_pack / 1e6, 1),
                   "from_torch_pack_melem_s_all_threads": round(k * n_s / pack_all_cores(FMT[fmt], w) / 1e6, 1),
                   "to_torch_unpack_melem_s_1thread": round(k * n_s / t_unpack / 1e6, 1)}
        else:
            fmt = capi.BFLOAT4_B if args.workload == "pack_bfp4_4k" else capi.BFLOAT8_B
            x = (workloads.stress_mixture((1, 1, 2048, 4096)) if args.workload == "pack_bfp4_4k" else workloads.roundtrip_1k())
            t = time.time()
            words = oracle.from_torch_bfp_tiles(fmt, x)
            t_pack = time.time() - t
            t = time.time()
            oracle.to_torch_bfp_tiles(fmt, words, x.shape)
            t_unpack = time.time() - t
            nb = x.size * 4 + words.size * 4
            cpu = {"value": round(2 * nb / (t_pack + t_unpack) / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
                   "sample": f"oracle from_torch + to_torch host sequences on fp32 {list(x.shape)}",
                   "from_torch_pack_melem_s_1thread": round(x.size / t_pack / 1e6, 1),
                   "from_torch_pack_melem_s_all_threads": round(x.size / pack_all_cores(fmt, x.reshape(-1, x.shape[-1])) / 1e6, 1),
                   "host_threads": host_threads,
                   "to_torch_unpack_melem_s_1thread": round(x.size / t_unpack / 1e6, 1)}

    from ttmi import counters

    measured_traffic = counters.read_traffic(TRAFFIC_SUMMARY)
    for leg in (l for wl in order for l in results[wl]):
        leg["roofline"]["traffic"] = measured_traffic.get(leg["workload"])

    note("measured ceilings")
    ceilings = measured_ceilings()
    line = {
        "metric": metric, "value": round(value, 3), "unit": unit, "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(total_ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic",
        "config": {"workload": WORKLOAD_NAMES[args.workload], "parts": [l["workload"] for l in prim],
                   "note": "weights rotate over distinct copies (>512 MiB) so the Infinity Cache cannot serve them"},
        "roofline": dict(dominant["roofline"], kernel=dominant["workload"], **{k: v for k, v in ceilings.items() if k != "how"}),
        "measured_ceilings": ceilings,
        "cpu_baseline": cpu,
        "legs": [l for wl in order for l in results[wl]],
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
