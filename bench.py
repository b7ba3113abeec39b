#!/usr/bin/env python3
"""Headline benchmark of the quantized-matmul path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-graph] [--no-cpu] [--no-detail]

Workload (BASELINE.json configs[1]): decode GEMV at Llama-3-8B FFN shapes —
gate and up 4096->14336, down 14336->4096 — with Q6_K and Q8_0 weights, int-dot
on q8_1 activations, batch 1.  One step = those six GEMV launches over one set of
weight matrices; consecutive steps rotate through several distinct weight sets
(> 1 GB in total) so that neither L2 nor the 256 MB Infinity Cache can serve the
weights.  Inputs (packed weights, quantized activations) are resident in HBM
before the timed region.  The timed steps are replayed from HIP graphs of up to 40
steps each (as a decode step of a 32- to 40-layer model is one graph).

Prints ONE JSON line: the metric is achieved HBM GB/s on algorithmic bytes
(weights once + q8 activations + fp16 outputs).  `roofline` prices the dominant
GEMV kernel against the 8 TB/s HBM peak, `roofline_gemm` the prefill quant-GEMM at
T = 2048 (BASELINE config 3) against the 2.5 PFLOP/s dense fp16 MFMA peak;
`cpu_baseline` times the reference's CPU path (dequant to fp32 + scalar fp32 dot,
restated in oracle/) on the host cores.  Every weight is a seeded N(0, 0.02) tensor
quantized in HBM (machx_inference_engine_amd.synth), every activation N(0, 1).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
H, FF = 4096, 14336
Q81X = 40


TRAFFIC_FILE = os.path.join(ROOT, "profiles", "pmc_traffic_gemv_q8_0_soa_and_gemm_q4_K.txt")


def counter_traffic(key):
    """HBM bytes per launch (read + written) of one kernel from the tracked counter summary: its line
    `traffic_bytes <key> read=<bytes> written=<bytes>` (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE per dispatch, scaled by a
    plain copy of known size; the file names the commit and the commands).  None when the file or the key is absent."""
    try:
        for line in open(TRAFFIC_FILE):
            f = line.split()
            if len(f) == 4 and f[0] == "traffic_bytes" and f[1] == key:
                return int(f[2].split("=")[1]) + int(f[3].split("=")[1])
    except OSError:
        pass
    return None


def gemv_bytes(fmt_row_bytes, K, N, T):
    """Algorithmic bytes of one GEMV launch: weights once, q8 activations, fp16 outputs."""
    return N * fmt_row_bytes + T * (K // 32) * Q81X + T * N * 2


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-graph", action="store_true", help="launch every step from Python instead of replaying HIP graphs")
    ap.add_argument("--unfused", action="store_true", help="gate and up as two launches instead of the fused gate+up launch")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-detail", action="store_true", help="skip the per-config detail table")
    ap.add_argument("--sets", type=int, default=4, help="distinct weight sets rotated through (331.7 MB each)")
    ap.add_argument("--probe", action="store_true",
                    help="counter probe for `rocprofv3 --pmc`: a few launches of the dominant kernels and of a plain copy of known size, no timing")
    ap.add_argument("--legs", default="all",
                    help="comma-separated detail legs to run (batched, gaps, ffn, c1, lm_head, c3, c4, c5); with a list the headline legs are skipped "
                         "and only the detail table is printed (development aid)")
    ap.add_argument("--shape", default=None, metavar="KIND:T:K:N",
                    help="profiling aid: only launches of one kernel at one shape (KIND in gemm_q4_K, gemv_q8_0_soa, gemv_q6_K, gemv_q4_K), "
                         "so that a rocprofv3 run holds exactly one (kernel, shape) pair; prints its HIP-event average")
    ap.add_argument("--yardstick", action="store_true",
                    help="read-only yardsticks of the device, as text: cold reads of the dominant launches' byte counts by launch shape, "
                         "and the per-CU rate of 16-byte loads by lane -> address pattern (cache-resident)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.stderr.write("bench.py: this build measures one GPU only (the path is data-parallel over output rows / experts, "
                         "so more GPUs would each take a slice of rows or experts); run with --gpus 1\n")
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        sys.stderr.write("bench.py: no GPU visible\n")
        sys.exit(3)
    import machx_inference_engine_amd as mx
    from machx_inference_engine_amd import synth
    ops = mx.ops
    dev = "cuda:0"
    torch.cuda.set_device(0)

    g = torch.Generator(device=dev)
    g.manual_seed(7)
    MFMA_PEAK = 2500.0   # dense fp16 MFMA, TFLOP/s

    def kernel_avg_us(fn, n_launch):
        """Average duration of one call of fn(i): HIP events around 5 replays of a graph of n_launch calls, on the stream
        the kernels are launched on (torch's current stream)."""
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        fn(0)
        torch.cuda.synchronize()
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            for i in range(n_launch):
                fn(i)
        gr.replay()
        torch.cuda.synchronize()
        e0.record()
        for _ in range(5):
            gr.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / (5 * n_launch) * 1e3

    def q6_planes(w, K, N):
        """Q6_K GGUF blocks (device) -> the natural-order planes of repack_q6_K_to_soa (device), through the host repacker."""
        return [torch.from_numpy(p).to(dev) for p in ops.repack_q6_K_to_soa(w.cpu().numpy(), K, N)]

    if args.yardstick:
        cus = torch.cuda.get_device_properties(0).multi_processor_count
        for n_bytes, what in ((124843008 // 1024 * 1024, "the fused Q8_0 gate + up launch"), (62390272 // 1024 * 1024, "one Q8_0 4096 -> 14336 matrix"),
                              (48200192 // 1024 * 1024, "one Q6_K 4096 -> 14336 matrix")):
            n_buf = max(2, (1200 << 20) // n_bytes)
            bufs = [torch.empty(n_bytes, dtype=torch.uint8, device=dev).random_(0, 255) for _ in range(n_buf)]
            print("cold read of %d bytes (%s), %d rotating buffers, %d CUs; cells: us per launch / TB/s" % (n_bytes, what, n_buf, cus))
            print("%-46s" % "variant \\ workgroups per CU" + "".join("%12d" % w for w in (2, 3, 4, 6, 8)))
            rows = [("registers, %2d x 16 B in flight per thread" % u, u, 0) for u in (2, 4, 8, 16)]
            rows += [("registers, %2d x 16 B, nontemporal" % u, u, 1) for u in (4, 8)]
            rows += [("LDS ring, %2d x 1 KB in flight per wave" % d, d, 2) for d in (4, 8, 16)]
            for name, u, mode in rows:
                cells = []
                for w in (2, 3, 4, 6, 8):
                    us = kernel_avg_us(lambda i: ops.probe_read_variant(bufs[i % n_buf], u, mode, cus * w), 2 * n_buf)
                    cells.append("%6.1f/%5.2f" % (us, n_bytes / us / 1e6))
                print("%-46s" % name + "".join(cells))
            cells = []
            for u in (4, 8, 16):   # not persistent: every workgroup reads one contiguous piece of u * 4 KB and leaves
                us = kernel_avg_us(lambda i: ops.probe_read_variant(bufs[i % n_buf], u, 0, n_bytes // (u * 4096)), 2 * n_buf)
                cells.append("%6.1f/%5.2f" % (us, n_bytes / us / 1e6))
            print("%-46s" % "one 16 / 32 / 64 KB piece per workgroup" + "".join(cells))
            print()
            del bufs
        pitch, rows_, iters, wgs = 2048, 4096, 20, 2 * cus
        region = torch.empty(rows_ * pitch + 16, dtype=torch.uint8, device=dev).random_(0, 255)
        print("16-byte-per-lane loads over a cache-resident region (%d rows of %d B), %d workgroups of 4 waves, %d passes" % (rows_, pitch, wgs, iters))
        names = ("one row per lane: 16 contiguous bytes", "2 adjacent lanes: 32 contiguous bytes", "4 adjacent lanes: 64 contiguous bytes",
                 "8 adjacent lanes: one 128-byte line", "128-byte line, pieces 2-byte aligned", "128-byte line, pieces 4-byte aligned",
                 "128-byte line, pieces 8-byte aligned")
        b = wgs * 4 * 64 * pitch * iters
        t = [kernel_avg_us(lambda i: ops.probe_lane_pattern(region, pitch, pat, iters, wgs), 4) for pat in range(len(names))]
        for name, us in zip(names, t):
            print("%-42s %8.1f us  %6.2f TB/s  %5.1f B/us/CU  %4.2f of the whole-line rate" % (name, us, b / us / 1e6, b / cus / us, t[3] / us))
        return

    if args.shape:
        kind, T, K, N = args.shape.split(":")
        T, K, N = int(T), int(K), int(N)
        if kind == "gemm_q4_K":
            wq = synth.normal_weights("q4_K", N, K, seed=900, device=dev)
            a16 = torch.randn((T, K), device=dev, generator=g).half()
            yg = torch.empty((T, N), dtype=torch.float16, device=dev)
            us = kernel_avg_us(lambda i: ops.gemm_q4_K(a16, wq, T, K, N, yg), 8)
            print(json.dumps({"shape": args.shape, "avg_launch_us": round(us, 2), "TFLOPs": round(2.0 * T * N * K / us / 1e6, 1),
                              "frac_mfma": round(2.0 * T * N * K / us / 1e6 / MFMA_PEAK, 4), "launches": 49}))
        else:
            fmt = kind[len("gemv_"):]
            x2 = fmt.endswith("_x2")     # two matrices sharing the activation row in one launch (gate + up), T = 1
            fmt = fmt[:-3] if x2 else fmt
            base = fmt.replace("_soa", "").replace("_planes", "")
            n_w = max(2, int(1.2e9 // (N * synth.row_bytes(base, K))))      # > 1 GB of weights in rotation
            wl = [synth.normal_weights(base, N, K, seed=70 + i, device=dev) for i in range(n_w)]
            if fmt.endswith("_soa"):
                wl = [synth.split_q8_0(w) for w in wl]
            xsq = ops.quantize_q8_1(torch.randn((T, K), device=dev, generator=g).half())
            yt = torch.empty((T, N), dtype=torch.float16, device=dev)
            if fmt == "q6_K_planes":   # the same Q6_K bits as natural-order planes (repack_q6_K_to_soa)
                wl = [q6_planes(w, K, N) for w in wl]
                fn = lambda i: ops.gemv_q6_soa_q8(xsq, wl[i % n_w], K, N, T, yt)
            elif fmt.endswith("_soa"):
                fn = lambda i: ops.gemv_q8_0_soa_q8_batched(xsq, wl[i % n_w][0], wl[i % n_w][1], K, N, T, yt)
            else:
                fn = lambda i: getattr(ops, "gemv_%s_q8_batched" % fmt)(xsq, wl[i % n_w], K, N, T, yt)
            if x2:
                assert T == 1
                yt2 = torch.empty((T, N), dtype=torch.float16, device=dev)
                kind2 = {"q6_K_planes": "q6_soa", "q8_0_soa": "q8_0_soa"}.get(fmt, fmt)
                fn = lambda i: ops.gemv_q8_x2(kind2, xsq, wl[i % n_w], wl[(i + 1) % n_w], K, N, yt, yt2)
            us = kernel_avg_us(fn, 2 * n_w)
            b = gemv_bytes(synth.row_bytes(base, K), K, N, T) * (2 if x2 else 1)
            print(json.dumps({"shape": args.shape, "avg_launch_us": round(us, 2), "GBps": round(b / us / 1e3, 1),
                              "frac_hbm": round(b / us / 1e3 / HBM_PEAK_GBS, 4), "launches": 12 * n_w + 1}))
        return

    legs = None if args.legs == "all" else set(args.legs.split(","))
    if legs is not None:
        args.no_cpu, args.sets, args.steps, args.warmup = True, 1, 8, 2
    want = lambda name: legs is None or name in legs

    # ---------------------------------------------------------------- inputs, resident in HBM
    fmts = ("q6_K", "q8_0")
    shapes = {"gate": (H, FF), "up": (H, FF), "down": (FF, H)}   # (K, N)
    sets = []
    for s in range(args.sets):
        ws = {}
        for fi, fmt in enumerate(fmts):
            for ni, (name, (K, N)) in enumerate(shapes.items()):
                ws[(fmt, name)] = synth.normal_weights(fmt, N, K, seed=1000 * s + 10 * fi + ni, device=dev)
        sets.append(ws)
    x = torch.randn((1, H), device=dev, generator=g).half()
    h = torch.randn((1, FF), device=dev, generator=g).half()
    xq, hq = ops.quantize_q8_1(x), ops.quantize_q8_1(h)
    y_ff = {(f, n): torch.empty(FF, dtype=torch.float16, device=dev) for f in fmts for n in ("gate", "up")}
    y_h = {f: torch.empty(H, dtype=torch.float16, device=dev) for f in fmts}
    # Q8_0 runs through the reference's own entry point for this format, gemv_q8_0_soa_q8: the
    # load-time split of block_q8_0 into an int8 plane and an fp16 scale plane (same bytes).
    for ws in sets:
        for n in shapes:
            ws[("q8_0_soa", n)] = synth.split_q8_0(ws[("q8_0", n)])

    def gemv(fmt, xq_, ws, name, K, N, y):
        if fmt == "q6_K":
            ops.gemv_q6_K_q8(xq_, ws[(fmt, name)], K, N, y)
        else:
            qs, d = ws[("q8_0_soa", name)]
            ops.gemv_q8_0_soa_q8(xq_, qs, d, K, N, y)

    def gate_up(fmt, ws):
        # gate and up share the activation row: one fused launch (as the reference fuses them for MXFP4 and Q4_K)
        if fmt == "q6_K":
            ops.gemv_q8_x2("q6_K", xq, ws[(fmt, "gate")], ws[(fmt, "up")], H, FF, y_ff[(fmt, "gate")], y_ff[(fmt, "up")])
        else:
            ops.gemv_q8_x2("q8_0_soa", xq, ws[("q8_0_soa", "gate")], ws[("q8_0_soa", "up")], H, FF, y_ff[(fmt, "gate")], y_ff[(fmt, "up")])

    def step(ws):
        for fmt in fmts:
            if args.unfused:
                gemv(fmt, xq, ws, "gate", H, FF, y_ff[(fmt, "gate")])
                gemv(fmt, xq, ws, "up", H, FF, y_ff[(fmt, "up")])
            else:
                gate_up(fmt, ws)
            gemv(fmt, hq, ws, "down", FF, H, y_h[fmt])

    bytes_per_step = sum(gemv_bytes(synth.row_bytes(f, K), K, N, 1) for f in fmts for (K, N) in shapes.values())
    if not args.unfused:
        bytes_per_step -= len(fmts) * (H // 32) * 40   # the fused launch reads the activation row once

    if args.probe:
        # plain copy of known size first (the scale for FETCH_SIZE / WRITE_SIZE), then the kernels under study
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        for i in range(8):
            step(sets[i % len(sets)])
        wq = synth.normal_weights("q4_K", FF, H, seed=900, device=dev)
        a16 = torch.randn((2048, H), device=dev, generator=g).half()
        for _ in range(4):
            ops.gemm_q4_K(a16, wq, 2048, H, FF)
        torch.cuda.synchronize()
        print(json.dumps({"probe": "copy 268435456 B x4; 8 decode steps; gemm_q4_K T=2048 K=4096 N=14336 x4"}))
        return

    # ---------------------------------------------------------------- warm-up, graphs
    for i in range(args.warmup):
        step(sets[i % len(sets)])
    torch.cuda.synchronize()
    graphs = None
    round_graph, rounds_per_graph = None, 0   # one graph holding several rounds of one step per weight set
    if not args.no_graph:
        graphs = []
        for ws in sets:
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr):
                step(ws)
            graphs.append(gr)
        for gr in graphs:
            gr.replay()
        # A decode step of a 32- to 40-layer model is one graph of that many FFN blocks; here: up to ten rounds over the
        # weight sets (40 steps with the default four sets) per graph, the largest count that divides the timed steps.
        # Kernels inside a graph follow each other without a gap; every graph launch costs about 3 us.
        rounds_per_graph = 0
        if args.steps % len(sets) == 0:
            rounds_per_graph = max(r for r in range(1, 11) if (args.steps // len(sets)) % r == 0)
        if rounds_per_graph > 0:
            round_graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(round_graph):
                for _ in range(rounds_per_graph):
                    for ws in sets:
                        step(ws)
            round_graph.replay()
        torch.cuda.synchronize()

    # ---------------------------------------------------------------- timed region: exactly K steps
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    if round_graph is not None:
        for i in range(args.steps // (len(sets) * rounds_per_graph)):
            round_graph.replay()
    else:
        for i in range(args.steps):
            if graphs:
                graphs[i % len(graphs)].replay()
            else:
                step(sets[i % len(sets)])
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    value = bytes_per_step * args.steps / elapsed / 1e9

    # ---------------------------------------------------------------- roofline of the dominant kernel (HIP events)
    # Dominant by time and bytes: the Q8_0 gate/up GEMV (K=4096, N=14336), 62,390,272 weight bytes per launch.
    if args.unfused:
        mats = [ws[("q8_0_soa", n)] for ws in sets for n in ("gate", "up")]
        dom_us = kernel_avg_us(lambda i: ops.gemv_q8_0_soa_q8(xq, mats[i % len(mats)][0], mats[i % len(mats)][1], H, FF, y_ff[("q8_0", "gate")]),
                               4 * len(mats))
        dom_bytes = gemv_bytes(synth.row_bytes("q8_0", H), H, FF, 1)
        dom_name, dom_traffic = "gemv_q8_kernel<FmtQ8SoaW,T=1> K=4096 N=14336", counter_traffic("gemv_q8_0_soa_T1_K4096_N14336")
    else:
        # the fused gate + up launch: two 4096 -> 14336 matrices, one activation row, two output rows
        dom_us = kernel_avg_us(lambda i: gate_up("q8_0", sets[i % len(sets)]), 4 * len(sets))
        dom_bytes = 2 * gemv_bytes(synth.row_bytes("q8_0", H), H, FF, 1) - (H // 32) * 40
        dom_name, dom_traffic = "gemv_q8_kernel<FmtQ8SoaW,T=1> gate+up fused, K=4096 N=2x14336", counter_traffic("gemv_q8_0_soa_gate_up_fused_T1")
    # yardstick: a pure read of the same number of bytes with the same launch geometry (rotating buffers, no arithmetic)
    n_read = (dom_bytes + 15) // 16 * 16
    rd = [torch.empty(n_read, dtype=torch.uint8, device=dev).random_(0, 255) for _ in range(8)]
    read_us = kernel_avg_us(lambda i: ops.probe_stream_read(rd[i % len(rd)]), 4 * len(rd))
    del rd
    achieved = dom_bytes / (dom_us * 1e-6) / 1e9
    roofline = {"bound": "hbm", "kernel": dom_name, "achieved": round(achieved, 1),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                # read from profiles/pmc_traffic_*.txt (counter run of `bench.py --probe`), not measured in this run
                "traffic": dom_traffic,
                "bytes_per_launch": dom_bytes, "avg_launch_us": round(dom_us, 3),
                # not part of the fraction above: what a read-only kernel reaches on the same bytes on this device
                "stream_read_same_bytes": {"avg_launch_us": round(read_us, 3), "GBps": round(n_read / read_us / 1e3, 1)}}

    # ---------------------------------------------------------------- the GEMM half of the metric: quant-GEMM at T = 2048
    # BASELINE config 3, Q4_K 14336 x 4096 (N(0, 0.02) weights encoded in HBM) x fp16 activations N(0, 1) [2048 x 4096]
    Tg, Kg, Ng = 2048, H, FF
    wq = synth.normal_weights("q4_K", Ng, Kg, seed=900, device=dev)
    a16 = torch.randn((Tg, Kg), device=dev, generator=g).half()
    yg = torch.empty((Tg, Ng), dtype=torch.float16, device=dev)
    gemm_us = kernel_avg_us(lambda i: ops.gemm_q4_K(a16, wq, Tg, Kg, Ng, yg), 8)
    gemm_flop = 2.0 * Tg * Ng * Kg
    gemm_tf = gemm_flop / gemm_us / 1e6
    roofline_gemm = {"bound": "mfma", "kernel": "gemm_kernel<GemmQ4K, dense, 128-token tiles> T=2048 K=4096 N=14336 (v_mfma_f32_32x32x16_f16)",
                     "achieved": round(gemm_tf, 1), "peak": MFMA_PEAK, "unit": "TFLOP/s", "frac": round(gemm_tf / MFMA_PEAK, 4),
                     "flop_per_launch": gemm_flop, "avg_launch_us": round(gemm_us, 2),
                     # read from profiles/pmc_traffic_*.txt; algorithmic bytes: W 33,030,144 + A 16,777,216 + Y 58,720,256
                     "traffic": counter_traffic("gemm_q4_K_T2048_K4096_N14336"), "algorithmic_bytes": Ng * synth.row_bytes("q4_K", Kg) + Tg * Kg * 2 + Tg * Ng * 2}
    del wq, a16, yg

    out = {"metric": "quant GEMV HBM GB/s (decode, Llama-3-8B FFN shapes, Q6_K + Q8_0, batch 1)", "value": round(value, 1),
           "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8 dot, fp32 fold", "data": "synthetic",
           "config": {"workload": "configs[1]: decode GEMV gate/up 4096->14336 + down 14336->4096, Q6_K and Q8_0, T=1, "
                                  "%s, %d rotating weight sets" % ("6 launches/step" if args.unfused else "gate+up fused: 4 launches/step", len(sets)),
                      "bytes_per_step": bytes_per_step, "hip_graph": bool(graphs),
                      "steps_per_graph": (len(sets) * rounds_per_graph) if round_graph is not None else (1 if graphs else 0),
                      "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4)},
           "roofline": roofline, "roofline_gemm": roofline_gemm}

    # ---------------------------------------------------------------- detail: the other batch sizes and formats
    if not args.no_detail:
        import numpy as np
        rng = np.random.default_rng(4)
        detail = {}
        if want('batched'):
            def soa_batched(xsq_, w, K, N, T, yt_):
                return ops.gemv_q8_0_soa_q8_batched(xsq_, w[0], w[1], K, N, T, yt_)

            for fmt, fn in (("q6_K", ops.gemv_q6_K_q8_batched), ("q8_0_soa", soa_batched), ("q8_0", ops.gemv_q8_0_q8_batched),
                            ("q4_K", ops.gemv_q4_K_q8_batched)):
                for name, (K, N) in (("gate_up", (H, FF)), ("down", (FF, H))):
                    if fmt == "q4_K":
                        ws_l = [synth.normal_weights(fmt, N, K, seed=77 + i, device=dev) for i in range(12)]
                    else:
                        # every matrix of every set, whatever its shape: the buffers are whole blocks and the same size for
                        # (K, N) and (N, K), and a dozen of them (0.6-0.75 GB) cannot stay in the 256 MB Infinity Cache
                        ws_l = [ws[(fmt, n)] for ws in sets for n in ("gate", "up", "down")]
                    for T in (1, 2, 4, 8):
                        xs = torch.randn((T, K), device=dev, generator=g).half()
                        xsq = ops.quantize_q8_1(xs)
                        yt = torch.empty((T, N), dtype=torch.float16, device=dev)
                        us = kernel_avg_us(lambda i: fn(xsq, ws_l[i % len(ws_l)], K, N, T, yt), 3 * len(ws_l))
                        b = gemv_bytes(synth.row_bytes(fmt.replace("_soa", ""), K), K, N, T)
                        detail["%s_%s_T%d" % (fmt, name, T)] = {"us": round(us, 2), "GBps": round(b / us / 1e3, 1),
                                                                "frac_hbm": round(b / us / 1e3 / HBM_PEAK_GBS, 4)}
                        if T == 1 and name == "gate_up":
                            # the same launch on one matrix over and over: served from the 256 MB Infinity Cache, not from HBM
                            us_c = kernel_avg_us(lambda i: fn(xsq, ws_l[0], K, N, T, yt), 24)
                            detail["%s_%s_T1_cache_resident" % (fmt, name)] = {"us": round(us_c, 2), "GBps": round(b / us_c / 1e3, 1)}
                    del ws_l
            # Q6_K as natural-order planes (repack_q6_K_to_soa, the reference's gemv_q6_soa_q8 layout), one token
            for name, (K, N) in (("gate_up", (H, FF)), ("down", (FF, H))):
                pl = [q6_planes(synth.normal_weights("q6_K", N, K, seed=177 + i, device=dev), K, N) for i in range(6)]   # 289 MB in rotation
                xsq = ops.quantize_q8_1(torch.randn((1, K), device=dev, generator=g).half())
                yt = torch.empty((1, N), dtype=torch.float16, device=dev)
                us = kernel_avg_us(lambda i: ops.gemv_q6_soa_q8(xsq, pl[i % len(pl)], K, N, 1, yt), 6 * len(pl))
                b = gemv_bytes(synth.row_bytes("q6_K", K), K, N, 1)
                detail["q6_K_planes_%s_T1" % name] = {"us": round(us, 2), "GBps": round(b / us / 1e3, 1), "frac_hbm": round(b / us / 1e3 / HBM_PEAK_GBS, 4)}
                del pl
        if want('gaps') and graphs:
            # What the dependencies between the four launches of a step cost: the same step recorded with the Q6_K chain and
            # the Q8_0 chain as two independent branches of the graph (gate + up -> down inside each), so that the tail of one
            # launch overlaps the ramp of another.  Not the headline (a decode step of one model is one chain).
            s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
            def step_branches(ws):
                cur = torch.cuda.current_stream()
                for st_, fmt in ((s1, "q6_K"), (s2, "q8_0")):
                    st_.wait_stream(cur)
                    with torch.cuda.stream(st_):
                        gate_up(fmt, ws)
                        gemv(fmt, hq, ws, "down", FF, H, y_h[fmt])
                cur.wait_stream(s1)
                cur.wait_stream(s2)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            gb = []
            for ws in sets:
                gr = torch.cuda.CUDAGraph()
                with torch.cuda.graph(gr):
                    step_branches(ws)
                gb.append(gr)
            res = {}
            for name, gl in (("one_chain", graphs), ("two_independent_chains", gb)):
                for gr in gl:
                    gr.replay()
                torch.cuda.synchronize()
                e0.record()
                for i in range(40):
                    gl[i % len(gl)].replay()
                e1.record()
                torch.cuda.synchronize()
                res[name + "_us"] = round(e0.elapsed_time(e1) / 40 * 1e3, 2)
            detail["step_launch_dependencies"] = res
        if want('ffn'):
            # one decode FFN (fp16 x in, fp16 y out) as the reference's launch chain and as the two fused launches
            xf = torch.randn(H, device=dev, generator=g).half()
            xq_b = torch.empty(H // 32 * 40, dtype=torch.uint8, device=dev)
            hq_b = torch.empty(FF // 32 * 40, dtype=torch.uint8, device=dev)
            g_b, u_b, h_b = (torch.empty(FF, dtype=torch.float16, device=dev) for _ in range(3))
            y_b = torch.empty(H, dtype=torch.float16, device=dev)
            for fmt, key in (("q8_0_soa", "q8_0_soa"), ("q6_K", "q6_K")):
                def chain(i):
                    ws = sets[i % len(sets)]
                    ops.quantize_q8_1(xf, xq_b)
                    ops.gemv_q8_x2(fmt, xq_b, ws[(key, "gate")], ws[(key, "up")], H, FF, g_b, u_b)
                    ops.swiglu_q8(g_b, u_b, out=(h_b, hq_b))
                    gemv(key.replace("_soa", ""), hq_b, ws, "down", FF, H, y_b)

                def fused(i):
                    ws = sets[i % len(sets)]
                    ops.gemv_x2_silu(fmt, xf, ws[(key, "gate")], ws[(key, "up")], H, FF, h_b)
                    ops.gemv_f16q8(fmt, h_b, ws[(key, "down")], FF, H, y_b)

                us_c, us_f = kernel_avg_us(chain, 2 * len(sets)), kernel_avg_us(fused, 2 * len(sets))
                detail["ffn_decode_%s_T1" % fmt] = {"chain_4_launches_us": round(us_c, 2), "fused_2_launches_us": round(us_f, 2)}
        if want('c1'):
            # BASELINE config 1: Q4_K 4096x4096, fp32 activations, fp32 out (9.4 MB: cache resident unless rotated)
            w1 = [synth.normal_weights("q4_K", 4096, 4096, seed=500 + i, device=dev) for i in range(40)]
            a32 = torch.randn(4096, device=dev, generator=g)
            y32 = torch.empty(4096, dtype=torch.float32, device=dev)
            us = kernel_avg_us(lambda i: ops.gemv_q4_K(a32, w1[i % len(w1)], 4096, 4096, y32), 2 * len(w1))
            b = 4096 * synth.row_bytes("q4_K", 4096) + 2 * 4096 * 4
            detail["config1_q4_K_4096x4096_f32"] = {"us": round(us, 2), "GBps": round(b / us / 1e3, 1), "frac_hbm": round(b / us / 1e3 / HBM_PEAK_GBS, 4)}
            aq = ops.quantize_q8_1(a32)
            y16 = torch.empty(4096, dtype=torch.float16, device=dev)
            us = kernel_avg_us(lambda i: ops.gemv_q4_K_q8(aq, w1[i % len(w1)], 4096, 4096, y16), 2 * len(w1))
            detail["config1_q4_K_4096x4096_q8"] = {"us": round(us, 2), "GBps": round(b / us / 1e3, 1), "frac_hbm": round(b / us / 1e3 / HBM_PEAK_GBS, 4)}
            del w1
        if want('lm_head'):
            # lm_head-sized decode GEMV (the largest single GEMV of a decode step): Q6_K, 4096 -> 151936, 510 MB
            NV = 151936
            wl = [synth.normal_weights("q6_K", NV, H, seed=700 + i, device=dev) for i in range(2)]
            yv = torch.empty(NV, dtype=torch.float16, device=dev)
            us = kernel_avg_us(lambda i: ops.gemv_q6_K_q8(xq, wl[i % 2], H, NV, yv), 4)
            b = gemv_bytes(synth.row_bytes("q6_K", H), H, NV, 1)
            detail["lm_head_q6_K_K4096_N151936_T1"] = {"us": round(us, 1), "GBps": round(b / us / 1e3, 1), "frac_hbm": round(b / us / 1e3 / HBM_PEAK_GBS, 4)}
            del wl, yv
        if want('c3'):
            # BASELINE config 3: prefill quant-GEMM, Q4_K, fp16 MFMA (peak 2.5 PFLOP/s dense fp16)
            for (K, N) in ((H, FF), (FF, H)):
                wq = synth.normal_weights("q4_K", N, K, seed=900, device=dev)
                for T in (512, 2048, 4096):
                    a16 = torch.randn((T, K), device=dev, generator=g).half()
                    yg = torch.empty((T, N), dtype=torch.float16, device=dev)
                    us = kernel_avg_us(lambda i: ops.gemm_q4_K(a16, wq, T, K, N, yg), 4)
                    tf = 2.0 * T * N * K / us / 1e6
                    ent = {"us": round(us, 1), "TFLOPs": round(tf, 1), "frac_mfma": round(tf / MFMA_PEAK, 4)}
                    if T >= 2048:
                        # the same product the reference's way on this box: dequantize W to an fp16 [K, N] matrix, then the
                        # vendor library's fp16 GEMM (rocBLAS here, oneDNN there); and that GEMM alone
                        bt = ops.dequant_to_Bt("q4_K", wq, K, N)
                        us_g = kernel_avg_us(lambda i: ops.gemm_fp16(a16, bt, T, N, K, torch.float16, yg), 4)
                        us_2 = kernel_avg_us(lambda i: (ops.dequant_to_Bt("q4_K", wq, K, N, bt), ops.gemm_fp16(a16, bt, T, N, K, torch.float16, yg)), 4)
                        ent["vendor_fp16_gemm_us"] = round(us_g, 1)
                        ent["vendor_fp16_gemm_TFLOPs"] = round(2.0 * T * N * K / us_g / 1e6, 1)
                        ent["dequant_plus_vendor_gemm_us"] = round(us_2, 1)
                        if T == 2048:   # the library's own tiled fp16 kernel (mx_gemm_fp16, fp32 out) on the same operands
                            y32 = torch.empty((T, N), dtype=torch.float32, device=dev)
                            us_t = kernel_avg_us(lambda i: ops.gemm_fp16(a16, bt, T, N, K, torch.float32, y32), 4)
                            ent["tiled_fp16_gemm_f32out_us"] = round(us_t, 1)
                            ent["tiled_fp16_gemm_TFLOPs"] = round(2.0 * T * N * K / us_t / 1e6, 1)
                            del y32
                        del bt
                    if T == 2048:
                        # the int-dot route over q8 rows (int8 matrix cores, fp32 fold per 32-element block): rows quantized once, outside the timing
                        aq8 = ops.quantize_q8_1s(a16)
                        us_q = kernel_avg_us(lambda i: ops.gemm_q8_rows("q4_K", aq8, (wq,), T, K, N, yg), 4)
                        ent["q8_rows_int8_mfma_us"] = round(us_q, 1)
                        ent["q8_rows_frac_int8_mfma"] = round(2.0 * T * N * K / us_q / 1e6 / 5000.0, 4)
                        del aq8
                    detail["config3_gemm_q4_K_T%d_K%d_N%d" % (T, K, N)] = ent
                    del a16, yg
                del wq
        if want('c4'):
            # BASELINE config 4: MXFP4 MoE decode at gpt-oss-20b shape (E=32, top-4, H=EF=2880), T=1 and T=32
            E4, K4, H4 = 32, 4, 2880
            nrep = 6   # rotate expert banks so a decode step cannot live in the Infinity Cache
            banks = []
            for i in range(nrep):
                gq, ge = synth.split_mxfp4(synth.normal_weights("mxfp4", E4 * H4, H4, seed=3000 + i, device=dev))
                uq, ue = synth.split_mxfp4(synth.normal_weights("mxfp4", E4 * H4, H4, seed=3100 + i, device=dev))
                dq, de = synth.split_mxfp4(synth.normal_weights("mxfp4", E4 * H4, H4, seed=3200 + i, device=dev))
                banks.append((gq, ge, uq, ue, dq, de))
            qs_st, e_st = H4 * H4 // 2, H4 * H4 // 32
            per_expert = 3 * (qs_st + e_st)
            for T in (1, 32):
                logits = rng.standard_normal((T, E4)).astype(np.float32)
                ids = np.sort(np.argsort(-logits, axis=1)[:, :K4], axis=1).astype(np.int32)
                wts = np.full((T, K4), 0.25, np.float32)
                off, si, wp, t2p = ops.build_moe_packing(ids, wts, E4)
                n_distinct = int((np.diff(off.astype(np.int64)) > 0).sum())
                xt = torch.randn((T, H4), device=dev, generator=g).half()
                TK = T * K4
                offd, sid = torch.from_numpy(off).to(dev), torch.from_numpy(si).to(dev)
                idsd = torch.from_numpy(ids.ravel().copy()).to(dev)
                hbuf = torch.empty((TK, H4), dtype=torch.float16, device=dev)
                obuf = torch.empty((TK, H4), dtype=torch.float16, device=dev)
                xq8 = ops.quantize_q8_1(xt)
                xpq = ops.quantize_q8_1(ops.moe_gather_rows(xt, sid, TK, H4))
                hq8 = ops.quantize_q8_1(hbuf)

                def layer(i):
                    b = banks[i % nrep]
                    if T == 1:    # device-side expert ids, one launch per stage
                        ops.moe_gate_up_oai_mxfp4(xq8, b[0], b[1], b[2], b[3], qs_st, e_st, None, None, idsd, T, K4, H4, H4, E4, h_out=hbuf)
                        if args.unfused:
                            ops.quantize_q8_1(hbuf, hq8)
                            ops.moe_down_mxfp4(hq8, b[4], b[5], qs_st, e_st, None, idsd, T, K4, H4, H4, E4, out_packed=obuf)
                        else:     # h quantized while the down launch stages it: same bits, one launch fewer
                            ops.moe_down_mxfp4_f16(hbuf, b[4], b[5], qs_st, e_st, None, idsd, T, K4, H4, H4, E4, out_packed=obuf)
                    else:         # expert-grouped rows, each routed expert streamed once
                        ops.moe_grouped_gate_up_oai_mxfp4(xpq, b[0], b[1], b[2], b[3], qs_st, e_st, None, None, offd, TK, E4, H4, H4, h_packed=hbuf)
                        # with 128 rows every workgroup would requantize all of them: the separate quantize launch is cheaper here
                        ops.quantize_q8_1(hbuf, hq8)
                        ops.moe_grouped_down_mxfp4(hq8, b[4], b[5], qs_st, e_st, None, offd, TK, E4, H4, H4, out_packed=obuf)

                us = kernel_avg_us(layer, 2 * nrep)
                bts = n_distinct * per_expert
                detail["config4_moe_mxfp4_T%d" % T] = {"us": round(us, 1), "distinct_experts": n_distinct, "GBps": round(bts / us / 1e3, 1),
                                                       "frac_hbm": round(bts / us / 1e3 / HBM_PEAK_GBS, 4)}
            del banks
        if want('c5'):
            # BASELINE config 5: Qwen3-MoE style grouped GEMM, E=128 top-8 H=2048 EF=768, 2048 tokens, Zipf(1.1), Q8_0 experts
            E5, K5, H5, EF5, T5 = 128, 8, 2048, 768, 2048
            gq5, gd5 = synth.split_q8_0(synth.normal_weights("q8_0", E5 * EF5, H5, seed=5000, device=dev))
            uq5, ud5 = synth.split_q8_0(synth.normal_weights("q8_0", E5 * EF5, H5, seed=5001, device=dev))
            dq5, dd5 = synth.split_q8_0(synth.normal_weights("q8_0", E5 * H5, EF5, seed=5002, device=dev))
            pz = np.arange(1, E5 + 1, dtype=np.float64) ** -1.1
            pz = pz[rng.permutation(E5)]
            pz /= pz.sum()
            ids5 = np.stack([np.sort(rng.choice(E5, size=K5, replace=False, p=pz)) for _ in range(T5)]).astype(np.int32)
            w5 = np.full(ids5.shape, 1.0 / K5, np.float32)
            off5, si5, wp5, t2p5 = ops.build_moe_packing(ids5, w5, E5)
            TK5 = T5 * K5
            x5 = torch.randn((T5, H5), device=dev, generator=g).half()
            off5d, wp5d = torch.from_numpy(off5).to(dev), torch.from_numpy(wp5).to(dev).half()
            xp5 = ops.moe_gather_rows(x5[:, :].contiguous(), torch.from_numpy(si5).to(dev), TK5, H5) if TK5 <= 65535 else None
            h5 = torch.empty((TK5, EF5), dtype=torch.float16, device=dev)
            o5 = torch.empty((TK5, H5), dtype=torch.float16, device=dev)

            def layer5(i):
                ops.moe_gemm_gate_up_silu_q8(xp5, gq5, gd5, uq5, ud5, EF5 * H5, EF5 * H5 // 32, off5d, TK5, E5, H5, EF5, h5)
                ops.moe_gemm_down_q8(h5, dq5, dd5, H5 * EF5, H5 * EF5 // 32, off5d, wp5d, TK5, E5, H5, EF5, o5)

            us = kernel_avg_us(layer5, 3)
            tf = 2.0 * TK5 * H5 * EF5 * 3 / us / 1e6
            detail["config5_moe_grouped_gemm_q8_0"] = {"us": round(us, 1), "TFLOPs": round(tf, 1), "frac_mfma": round(tf / MFMA_PEAK, 4),
                                                       "route": "fp16 rows, fp16 MFMA (mx_moe_gemm_*)"}
            # the same layer from the unsorted token rows: gather launch + the two GEMMs, against the gather folded into the row loads
            si5d = torch.from_numpy(si5).to(dev)

            def layer5_gather(i):
                ops.moe_gather_rows(x5, si5d, TK5, H5, xp5)
                layer5(i)

            def layer5_fused(i):
                ops.moe_gemm_gate_up_silu_q8(x5, gq5, gd5, uq5, ud5, EF5 * H5, EF5 * H5 // 32, off5d, TK5, E5, H5, EF5, h5, sorted_idx=si5d)
                ops.moe_gemm_down_q8(h5, dq5, dd5, H5 * EF5, H5 * EF5 // 32, off5d, wp5d, TK5, E5, H5, EF5, o5)

            detail["config5_from_unsorted_rows"] = {"gather_launch_plus_gemms_us": round(kernel_avg_us(layer5_gather, 3), 1),
                                                    "gather_in_the_row_loads_us": round(kernel_avg_us(layer5_fused, 3), 1)}
            # the same layer through the reference's own signatures: q8 rows (quantize_q8_1) -> moe_prefill_gate_up_silu_q8 ->
            # quantize_q8_1 -> moe_prefill_down_q8, int8 MFMA with the per-block fp32 fold (peak 5 POP/s dense int8)
            xq5 = torch.empty(TK5 * (H5 // 32) * 40, dtype=torch.uint8, device=dev)
            hq5 = torch.empty(TK5 * (EF5 // 32) * 40, dtype=torch.uint8, device=dev)

            def layer5_q8(i):
                ops.quantize_q8_1(xp5, xq5)
                ops.moe_prefill_gate_up_silu_q8(xq5, gq5, gd5, uq5, ud5, EF5 * H5, EF5 * H5 // 32, off5d, TK5, E5, H5, EF5, h5)
                ops.quantize_q8_1(h5, hq5)
                ops.moe_prefill_down_q8(hq5, dq5, dd5, H5 * EF5, H5 * EF5 // 32, off5d, wp5d, TK5, E5, H5, EF5, o5)

            us8 = kernel_avg_us(layer5_q8, 3)
            to8 = 2.0 * TK5 * H5 * EF5 * 3 / us8 / 1e6
            detail["config5_moe_grouped_q8_rows"] = {"us": round(us8, 1), "TOPs": round(to8, 1), "frac_int8_mfma": round(to8 / 5000.0, 4),
                                                     "route": "q8 rows through the reference's signatures, int8 MFMA + fp32 fold (incl. the two quantize launches)"}
        out["detail"] = detail

    # ---------------------------------------------------------------- CPU baseline (reported only)
    if not args.no_cpu:
        import numpy as np
        import oracle as O   # the checker, used here only as the timed CPU baseline
        # Sample: the down projection of both formats plus gate (one step's shapes), T=1, one thread,
        # exactly the reference's loop: dequant row to fp32, sequential fp32 dot.
        xh = x.float().cpu().numpy()
        hh = h.float().cpu().numpy()
        work = [("q6_K", O.Q6_K, sets[0][("q6_K", "gate")], xh, H, FF), ("q6_K", O.Q6_K, sets[0][("q6_K", "down")], hh, FF, H),
                ("q8_0", O.Q8_0, sets[0][("q8_0", "gate")], xh, H, FF), ("q8_0", O.Q8_0, sets[0][("q8_0", "down")], hh, FF, H)]
        host = [(f, w.cpu().numpy(), a, K, N) for (_, f, w, a, K, N) in work]
        os.environ["OMP_NUM_THREADS"] = "1"
        tot_b, t_cpu, reps = 0, 0.0, 0
        try:
            import ctypes
            omp = ctypes.CDLL("libgomp.so.1")
            omp.omp_set_num_threads(1)
        except OSError:
            omp = None
        # Where oracle/_ref (the reference's own host code, built where the reference tree was mounted) is present,
        # the timed loop runs the reference's ie::ref::dequant_*_buffer itself; otherwise the oracle's restatement.
        ref = O.load_ref()
        ybuf = np.empty(max(H, FF), np.float32)

        def cpu_gemv(f, w, a, K, N):
            if ref is not None:
                a32 = np.ascontiguousarray(a, np.float32).ravel()
                assert ref.ref_gemv_cpu(f, w.ctypes.data, a32.ctypes.data, ybuf.ctypes.data, K, N) == 0
            else:
                O.gemv_f32chain(f, w, a, K, N)

        while t_cpu < 10.0 and reps < 50:
            for f, w, a, K, N in host:
                c0 = time.perf_counter()
                cpu_gemv(f, w, a, K, N)
                t_cpu += time.perf_counter() - c0
                tot_b += w.nbytes
            reps += 1
        out["cpu_baseline"] = {"value": round(tot_b / t_cpu / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "reference" if ref is not None else "port",
                               "sample": "gate (4096->14336) and down (14336->4096) GEMV in Q6_K and Q8_0, T=1, %d repetitions, "
                                         "weight bytes / time; dequant-to-fp32 (%s) + sequential fp32 dot as in the reference's "
                                         "tests/unit/gemv_q4k_test.cpp" % (reps, "the reference's ie::ref::dequant_*_buffer, oracle/_ref"
                                                                           if ref is not None else "oracle restatement")}
        if omp is not None:
            n_thr = min(16, os.cpu_count() or 1)
            omp.omp_set_num_threads(n_thr)
            c0 = time.perf_counter()
            nb = 0
            for _ in range(3):
                for f, w, a, K, N in host:
                    O.gemv_f32chain(f, w, a, K, N)
                    nb += w.nbytes
            out["cpu_baseline_mt"] = {"value": round(nb / (time.perf_counter() - c0) / 1e9, 3), "unit": "GB/s", "cores": n_thr,
                                      "kind": "port", "sample": "same work, rows split over OpenMP threads"}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
