#!/usr/bin/env python3
"""Benchmark driver.

Headline metric (BASELINE.json): w1a2 GEMM effective TOPS at M=64, N=K=1024, weights {-1,+1} stored
as one bit (w = 2b-1), activations unsigned 2-bit, bit-packed along K, int32 output.  One "step" is
one launch of that GEMM through the C ABI with all operands resident in HBM.  The timed loop runs in
C++ (libapnn_bench.so), like the timing section of the reference's benchmark main
(APNN-TC-lib/bmmaTensorCoreGemm/src/71_bmmaTensorCoreGemm.cu:526-549).  The launches of the
latency-bound shapes (headline, M=64 sweep, batch-1 convolutions) are replayed from HIP graphs of
GRAPH_BATCH launches each: a plain host loop of thousands of ~3 us launches is throttled by the host
side of the queue (3.0-4.4 us per launch depending on the loop length), graph replay issues the same
kernels at the device's own rate.  The plain-loop figure is reported beside it.

--steps K / --warmup W: the headline's timed region is ceil(2000 / K) repetitions of K launches (at
least 2000 launches, so that one graph launch and one synchronisation do not dominate a short run),
after max(W, 200) untimed launches; it is measured three times and the median block is reported.
`value`, `ms_per_step` and `roofline` all come from the same clock: HIP events on the launch stream.

Prints ONE JSON line.  Besides the contract fields it carries
  roofline     : the GEMM kernel against the HBM roofline (algorithmic bytes / HIP-event time per launch)
  cpu_baseline : the scalar CPU oracle timed on the host cores on the same inputs
  extra        : the reference-compatible unsigned result, the launch floor, and the other shapes of
                 the sweep with their own roofline fractions.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
INT8_MFMA_PEAK_TOPS = 5000.0   # MI355X dense int8 MFMA
FP4_MFMA_PEAK_TOPS = 10100.0   # MI355X dense fp4 MFMA (the matrix-core path feeds 2-bit digits as e2m1 codes)
# HBM bytes per launch of the headline kernel from the hardware counters (FETCH_SIZE 184.50 KiB x 2.0
# calibration, WRITE_SIZE 256 KiB x 1.0): see profiles/gemm_w1a2_m64_n1024_k1024.md
HEADLINE_TRAFFIC_BYTES = 640000
BASELINE_TOPS = 18.66          # reference README.md:142 (w1a2, M=64, N=K=1024, sm_86)
GRAPH_BATCH = 200              # kernel launches per captured HIP graph
MIN_TIMED_LAUNCHES = 2000      # the timed region of a latency-bound shape never holds fewer launches
MIN_WARMUP_LAUNCHES = 200      # nor its warm-up fewer than this (clock ramp, first-touch of the code object)
HEADLINE_BLOCKS = 3            # the headline is timed this many times; the median block is reported


def gemm_bytes(M, N, K, wb, xb):
    return (wb * M * K + xb * N * K) // 8 + 4 * M * N


def crossover_table(A, G, O, benchlib, stream):
    """Every kernel path / tile shape pinned in turn on the shapes around which the library's own choice
    (APNN_PATH_AUTO) changes: the M=64 sweep end point, the small-GEMM cross-over to the matrix cores,
    large GEMMs, the 16x16 convolution family and the ResNet18 layer shapes at batch 8 and 64.  Each entry
    lists the time of every candidate that is built, the library's choice (from apnn_*_plan) and how far
    that choice is from the fastest candidate."""
    import numpy as np
    import torch
    KN = {A.KERNEL_VALU_TILE: "valu", A.KERNEL_VALU_DIRECT: "valu-direct", A.KERNEL_MFMA_FP4: "fp4",
          A.KERNEL_MFMA_I8: "i8", A.KERNEL_PATCH_FP4: "patch", A.KERNEL_MFMA_FP4_XS: "xs"}
    rng = np.random.default_rng(0x5EED0004)

    def run(desc, fn_graph, fn_plain, small):
        ev, wall = ctypes.c_float(), ctypes.c_double()
        if small:
            rc = fn_graph(ctypes.byref(desc), 200, 1000, GRAPH_BATCH, ctypes.byref(ev), ctypes.byref(wall))
            n = 1000
        else:
            rc = fn_plain(ctypes.byref(desc), 3, 20, stream, ctypes.byref(ev), ctypes.byref(wall))
            n = 20
        torch.cuda.synchronize()
        return None if rc != 0 else ev.value / n * 1e3

    def sweep(name, desc, plan_fn, fn_graph, fn_plain, small, cands):
        plan = A.Plan()
        desc.path = A.PATH_AUTO
        assert plan_fn(ctypes.byref(desc), ctypes.byref(plan)) == 0
        auto = "%s/%d" % (KN[plan.kernel], plan.tile)
        times = {}
        for pth, tile in cands:
            desc.path = pth | ((tile + 1) << 8)
            p2 = A.Plan()
            if plan_fn(ctypes.byref(desc), ctypes.byref(p2)) != 0:
                continue        # not built for this precision / load width, or does not fit
            t = run(desc, fn_graph, fn_plain, small)
            if t is not None:
                times["%s/%d" % (KN[p2.kernel], p2.tile)] = round(t, 2)
        desc.path = A.PATH_AUTO
        t_auto = run(desc, fn_graph, fn_plain, small)
        best = min(times, key=times.get)
        return {"shape": name, "auto": auto, "auto_us": round(t_auto, 2), "best": best, "best_us": times[best],
                "auto_over_best": round(t_auto / times[best], 3), "candidates_us": times}

    L = A.lib()
    out = []
    gemm_cands = ([(A.PATH_VALU, t) for t in range(5)] + [(A.PATH_MFMA, t) for t in (1, 2, 3, 4, 5, 6, 9)] +
                  [(A.PATH_MFMA_I8, t) for t in (1, 2, 6)] + [(A.PATH_MFMA_XS, t) for t in (1, 2, 3, 6)])
    for (wb, xb, M, N, K) in [(1, 2, 64, 1024, 1024), (1, 4, 64, 1024, 1024), (1, 2, 128, 128, 2048), (1, 2, 256, 256, 1024),
                              (1, 2, 256, 256, 4096), (1, 2, 512, 512, 1024), (1, 2, 1024, 1024, 1024),
                              (1, 2, 2048, 2048, 2048), (1, 4, 2048, 2048, 2048), (1, 2, 4096, 4096, 4096),
                              (1, 4, 4096, 4096, 4096), (1, 2, 8192, 8192, 8192), (2, 2, 8192, 8192, 8192)]:
        W = G.to_dev(O.random_planes(rng, wb, M, K // 32))
        X = G.to_dev(O.random_planes(rng, xb, N, K // 32))
        D = G.dev_empty_i32(M * N)
        d = A.GemmDesc(W=W.data_ptr(), X=X.data_ptr(), D=D.data_ptr(), M=M, N=N, K=K, wb=wb, xb=xb)
        cands = [c for c in gemm_cands if not (c[0] == A.PATH_VALU and M * N > 1024 * 1024 and c[1] != 0)]
        out.append(sweep("gemm w%da%d %dx%dx%d" % (wb, xb, M, N, K), d, L.apnn_gemm_plan, benchlib.apnn_bench_gemm_graph,
                         benchlib.apnn_bench_gemm, M * N <= 512 * 512, cands))
    conv_cands = ([(A.PATH_VALU, t) for t in range(4)] + [(A.PATH_MFMA, t) for t in (1, 2, 3, 4, 5, 7, 8, 9)] +
                  [(A.PATH_MFMA_I8, t) for t in (1, 2, 3, 4, 7)] + [(A.PATH_MFMA_PATCH, t) for t in range(5)] +
                  [(A.PATH_MFMA_XS, t) for t in (1, 2, 3, 7)])
    geoms = [("conv16 b1 C=%d" % c, 1, 16, c, c, 3, 1, 1) for c in (128, 512, 1024)]
    geoms += [("conv16 b16 C=%d" % c, 16, 16, c, c, 3, 1, 1) for c in (128, 256, 512, 1024)]
    for b in (8, 64):
        geoms += [("resnet b%d 56x56 64->64" % b, b, 56, 64, 64, 3, 1, 1), ("resnet b%d 56x56 64->128 /2" % b, b, 56, 64, 128, 3, 2, 1),
                  ("resnet b%d 28x28 128->128" % b, b, 28, 128, 128, 3, 1, 1), ("resnet b%d 28x28 128->256 /2" % b, b, 28, 128, 256, 3, 2, 1),
                  ("resnet b%d 14x14 256->256" % b, b, 14, 256, 256, 3, 1, 1), ("resnet b%d 14x14 256->512 /2" % b, b, 14, 256, 512, 3, 2, 1),
                  ("resnet b%d 7x7 512->512" % b, b, 7, 512, 512, 3, 1, 1), ("resnet b%d 56x56 64->128 1x1 /2" % b, b, 56, 64, 128, 1, 2, 0)]
    for (name, batch, H, cin, cout, R, stride, pad) in geoms:
        X = G.to_dev(O.random_planes(rng, 2, batch * H * H, cin // 32))
        Wt = G.to_dev(O.random_planes(rng, 1, cout * R * R, cin // 32))
        Ho = (H + 2 * pad - R) // stride + 1
        thr = G.to_dev(np.sort(rng.integers(-200, 200, size=(cout, 3)), axis=1).astype(np.int32))
        outp = G.dev_empty_i32(2 * batch * Ho * Ho * cout // 32)
        E = G.epilogue(mode=A.EPI_BN, out_bits=2, thr=thr)
        d = A.ConvDesc(W=Wt.data_ptr(), X=X.data_ptr(), O=outp.data_ptr(), batch=batch, H=H, Wd=H, cin_pad=cin, COUT=cout,
                       R=R, S=R, stride=stride, pad=pad, halo=0, wb=1, xb=2, weight_mode=A.WEIGHT_SYMMETRIC, epi=E)
        rows = batch * Ho * Ho
        cands = [c for c in conv_cands if not (c[0] == A.PATH_VALU and rows * cout > 1024 * 1024 and c[1] != 0)]
        out.append(sweep(name + " w1a2 bn-packed", d, L.apnn_conv_plan, benchlib.apnn_bench_conv_graph,
                         benchlib.apnn_bench_conv, rows * cout <= 512 * 512, cands))
    return out


def crossover_sweep(A, G, O, benchlib):
    """The library's own choice against every FP4 matrix-core tile that is built, over the whole 16x16
    convolution sweep (four precisions x batch 1 / 16 x eight channel counts x int32 / quantized output) and
    ten GEMM sizes per precision: the measurement behind the per-precision tile rules of the dispatcher.
    Every candidate and AUTO are replayed from HIP graphs in the same process; `ratio` = AUTO / fastest tile."""
    import numpy as np
    import torch
    KN = {A.KERNEL_VALU_TILE: "valu", A.KERNEL_VALU_DIRECT: "valu-direct", A.KERNEL_MFMA_FP4: "fp4",
          A.KERNEL_MFMA_I8: "i8", A.KERNEL_PATCH_FP4: "patch", A.KERNEL_MFMA_FP4_XS: "xs"}
    rng = np.random.default_rng(0x5EED0005)
    L = A.lib()

    def run(fn, desc, n):
        ev, wall = ctypes.c_float(), ctypes.c_double()
        rc = fn(ctypes.byref(desc), max(20, n // 5), n, min(GRAPH_BATCH, n), ctypes.byref(ev), ctypes.byref(wall))
        torch.cuda.synchronize()
        return None if rc != 0 else ev.value / n * 1e3

    def sweep(name, desc, plan_fn, fn, n, tiles):
        plan = A.Plan()
        desc.path = A.PATH_AUTO
        assert plan_fn(ctypes.byref(desc), ctypes.byref(plan)) == 0
        times = {}
        for t in tiles:
            desc.path = A.PATH_MFMA | ((t + 1) << 8)
            if plan_fn(ctypes.byref(desc), ctypes.byref(A.Plan())) != 0:
                continue
            v = run(fn, desc, n)
            if v is not None:
                times[t] = round(v, 2)
        desc.path = A.PATH_AUTO
        ta = run(fn, desc, n)
        best = min(times, key=times.get)
        return {"shape": name, "auto": "%s/%d" % (KN[plan.kernel], plan.tile), "auto_us": round(ta, 2), "best_tile": best,
                "best_us": times[best], "ratio": round(ta / times[best], 3), "tiles_us": times}

    out = []
    for (wb, xb) in [(1, 2), (1, 3), (1, 4), (2, 2)]:
        for batch in (1, 16):
            for C in (128, 256, 384, 512, 640, 768, 896, 1024):
                for fused in (False, True):
                    H = 16
                    rows = batch * H * H
                    X = G.to_dev(O.random_planes(rng, xb, rows, C // 32))
                    Wt = G.to_dev(O.random_planes(rng, wb, C * 9, C // 32))
                    thr = G.to_dev(np.sort(rng.integers(-200, 200, size=(C, 2 ** xb - 1)), axis=1).astype(np.int32))
                    outp = G.dev_empty_i32(max(xb * rows * C // 32, rows * C))
                    E = G.epilogue(mode=A.EPI_BN, out_bits=xb, thr=thr) if fused else G.epilogue()
                    d = A.ConvDesc(W=Wt.data_ptr(), X=X.data_ptr(), O=outp.data_ptr(), batch=batch, H=H, Wd=H, cin_pad=C,
                                   COUT=C, R=3, S=3, stride=1, pad=1, halo=0, wb=wb, xb=xb,
                                   weight_mode=A.WEIGHT_UNSIGNED, epi=E)
                    out.append(sweep("conv w%da%d 16x16 b%d C=%d %s" % (wb, xb, batch, C, "bn-packed" if fused else "int32"),
                                     d, L.apnn_conv_plan, benchlib.apnn_bench_conv_graph,
                                     1000 if rows * C * C < 3e9 else 200, (1, 2, 3, 4, 5, 7, 8, 9)))
        for (M, N, K) in [(512, 512, 1024), (1024, 1024, 1024), (1024, 1024, 4096), (2048, 2048, 2048), (1024, 4096, 2048),
                          (4096, 1024, 2048), (3072, 3072, 3072), (4096, 4096, 4096), (2048, 8192, 4096), (6144, 6144, 6144)]:
            W = G.to_dev(O.random_planes(rng, wb, M, K // 32))
            X = G.to_dev(O.random_planes(rng, xb, N, K // 32))
            D = G.dev_empty_i32(M * N)
            d = A.GemmDesc(W=W.data_ptr(), X=X.data_ptr(), D=D.data_ptr(), M=M, N=N, K=K, wb=wb, xb=xb)
            out.append(sweep("gemm w%da%d %dx%dx%d" % (wb, xb, M, N, K), d, L.apnn_gemm_plan, benchlib.apnn_bench_gemm_graph,
                             500 if M * N * K < 2e10 else 40, (1, 2, 3, 4, 5, 6, 9)))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary shapes (same as --extra none)")
    ap.add_argument("--extra", default="all",
                    help="comma list of secondary workloads to run after the headline: all, none, gemm_sweep, "
                         "gemm_large, gemm8192 (w1a2 only), conv, nets, resnet18_b8, resnet18_b64, alexnet_b8, "
                         "alexnet_b64, vgg_b8, vgg_b64; crossover (not part of all): every kernel path / tile "
                         "pinned in turn on the shapes where the library's choice changes; crossover_sweep (not part "
                         "of all): AUTO against every FP4 matrix-core tile over the whole convolution sweep and ten "
                         "GEMM sizes, all four precisions")
    ap.add_argument("--path", default="auto")
    ap.add_argument("--shape", action="append", default=[],
                    help="extra workload on --path (repeatable; used by the profile commands): "
                         "gemm:w1a2:M:N:K or conv:w1a2:b16:c1024:int32|fused[:hN] (3x3 on an NxN map, "
                         "default 16x16); --path may carry a pinned tile as path/tile, e.g. mfma/5")
    ap.add_argument("--copy-calib", action="store_true",
                    help="also launch one 256 MiB device copy and one 256 MiB store in the matrix-core kernels' "
                         "int32 store pattern (known traffic) for counter calibration")
    ap.add_argument("--headline-only", action="store_true",
                    help="run nothing but the headline's graph-replayed launches (warm-up + timed blocks): the "
                         "command the headline kernel is traced with, so that every traced launch of the kernel "
                         "belongs to the timed configuration")
    args = ap.parse_args()
    want = set(x for x in ("none" if args.no_extra else args.extra).split(",") if x)
    def on(*names):
        return "all" in want or any(n in want for n in names)
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (no collectives, no sharding); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import gpu_util as G
    import oracle_lib as O

    A = G.A
    L = A.lib()
    benchlib = ctypes.CDLL(os.path.join(os.path.dirname(A.LIB_PATH), "libapnn_bench.so"))
    benchlib.apnn_bench_gemm.argtypes = [ctypes.POINTER(A.GemmDesc), ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                         ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_double)]
    benchlib.apnn_bench_conv.argtypes = [ctypes.POINTER(A.ConvDesc), ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                         ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_double)]
    benchlib.apnn_bench_gemm_graph.argtypes = [ctypes.POINTER(A.GemmDesc), ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                               ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_double)]
    benchlib.apnn_bench_conv_graph.argtypes = [ctypes.POINTER(A.ConvDesc), ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                               ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_double)]
    benchlib.apnn_bench_gemm_graph_rotate.argtypes = [ctypes.POINTER(A.GemmDesc), ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                      ctypes.c_int, ctypes.POINTER(ctypes.c_float),
                                                      ctypes.POINTER(ctypes.c_double)]
    benchlib.apnn_bench_empty.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                          ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_double)]
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    pname, _, ptile = args.path.partition("/")
    path = {"auto": A.PATH_AUTO, "valu": A.PATH_VALU, "mfma": A.PATH_MFMA, "mfma_i8": A.PATH_MFMA_I8,
            "patch": A.PATH_MFMA_PATCH, "mfma_xs": A.PATH_MFMA_XS}[pname]
    if ptile:
        path |= (int(ptile) + 1) << 8
    # the headline and the standard extra workloads run on the plain path; a pinned tile or a
    # convolution-only / GEMM-subset path applies to the --shape workloads only
    plain = not ptile and pname in ("auto", "valu", "mfma", "mfma_i8")
    cur = {"path": path if plain else A.PATH_AUTO}

    def make_inputs(M, N, K, wb, xb):
        W = O.random_planes(np.random.default_rng(0x5EED0001), wb, M, K // 32)
        X = O.random_planes(np.random.default_rng(0x5EED0002), xb, N, K // 32)
        return W, X

    def time_gemm(M, N, K, wb, xb, sym, warmup, iters, verify_rows=None, graph=False, colsum=False):
        W, X = make_inputs(M, N, K, wb, xb)
        dW, dX = G.to_dev(W), G.to_dev(X)
        out = G.dev_empty_i32(M * N, fill=-7)
        d = A.GemmDesc(W=dW.data_ptr(), X=dX.data_ptr(), D=out.data_ptr(), M=M, N=N, K=K, wb=wb, xb=xb,
                       weight_mode=sym, path=cur["path"])
        ev, wall = ctypes.c_float(), ctypes.c_double()
        torch.cuda.synchronize()
        if graph:
            A.check(benchlib.apnn_bench_gemm_graph(ctypes.byref(d), warmup, iters, GRAPH_BATCH, ctypes.byref(ev),
                                                   ctypes.byref(wall)), "apnn_bench_gemm_graph")
        else:
            A.check(benchlib.apnn_bench_gemm(ctypes.byref(d), warmup, iters, stream, ctypes.byref(ev),
                                             ctypes.byref(wall)), "apnn_bench_gemm")
        torch.cuda.synchronize()
        got = G.to_host(out).reshape(M, N)
        if verify_rows is None:
            ok = bool(np.array_equal(got, O.gemm(W, X, M, N, K, wb, xb, sym_w=sym, nthreads=os.cpu_count() or 1)))
        else:
            ok = True
            for m in verify_rows:
                ref = O.gemm_rows(W, X, M, N, K, wb, xb, m, m + 1, sym_w=sym, nthreads=os.cpu_count() or 1)[0]
                ok = ok and bool(np.array_equal(got[m], ref))
        if colsum and not sym:
            # sum_m D[m][n] = sum_k (sum_m w[m][k]) x[n][k]: every output element takes part
            ok = ok and bool(np.array_equal(got.sum(0, dtype=np.int64), O.gemm_column_sums(W, X)))
        return dict(event_ms=ev.value / iters, wall_ms=wall.value / iters, verified=ok, W=W, X=X)

    if args.copy_calib:
        nbytes_c = 256 << 20
        src = torch.zeros(nbytes_c // 4, dtype=torch.int32, device="cuda")
        dst = torch.empty_like(src)
        benchlib.apnn_bench_copy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_longlong, ctypes.c_void_p]
        A.check(benchlib.apnn_bench_copy(src.data_ptr(), dst.data_ptr(), nbytes_c, stream), "apnn_bench_copy")
        benchlib.apnn_bench_store_blocks.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
        A.check(benchlib.apnn_bench_store_blocks(dst.data_ptr(), 8192, 8192, stream), "apnn_bench_store_blocks")
        torch.cuda.synchronize()

    # ---- headline -----------------------------------------------------------------------------
    M, N, K, wb, xb = 64, 1024, 1024, 1, 2
    ops = 2.0 * M * N * K
    nbytes = gemm_bytes(M, N, K, wb, xb)
    reps = -(-MIN_TIMED_LAUNCHES // max(1, args.steps))
    timed = reps * max(1, args.steps)
    warm = max(args.warmup, MIN_WARMUP_LAUNCHES)

    def headline(sym, graph=True):
        blocks = [time_gemm(M, N, K, wb, xb, sym, warm, timed, graph=graph) for _ in range(HEADLINE_BLOCKS)]
        blocks.sort(key=lambda b: b["event_ms"])
        mid = blocks[len(blocks) // 2]
        mid["verified"] = all(b["verified"] for b in blocks)
        mid["block_us"] = [round(b["event_ms"] * 1e3, 4) for b in blocks]
        return mid

    r = headline(A.WEIGHT_SYMMETRIC)
    step_ms = r["event_ms"]                       # HIP-event time per launch
    tops = ops / (step_ms * 1e-3) / 1e12
    achieved_gbs = nbytes / (step_ms * 1e-3) / 1e9
    result = {
        "metric": "w1a2 GEMM effective TOPS at M=64,N=K=1024",
        "value": round(tops, 4),
        "unit": "TOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_ms, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": round(tops / BASELINE_TOPS, 4),
        "dtype": "int32 accumulate over 1-bit x 2-bit planes",
        "data": "synthetic",
        "config": {"workload": "apnn_gemm w1a2 M=64 N=1024 K=1024, weights 2b-1 (symmetric), int32 out",
                   "path": args.path, "launch": "HIP graph replay, %d launches per graph" % GRAPH_BATCH,
                   "timed_launches": timed, "warmup_launches": warm, "clock": "HIP events on the launch stream",
                   "blocks_us_per_launch": r["block_us"], "host_wall_us_per_launch": round(r["wall_ms"] * 1e3, 4),
                   "verified_bit_exact": r["verified"]},
        "roofline": {"bound": "hbm", "achieved": round(achieved_gbs, 3), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved_gbs / HBM_PEAK_GBS, 6), "traffic": HEADLINE_TRAFFIC_BYTES,
                     "algorithmic_bytes": nbytes, "kernel_us": round(step_ms * 1e3, 4)},
    }

    if args.headline_only:
        print(json.dumps(result))
        return

    extra = {}
    # the reference's unsigned arithmetic right after the headline run (same clock state: a loop of
    # empty kernels in between lets the GPU clock down and the next short measurement pays for it)
    ru = headline(A.WEIGHT_UNSIGNED)
    extra["unsigned_reference_arithmetic"] = {"tops": round(ops / (ru["event_ms"] * 1e-3) / 1e12, 4),
                                              "us": round(ru["event_ms"] * 1e3, 4), "verified": ru["verified"]}
    re_ = time_gemm(M, N, K, wb, xb, A.WEIGHT_SYMMETRIC, warm, timed)
    extra["plain_launch_loop"] = {"tops": round(ops / (re_["wall_ms"] * 1e-3) / 1e12, 4),
                                  "us": round(re_["wall_ms"] * 1e3, 4), "verified": re_["verified"]}
    ev, wall = ctypes.c_float(), ctypes.c_double()
    benchlib.apnn_bench_empty(warm, timed, stream, ctypes.byref(ev), ctypes.byref(wall))
    extra["empty_kernel_us_per_launch"] = round(wall.value / timed * 1e3, 4)

    # Cold caches: the same launch rotating over COLD_SETS buffer sets (weights, activations and output of
    # their own each; COLD_SETS x 520 KiB = 333 MB, more than the 256 MB last-level cache), one graph of
    # COLD_SETS launches replayed, so a buffer set is touched again only after all the others.
    COLD_SETS = 640
    Wc, Xc = r["W"], r["X"]
    cW = torch.from_numpy(np.ascontiguousarray(Wc).view(np.int32)).cuda().repeat(COLD_SETS, 1, 1, 1)
    cX = torch.from_numpy(np.ascontiguousarray(Xc).view(np.int32)).cuda().repeat(COLD_SETS, 1, 1, 1)
    cD = torch.full((COLD_SETS, M * N), -7, dtype=torch.int32, device="cuda")
    descs = (A.GemmDesc * COLD_SETS)()
    for i in range(COLD_SETS):
        descs[i] = A.GemmDesc(W=cW[i].data_ptr(), X=cX[i].data_ptr(), D=cD[i].data_ptr(), M=M, N=N, K=K, wb=wb, xb=xb,
                              weight_mode=A.WEIGHT_SYMMETRIC, path=cur["path"])
    ev, wall = ctypes.c_float(), ctypes.c_double()
    A.check(benchlib.apnn_bench_gemm_graph_rotate(descs, COLD_SETS, COLD_SETS, 4 * COLD_SETS, COLD_SETS,
                                                  ctypes.byref(ev), ctypes.byref(wall)), "apnn_bench_gemm_graph_rotate")
    torch.cuda.synchronize()
    cold_ok = bool((cD == cD[0]).all().item()) and bool(
        np.array_equal(cD[0].cpu().numpy().reshape(M, N), O.gemm(Wc, Xc, M, N, K, wb, xb, sym_w=1)))
    cold_us = ev.value / (4 * COLD_SETS) * 1e3
    extra["cold_cache"] = {"us": round(cold_us, 4), "tops": round(ops / (cold_us * 1e-6) / 1e12, 4),
                           "frac_hbm_peak": round(nbytes / (cold_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 6),
                           "buffer_sets": COLD_SETS, "bytes_rotated": COLD_SETS * nbytes, "verified": cold_ok}
    result["config"]["cold_us_per_launch"] = round(cold_us, 4)
    del cW, cX, cD

    conv_ref_cache = {}

    def time_conv(batch, C, w_, a_, fused, warmup, iters, H=16):
        """3x3, stride 1, stored halo, 16x16 feature map, Cin = Cout = C (the reference's conv benchmark,
        APNN-TC-lib/bmmaTensorCoreGemm/src/51_conv_w1a2_small.cu:478-512, with a batch dimension).  Every
        row is checked against the oracle: the int32 output as is, the fused output against the oracle's
        threshold quantizer + packer applied to the oracle convolution."""
        Wd = H
        rng = np.random.default_rng(0x5EED0003)
        X = O.random_planes(rng, a_, batch * (H + 2) * (Wd + 2), C // 32)
        # the halo ring holds zeros, as the reference's padded input does
        Xv = X.reshape(a_, batch, H + 2, Wd + 2, C // 32)
        Xv[:, :, 0], Xv[:, :, -1], Xv[:, :, :, 0], Xv[:, :, :, -1] = 0, 0, 0, 0
        Wt = O.random_planes(rng, w_, C * 9, C // 32)
        dW, dX = G.to_dev(Wt), G.to_dev(X)
        key = (batch, C, w_, a_, H)
        if key not in conv_ref_cache:
            conv_ref_cache.clear()      # rows of one shape are adjacent: keep one reference at a time
            conv_ref_cache[key] = O.conv(Wt, X, batch=batch, H=H, W=Wd, cwords=C // 32, cout=C, R=3, S=3, stride=1,
                                         pad=1, halo=1, wb=w_, xb=a_, sym_w=0, nthreads=os.cpu_count() or 1)
        ref = conv_ref_cache[key]
        if fused:
            hi = 9 * C * ((1 << a_) - 1) * ((1 << w_) - 1) // 2
            thr = np.sort(rng.integers(0, hi + 1, size=(C, (1 << a_) - 1)), axis=1).astype(np.int32)
            dT = G.to_dev(thr)
            out = G.dev_empty_i32(a_ * batch * H * Wd * C // 32, fill=-7)
            E = G.epilogue(mode=A.EPI_BN, out_bits=a_, thr=dT)
            nbytes = (a_ * batch * H * Wd * C + w_ * 9 * C * C + a_ * batch * H * Wd * C) // 8 + 4 * ((1 << a_) - 1) * C
        else:
            out = G.dev_empty_i32(batch * H * Wd * C, fill=-7)
            E = G.epilogue()
            nbytes = (a_ * batch * H * Wd * C + w_ * 9 * C * C) // 8 + 4 * batch * H * Wd * C
        d = A.ConvDesc(W=dW.data_ptr(), X=dX.data_ptr(), O=out.data_ptr(), batch=batch, H=H, Wd=Wd, cin_pad=C, COUT=C,
                       R=3, S=3, stride=1, pad=1, halo=1, wb=w_, xb=a_, weight_mode=A.WEIGHT_UNSIGNED, epi=E,
                       path=cur["path"])
        ev, wall = ctypes.c_float(), ctypes.c_double()
        # graph replay at both batch sizes: a plain launch loop issues a kernel every 3-5 us at best, which
        # would hide every batch-16 row that runs faster than that
        A.check(benchlib.apnn_bench_conv_graph(ctypes.byref(d), warmup, iters, min(GRAPH_BATCH, iters), ctypes.byref(ev),
                                               ctypes.byref(wall)), "apnn_bench_conv_graph")
        torch.cuda.synchronize()
        rows = batch * H * Wd
        if fused:
            got = G.to_host(out, np.uint32).reshape(a_, rows, C // 32)
            q = O.bn_quantize(ref.reshape(rows, C), None, thr, None, a_)
            ok = bool(np.array_equal(got, O.lowbits_pack(q, rows, C, a_)))
        else:
            ok = bool(np.array_equal(G.to_host(out).reshape(ref.shape), ref))
        ops_c = 2.0 * batch * H * Wd * C * 9 * C
        t_s = ev.value / iters * 1e-3
        tops_c = ops_c / t_s / 1e12
        gbs = nbytes / t_s / 1e9
        # fractions of the two rooflines of this path: HBM (algorithmic bytes) and the matrix cores the
        # kernels issue on (FP4 operands; the int8 figure is the chip's integer peak, for comparison)
        return {"us": round(t_s * 1e6, 3), "tops": round(tops_c, 2), "hbm_gbs": round(gbs, 1),
                "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4), "frac_fp4_mfma_peak": round(tops_c / FP4_MFMA_PEAK_TOPS, 4),
                "frac_int8_mfma_peak": round(tops_c / INT8_MFMA_PEAK_TOPS, 4), "verified": ok}

    if want != {"none"}:
        shapes = []
        for (w_, a_) in [(1, 2), (1, 3), (1, 4), (2, 2)]:
            for nk in (128, 256, 384, 512, 640, 768, 896, 1024) if on("gemm_sweep") else ():
                t = time_gemm(64, nk, nk, w_, a_, A.WEIGHT_UNSIGNED, 200, 2000, graph=True)
                nb = gemm_bytes(64, nk, nk, w_, a_)
                shapes.append({"shape": "w%da%d M=64 N=K=%d" % (w_, a_, nk),
                               "us": round(t["event_ms"] * 1e3, 3),
                               "tops": round(2.0 * 64 * nk * nk / (t["event_ms"] * 1e-3) / 1e12, 3),
                               "frac_hbm_peak": round(nb / (t["event_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 5),
                               "verified": t["verified"]})
            large = (2048, 4096, 8192) if on("gemm_large") else ((8192,) if (w_, a_) == (1, 2) and on("gemm8192") else ())
            for n in large if (w_, a_) == (1, 2) else ():
                # the same GEMM with the low a bits packed (apmm_w1a2_decompose): no 4*M*N-byte int32 store
                W, X = make_inputs(n, n, n, w_, a_)
                dW, dX = G.to_dev(W), G.to_dev(X)
                outp = G.dev_empty_i32(a_ * n * n // 32, fill=-7)
                dd = A.GemmDesc(W=dW.data_ptr(), X=dX.data_ptr(), D=outp.data_ptr(), M=n, N=n, K=n, wb=w_, xb=a_,
                                epi=G.epilogue(mode=A.EPI_LOWBITS, out_bits=a_), path=cur["path"])
                ev, wall = ctypes.c_float(), ctypes.c_double()
                iters = {2048: 20, 4096: 10, 8192: 3}[n]
                A.check(benchlib.apnn_bench_gemm(ctypes.byref(dd), 2, iters, stream, ctypes.byref(ev), ctypes.byref(wall)),
                        "apnn_bench_gemm(packed)")
                torch.cuda.synchronize()
                gotp = G.to_host(outp, np.uint32).reshape(a_, n, n // 32)
                okp = True
                for m in (0, n // 2 + 1, n - 1):
                    ref = O.gemm_rows(W, X, n, n, n, w_, a_, m, m + 1, nthreads=os.cpu_count() or 1)
                    okp = okp and bool(np.array_equal(gotp[:, m], O.lowbits_pack(ref, 1, n, a_)[:, 0]))
                tt = 2.0 * n ** 3 / (ev.value / iters * 1e-3) / 1e12
                shapes.append({"shape": "w%da%d M=N=K=%d low-bit packed out" % (w_, a_, n), "ms": round(ev.value / iters, 4),
                               "tops": round(tt, 2), "frac_fp4_mfma_peak": round(tt / FP4_MFMA_PEAK_TOPS, 4),
                               "verified": okp})
            for n in large:
                iters = {2048: 20, 4096: 10, 8192: 3}[n]
                vrows = sorted(set([0, n - 1] + [int(v) for v in np.random.default_rng(n).integers(0, n, 14)]))
                t = time_gemm(n, n, n, w_, a_, A.WEIGHT_UNSIGNED, 2, iters, verify_rows=vrows, colsum=True)
                tt = 2.0 * n ** 3 / (t["event_ms"] * 1e-3) / 1e12
                shapes.append({"shape": "w%da%d M=N=K=%d" % (w_, a_, n), "ms": round(t["event_ms"], 4),
                               "tops": round(tt, 2), "frac_int8_mfma_peak": round(tt / INT8_MFMA_PEAK_TOPS, 4),
                               "frac_fp4_mfma_peak": round(tt / FP4_MFMA_PEAK_TOPS, 4),
                               "hbm_gbs": round(gemm_bytes(n, n, n, w_, a_) / (t["event_ms"] * 1e-3) / 1e9, 1),
                               "verified": t["verified"],
                               "verified_how": "%d sampled rows vs oracle + all column sums (linearity)" % len(vrows)})
        if shapes:
            extra["shapes"] = shapes
        if on("conv"):
            convs = []
            for (w_, a_) in [(1, 2), (1, 3), (1, 4), (2, 2)]:
                for batch in (1, 16):
                    # every channel count of the reference's published list (README.md:160-167), at both batch
                    # sizes, for all four precisions
                    for C in (128, 256, 384, 512, 640, 768, 896, 1024):
                        for fused in (False, True):
                            t = time_conv(batch, C, w_, a_, fused, 200 if batch == 1 else 20, 1000 if batch == 1 else 100)
                            t["shape"] = "w%da%d 3x3 16x16 b%d Cin=Cout=%d %s" % (
                                w_, a_, batch, C, "bn-quantize packed out" if fused else "int32 out")
                            convs.append(t)
            extra["conv"] = convs
        # ---- second headline metric: end-to-end w1a2 ResNet18 (and the AlexNet-style net) --------
        nets = {}
        for kind, nm in ((A.NET_RESNET18, "resnet18"), (A.NET_ALEXNET, "alexnet"), (A.NET_VGG, "vgg")):
            for batch in (8, 64):
                if not on("nets", "%s_b%d" % (nm, batch)):
                    continue
                NL = A.nn_lib()
                net = NL.apnn_net_create(kind, batch, 1, cur["path"])
                assert net, "network construction failed"
                img = torch.randint(0, 256, (batch, 224, 224, 3), dtype=torch.uint8, device="cuda")
                lg = torch.empty((batch, 1000), dtype=torch.float32, device="cuda")
                ev, wall = ctypes.c_float(), ctypes.c_double()
                iters = 200 if batch == 8 else 50
                A.check(NL.apnn_net_bench(net, img.data_ptr(), lg.data_ptr(), 10, iters, 0, stream, ctypes.byref(ev),
                                          ctypes.byref(wall)), "apnn_net_bench")
                # effective operations of one image: 2 x MACs of every convolution / FC / classifier layer
                ops_img = 0.0
                for li in range(NL.apnn_net_layer_count(net)):
                    ld = A.LayerDesc()
                    NL.apnn_net_layer(net, li, ctypes.byref(ld))
                    if ld.kind == A.LAYER_OUT_I8:
                        ops_img += 2.0 * ld.in_c * ld.out_c
                    elif ld.kind == A.LAYER_IMAGE_QUANT or ld.stride <= 0:
                        continue    # quantize-and-pack of the input image: no multiply-accumulates
                    else:
                        ho = (ld.in_h + 2 * ld.pad - ld.R) // ld.stride + 1
                        wo = (ld.in_w + 2 * ld.pad - ld.S) // ld.stride + 1
                        ops_img += 2.0 * ho * wo * ld.out_c * ld.R * ld.S * ld.in_c
                entry = {"ms_per_forward": round(wall.value / iters, 4),
                         "images_per_sec": round(batch * iters / wall.value * 1e3, 1),
                         "gops_per_image": round(ops_img / 1e9, 3)}
                # the same forward replayed as one HIP graph (no per-kernel launch from the host)
                A.check(NL.apnn_net_bench(net, img.data_ptr(), lg.data_ptr(), 10, iters, 1, stream, ctypes.byref(ev),
                                          ctypes.byref(wall)), "apnn_net_bench(graph)")
                entry["graph_ms_per_forward"] = round(ev.value / iters, 4)
                entry["graph_images_per_sec"] = round(batch * iters / ev.value * 1e3, 1)
                best_tops = ops_img * entry["graph_images_per_sec"] / 1e12
                entry["effective_tops"] = round(best_tops, 1)
                entry["frac_fp4_mfma_peak"] = round(best_tops / FP4_MFMA_PEAK_TOPS, 4)
                entry["frac_int8_mfma_peak"] = round(best_tops / INT8_MFMA_PEAK_TOPS, 4)
                nets["%s_w1a2_b%d" % (nm, batch)] = entry
                NL.apnn_net_destroy(net)
        if nets:
            extra["networks"] = nets
    cur["path"] = path
    for spec in args.shape:
        f = spec.split(":")
        w_, a_ = int(f[1][1]), int(f[1][3])
        if f[0] == "gemm":
            Mg, Ng, Kg = int(f[2]), int(f[3]), int(f[4])
            small = Mg * Ng <= 512 * 512
            vr = None if Mg * Ng <= 1024 * 1024 else [0, Mg // 2 + 1, Mg - 1]
            t = time_gemm(Mg, Ng, Kg, w_, a_, A.WEIGHT_UNSIGNED, 200 if small else 2, 2000 if small else 5,
                          verify_rows=vr, graph=small)
            tt = 2.0 * Mg * Ng * Kg / (t["event_ms"] * 1e-3) / 1e12
            extra.setdefault("requested", []).append({"shape": spec, "path": args.path, "us": round(t["event_ms"] * 1e3, 3),
                                                      "tops": round(tt, 2), "verified": t["verified"]})
        else:
            bt, Cc = int(f[2][1:]), int(f[3][1:])
            Hm = int(f[5][1:]) if len(f) > 5 else 16
            t = time_conv(bt, Cc, w_, a_, f[4] == "fused", 200 if bt == 1 else 20, 1000 if bt == 1 else 100, H=Hm)
            t.update(shape=spec, path=args.path)
            extra.setdefault("requested", []).append(t)
    if "crossover" in want:
        extra["crossover"] = crossover_table(A, G, O, benchlib, stream)
    if "crossover_sweep" in want:
        extra["crossover_sweep"] = crossover_sweep(A, G, O, benchlib)
    result["extra"] = extra

    # ---- CPU baseline: the scalar oracle on the same inputs, host cores ---------------------------
    if not args.no_cpu:
        W, X = r["W"], r["X"]
        ncores = os.cpu_count() or 1
        def cpu_time(nthreads, budget_s):
            n, t0 = 0, time.perf_counter()
            while True:
                O.gemm(W, X, M, N, K, wb, xb, sym_w=1, nthreads=nthreads)
                n += 1
                el = time.perf_counter() - t0
                if el > budget_s:
                    return el / n, n
        t1, n1 = cpu_time(1, 6.0)
        tn, nn = cpu_time(ncores, 6.0)
        result["cpu_baseline"] = {
            "value": round(ops / tn / 1e12, 5), "unit": "TOPS", "cores": ncores, "kind": "port",
            "sample": "full headline GEMM (M=64,N=K=1024, +-1 weights), %d runs on %d threads; "
                      "single thread: %.5f TOPS over %d runs" % (nn, ncores, ops / t1 / 1e12, n1),
            "single_thread_tops": round(ops / t1 / 1e12, 5),
        }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
