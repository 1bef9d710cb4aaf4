#!/usr/bin/env python3
"""Benchmark of the bitplane GEMV (matmul_kbit) on one MI355X.

Workload (the configuration the headline metric is quoted on): the seven linears of one
Llama-2-7B decoder layer at batch 1 -- q,k,v,o 4096x4096, gate,up 11008x4096, down
4096x11008 -- parent 8 bits, every w_bits in 3..8.  One "step" is one pass over those
7 x 6 = 42 GEMVs.  Weights live in HBM before the timed region; consecutive steps walk a
pool of distinct weight sets (>= 1.5 GB of touched planes per shape) so that no launch finds
its planes in the 256 MB last-level cache.

Prints ONE JSON line: whole-step effective bandwidth (algorithmic bytes / time), the
per-kernel roofline of the kernel that dominates the step, and the CPU baseline (the C
oracle's host-speed GEMV on the same shapes, timed on this box's cores).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "any-precision-llm_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, published
BITS = (3, 4, 5, 6, 7, 8)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--workload", default="llama2_7b_layer_batch1",
                    choices=("llama2_7b_layer_batch1", "llama3_8b_layer_batches", "llama2_7b_dequant_full_model",
                             "llama2_7b_decode", "llama2_7b_prefill", "llama2_7b_gemm_rows", "gemv_kernel_variants",
                             "routing_audit", "profile_set"),
                    help="default: the headline (42 GEMVs of a Llama-2-7B layer at batch 1).  "
                         "llama3_8b_layer_batches: matmul_kbit on the Llama-3-8B shapes at M = 1, 2, 4, 8.  "
                         "llama2_7b_dequant_full_model: dequant_kbit over all 224 linears of Llama-2-7B.  "
                         "llama2_7b_decode: batch-1 greedy decoding of a random-init Llama-2-7B-shaped model, "
                         "256 tokens after a 128-token prompt, per w_bits.  "
                         "llama2_7b_prefill: the seven linears of a layer on 32 x 512 = 16384 activation rows "
                         "(dequant_kbit + library GEMM, the large-batch branch of AnyPrecisionLinear).  "
                         "llama2_7b_gemm_rows: ap_gemm_kbit on the three linear shapes of the layer at 64..512 activation "
                         "rows: its default launch, the K-split and the tiled kernel forced, dequant_kbit + library GEMM "
                         "beside them; with --eager one launch of the tiled kernel per case only (for counter runs).  "
                         "gemv_kernel_variants: the four dot-product GEMV kernels forced in turn (tuning knobs) on "
                         "the headline shapes and on 28672 x 8192, batch 1, beside the read-only stream; with "
                         "--eager the launches go out one by one (the form rocprofv3 counter runs need).  "
                         "profile_set: one eager launch list for rocprofv3 runs -- every kernel the default routes of the "
                         "Llama-2-7B layer use: the 18 single GEMVs, the q/k/v and gate/up group launches, the SwiGLU pair "
                         "launch, dequant_kbit per linear and per layer set, the fused GEMM at 16 and 16384 rows; "
                         "--kernel-reps launches per case on rotating weight sets, a manifest of the cases on stdout.  "
                         "routing_audit: for the linears of the models named by --audit-models, at 1..8 activation "
                         "rows and 3, 4, 5, 8 bits, the time of what ap_matmul_kbit launches by default beside every "
                         "kernel and geometry the tuning knobs can force: where is the default not the fastest.")
    ap.add_argument("--audit-models", default="7b,8b", help="routing_audit: comma list out of 7b, 8b, 13b, 70b")
    ap.add_argument("--audit-rows", default="1,2,3,4,5,8", help="routing_audit: activation row counts")
    ap.add_argument("--audit-sets", action="store_true", help="routing_audit: also the q/k/v and gate/up sets (ap_matmul_kbit_group)")
    ap.add_argument("--audit-gemm", action="store_true", help="routing_audit: also ap_gemm_kbit at 16, 32, 48, 64, 96, 128 rows")
    ap.add_argument("--audit-decode", action="store_true",
                    help="llama2_7b_decode: instead of the sweep over w_bits, the decode graph re-recorded under each global "
                         "override of the GEMV launch rules (ap_set_tuning), tokens/s against the default rules'")
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--pool", type=int, default=4, help="at least this many distinct decoder layers in the pool")
    ap.add_argument("--pool-gb", type=float, default=1.5,
                    help="per shape, GB of the three top planes over all weight sets of the pool")
    ap.add_argument("--kernel-reps", type=int, default=40, help="launches per (shape, w_bits) for the per-kernel table")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--table", default="", help="also write the per-layer table (markdown) to this file")
    ap.add_argument("--only-step", action="store_true", help="skip the per-kernel table (used under rocprofv3)")
    ap.add_argument("--no-extras", action="store_true", help="skip the dequant and batch tables")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three plain 256 MiB device copies, so a counter run has a kernel of known "
                         "HBM traffic (read 256 MiB, write 256 MiB) to scale FETCH_SIZE / WRITE_SIZE with")
    ap.add_argument("--eager", action="store_true",
                    help="launch the timed steps one by one instead of replaying a HIP graph (rocprofv3 inflates "
                         "the durations of graph-launched kernels, so profiles are taken in this mode)")
    return ap.parse_args()


class WeightPool:
    """`sets` device-resident synthetic linears of one shape.  Uniform parent codes are
    uniform plane bits, so planes are drawn directly as random words; tables are ascending
    N(0, 0.02) draws (std 0.02), one per set and precision."""

    def __init__(self, torch, N, K, sets, gen, bits=BITS):
        self.N, self.K, self.sets = N, K, sets
        self.qweight = torch.randint(-2**31, 2**31 - 1, (sets, 8, N, K // 32), dtype=torch.int32, device="cuda",
                                     generator=gen)
        self.luts = {}
        for b in bits:
            t = torch.randn((sets, N, 1 << b), device="cuda", generator=gen) * 0.02
            self.luts[b] = torch.sort(t, dim=2).values.to(torch.float16).contiguous()
        self.out = torch.empty((8, N), dtype=torch.float16, device="cuda")


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from any_precision_amd import _capi, synth

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    if args.workload == "llama3_8b_layer_batches":
        return batch_sweep(args, torch, _capi, synth)
    if args.workload == "llama2_7b_dequant_full_model":
        return dequant_full_model(args, torch, _capi, synth)
    if args.workload == "llama2_7b_prefill":
        return prefill_linears(args, torch, _capi, synth)
    if args.workload == "gemv_kernel_variants":
        return gemv_kernel_variants(args, torch, _capi, synth)
    if args.workload == "routing_audit":
        return routing_audit(args, torch, _capi, synth)
    if args.workload == "profile_set":
        return profile_set(args, torch, _capi, synth)
    if args.workload == "llama2_7b_gemm_rows":
        return gemm_rows(args, torch, _capi, synth)
    if args.workload == "llama2_7b_decode":
        with torch.inference_mode():     # the decoder captures its graphs in inference mode; stay in it
            return decode_tokens(args, torch, _capi, synth)
    lib = _capi.lib
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0)
    shapes = [(n, N, K) for n, N, K in synth.LLAMA2_7B_LAYER]
    uniq = {}
    for idx, (name, N, K) in enumerate(shapes):
        uniq.setdefault((N, K), []).append(idx)

    # Cold-cache discipline: every launch reads a weight set that no recent launch touched.  Per
    # shape the pool holds enough sets that even the 3 top planes of all sets exceed
    # `--pool-gb` (default 1.5 GB, six times the 256 MB last-level cache).
    pools = {}
    for (N, K), idxs in uniq.items():
        need = int(args.pool_gb * 1e9 / (3 * N * K / 8)) + 1
        sets = max(need, len(idxs) * args.pool)
        pools[(N, K)] = WeightPool(torch, N, K, sets, gen)
    batches = (1, 2, 4, 8, 16, 32, 128, 256)
    xb = {(M, K): torch.randn((M, K), device="cuda", generator=gen).to(torch.float16)
          for K in {K for _, _, K in shapes} for M in batches}
    for P in pools.values():
        P.out = torch.empty((max(batches), P.N), dtype=torch.float16, device="cuda")
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    cursor = {k: 0 for k in pools}

    def launch(N: int, K: int, b: int, stream: int, M: int = 1, fn=None):
        """One GEMV (or `fn`: another entry point with the same signature) on the next weight set of its shape."""
        P = pools[(N, K)]
        j = cursor[(N, K)] = (cursor[(N, K)] + 1) % P.sets
        rc = (fn or lib.ap_matmul_kbit)(xb[(M, K)].data_ptr(), P.qweight[j].data_ptr(), P.luts[b][j].data_ptr(),
                                        P.out.data_ptr(), M, N, K, b, stream)
        if rc != 0:
            raise RuntimeError(_capi.strerror(rc))

    sink = torch.zeros(16, dtype=torch.int32, device="cuda")

    def read_only(N: int, K: int, b: int, stream: int):
        """ap_probe_stream over the planes 0..b-1 and the table of the next weight set of the shape."""
        P = pools[(N, K)]
        j = cursor[(N, K)] = (cursor[(N, K)] + 1) % P.sets
        rc = lib.ap_probe_stream(P.qweight[j].data_ptr(), b * N * K // 8, P.luts[b][j].data_ptr(), N * (2 << b),
                                 sink.data_ptr(), 32, stream)
        if rc != 0:
            raise RuntimeError(_capi.strerror(rc))

    def time_graph(enqueue, reps, replays=5):
        """us per call of `enqueue(stream)`: `reps` calls captured in one HIP graph; median over `replays`
        timed replays after an untimed one (with --eager: launched one by one, host launch cost included)."""
        with torch.cuda.stream(side):
            if args.eager:
                enqueue(side.cuda_stream)
                side.synchronize()
                a0, a1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a0.record(side)
                for _ in range(reps):
                    enqueue(side.cuda_stream)
                a1.record(side)
                side.synchronize()
                return a0.elapsed_time(a1) * 1e3 / reps
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                for _ in range(reps):
                    enqueue(torch.cuda.current_stream().cuda_stream)
            g.replay()
            side.synchronize()
            times = []
            for _ in range(replays):
                a0, a1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a0.record(side)
                g.replay()
                a1.record(side)
                side.synchronize()
                times.append(a0.elapsed_time(a1) * 1e3 / reps)
        times.sort()
        time_graph.spread = (times[0], times[-1])
        return times[len(times) // 2]

    def step(i: int, stream: int):
        for b in BITS:
            for _, N, K in shapes:
                launch(N, K, b, stream)

    step_bytes = sum(synth.gemv_bytes(N, K, b, 1) for _, N, K in shapes for b in BITS)

    # the same 42 GEMVs with the linears that share an input issued as one launch each (q,k,v; gate,up):
    # 24 launches per step.  Reported beside the headline, which stays one launch per linear.
    names = [n for n, _, _ in shapes]
    groups = [[names.index(n) for n in g] for g in (("q_proj", "k_proj", "v_proj"), ("o_proj",),
                                                    ("gate_proj", "up_proj"), ("down_proj",))]
    lin_out = [torch.empty((1, N), dtype=torch.float16, device="cuda") for _, N, _ in shapes]

    def grouped_step(stream: int):
        for b in BITS:
            for g in groups:
                qs, ts = [], []
                for li in g:
                    _, N, K = shapes[li]
                    P = pools[(N, K)]
                    j = cursor[(N, K)] = (cursor[(N, K)] + 1) % P.sets
                    qs.append(P.qweight[j].data_ptr())
                    ts.append(P.luts[b][j].data_ptr())
                K = shapes[g[0]][2]
                rc = _capi.matmul_group(xb[(1, K)].data_ptr(), qs, ts, [lin_out[li].data_ptr() for li in g],
                                        [shapes[li][1] for li in g], 1, K, b, stream)
                if rc != 0:
                    raise RuntimeError(_capi.strerror(rc))

    if args.calibrate_copy:
        src = torch.ones(64 << 20, dtype=torch.int32, device="cuda")      # 256 MiB
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1, out=dst)      # one elementwise kernel: reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    # ---- whole-step timing: the K steps are captured in one HIP graph so the host never starves the GPU
    with torch.cuda.stream(side):
        for i in range(args.warmup):
            step(i, side.cuda_stream)
        side.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        if args.eager:
            torch.cuda.synchronize()
            e0.record(side)
            for i in range(args.steps):
                step(args.warmup + i, side.cuda_stream)
            e1.record(side)
        else:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for i in range(args.steps):
                    step(args.warmup + i, torch.cuda.current_stream().cuda_stream)
            graph.replay()                      # untimed: first replay pays graph upload
            side.synchronize()
            torch.cuda.synchronize()
            e0.record(side)
            graph.replay()
            e1.record(side)
        torch.cuda.synchronize()
        total_ms = e0.elapsed_time(e1)
    ms_per_step = total_ms / args.steps
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    grouped = None
    if not args.eager and not args.only_step:
        us = time_graph(grouped_step, max(2, args.steps // 2))
        grouped = {"launches_per_step": len(BITS) * len(groups), "ms_per_step": round(us / 1e3, 5),
                   "GBps": round(step_bytes / us / 1e3, 1), "frac": round(step_bytes / us / 1e3 / HBM_PEAK_GBS, 4),
                   "note": "same 42 GEMVs, q/k/v and gate/up each as one ap_matmul_kbit_group launch"}

    # ---- per-kernel table: each (shape, w_bits) alone, rotating over the pool (cold planes)
    table, dequant_table, batch_table = [], [], []
    if not args.only_step:
        for (N, K), idxs in uniq.items():
            for b in BITS:
                by = synth.gemv_bytes(N, K, b, 1)
                # enough launches that a replay streams >= 1 GB before it returns to its first weight set
                reps = min(pools[(N, K)].sets, max(args.kernel_reps, int(1e9 / by) + 1))
                us = time_graph(lambda st: launch(N, K, b, st), reps)
                geo = _capi.matmul_geometry(1, N, K, b)
                lo, hi = getattr(time_graph, "spread", (us, us))
                # the same launch on ONE weight set over and over: planes resident in the last-level cache
                P0 = pools[(N, K)]
                us_warm = time_graph(lambda st: lib.ap_matmul_kbit(xb[(1, K)].data_ptr(), P0.qweight[0].data_ptr(),
                                                                   P0.luts[b][0].data_ptr(), P0.out.data_ptr(), 1, N, K,
                                                                   b, st), args.kernel_reps)
                # a kernel that only READS the same planes and tables (16-byte loads, no arithmetic, no
                # output), launched over the same rotating pool: what the machine does for these bytes
                us_read = time_graph(lambda st: read_only(N, K, b, st), reps)
                table.append({"N": N, "K": K, "w_bits": b, "us": round(us, 3), "us_min": round(lo, 3),
                              "us_max": round(hi, 3), "us_cache_resident": round(us_warm, 3),
                              "stream_only_us": round(us_read, 3),
                              "frac_of_stream_ceiling": round(us_read / us, 4),
                              "GBps": round(by / us / 1e3, 1),
                              "frac": round(by / us / 1e3 / HBM_PEAK_GBS, 4), "bytes": by,
                              "count_in_step": len(idxs), "kernel": _capi.matmul_route(1, N, K, b), "geometry": geo})

    # ---- further kernels of the path (reported beside the headline, not part of `value`)
    if not args.only_step and not args.no_extras:
        # dequant_kbit: planes + table in, fp16 [N, K] out; outputs rotate over >= 512 MB of buffers
        for (N, K), P in pools.items():
            nout = max(2, int(512e6 / (2 * N * K)) + 1)
            outs = [torch.empty((N, K), dtype=torch.float16, device="cuda") for _ in range(nout)]
            state = {"i": 0}

            def deq(st, b):
                j = cursor[(N, K)] = (cursor[(N, K)] + 1) % P.sets
                state["i"] = (state["i"] + 1) % nout
                rc = lib.ap_dequant_kbit(P.qweight[j].data_ptr(), P.luts[b][j].data_ptr(),
                                         outs[state["i"]].data_ptr(), N, K, b, st)
                if rc != 0:
                    raise RuntimeError(_capi.strerror(rc))

            def write_only(st):
                state["i"] = (state["i"] + 1) % nout
                rc = lib.ap_probe_write(outs[state["i"]].data_ptr(), 2 * N * K, 7, 32, st)
                if rc != 0:
                    raise RuntimeError(_capi.strerror(rc))

            # a kernel that only WRITES the fp16 output (no planes, no lookups): the store floor of this box
            us_write = time_graph(write_only, 12)
            for b in BITS:
                us = time_graph(lambda st: deq(st, b), 12)
                by = synth.dequant_bytes(N, K, b)
                us_read = next((r["stream_only_us"] for r in table if (r["N"], r["K"], r["w_bits"]) == (N, K, b)), None)
                dequant_table.append({"N": N, "K": K, "w_bits": b, "us": round(us, 2),
                                      "GBps": round(by / us / 1e3, 1), "frac": round(by / us / 1e3 / HBM_PEAK_GBS, 4),
                                      "write_only_us": round(us_write, 2), "read_only_us": us_read,
                                      "frac_of_write_floor": round(us_write / us, 4)})
            del outs
        # batches: matmul_kbit for M <= 8 (MFMA kernel from 5 rows on), fused gemm_kbit beyond (K-split kernel at 16 and
        # 32 rows, tiled kernel at 128 and 256), there beside dequant_kbit + library GEMM on the same weight sets
        import any_precision_ext as ext
        for (N, K) in pools:
            for b in (3, 4, 8):
                row = {"N": N, "K": K, "w_bits": b}
                for M in batches:
                    fn = lib.ap_matmul_kbit if M <= 8 else lib.ap_gemm_kbit
                    row[f"us_M{M}"] = round(time_graph(lambda st: launch(N, K, b, st, M, fn), 24 if M <= 32 else 8), 2)
                    if M >= 128:
                        P = pools[(N, K)]

                        def pair(st):
                            j = cursor[(N, K)] = (cursor[(N, K)] + 1) % P.sets
                            torch.matmul(xb[(M, K)], ext.dequant_kbit(P.qweight[j], P.luts[b][j], b).T, out=P.out[:M])

                        with torch.cuda.stream(side):   # the library GEMM sets itself up on first use: not inside a capture
                            pair(side.cuda_stream)
                            side.synchronize()
                        row[f"dequant_matmul_us_M{M}"] = round(time_graph(pair, 8), 2)
                batch_table.append(row)

    # ---- compact figures for the other configurations (each has a --workload of its own with the full
    # tables): the Llama-3-8B shapes at M = 1, 2, 4, 8 and dequant_kbit over a whole Llama-2-7B layer set
    llama3, dequant_layer = None, None
    if not args.only_step and not args.no_extras and not args.eager:
        llama3 = []
        for (N, K) in ((1024, 4096), (14336, 4096), (4096, 14336)):
            sets = max(3, int(0.6e9 / (3 * N * K / 8)) + 1)
            P3 = WeightPool(torch, N, K, sets, gen, bits=(3, 8))
            cur = {"j": 0}
            for b in (3, 8):
                row = {"N": N, "K": K, "w_bits": b}
                for M in (1, 2, 4, 8):
                    x3 = xb[(M, 4096)] if K == 4096 else torch.randn((M, K), device="cuda", generator=gen).to(torch.float16)
                    out3 = torch.empty((M, N), dtype=torch.float16, device="cuda")

                    def call3(st):
                        cur["j"] = (cur["j"] + 1) % P3.sets
                        rc = lib.ap_matmul_kbit(x3.data_ptr(), P3.qweight[cur["j"]].data_ptr(), P3.luts[b][cur["j"]].data_ptr(),
                                                out3.data_ptr(), M, N, K, b, st)
                        if rc != 0:
                            raise RuntimeError(_capi.strerror(rc))
                    us = time_graph(call3, min(24, 2 * sets))
                    row[f"us_M{M}"] = round(us, 2)
                    row[f"frac_M{M}"] = round(synth.gemv_bytes(N, K, b, M) / us / 1e3 / HBM_PEAK_GBS, 4)
                llama3.append(row)
            del P3
            torch.cuda.empty_cache()
        # dequant_kbit of the 7 linears of a layer, outputs rotating over >= 512 MB per shape: bytes read + written
        # over time, per w_bits -- 32 such layer sets are the full model (configuration 4)
        outs = {(N, K): [torch.empty((N, K), dtype=torch.float16, device="cuda")
                         for _ in range(max(2, int(512e6 / (2 * N * K)) + 1))] for (N, K) in pools}
        oi = {k: 0 for k in pools}

        def dequant_layer_set(st, b):
            for _, N, K in shapes:
                P = pools[(N, K)]
                j = cursor[(N, K)] = (cursor[(N, K)] + 1) % P.sets
                oi[(N, K)] = (oi[(N, K)] + 1) % len(outs[(N, K)])
                rc = lib.ap_dequant_kbit(P.qweight[j].data_ptr(), P.luts[b][j].data_ptr(), outs[(N, K)][oi[(N, K)]].data_ptr(),
                                         N, K, b, st)
                if rc != 0:
                    raise RuntimeError(_capi.strerror(rc))
        def dequant_layer_one_launch(st, b):
            """The same seven linears through ap_dequant_kbit_group: one launch per layer set."""
            qs, ts, os_ = [], [], []
            for _, N, K in shapes:
                P = pools[(N, K)]
                j = cursor[(N, K)] = (cursor[(N, K)] + 1) % P.sets
                oi[(N, K)] = (oi[(N, K)] + 1) % len(outs[(N, K)])
                qs.append(P.qweight[j].data_ptr())
                ts.append(P.luts[b][j].data_ptr())
                os_.append(outs[(N, K)][oi[(N, K)]].data_ptr())
            rc = _capi.dequant_group(qs, ts, os_, [N for _, N, _ in shapes], [K for _, _, K in shapes], b, st)
            if rc != 0:
                raise RuntimeError(_capi.strerror(rc))
        dequant_layer = []
        for b in BITS:
            us1 = time_graph(lambda st: dequant_layer_set(st, b), 4)
            us = time_graph(lambda st: dequant_layer_one_launch(st, b), 4)
            by = sum(synth.dequant_bytes(N, K, b) for _, N, K in shapes)
            dequant_layer.append({"w_bits": b, "us_per_layer_set": round(us, 1), "GBps": round(by / us / 1e3, 1),
                                  "frac": round(by / us / 1e3 / HBM_PEAK_GBS, 4),
                                  "full_model_ms": round(32 * us / 1e3, 3),
                                  "launches": "one ap_dequant_kbit_group launch per layer set (7 linears)",
                                  "one_launch_per_linear": {"us_per_layer_set": round(us1, 1), "GBps": round(by / us1 / 1e3, 1),
                                                            "frac": round(by / us1 / 1e3 / HBM_PEAK_GBS, 4)}})
        del outs
        torch.cuda.empty_cache()

    # ---- what this box gives a trivial kernel, in this run: a plain device copy (read 512 MiB + write
    # 512 MiB per launch) and an elementwise op on one element (the fixed cost of a graph node)
    machine = None
    if not args.only_step and not args.eager:
        src = torch.empty(128 << 20, dtype=torch.int32, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        us_copy = time_graph(lambda st: dst.copy_(src), 4)
        one = torch.zeros(1, device="cuda")
        us_node = time_graph(lambda st: one.add_(1.0), 200)
        us_empty = time_graph(lambda st: lib.ap_probe_empty(sink.data_ptr(), st), 200)
        # the GEMV itself with nothing to stream: 64 rows of 4096 elements (launch + first loads + table
        # staging + lookups of one word per lane + reduction + store), the fixed cost every launch carries
        P0 = pools[(4096, 4096)]
        fixed = {}
        for b in (3, 8):
            fixed[f"w{b}"] = round(time_graph(
                lambda st: lib.ap_matmul_kbit(xb[(1, 4096)].data_ptr(), P0.qweight[0].data_ptr(), P0.luts[b][0].data_ptr(),
                                              P0.out.data_ptr(), 1, 64, 4096, b, st), 100), 3)
        machine = {"copy_GBps": round(2 * src.numel() * 4 / us_copy / 1e3, 1), "copy_bytes": 2 * src.numel() * 4,
                   "graph_node_us": round(us_node, 3), "empty_kernel_us": round(us_empty, 3),
                   "gemv_64_rows_us": fixed,
                   "note": "torch copy of 512 MiB (read + write), a 1-element add, an empty kernel and the GEMV on 64 "
                           "rows (whose planes are not 64 rows of a real layer but the first rows of one: same "
                           "launch, nothing to stream), all as HIP-graph nodes"}
        if table:
            read_ms = sum(r["stream_only_us"] * r["count_in_step"] for r in table) / 1e3
            machine["stream_only_step_ms"] = round(read_ms, 5)
            machine["stream_only_GBps"] = round(step_bytes / read_ms / 1e6, 1)
            machine["value_over_stream_only"] = round(read_ms / ms_per_step, 4)
        del src, dst

    # what any-precision sells: a 3-bit launch should cost what its bytes cost.  Per shape: time at 3 bits over time at
    # 8 bits, next to the ratio of the algorithmic bytes (0.34-0.36)
    low_bits = None
    if table:
        low_bits = []
        for (N, K) in uniq:
            r3 = next(r for r in table if (r["N"], r["K"], r["w_bits"]) == (N, K, 3))
            r8 = next(r for r in table if (r["N"], r["K"], r["w_bits"]) == (N, K, 8))
            low_bits.append({"N": N, "K": K, "t3_over_t8": round(r3["us"] / r8["us"], 3),
                             "bytes3_over_bytes8": round(r3["bytes"] / r8["bytes"], 3)})

    roofline = None
    if table:
        dom = max(table, key=lambda r: r["us"] * r["count_in_step"])
        # HBM bytes per launch measured with rocprofv3 counters in separate runs (profiles/), if recorded
        traffic = None
        tfile = os.path.join(ROOT, "profiles", "gemv_kbit_hbm_traffic.json")
        if os.path.exists(tfile):
            with open(tfile) as f:
                traffic = json.load(f)["bytes"].get(f"{dom['N']}x{dom['K']}:{dom['w_bits']}")
        roofline = {"bound": "hbm", "achieved": dom["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": dom["frac"], "traffic": traffic,
                    "kernel": (f"gemv_kbit_kernel<{dom['w_bits']},1,{dom['geometry']['wpl']},*>" if dom["kernel"] == "dot"
                               else f"{dom['kernel']} kernel, w_bits {dom['w_bits']}") + f" {dom['N']}x{dom['K']}",
                    "stream_only_us": dom["stream_only_us"], "frac_of_stream_ceiling": dom["frac_of_stream_ceiling"],
                    "us_per_launch": dom["us"], "algorithmic_bytes_per_launch": dom["bytes"]}

    # ---- CPU baseline: the oracle's host-speed GEMV (unpack + gather + dot), and the reference semantics
    # written with PyTorch CPU ops, both timed on this box's host cores
    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(torch, synth, shapes)

    # ---- the model-level figure of the same path: batch-1 decode of the Llama-2-7B-shaped model (3 and 8 bits)
    decode = prefill = None
    sets_per_shape = {f"{N}x{K}": P.sets for (N, K), P in pools.items()}
    if not args.only_step and not args.no_extras and not args.eager:
        pools.clear()               # the weight pools are no longer needed: make room for the model
        torch.cuda.empty_cache()
        decode = decode_summary(torch)
        prefill = {"workload": PREFILL_WORKLOAD, "per_w_bits": prefill_rows(torch, synth, reps=3)}

    if machine:
        # how much of a step is the fixed cost of its 42 dependent launches, and the rate of the rest
        floor_ms = len(BITS) * len(shapes) * machine["graph_node_us"] / 1e3
        machine["step_launch_floor_ms"] = round(floor_ms, 4)
        if ms_per_step > floor_ms:
            machine["GBps_beyond_launch_floor"] = round(step_bytes / (ms_per_step - floor_ms) / 1e6, 1)
    result = {
        "metric": "bitplane GEMV effective HBM GB/s, Llama-2-7B layer set, w_bits 3-8, batch 1",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp16 tables/activations, u32 bitplanes, fp32 accumulate", "data": "synthetic",
        "config": {"workload": "Llama-2-7B decoder-layer linear set (q,k,v,o 4096x4096; gate,up 11008x4096; "
                               "down 4096x11008), batch 1, parent 8 bits, w_bits 3..8 = 42 GEMVs per step",
                   "weight_sets_per_shape": sets_per_shape,
                   "bytes_per_step": step_bytes,
                   "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4)},
        "roofline": roofline, "cpu_baseline": cpu, "grouped_launches": grouped, "machine_reference": machine,
        "layers": table,
        "dequant_kbit": dequant_table, "batch_us": batch_table,
        "llama3_8b_batches": llama3, "dequant_layer_set": dequant_layer, "llama2_7b_decode": decode,
        "llama2_7b_prefill": prefill, "low_bit_time_ratio": low_bits,
    }
    if args.table and table:
        with open(args.table, "w") as f:
            f.write("GEMV batch 1 (matmul_kbit)\n\n")
            f.write("| N x K | w_bits | us/launch | GB/s | % of 8 TB/s | us, planes cache-resident |\n|---|---|---|---|---|---|\n")
            for r in table:
                f.write(f"| {r['N']}x{r['K']} | {r['w_bits']} | {r['us']:.2f} | {r['GBps']:.0f} | {100 * r['frac']:.1f} | "
                        f"{r['us_cache_resident']:.2f} |\n")
            if dequant_table:
                f.write("\ndequant_kbit (read planes + table, write fp16)\n\n")
                f.write("| N x K | w_bits | us/launch | GB/s | % of 8 TB/s |\n|---|---|---|---|---|\n")
                for r in dequant_table:
                    f.write(f"| {r['N']}x{r['K']} | {r['w_bits']} | {r['us']:.1f} | {r['GBps']:.0f} | {100 * r['frac']:.1f} |\n")
            if batch_table:
                f.write("\nus per launch by batch (M <= 8: matmul_kbit; 16 and more: gemm_kbit)\n\n")
                f.write("| N x K | w_bits | " + " | ".join(f"M={M}" for M in batches) + " |\n|---|---|" + "---|" * len(batches) + "\n")
                for r in batch_table:
                    f.write(f"| {r['N']}x{r['K']} | {r['w_bits']} | " + " | ".join(f"{r[f'us_M{M}']:.1f}" for M in batches) + " |\n")
    print(json.dumps(result))


def _cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(torch, synth, shapes):
    """Two CPU legs, about 10 s together.  (1) `value`: the C oracle's host-speed GEMV (unpack + gather + fp32
    dot, OpenMP over rows) on two shapes x two bit-widths.  (2) `torch_reference_semantics`: the reference's
    semantics written with PyTorch CPU ops on 4096 x 4096 at batch 1 -- bitplane unpack (shifts and masks on
    the int32 tensor), table gather (any_precision/evaluate/eval.py:104-105), fp32 matmul
    (any_precision/modules/AnyPrecisionLinear.py:60-62) -- for every w_bits 3..8: one warm-up, five timed
    runs, median; end to end and the matmul alone on the dequantised weight."""
    import numpy as np
    import oracle
    oracle.build()
    rng = np.random.default_rng(0)
    t_cpu, b_cpu = 0.0, 0
    for _, N, K in [shapes[0], shapes[4]]:
        qw = rng.integers(-2**31, 2**31 - 1, size=(8, N, K // 32), dtype=np.int64).astype(np.int32)
        x = rng.normal(0, 1, size=(1, K)).astype(np.float16)
        for b in (3, 8):
            lut = np.sort(rng.normal(0, 0.02, size=(N, 1 << b)), axis=1).astype(np.float16)
            oracle.matmul_kbit_fast(x, qw, lut, b)                  # warm
            reps, t0 = 0, time.perf_counter()
            while reps < 3 or time.perf_counter() - t0 < 1.0:       # about 1 s per case
                oracle.matmul_kbit_fast(x, qw, lut, b)
                reps += 1
            t_cpu += (time.perf_counter() - t0) / reps
            b_cpu += synth.gemv_bytes(N, K, b, 1)
    cpu = {"value": round(b_cpu / t_cpu / 1e9, 3), "unit": "GB/s", "cores": oracle.num_threads(), "kind": "port",
           "sample": "C oracle GEMV (unpack+gather+fp32 dot, OpenMP over rows): 4096x4096 and 11008x4096 at w_bits "
                     "3 and 8, batch 1, each repeated for about 1 s (mean)"}

    N = K = 4096
    torch.set_num_threads(os.cpu_count() or 1)
    qw_t = torch.from_numpy(rng.integers(-2**31, 2**31 - 1, size=(8, N, K // 32), dtype=np.int64).astype(np.int32))
    x_t = torch.from_numpy(rng.normal(0, 1, size=(1, K)).astype(np.float32))
    shifts = torch.arange(7, -1, -1, dtype=torch.uint8)

    def torch_unpack(b):
        by = qw_t[:b].contiguous().view(torch.uint8).view(b, N, K // 1024, 32, 4).flip(-1)        # [p,n,c,t,j]
        bits = (by.unsqueeze(-1) >> shifts) & 1                                                   # [p,n,c,t,j,e]
        bits = bits.permute(0, 1, 2, 4, 3, 5).reshape(b, N, K)
        w = (1 << torch.arange(b - 1, -1, -1, dtype=torch.int64)).view(b, 1, 1)
        return (bits.to(torch.int64) * w).sum(0)

    per_bits = []
    for b in BITS:
        lut_t = torch.from_numpy(np.sort(rng.normal(0, 0.02, size=(N, 1 << b)), axis=1).astype(np.float32))
        e2e, mm = [], []
        for rep in range(6):                                        # the first run is the warm-up
            t0 = time.perf_counter()
            wdq = torch.gather(lut_t, 1, torch_unpack(b))
            y = x_t @ wdq.T
            t1 = time.perf_counter()
            y = x_t @ wdq.T
            t2 = time.perf_counter()
            if rep:
                e2e.append(t1 - t0)
                mm.append(t2 - t1)
        e2e.sort()
        mm.sort()
        by_b = synth.gemv_bytes(N, K, b, 1)
        per_bits.append({"w_bits": b, "ms_end_to_end": round(e2e[len(e2e) // 2] * 1e3, 2),
                         "ms_matmul_only": round(mm[len(mm) // 2] * 1e3, 3),
                         "GBps_end_to_end": round(by_b / e2e[len(e2e) // 2] / 1e9, 4)})
    cpu["torch_reference_semantics"] = {
        "per_w_bits": per_bits, "os_cpu_count": os.cpu_count(), "torch_threads": torch.get_num_threads(),
        "cpu_model": _cpu_model(),
        "sample": "torch CPU ops, 4096x4096, batch 1, every w_bits 3..8: unpack + gather + fp32 matmul end to end, "
                  "and the matmul alone on the dequantised fp32 weight; one warm-up, median of five"}
    return cpu


def _graph_us(torch, side, enqueue, reps):
    """us per call of `enqueue(stream)`: `reps` calls in one HIP graph, best of three timed replays."""
    with torch.cuda.stream(side):
        enqueue(side.cuda_stream)
        side.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            for _ in range(reps):
                enqueue(torch.cuda.current_stream().cuda_stream)
        g.replay()
        side.synchronize()
        best = float("inf")
        for _ in range(3):
            a0, a1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a0.record(side)
            g.replay()
            a1.record(side)
            side.synchronize()
            best = min(best, a0.elapsed_time(a1) * 1e3 / reps)
    return best


def batch_sweep(args, torch, _capi, synth):
    """matmul_kbit on the Llama-3-8B linear shapes at M = 1, 2, 4, 8, every w_bits, cold planes."""
    lib = _capi.lib
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0)
    side = torch.cuda.Stream()
    rows = []
    for N, K in sorted({(N, K) for _, N, K in synth.LLAMA3_8B_LAYER}):
        sets = int(args.pool_gb * 1e9 / (3 * N * K / 8)) + 1
        P = WeightPool(torch, N, K, sets, gen)
        cur = {"j": 0}
        for M in (1, 2, 4, 8):
            x = torch.randn((M, K), device="cuda", generator=gen).to(torch.float16)
            for b in BITS:
                def call(st):
                    cur["j"] = (cur["j"] + 1) % P.sets
                    rc = lib.ap_matmul_kbit(x.data_ptr(), P.qweight[cur["j"]].data_ptr(), P.luts[b][cur["j"]].data_ptr(),
                                            P.out.data_ptr(), M, N, K, b, st)
                    if rc != 0:
                        raise RuntimeError(_capi.strerror(rc))
                us = _graph_us(torch, side, call, min(args.kernel_reps, P.sets))
                by = synth.gemv_bytes(N, K, b, M)
                rows.append({"N": N, "K": K, "M": M, "w_bits": b, "us": round(us, 2), "GBps": round(by / us / 1e3, 1),
                             "frac": round(by / us / 1e3 / HBM_PEAK_GBS, 4)})
        del P
        torch.cuda.empty_cache()
    if args.table:
        with open(args.table, "w") as f:
            f.write("matmul_kbit, Llama-3-8B linear shapes: us per launch (GB/s of algorithmic bytes)\n\n")
            f.write("| N x K | M | " + " | ".join(f"b={b}" for b in BITS) + " |\n|---|---|" + "---|" * len(BITS) + "\n")
            for (N, K, M) in sorted({(r["N"], r["K"], r["M"]) for r in rows}):
                cells = [next(r for r in rows if (r["N"], r["K"], r["M"], r["w_bits"]) == (N, K, M, b)) for b in BITS]
                f.write(f"| {N}x{K} | {M} | " + " | ".join(f"{c['us']:.1f} ({c['GBps']:.0f})" for c in cells) + " |\n")
    # one figure for the sweep: bytes over time of one pass over a layer (7 linears) at every M and w_bits
    tot_b = tot_t = 0.0
    for _, N, K in synth.LLAMA3_8B_LAYER:
        for r in rows:
            if (r["N"], r["K"]) == (N, K):
                tot_b += synth.gemv_bytes(N, K, r["w_bits"], r["M"])
                tot_t += r["us"]
    print(json.dumps({
        "metric": "bitplane GEMV effective HBM GB/s, Llama-3-8B layer set, w_bits 3-8, batches 1,2,4,8",
        "value": round(tot_b / tot_t / 1e3, 1), "unit": "GB/s", "n_gpus": 1, "higher_is_better": True,
        "vs_baseline": None, "dtype": "fp16 tables/activations, u32 bitplanes, fp32 accumulate", "data": "synthetic",
        "config": {"workload": "Llama-3-8B decoder-layer linear set (q,o 4096x4096; k,v 1024x4096; gate,up 14336x4096; "
                               "down 4096x14336), M in 1,2,4,8, parent 8 bits, w_bits 3..8; per-kernel graphs of "
                               f"{args.kernel_reps} launches over cold weight sets"},
        "kernels": rows}))


def gemv_kernel_variants(args, torch, _capi, synth):
    """Batch-1 GEMV with each of the four dot-product kernels forced in turn, cold weight sets: us per launch
    and fraction of the HBM peak per (shape, w_bits, kernel), beside a kernel that only reads the same bytes.
    With --eager nothing is timed in a graph: every launch goes out on its own (kernel names and counters
    of a rocprofv3 run then belong to single launches); the printed times then include host launch cost."""
    lib = _capi.lib
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0)
    side = torch.cuda.Stream()
    sink = torch.zeros(16, dtype=torch.int32, device="cuda")
    variants = (("dot", {}), ("fine", {"gemv_fine": 2}), ("stream", {"gemv_stream": 2}))
    off = {"gemv_fine": 0, "gemv_stream": 0}
    bits = (3, 5, 8)
    rows = []
    for N, K in ((4096, 4096), (11008, 4096), (4096, 11008), (28672, 8192)):
        sets = max(3, int(args.pool_gb * 1e9 / (3 * N * K / 8)) + 1)
        if args.eager:
            sets = min(sets, 12)
        P = WeightPool(torch, N, K, sets, gen, bits=bits)
        x = torch.randn((1, K), device="cuda", generator=gen).to(torch.float16)
        cur = {"j": 0}
        for b in bits:
            by = synth.gemv_bytes(N, K, b, 1)
            reps = min(P.sets, max(8, int(1e9 / by) + 1))

            def read_only(st):
                cur["j"] = (cur["j"] + 1) % P.sets
                rc = lib.ap_probe_stream(P.qweight[cur["j"]].data_ptr(), b * N * K // 8, P.luts[b][cur["j"]].data_ptr(),
                                         N * (2 << b), sink.data_ptr(), 32, st)
                if rc != 0:
                    raise RuntimeError(_capi.strerror(rc))

            def gemv(st):
                cur["j"] = (cur["j"] + 1) % P.sets
                rc = lib.ap_matmul_kbit(x.data_ptr(), P.qweight[cur["j"]].data_ptr(), P.luts[b][cur["j"]].data_ptr(),
                                        P.out.data_ptr(), 1, N, K, b, st)
                if rc != 0:
                    raise RuntimeError(_capi.strerror(rc))

            def timed(fn):
                if not args.eager:
                    return _graph_us(torch, side, fn, reps)
                with torch.cuda.stream(side):
                    fn(side.cuda_stream)
                    side.synchronize()
                    t0 = time.perf_counter()
                    for _ in range(reps):
                        fn(side.cuda_stream)
                    side.synchronize()
                return (time.perf_counter() - t0) * 1e6 / reps

            row = {"N": N, "K": K, "w_bits": b, "bytes": by, "stream_only_us": round(timed(read_only), 2)}
            for name, knobs in variants:
                with _capi.tuning(**{**off, **knobs}):
                    if _capi.matmul_route(1, N, K, b) != name:
                        continue
                    us = timed(gemv)
                row[f"{name}_us"] = round(us, 2)
                row[f"{name}_frac"] = round(by / us / 1e3 / HBM_PEAK_GBS, 4)
            row["default_kernel"] = _capi.matmul_route(1, N, K, b)
            rows.append(row)
        del P
        torch.cuda.empty_cache()
    print(json.dumps({
        "metric": "bitplane GEMV us per launch by kernel variant, batch 1", "unit": "us", "n_gpus": 1,
        "higher_is_better": False, "vs_baseline": None, "data": "synthetic",
        "dtype": "fp16 tables/activations, u32 bitplanes, fp32 accumulate",
        "config": {"workload": "4096x4096, 11008x4096, 4096x11008, 28672x8192 at w_bits 3, 5, 8, batch 1; each of the "
                               "dot / fine / stream kernels forced through ap_set_tuning; cold weight sets; "
                               + ("eager launches" if args.eager else "HIP graphs")},
        "value": None, "kernels": rows}))


AUDIT_SETS = {     # linears of a decoder layer that share their input: ((rows of each member), elements per row)
    "7b": (((4096, 4096, 4096), 4096), ((11008, 11008), 4096)),
    "8b": (((4096, 1024, 1024), 4096), ((14336, 14336), 4096)),
    "13b": (((5120, 5120, 5120), 5120), ((13824, 13824), 5120)),
    "70b": (((8192, 1024, 1024), 8192), ((28672, 28672), 8192)),
}
AUDIT_SHAPES = {   # (rows, elements per row) of the distinct linears of a decoder layer
    "7b": ((4096, 4096), (11008, 4096), (4096, 11008)),
    "8b": ((4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336)),
    "13b": ((5120, 5120), (13824, 5120), (5120, 13824)),
    "70b": ((8192, 8192), (1024, 8192), (28672, 8192), (8192, 28672)),
}


def routing_audit(args, torch, _capi, synth):
    """ap_matmul_kbit's own choice of kernel and launch geometry against every alternative the tuning knobs can
    force, on cold weight sets: per (shape, activation rows, w_bits) the default's time, the fastest candidate's,
    and which it was.  The routing rules are thresholds fitted to measurements; this is the measurement."""
    lib = _capi.lib
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0)
    side = torch.cuda.Stream()
    bits = (3, 4, 5, 8)
    dot = {"gemv_stream": 0, "gemv_fine": 0, "matmul_mfma4": 0}
    few = [("dot_1row", dict(dot, gemv_rows=1)), ("dot_2rows", dict(dot, gemv_rows=2)), ("dot_4rows", dict(dot, gemv_rows=4)),
           ("stream", {"gemv_stream": 2}), ("fine", {"gemv_fine": 2}), ("mfma4", {"matmul_mfma4": 2, "gemv_stream": 0, "gemv_fine": 0})]
    many = [("dot", dict(dot, matmul_mfma_from=9)), ("mfma16", {"matmul_mfma4": 0, "matmul_mfma_from": 4}),
            ("mfma16_2blocks", {"matmul_mfma4": 0, "matmul_mfma_from": 4, "gemm_rb2": 2, "gemm_walk": 0}),
            ("mfma4", {"matmul_mfma4": 2})]
    shapes = []
    for m in args.audit_models.split(","):
        for sh in AUDIT_SHAPES[m.strip()]:
            if sh not in shapes:
                shapes.append(sh)
    Ms = [int(v) for v in args.audit_rows.split(",")]
    cases, losses = [], []
    for N, K in shapes:
        sets = max(4, int(args.pool_gb * 1e9 / (N * K)) + 1)
        P = WeightPool(torch, N, K, sets, gen, bits=bits)
        cur = {"j": 0}
        for b in bits:
            for M in Ms:
                x = torch.randn((M, K), device="cuda", generator=gen).to(torch.float16)

                def gemv(st):
                    cur["j"] = (cur["j"] + 1) % P.sets
                    rc = lib.ap_matmul_kbit(x.data_ptr(), P.qweight[cur["j"]].data_ptr(), P.luts[b][cur["j"]].data_ptr(),
                                            P.out.data_ptr(), M, N, K, b, st)
                    if rc != 0:
                        raise RuntimeError(_capi.strerror(rc))

                reps = min(P.sets, 24)
                us = {"default": _graph_us(torch, side, gemv, reps)}
                for name, knobs in (few if M <= 4 else many):
                    if name == "mfma4" and M < 2:
                        continue
                    with _capi.tuning(**knobs):
                        if _capi.matmul_route(M, N, K, b) != name.split("_")[0]:
                            continue                      # the kernel does not serve this shape
                        if name.startswith("dot_") and _capi.matmul_geometry(M, N, K, b)["rows"] != int(name[4]):
                            continue                      # nor with this many rows per workgroup
                        us[name] = _graph_us(torch, side, gemv, reps)
                us["default"] = min(us["default"], _graph_us(torch, side, gemv, reps))   # measured first and last
                best = min((k for k in us if k != "default"), key=lambda k: us[k], default="default")
                case = {"N": N, "K": K, "w_bits": b, "M": M, "route": _capi.matmul_route(M, N, K, b),
                        "default_us": round(us["default"], 2), "best": best, "best_us": round(us[best], 2)}
                cases.append(case)
                if us["default"] > 1.05 * us[best]:
                    losses.append(dict(case, excess=round(us["default"] / us[best] - 1, 3)))
        # the fused GEMM of ap_gemm_kbit on the same weights: one or two row blocks per workgroup, the row-walking kernel,
        # the tiled kernel
        for b in bits:
            for M in ((16, 32, 48, 64, 96, 128) if args.audit_gemm else ()):
                x = torch.randn((M, K), device="cuda", generator=gen).to(torch.float16)
                big_out = torch.empty((M, N), dtype=torch.float16, device="cuda")

                def gemm(st):
                    cur["j"] = (cur["j"] + 1) % P.sets
                    rc = lib.ap_gemm_kbit(x.data_ptr(), P.qweight[cur["j"]].data_ptr(), P.luts[b][cur["j"]].data_ptr(),
                                          big_out.data_ptr(), M, N, K, b, st)
                    if rc != 0:
                        raise RuntimeError(_capi.strerror(rc))

                reps = min(P.sets, 16)
                us = {"default": _graph_us(torch, side, gemm, reps)}
                for name, knobs in (("one_block", {"gemm_tiled": 0, "gemm_walk": 0, "gemm_rb2": 0}),
                                    ("two_blocks", {"gemm_tiled": 0, "gemm_walk": 0, "gemm_rb2": 2}),
                                    ("walking", {"gemm_tiled": 0, "gemm_walk": 2}), ("tiled", {"gemm_tiled": 2})):
                    if name == "tiled" and K % 128:
                        continue
                    with _capi.tuning(**knobs):
                        us[name] = _graph_us(torch, side, gemm, reps)
                us["default"] = min(us["default"], _graph_us(torch, side, gemm, reps))
                best = min((k for k in us if k != "default"), key=lambda k: us[k])
                case = {"entry": "ap_gemm_kbit", "N": N, "K": K, "w_bits": b, "M": M, "default_us": round(us["default"], 2),
                        "best": best, "best_us": round(us[best], 2)}
                cases.append(case)
                if us["default"] > 1.05 * us[best]:
                    losses.append(dict(case, excess=round(us["default"] / us[best] - 1, 3)))
        del P
        torch.cuda.empty_cache()
    # sets of linears that share their input (q/k/v, gate/up) through ap_matmul_kbit_group: the default against one
    # dot-product launch with 2 or 4 rows per workgroup and against a launch per member
    import ctypes
    for m in (args.audit_models.split(",") if args.audit_sets else ()):
        for Ns, K in AUDIT_SETS[m.strip()]:
            pools = [WeightPool(torch, N, K, max(3, int(args.pool_gb * 0.5e9 / (sum(Ns) * K)) + 1), gen, bits=bits) for N in Ns]
            n = len(Ns)
            arr, rows_arr = ctypes.c_void_p * n, (ctypes.c_int * n)(*Ns)
            cur = {"j": 0}
            for b in bits:
                for M in Ms:
                    x = torch.randn((M, K), device="cuda", generator=gen).to(torch.float16)
                    outs = arr(*[P.out.data_ptr() for P in pools])

                    def group(st):
                        cur["j"] = (cur["j"] + 1) % pools[0].sets
                        j = cur["j"]
                        rc = lib.ap_matmul_kbit_group(x.data_ptr(), n, arr(*[P.qweight[j].data_ptr() for P in pools]),
                                                      arr(*[P.luts[b][j].data_ptr() for P in pools]), outs, rows_arr, M, K, b, st)
                        if rc != 0:
                            raise RuntimeError(_capi.strerror(rc))

                    def per_member(st):
                        cur["j"] = (cur["j"] + 1) % pools[0].sets
                        for P in pools:
                            rc = lib.ap_matmul_kbit(x.data_ptr(), P.qweight[cur["j"]].data_ptr(), P.luts[b][cur["j"]].data_ptr(),
                                                    P.out.data_ptr(), M, P.N, K, b, st)
                            if rc != 0:
                                raise RuntimeError(_capi.strerror(rc))

                    reps = min(pools[0].sets, 12)
                    us = {"default": _graph_us(torch, side, group, reps), "launch_per_member": _graph_us(torch, side, per_member, reps)}
                    forced = dict(dot, matmul_mfma_from=9)
                    for name, knobs in (("one_launch_2rows", dict(forced, gemv_rows=2)), ("one_launch_4rows", dict(forced, gemv_rows=4))):
                        if name == "one_launch_4rows" and M > 4:
                            continue
                        with _capi.tuning(**knobs):
                            routes, per_wg = _capi.matmul_group_route(M, list(Ns), K, b)
                            if set(routes) == {"dot"} and per_wg == int(name[11]):
                                us[name] = _graph_us(torch, side, group, reps)
                    us["default"] = min(us["default"], _graph_us(torch, side, group, reps))
                    best = min((k for k in us if k != "default"), key=lambda k: us[k])
                    case = {"entry": "ap_matmul_kbit_group", "N": list(Ns), "K": K, "w_bits": b, "M": M,
                            "route": _capi.matmul_group_route(M, list(Ns), K, b)[0][0], "default_us": round(us["default"], 2),
                            "best": best, "best_us": round(us[best], 2)}
                    cases.append(case)
                    if us["default"] > 1.05 * us[best]:
                        losses.append(dict(case, excess=round(us["default"] / us[best] - 1, 3)))
            # the same sets through ap_gemm_kbit_group at 16, 32, 48 and 128 rows: the default against one launch of the
            # tiled kernel and against a launch per member
            for b in (bits if args.audit_gemm else ()):
                for M in (16, 32, 48, 128):
                    x = torch.randn((M, K), device="cuda", generator=gen).to(torch.float16)
                    big = [torch.empty((M, N), dtype=torch.float16, device="cuda") for N in Ns]
                    outs = arr(*[o.data_ptr() for o in big])

                    def gemm_set(st):
                        cur["j"] = (cur["j"] + 1) % pools[0].sets
                        j = cur["j"]
                        rc = lib.ap_gemm_kbit_group(x.data_ptr(), n, arr(*[P.qweight[j].data_ptr() for P in pools]),
                                                    arr(*[P.luts[b][j].data_ptr() for P in pools]), outs, rows_arr, None, M, K, b, st)
                        if rc != 0:
                            raise RuntimeError(_capi.strerror(rc))

                    def gemm_members(st):
                        cur["j"] = (cur["j"] + 1) % pools[0].sets
                        for P, o in zip(pools, big):
                            rc = lib.ap_gemm_kbit(x.data_ptr(), P.qweight[cur["j"]].data_ptr(), P.luts[b][cur["j"]].data_ptr(),
                                                  o.data_ptr(), M, P.N, K, b, st)
                            if rc != 0:
                                raise RuntimeError(_capi.strerror(rc))

                    reps = min(pools[0].sets, 8)
                    us = {"default": _graph_us(torch, side, gemm_set, reps), "launch_per_member": _graph_us(torch, side, gemm_members, reps)}
                    if K % 128 == 0:
                        with _capi.tuning(gemm_tiled=2):
                            us["one_tiled_launch"] = _graph_us(torch, side, gemm_set, reps)
                    us["default"] = min(us["default"], _graph_us(torch, side, gemm_set, reps))
                    best = min((k for k in us if k != "default"), key=lambda k: us[k])
                    case = {"entry": "ap_gemm_kbit_group", "N": list(Ns), "K": K, "w_bits": b, "M": M,
                            "default_us": round(us["default"], 2), "best": best, "best_us": round(us[best], 2)}
                    cases.append(case)
                    if us["default"] > 1.05 * us[best]:
                        losses.append(dict(case, excess=round(us["default"] / us[best] - 1, 3)))
            del pools
            torch.cuda.empty_cache()
    within = 1 - len(losses) / len(cases)
    print(json.dumps({
        "metric": "share of (shape, rows, w_bits) cases where ap_matmul_kbit's default launch is within 5 % of the fastest forced alternative",
        "value": round(within, 4), "unit": "fraction", "n_gpus": 1, "higher_is_better": True, "vs_baseline": None,
        "data": "synthetic", "dtype": "fp16 tables/activations, u32 bitplanes, fp32 accumulate",
        "config": {"workload": f"linears of {args.audit_models} at {args.audit_rows} activation rows, w_bits 3, 4, 5, 8"
                               + (", their q/k/v and gate/up sets" + (" (also through ap_gemm_kbit_group at 16, 32, 48 and 128 rows)" if args.audit_gemm else "")
                                  if args.audit_sets else "")
                               + (", ap_gemm_kbit at 16, 32, 48, 64, 96, 128 rows" if args.audit_gemm else "")
                               + "; cold weight sets; HIP graphs; alternatives forced through ap_set_tuning"},
        "cases": len(cases), "worst_excess": max((l["excess"] for l in losses), default=0.0),
        "losses": sorted(losses, key=lambda l: -l["excess"]), "all_cases": cases}))


def profile_set(args, torch, _capi, synth):
    """Eager launches of every kernel the default routes of the Llama-2-7B layer use, `--kernel-reps` per case on
    rotating (cold) weight sets, each case exactly one kernel dispatch per launch; prints the ordered manifest of the
    cases so that the dispatches of a rocprofv3 trace or counter run can be attributed (the library's kernels appear
    in launch order; with --calibrate-copy three 256 MiB torch.add launches of known traffic come first)."""
    lib = _capi.lib
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0)
    reps = max(1, min(args.kernel_reps, 8))
    shapes = sorted({(N, K) for _, N, K in synth.LLAMA2_7B_LAYER})
    pools = {(N, K): WeightPool(torch, N, K, max(reps, 3), gen) for N, K in shapes}
    x1 = {K: torch.randn((1, K), device="cuda", generator=gen).half() for K in (4096, 11008)}
    out = torch.empty((16, 3 * 11008), dtype=torch.float16, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    manifest = []

    def case(label, launch):
        for i in range(reps):
            rc = launch(i)
            if rc not in (0, None):
                raise RuntimeError(f"{label}: {_capi.strerror(rc)}")
        torch.cuda.synchronize()
        manifest.append({"case": label, "dispatches": reps})

    if args.calibrate_copy:
        src = torch.ones(64 << 20, dtype=torch.int32, device="cuda")      # 256 MiB
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1, out=dst)      # one elementwise kernel: reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst
    for b in BITS:
        for N, K in shapes:
            P = pools[(N, K)]
            case(f"matmul_kbit {N}x{K} M=1 b={b} [{_capi.matmul_route(1, N, K, b)}]",
                 lambda i: lib.ap_matmul_kbit(x1[K].data_ptr(), P.qweight[i].data_ptr(), P.luts[b][i].data_ptr(), out.data_ptr(),
                                              1, N, K, b, st))
    for b in BITS:
        P = pools[(4096, 4096)]
        case(f"matmul_kbit_group q,k,v 3x4096x4096 M=1 b={b}",
             lambda i: _capi.matmul_group(x1[4096].data_ptr(), [P.qweight[(i + g) % P.sets].data_ptr() for g in range(3)],
                                          [P.luts[b][(i + g) % P.sets].data_ptr() for g in range(3)],
                                          [out.data_ptr() + 2 * 4096 * g for g in range(3)], [4096] * 3, 1, 4096, b, st))
        P = pools[(11008, 4096)]
        case(f"matmul_kbit_group gate,up 2x11008x4096 M=1 b={b}",
             lambda i: _capi.matmul_group(x1[4096].data_ptr(), [P.qweight[(i + g) % P.sets].data_ptr() for g in range(2)],
                                          [P.luts[b][(i + g) % P.sets].data_ptr() for g in range(2)],
                                          [out.data_ptr() + 2 * 11008 * g for g in range(2)], [11008] * 2, 1, 4096, b, st))
        case(f"matmul_kbit_swiglu gate,up 2x11008x4096 M=1 b={b}",
             lambda i: lib.ap_matmul_kbit_swiglu(x1[4096].data_ptr(), P.qweight[i].data_ptr(), P.luts[b][i].data_ptr(),
                                                 P.qweight[(i + 1) % P.sets].data_ptr(), P.luts[b][(i + 1) % P.sets].data_ptr(),
                                                 out.data_ptr(), 1, 11008, 4096, b, st))
    # dequant: per linear and the seven linears of a layer in one launch
    wout = {(N, K): torch.empty((2, N, K), dtype=torch.float16, device="cuda") for N, K in shapes}
    for b in BITS:
        for N, K in shapes:
            P = pools[(N, K)]
            case(f"dequant_kbit {N}x{K} b={b}",
                 lambda i: lib.ap_dequant_kbit(P.qweight[i].data_ptr(), P.luts[b][i].data_ptr(), wout[(N, K)][i & 1].data_ptr(), N, K, b, st))
    layer = [(N, K) for _, N, K in synth.LLAMA2_7B_LAYER]
    wlayer = [torch.empty((N, K), dtype=torch.float16, device="cuda") for N, K in layer]
    for b in (3, 8):
        case(f"dequant_kbit_group 7 linears of a layer b={b}",
             lambda i: _capi.dequant_group([pools[s].qweight[(i + g) % pools[s].sets].data_ptr() for g, s in enumerate(layer)],
                                           [pools[s].luts[b][(i + g) % pools[s].sets].data_ptr() for g, s in enumerate(layer)],
                                           [w.data_ptr() for w in wlayer], [N for N, _ in layer], [K for _, K in layer], b, st))
    del wout, wlayer
    # fused GEMM: 16 rows (K-split kernel) and 16384 rows (tiled kernel, one launch)
    x16 = torch.randn((16, 4096), device="cuda", generator=gen).half()
    xp = torch.randn((32 * 512, 4096), device="cuda", generator=gen).half()
    outp = torch.empty((32 * 512, 11008), dtype=torch.float16, device="cuda")
    for b in (3, 8):
        for N, K in ((4096, 4096), (11008, 4096)):
            P = pools[(N, K)]
            case(f"gemm_kbit {N}x{K} M=16 b={b}",
                 lambda i: lib.ap_gemm_kbit(x16.data_ptr(), P.qweight[i].data_ptr(), P.luts[b][i].data_ptr(), outp.data_ptr(),
                                            16, N, K, b, st))
            case(f"gemm_kbit {N}x{K} M=16384 b={b}",
                 lambda i: lib.ap_gemm_kbit(xp.data_ptr(), P.qweight[i].data_ptr(), P.luts[b][i].data_ptr(), outp.data_ptr(),
                                            32 * 512, N, K, b, st))
    print(json.dumps({"metric": "profile launch list (no timing)", "value": None, "unit": None, "n_gpus": 1,
                      "higher_is_better": True, "vs_baseline": None, "data": "synthetic",
                      "config": {"workload": "every kernel of the default routes of the Llama-2-7B layer, eager, "
                                             f"{reps} launches per case"},
                      "calibration_dispatches": 3 if args.calibrate_copy else 0, "manifest": manifest}))


def gemm_rows(args, torch, _capi, synth):
    """ap_gemm_kbit at 64..512 activation rows on 4096 x 4096, 11008 x 4096, 4096 x 11008 (cold weight sets, HIP graphs):
    the default launch, the K-split kernel (chunks of 128 rows beyond 128), the tiled kernel with either tile, and
    dequant_kbit + torch.matmul, which is what AnyPrecisionLinear falls back to."""
    import any_precision_ext as ext
    lib = _capi.lib
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0)
    side = torch.cuda.Stream()
    bits, Ms = (3, 4, 5, 8), (64, 128, 256, 512)
    cases = []
    for N, K in ((4096, 4096), (11008, 4096), (4096, 11008)):
        P = WeightPool(torch, N, K, max(4, int(args.pool_gb * 1e9 / (N * K)) + 1), gen, bits=bits)
        cur = {"j": 0}
        for b in bits:
            for M in Ms:
                x = torch.randn((M, K), device="cuda", generator=gen).to(torch.float16)
                out = torch.empty((M, N), dtype=torch.float16, device="cuda")

                def fused(st):
                    cur["j"] = (cur["j"] + 1) % P.sets
                    rc = lib.ap_gemm_kbit(x.data_ptr(), P.qweight[cur["j"]].data_ptr(), P.luts[b][cur["j"]].data_ptr(),
                                          out.data_ptr(), M, N, K, b, st)
                    if rc != 0:
                        raise RuntimeError(_capi.strerror(rc))

                def pair(st):
                    cur["j"] = (cur["j"] + 1) % P.sets
                    torch.matmul(x, ext.dequant_kbit(P.qweight[cur["j"]], P.luts[b][cur["j"]], b).T, out=out)

                if args.eager:
                    with _capi.tuning(gemm_tiled=2):
                        fused(torch.cuda.current_stream().cuda_stream)
                    torch.cuda.synchronize()
                    continue
                reps = min(P.sets, 12)
                us = {"default": _graph_us(torch, side, fused, reps), "dequant_matmul": _graph_us(torch, side, pair, reps)}
                for name, knobs in (("k_split", {"gemm_tiled": 0}), ("tiled_64", {"gemm_tiled": 2, "gemm_tile": 4}),
                                    ("tiled_128", {"gemm_tiled": 2, "gemm_tile": 8})):
                    with _capi.tuning(**knobs):
                        us[name] = _graph_us(torch, side, fused, reps)
                fastest = min(us[k] for k in us if k not in ("default", "dequant_matmul"))
                cases.append(dict({"N": N, "K": K, "w_bits": b, "M": M}, **{k + "_us": round(v, 1) for k, v in us.items()},
                                  default_TFLOPs=round(2.0 * M * N * K / us["default"] / 1e6, 1),
                                  default_over_fastest_fused=round(us["default"] / fastest, 3),
                                  fused_over_dequant_matmul=round(us["default"] / us["dequant_matmul"], 3)))
        del P
        torch.cuda.empty_cache()
    if args.eager:
        print(json.dumps({"metric": "one eager launch of the tiled fused GEMM per (shape, w_bits, rows)", "value": None,
                          "unit": "", "n_gpus": 1, "higher_is_better": True, "vs_baseline": None, "data": "synthetic",
                          "config": {"workload": "llama2_7b_gemm_rows --eager"}}))
        return
    wins = [c for c in cases if c["fused_over_dequant_matmul"] < 1.0]
    print(json.dumps({
        "metric": "share of (shape, w_bits, rows) cases where ap_gemm_kbit's default launch beats dequant_kbit + library GEMM",
        "value": round(len(wins) / len(cases), 4), "unit": "fraction", "n_gpus": 1, "higher_is_better": True,
        "vs_baseline": None, "data": "synthetic", "dtype": "fp16 operands, u32 bitplanes, fp32 accumulate",
        "config": {"workload": "ap_gemm_kbit on 4096x4096, 11008x4096, 4096x11008 at 64, 128, 256, 512 activation rows, "
                               "w_bits 3, 4, 5, 8; cold weight sets; HIP graphs"},
        "worst_default_over_fastest_fused": max(c["default_over_fastest_fused"] for c in cases), "cases": cases}))


def dequant_full_model(args, torch, _capi, synth):
    """dequant_kbit over every linear of a Llama-2-7B-shaped model (32 layers x 7 linears, 6.476 G weights)."""
    lib = _capi.lib
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0)
    side = torch.cuda.Stream()
    layers = 32
    linears = []   # (N, K, qweight [8,N,W], luts {b: [N, 2^b]})
    for li in range(layers):
        for _, N, K in synth.LLAMA2_7B_LAYER:
            q = torch.randint(-2**31, 2**31 - 1, (8, N, K // 32), dtype=torch.int32, device="cuda", generator=gen)
            luts = {b: torch.sort(torch.randn((N, 1 << b), device="cuda", generator=gen) * 0.02, dim=1).values
                    .to(torch.float16).contiguous() for b in BITS}
            linears.append((N, K, q, luts))
    # outputs rotate over ~1 GB of buffers per shape so that no store lands on a line still in the last-level cache
    outs = {}
    for N, K in {(N, K) for N, K, _, _ in linears}:
        outs[(N, K)] = [torch.empty((N, K), dtype=torch.float16, device="cuda") for _ in range(int(1e9 / (2 * N * K)) + 1)]
    turn = {k: 0 for k in outs}
    weights = sum(N * K for N, K, _, _ in linears)
    results = []
    for b in BITS:
        def pass_(st):
            for N, K, q, luts in linears:
                turn[(N, K)] = (turn[(N, K)] + 1) % len(outs[(N, K)])
                rc = lib.ap_dequant_kbit(q.data_ptr(), luts[b].data_ptr(), outs[(N, K)][turn[(N, K)]].data_ptr(), N, K, b, st)
                if rc != 0:
                    raise RuntimeError(_capi.strerror(rc))
        us = _graph_us(torch, side, pass_, 1)
        by = sum(synth.dequant_bytes(N, K, b) for N, K, _, _ in linears)
        results.append({"w_bits": b, "ms": round(us / 1e3, 3), "GBps": round(by / us / 1e3, 1),
                        "frac": round(by / us / 1e3 / HBM_PEAK_GBS, 4), "bytes": by})
    tot_b, tot_t = sum(r["bytes"] for r in results), sum(r["ms"] for r in results)
    print(json.dumps({
        "metric": "dequant_kbit effective HBM GB/s (read planes + table, write fp16), Llama-2-7B full model, w_bits 3-8",
        "value": round(tot_b / tot_t / 1e6, 1), "unit": "GB/s", "n_gpus": 1, "higher_is_better": True,
        "vs_baseline": None, "dtype": "fp16 tables, u32 bitplanes (table copy, bit-exact)", "data": "synthetic",
        "config": {"workload": f"dequant_kbit over 32 layers x 7 linears = {weights} weights, one HIP graph of 224 "
                               "launches per w_bits, best of three replays"},
        "per_w_bits": results}))



def _llama2_7b_config():
    from transformers import LlamaConfig
    return LlamaConfig(hidden_size=4096, intermediate_size=11008, num_hidden_layers=32, num_attention_heads=32,
                       num_key_value_heads=32, vocab_size=32000, max_position_embeddings=4096, rms_norm_eps=1e-5,
                       tie_word_embeddings=False)


def decode_summary(torch, prompt_len=128, new_tokens=256):
    """tokens/s of the graph-replayed decode step on a random-init Llama-2-7B-shaped model: 256 tokens after a
    128-token prompt at every w_bits 3..8, the loop of the reference's demo.py:59-80 (--workload llama2_7b_decode
    adds the prompt time and the other decode modes)."""
    from any_precision_amd import AnyPrecisionForCausalLM, GraphDecoder
    model = AnyPrecisionForCausalLM.from_config(_llama2_7b_config(), seed=0, device="cuda")
    dec = GraphDecoder(model, max_len=prompt_len + new_tokens + 8)
    ids = torch.randint(0, 32000, (prompt_len,), generator=torch.Generator().manual_seed(0)).cuda()
    rows = []
    for b in BITS:
        dec.prefill(ids, b)
        dec.capture(b)
        dec.decode(8, b)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        dec.decode(new_tokens - 9, b)
        torch.cuda.synchronize()
        tok_s = (new_tokens - 9) / (time.perf_counter() - t0)
        rows.append({"w_bits": b, "tokens_per_s": round(tok_s, 1), "ms_per_token": round(1e3 / tok_s, 3)})
    del dec, model
    torch.cuda.empty_cache()
    return {"workload": f"greedy decode of {new_tokens} tokens after a {prompt_len}-token prompt, batch 1, 32 layers / hidden "
                        "4096 / FFN 11008 / 32 heads / vocab 32000, random-init, decode step replayed from one HIP graph",
            "per_w_bits": rows}


def decode_tokens(args, torch, _capi, synth):
    """Batch-1 greedy decoding, random-init Llama-2-7B-shaped model: tokens/s per w_bits, the decode
    step replayed from a HIP graph; beside it the 224 GEMVs of a token alone and the eager loop."""
    from any_precision_amd import AnyPrecisionForCausalLM, GraphDecoder
    cfg = _llama2_7b_config()
    model = AnyPrecisionForCausalLM.from_config(cfg, seed=0, device="cuda")
    prompt_len, new_tokens = 128, 256
    dec = GraphDecoder(model, max_len=prompt_len + new_tokens + 8)
    dec_single = GraphDecoder(model, max_len=prompt_len + new_tokens + 8, group_launches=False)
    dec_stock = GraphDecoder(model, max_len=prompt_len + new_tokens + 8, fused_ops=False)
    ids = torch.randint(0, cfg.vocab_size, (prompt_len,), generator=torch.Generator().manual_seed(0)).cuda()
    lib = _capi.lib
    side = torch.cuda.Stream()
    rows = []
    if args.eager:
        # for a kernel trace: the prompt, then 16 tokens launched one kernel at a time, at 3 and 8 bits
        for b in (3, 8):
            dec.prefill(ids, b)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            dec.decode(16, b, use_graph=False)
            torch.cuda.synchronize()
            rows.append({"w_bits": b, "eager_tokens_per_s": round(16 / (time.perf_counter() - t0), 1)})
        print(json.dumps({"metric": "batch-1 decode tokens/s, eager launches (for profiling)", "value": None, "unit": "tokens/s",
                          "n_gpus": 1, "higher_is_better": True, "vs_baseline": None, "data": "synthetic",
                          "config": {"workload": f"{prompt_len}-token prompt + 16 eager tokens, Llama-2-7B-shaped model"},
                          "per_w_bits": rows}))
        return
    if args.audit_decode:
        # the launch rules were fitted to launches timed alone; this times the whole step with one rule overridden at a time
        overrides = [("rows_1", {"gemv_rows": 1}), ("rows_2", {"gemv_rows": 2}), ("rows_4", {"gemv_rows": 4}),
                     ("no_stream", {"gemv_stream": 0}), ("stream_everywhere", {"gemv_stream": 2}), ("no_fine", {"gemv_fine": 0}),
                     ("fine_everywhere", {"gemv_fine": 2}),
                     ("target_waves_8192", {"gemv_target_waves": 8192}), ("target_waves_32768", {"gemv_target_waves": 32768})]

        def tokens_per_s(b, knobs):
            dec.graphs.clear()                              # the launch geometry is fixed when the step is recorded
            with _capi.tuning(**knobs):
                dec.prefill(ids, b)
                dec.capture(b)
            dec.decode(8, b)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            dec.decode(200, b)
            torch.cuda.synchronize()
            return 200 / (time.perf_counter() - t0)

        worst = 0.0
        for b in BITS:
            first = tokens_per_s(b, {})
            forced = {name: round(tokens_per_s(b, knobs), 1) for name, knobs in overrides}
            default = max(first, tokens_per_s(b, {}))       # measured first and last
            best = max(forced, key=forced.get)
            worst = max(worst, forced[best] / default - 1)
            rows.append({"w_bits": b, "default_tokens_per_s": round(default, 1), "best_override": best,
                         "best_override_tokens_per_s": forced[best], "overrides": forced})
        print(json.dumps({"metric": "largest gain of any single global override of the GEMV launch rules over the default rules, "
                                    "batch-1 decode tokens/s, Llama-2-7B-shaped model", "value": round(worst, 4), "unit": "fraction",
                          "n_gpus": 1, "higher_is_better": False, "vs_baseline": None, "data": "synthetic",
                          "dtype": "fp16 (fp32 accumulate), u32 bitplanes",
                          "config": {"workload": f"{prompt_len}-token prompt + 200 timed tokens per setting, decode step re-recorded "
                                                 "into a HIP graph under each override, w_bits 3-8"},
                          "per_w_bits": rows}))
        return
    for b in BITS:
        dec.prefill(ids, b)
        torch.cuda.synchronize()
        prefill_ms = float("inf")
        for _ in range(3):                                     # the prompt again, warm (best of three: its launches
            t0 = time.perf_counter()                           # come from Python one by one); its linears take the
            dec.prefill(ids, b)                                # fused GEMM or dequant + library GEMM as
            torch.cuda.synchronize()                           # AnyPrecisionLinear decides
            prefill_ms = min(prefill_ms, (time.perf_counter() - t0) * 1e3)
        dec.capture(b)
        dec.decode(8, b)                                   # warm replays
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        dec.decode(new_tokens - 9, b)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        tok_s = (new_tokens - 9) / dt
        single = stock = None
        if b in (3, 8):
            for which in ("single", "stock"):
                d = dec_single if which == "single" else dec_stock
                d.prefill(ids, b)
                d.capture(b)
                d.decode(8, b)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                d.decode(64, b)
                torch.cuda.synchronize()
                if which == "single":
                    single = 64 / (time.perf_counter() - t0)
                else:
                    stock = 64 / (time.perf_counter() - t0)
        eager = None
        if b in (3, 8):
            dec.prefill(ids, b)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            dec.decode(32, b, use_graph=False)
            torch.cuda.synchronize()
            eager = 32 / (time.perf_counter() - t0)
        # the linears of one token alone (224 GEMVs on this model's own weights, one graph)
        x = {K: torch.randn((1, K), device="cuda").half() for K in (4096, 11008)}
        outs = {N: torch.empty((1, N), dtype=torch.float16, device="cuda") for N in (4096, 11008)}

        def token_linears(st):
            for lin in model.ap_linears:
                rc = lib.ap_matmul_kbit(x[lin.in_features].data_ptr(), lin.qweight.data_ptr(),
                                        lin._buffers[f"lut{b}"].data_ptr(), outs[lin.out_features].data_ptr(),
                                        1, lin.out_features, lin.in_features, b, st)
                if rc != 0:
                    raise RuntimeError(_capi.strerror(rc))
        lin_us = _graph_us(torch, side, token_linears, 1)
        lin_bytes = sum(synth.gemv_bytes(l.out_features, l.in_features, b, 1) for l in model.ap_linears)
        rows.append({"w_bits": b, "tokens_per_s": round(tok_s, 1), "ms_per_token": round(1e3 / tok_s, 3),
                     "prompt_ms": round(prefill_ms, 2),
                     "eager_tokens_per_s": None if eager is None else round(eager, 1),
                     "one_launch_per_linear_tokens_per_s": None if single is None else round(single, 1),
                     "stock_pytorch_ops_between_linears_tokens_per_s": None if stock is None else round(stock, 1),
                     "linears_ms_per_token": round(lin_us / 1e3, 3),
                     "linears_GBps": round(lin_bytes / lin_us / 1e3, 1),
                     "linears_frac_of_hbm_peak": round(lin_bytes / lin_us / 1e3 / HBM_PEAK_GBS, 4)})
    print(json.dumps({
        "metric": "batch-1 decode tokens/s, random-init Llama-2-7B-shaped model, mean over w_bits 3-8",
        "value": round(sum(r["tokens_per_s"] for r in rows) / len(rows), 1), "unit": "tokens/s", "n_gpus": 1,
        "higher_is_better": True, "vs_baseline": None, "dtype": "fp16 (fp32 accumulate), u32 bitplanes",
        "data": "synthetic (random-init weights, random prompt ids)",
        "config": {"workload": f"greedy decode of {new_tokens} tokens after a {prompt_len}-token prompt, batch 1, "
                               "32 layers / hidden 4096 / FFN 11008 / 32 heads / vocab 32000; decode step replayed "
                               "from one HIP graph, 7 launches per layer, all this library's (7 linears in 4 launches, "
                               "add + RMSNorm twice, rotary + cache append + attention; SiLU * up rides on the gate/up launch); argmax and the position / token "
                               "bookkeeping are one library kernel; embedding lookup and head are PyTorch ops"},
        "per_w_bits": rows}))



MFMA_PEAK_TFLOPS = 2500.0   # dense fp16 matrix-core peak of MI355X


def prefill_rows(torch, synth, bits=(3, 8), reps=5):
    """The seven linears of a Llama-2-7B layer on M = 32 x 512 = 16384 activation rows, two routes per w_bits:
    the module's forward (AnyPrecisionLinear's branch for many rows: dequant_kbit to fp16, then the library GEMM --
    the reference's AnyPrecisionLinear.py:60-62) and ap_gemm_kbit (the fused tiled dequant -> LDS -> MFMA kernel, one
    launch per linear).  ms per layer set, TFLOP/s and the fraction of the 2.5 PFLOP/s fp16 matrix-core peak."""
    from any_precision_amd import AnyPrecisionLinear
    import any_precision_ext as ext
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0)
    M = 32 * 512
    side = torch.cuda.Stream()
    rows = []
    with torch.inference_mode():
        for b in bits:
            t_total = t_deq = t_fused = flops = 0.0
            for name, N, K in synth.LLAMA2_7B_LAYER:
                lin = AnyPrecisionLinear(K, N, [b], bias=False, device="cuda", dtype=torch.float16)
                lin.qweight.copy_(torch.randint(-2**31, 2**31 - 1, lin.qweight.shape, dtype=torch.int32, device="cuda",
                                                generator=gen))
                lin._buffers[f"lut{b}"].copy_(torch.sort(torch.randn((N, 1 << b), device="cuda", generator=gen) * 0.02,
                                                         dim=1).values.half())
                x = torch.randn((M, K), device="cuda", generator=gen).half()

                def run(fn, n):
                    with torch.cuda.stream(side):
                        fn()
                        side.synchronize()
                        a0, a1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                        a0.record(side)
                        for _ in range(n):
                            fn()
                        a1.record(side)
                        side.synchronize()
                    return a0.elapsed_time(a1) / n
                t_total += run(lambda: lin(x, precision=b), reps)
                t_deq += run(lambda: ext.dequant_kbit(lin.qweight, lin._buffers[f"lut{b}"], b), reps)
                t_fused += run(lambda: ext.gemm_kbit(x, lin.qweight, lin._buffers[f"lut{b}"], b), max(2, reps // 2))
                flops += 2.0 * M * N * K
                del lin, x
            rows.append({"w_bits": b, "ms_per_layer_linears": round(t_total, 3), "ms_dequant": round(t_deq, 3),
                         "dequant_share": round(t_deq / t_total, 4), "TFLOPs": round(flops / t_total / 1e9, 1),
                         "frac_of_mfma_peak": round(flops / t_total / 1e9 / MFMA_PEAK_TFLOPS, 4),
                         "fused_tiled_gemm_ms": round(t_fused, 3), "fused_tiled_gemm_TFLOPs": round(flops / t_fused / 1e9, 1),
                         "fused_tiled_gemm_frac_of_mfma_peak": round(flops / t_fused / 1e9 / MFMA_PEAK_TFLOPS, 4)})
    torch.cuda.empty_cache()
    return rows


PREFILL_WORKLOAD = ("7 linears of a Llama-2-7B decoder layer, M = 32 x 512 = 16384 activation rows, eager launches: the "
                    "module's route (dequant_kbit + torch.matmul per call, weight rebuilt on every call) and, beside it, "
                    "ap_gemm_kbit (fused tiled kernel)")


def prefill_linears(args, torch, _capi, synth):
    rows = prefill_rows(torch, synth)
    print(json.dumps({
        "metric": "prefill linears TFLOP/s, Llama-2-7B layer set, 16384 activation rows",
        "value": round(sum(r["TFLOPs"] for r in rows) / len(rows), 1), "unit": "TFLOP/s", "n_gpus": 1,
        "higher_is_better": True, "vs_baseline": None, "dtype": "fp16 (library GEMM) on dequantised weights",
        "data": "synthetic",
        "config": {"workload": PREFILL_WORKLOAD},
        "per_w_bits": rows}))


if __name__ == "__main__":
    main()
