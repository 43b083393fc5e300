#!/usr/bin/env python3
"""Benchmark of the CuSync hot path on one MI355X.

Workload: the GPT-3 175B MLP, one GPU's 1/8 shard — X[B,12288] fp16 x
W1[12288,6144] with GeLU fused -> H[B,6144] x W2[6144,12288] — as two dependent
GEMMs, stream-ordered (kernel-boundary sync) versus CuSync RowSync / TileSync on
two streams.  A "step" is one pass of the chain at B = 2048 under the better
CuSync policy; inputs are resident in HBM before the timed region.

Prints ONE JSON line.  `value` is the step latency in microseconds (lower is
better); `per_batch` holds the metric proper: latency per B in {1..2048} for the
three modes, % gain over stream-ordered, TFLOP/s and roofline fraction, measured
with the reference's protocol (10 warm-up runs, 20 timed, slowest 10 % dropped;
src/ml-bench/transformer/mlp.cu:954-955, eval_mlp.py:40-50).

Every comparison is timed INTERLEAVED: the handles of all modes of one shape are
alive together and take turns step by step (stream, row, tile, stream, row, ...),
after a fixed number of untimed steps that lets the device's clock settle, so that
clock drift, the memory-side cache and the order of the legs cannot favour a mode.
"""
import argparse
import json
import os
import statistics
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HIDDEN, INNER = 12288, 6144
BATCHES = [1, 16, 64, 256, 512, 1024, 2048]
PEAK_FP16_TFLOPS = 2500.0      # MI355X dense fp16 MFMA
PEAK_HBM_GBS = 8000.0          # MI355X HBM3E
SETTLE_STEPS = 40              # untimed steps of the timed shape before anything is measured: after a light load
                               # the device needs about 30 steps of this size until its clock settles
MIN_WARM_S = 0.025             # the slow phase after an idle gap (handles being created) is over after about 15 ms of load
TRAFFIC_TABLE = os.path.join(ROOT, "profiles", "gemm_hbm_traffic_by_tile.md")
MFMA_TABLE = os.path.join(ROOT, "profiles", "gemm_mfma_by_batch.md")


def table_row(path, tiles, batch):
    """The cells of the row of a committed profile table whose first three columns are the tile ids of the two
    launches and the batch; None if that combination was never profiled."""
    try:
        with open(path) as f:
            for line in f:
                cells = [c.strip() for c in line.strip().strip("|").split("|")]
                if len(cells) >= 4 and cells[0].isdigit() and cells[1].isdigit() and cells[2].isdigit():
                    if (int(cells[0]), int(cells[1]), int(cells[2])) == (tiles[0], tiles[1], batch):
                        return cells
    except OSError:
        pass
    return None


def traffic_bytes(tiles, batch):
    """HBM bytes per GEMM launch from the committed counter runs (rocprofv3 FETCH_SIZE / WRITE_SIZE scaled by a
    plain copy of known size), looked up by the tile ids of the two launches and the batch; None if that
    combination was never profiled."""
    row = table_row(TRAFFIC_TABLE, tiles, batch)
    return float(row[3]) * 1e6 if row else None


def mfma_busy(tiles, batch):
    """From the committed SQ counter runs, for the tile ids of the two launches and the batch: the share of SIMD
    cycles the matrix pipes were busy over the launch, at the clock the launch ran at (SQ_VALU_MFMA_BUSY_CYCLES per
    SIMD over SQ_BUSY_CYCLES per shader engine), that clock, and the share of wave time spent waiting
    (SQ_WAIT_INST_ANY / SQ_WAVE_CYCLES).  None if that combination was never profiled."""
    row = table_row(MFMA_TABLE, tiles, batch)
    return {"mfma_busy_pct": float(row[3]), "clock_ghz": float(row[4]), "wait_inst_any_pct": float(row[5])} if row else None


def trimmed(times):
    """Mean and stdev after dropping the slowest 10 % (eval_mlp.py:40-50)."""
    t = sorted(times)
    keep = t[:max(1, len(t) - len(t) // 10)]
    return statistics.fmean(keep), (statistics.pstdev(keep) if len(keep) > 1 else 0.0)


def mlp_flops(b):
    return 4.0 * b * HIDDEN * INNER


def mlp_bytes(b):
    # each operand/result once in fp16; the intermediate is written once and read once
    return 2.0 * (2 * HIDDEN * INNER + b * HIDDEN * 2 + 2 * b * INNER)


def ideal_us(b):
    return max(mlp_flops(b) / (PEAK_FP16_TFLOPS * 1e12), mlp_bytes(b) / (PEAK_HBM_GBS * 1e9)) * 1e6


def cpu_baseline(x_host, w1_host, w2_host, budget_s=15.0):
    """Times the CPU oracle (the restatement of the reference's host GEMM,
    src/ml-bench/transformer/common.h:89-102) on a bounded number of rows of the
    same workload and scales to the B = 2048 shard."""
    import numpy as np
    import oracle as orc
    t0 = time.perf_counter()
    h = orc.gemm(x_host[:1], w1_host, orc.EPI_GELU)
    orc.gemm(h, w2_host)
    t1 = time.perf_counter() - t0
    rows = int(max(1, min(512, budget_s / max(t1, 1e-3))))
    t0 = time.perf_counter()
    h = orc.gemm(np.ascontiguousarray(x_host[:rows]), w1_host, orc.EPI_GELU)
    orc.gemm(h, w2_host)
    t = time.perf_counter() - t0
    per_row_us = t / rows * 1e6
    return {
        "value": per_row_us * 2048, "unit": "us", "cores": orc.num_threads(), "kind": "port",
        "sample": "%d of 2048 rows of the same MLP (%.1f s of CPU time), scaled linearly; %.2f GFLOP/s" % (
            rows, t, mlp_flops(rows) / t / 1e9),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10,
                    help="untimed rounds before the timed ones, on top of a fixed settling preamble")
    ap.add_argument("--batch", type=int, default=2048, help="B of the timed step")
    ap.add_argument("--no-sweep", action="store_true", help="skip the per-batch table")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--roofline-only", action="store_true",
                    help="run only the leg that times the dominant kernel (stream-ordered GEMM1/GEMM2 at --batch) "
                         "plus a plain copy of known size; used under rocprofv3 so its per-kernel averages match")
    ap.add_argument("--profile-chain", choices=["attention", "conv", "mlp"], default=None,
                    help="run only the stream-ordered attention chain (S = 2048) or convolution pairs, or (mlp) --steps rounds of "
                         "the GPT-3 MLP at --batch stream-ordered / RowSync / TileSync in turn, for rocprofv3")
    ap.add_argument("--timeline", action="store_true",
                    help="with --roofline-only: one more step with the kernels' per-workgroup clock records switched on "
                         "(cusync_rt_set_timeline); prints where a workgroup's time goes per launch")
    ap.add_argument("--zero-operands", action="store_true",
                    help="with --roofline-only: X, W1 and W2 all zero.  Same instruction stream, far less switching in the "
                         "matrix pipes: what the kernels take when the device's power limit does not set the clock")
    ap.add_argument("--tile1", type=int, default=-1)
    ap.add_argument("--tile2", type=int, default=-1)
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (CuSync is a single-GPU mechanism); "
                 "run with --gpus 1")

    import numpy as np
    import torch
    from cusync_amd import api

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = api.device_info()

    # Synthetic shard: X ~ U[-1,1], W ~ N(0, 0.02), seeds X 1 / W1 2 / W2 3, rounded to fp16.
    def normal(shape, seed):
        return (np.random.default_rng(seed).standard_normal(shape, dtype=np.float32) * 0.02).astype(np.float16)

    w1_host, w2_host = normal((HIDDEN, INNER), 2), normal((INNER, HIDDEN), 3)
    x_host = np.random.default_rng(1).uniform(-1, 1, (max(BATCHES), HIDDEN)).astype(np.float32).astype(np.float16)
    w1, w2, x_all = (torch.from_numpy(a).cuda() for a in (w1_host, w2_host, x_host))
    if args.zero_operands:
        if not args.roofline_only:
            sys.exit("bench.py: --zero-operands is a diagnosis of the --roofline-only leg")
        for t in (w1, w2, x_all):
            t.zero_()
    torch.cuda.synchronize()

    class Chain:
        """One MLP handle with its intermediate and output buffers."""

        def __init__(self, batch, sync, one_launch=False, repack=False, operands=None):
            xs, wa, wb = operands or (x_all, w1, w2)
            self.h = torch.empty((batch, INNER), dtype=torch.float16, device="cuda")
            self.y = torch.empty((batch, HIDDEN), dtype=torch.float16, device="cuda")
            self.x = xs[:batch]
            torch.cuda.synchronize()
            self.m = api.Mlp(api.MODEL.GPT3, batch, HIDDEN, INNER, sync, wa.data_ptr(), wb.data_ptr(),
                             tile1=args.tile1, tile2=args.tile2, one_launch=one_launch, repack_weights=repack)
            self.tiles = self.m.tiles()

        def step(self, split=False):
            """One pass; elapsed microseconds by HIP events on the chain's own streams (a wait that gave up raises)."""
            out = self.m.run(self.x.data_ptr(), self.h.data_ptr(), self.y.data_ptr(), runs=1, split=split)
            return (out[0][0], out[1][0], out[2][0]) if split else out[0]

        def close(self):
            self.m.destroy()

    def default_one_launch(batch, sync):
        """Whether the tile table runs this batch size in one launch when the caller leaves it open."""
        import ctypes
        from cusync_amd import _lib
        cfg = _lib.MlpConfig(api.MODEL.GPT3, batch, HIDDEN, INNER, sync, args.tile1, args.tile2, -1, 1, 0, 0, 0, 0, -1, 0, 0)
        one = ctypes.c_int(0)
        if _lib.load().cusync_mlp_choice(ctypes.byref(cfg), None, None, None, None, ctypes.byref(one)) != 0:
            raise RuntimeError("cusync_mlp_choice: " + api.last_error())
        return bool(one.value)

    def interleaved(chains, warm, timed, split_first=False):
        """Runs the chains in turn, one step each per round: `warm` untimed rounds (and as many more as it takes to
        keep the device under this load for MIN_WARM_S), then `timed` rounds.  Returns
        one list of step times per chain (for the first chain, with split_first, triples: step, GEMM1, GEMM2)."""
        t0, done = time.perf_counter(), 0
        while done < warm or time.perf_counter() - t0 < MIN_WARM_S:      # (steps return when their last kernel has ended)
            for c in chains:
                c.step()
            done += 1
        times = [[] for _ in chains]
        for _ in range(timed):
            for i, c in enumerate(chains):
                times[i].append(c.step(split=split_first and i == 0))
        return times

    def rounds(objs, step, warm=10, timed=20):
        """The same turn-taking for the other chains' handles: `step(obj)` runs one pass and returns ([us], extra).
        Returns the step times and the extras, one list per object."""
        t0, done = time.perf_counter(), 0
        while done < warm or time.perf_counter() - t0 < MIN_WARM_S:
            for o in objs:
                step(o)
            done += 1
        times, extras = [[] for _ in objs], [[] for _ in objs]
        for _ in range(timed):
            for i, o in enumerate(objs):
                t, e = step(o)
                times[i].append(t[0])
                extras[i].append(e[0] if e else None)
        return times, extras

    def settle(batch, steps=SETTLE_STEPS):
        """Untimed steps of the timed shape: brings the clock to where it stays under this load."""
        c = Chain(batch, api.SYNC.STREAM)
        for _ in range(steps):
            c.step()
        c.close()

    def roofline_leg(B, warm, timed):
        """Durations of the two GEMM launches, HIP events on the stream they run on."""
        c = Chain(B, api.SYNC.STREAM)
        # The settling steps run on this very chain, with nothing between them and the timed ones: after an idle gap of
        # tens of milliseconds (a handle being created is one) the device runs these launches at boost for 2 ms, then
        # up to a quarter slower for several, and is back at its steady rate only after about 15 ms of load.
        (t3,) = interleaved([c], max(warm, SETTLE_STEPS), timed, split_first=True)
        tiles = c.tiles
        timeline = None
        if args.timeline or not args.roofline_only:      # (left out of the bare --roofline-only run the profiler's counters average over)
            # one record per finished tile: 100 MHz clock at kernel entry of the workgroup, tile drawn, first loads
            # issued, main loop done, epilogue (and post) done
            from cusync_amd import _lib
            buf = torch.zeros(1 + 8 * 8192, dtype=torch.int64, device="cuda")
            torch.cuda.synchronize()
            _lib.load().cusync_rt_set_timeline(buf.data_ptr(), buf.numel() * 8)
            c.step()
            _lib.load().cusync_rt_set_timeline(None, 0)
            r = buf.cpu().numpy()
            rec = r[1:1 + 8 * int(r[0])].reshape(-1, 8)
            entry = np.sort(np.unique(rec[:, 6]))
            cut = entry[int(np.argmax(np.diff(entry))) + 1] if len(entry) > 1 else entry[0] + 1      # first workgroup of GEMM2
            timeline = {}
            for name, m in (("gemm1", rec[:, 6] < cut), ("gemm2", rec[:, 6] >= cut)):
                q = rec[m]
                if len(q) == 0:
                    continue
                t0 = q[:, 6].min()
                first = q[(q[:, 1] >> 48) == 0]          # a workgroup's first tile: its prologue starts at kernel entry
                def med(v):
                    return round(float(np.median(v)) / 100.0, 2)
                timeline[name] = {
                    "tiles": int(len(q)), "workgroups": int(len(np.unique(q[:, 0] >> 8 & 0xffffffff))),
                    "entry_spread_us": round(float(q[:, 6].max() - t0) / 100.0, 2),
                    "entry_to_first_loads_us": med(first[:, 3] - first[:, 6]),
                    "k_loop_us": {"median": med(q[:, 4] - q[:, 3]), "min": round(float((q[:, 4] - q[:, 3]).min()) / 100.0, 2),
                                  "max": round(float((q[:, 4] - q[:, 3]).max()) / 100.0, 2)},
                    "epilogue_us": med(q[:, 5] - q[:, 4]),
                    # the eight XCDs do not run at one speed: a launch of one tile per CU is as long as its slowest XCD
                    "k_loop_us_by_xcd": [med((q[:, 4] - q[:, 3])[(q[:, 0] >> 40) & 0xf == x]) if np.any((q[:, 0] >> 40) & 0xf == x) else None
                                         for x in range(8)],
                    "last_tile_done_us": round(float(q[:, 5].max() - t0) / 100.0, 2),
                }
        c.close()
        t_s, g1, g2 = [v[0] for v in t3], [v[1] for v in t3], [v[2] for v in t3]
        k_us = (statistics.fmean(g1) + statistics.fmean(g2)) / 2
        flops_per_launch = 2.0 * B * HIDDEN * INNER
        achieved = flops_per_launch / (k_us * 1e-6) / 1e12
        shapes = ["%dx%dx%d" % api.tile_shape(t) for t in tiles[:2]]
        # plain copy of known size: the scale for the FETCH_SIZE / WRITE_SIZE counters
        a = torch.zeros(64 << 20, dtype=torch.float16, device="cuda")      # 128 MiB read + 128 MiB written
        b = torch.empty_like(a)
        for _ in range(3):
            torch.add(a, 1, out=b)
        torch.cuda.synchronize()
        # few rows: a launch streams its weight matrix once and that bounds it (algorithmic bytes: the operands once)
        bytes_per_launch = 2.0 * (HIDDEN * INNER + B * HIDDEN + B * INNER)
        hbm_bound = bytes_per_launch / (PEAK_HBM_GBS * 1e9) > flops_per_launch / (PEAK_FP16_TFLOPS * 1e12)
        gbs = bytes_per_launch / (k_us * 1e-6) / 1e9
        head = ({"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4)}
                if hbm_bound else
                {"bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s",
                 "frac": round(achieved / PEAK_FP16_TFLOPS, 4)})
        busy = mfma_busy(tiles, B)
        return {**head, "traffic": traffic_bytes(tiles, B), "mfma_busy_pct": busy["mfma_busy_pct"] if busy else None,
                "clock_ghz_under_load": busy["clock_ghz"] if busy else None, **({"timeline": timeline} if timeline else {}),
                **({"operands": "all zero"} if args.zero_operands else {}),
                "kernel": "gemmDmaKernel, mean of the two launches of the step: GEMM1 tile %s %.1f us, GEMM2 tile %s %.1f us "
                          "(stream-ordered, %.1f GFLOP per launch)" % (shapes[0], statistics.fmean(g1), shapes[1], statistics.fmean(g2),
                                                                       flops_per_launch / 1e9),
                }, statistics.fmean(t_s), tiles

    if args.profile_chain == "mlp":
        # every round enqueues six GEMM launches in this order: stream-ordered GEMM1, GEMM2; RowSync producer, consumer;
        # TileSync producer, consumer.  A kernel trace of this run shows when each started and ended.
        settle(args.batch)
        chains = [Chain(args.batch, api.SYNC.STREAM), Chain(args.batch, api.SYNC.ROW), Chain(args.batch, api.SYNC.TILE)]
        times = interleaved(chains, args.warmup, args.steps)
        for c in chains:
            c.close()
        def dist(v):
            med = statistics.median(v)
            lo = int(min(v) // 10 * 10)
            bins = {}
            for t in v:
                b = int((t - lo) // 10)
                bins[b] = bins.get(b, 0) + 1
            return {"mean": round(statistics.fmean(v), 2), "median": round(med, 2), "min": round(min(v), 2), "max": round(max(v), 2),
                    "p99": round(sorted(v)[min(len(v) - 1, int(len(v) * 0.99))], 2), "steps_over_1.05_median": sum(1 for t in v if t > 1.05 * med),
                    "histogram_10us_bins_from_%d" % lo: [bins.get(i, 0) for i in range(max(bins) + 1)]}
        print(json.dumps({"metric": "GPT-3 MLP rounds of stream / rowsync / tilesync", "batch": args.batch, "warmup_rounds": args.warmup,
                          "rounds": args.steps, "settle_steps": SETTLE_STEPS, "wait_kernel_forced": os.environ.get("CUSYNC_WAIT_KERNEL", "0") not in ("", "0"),
                          "event_us": {n: round(statistics.fmean(t), 2) for n, t in zip(("stream", "rowsync", "tilesync"), times)},
                          "step_us": {n: dist(t) for n, t in zip(("stream", "rowsync", "tilesync"), times)}}))
        return
    if args.profile_chain == "attention":
        heads, e, seq = 12, 12 * 128, 2048
        g = torch.Generator(device="cuda").manual_seed(4)
        wqkv = (torch.randn((HIDDEN, 3 * e), device="cuda", generator=g) * 0.02).half()
        wo = (torch.randn((e, HIDDEN), device="cuda", generator=g) * 0.02).half()
        qkv = torch.empty((seq, 3 * e), dtype=torch.float16, device="cuda")
        o = torch.empty((seq, e), dtype=torch.float16, device="cuda")
        y = torch.empty((seq, HIDDEN), dtype=torch.float16, device="cuda")
        torch.cuda.synchronize()
        layer = api.AttnLayer(seq, HIDDEN, heads, api.SYNC.STREAM, wqkv.data_ptr(), wo.data_ptr())
        layer.run(x_all[:seq].data_ptr(), qkv.data_ptr(), o.data_ptr(), y.data_ptr(), runs=args.warmup)
        t, st = layer.run(x_all[:seq].data_ptr(), qkv.data_ptr(), o.data_ptr(), y.data_ptr(), runs=max(10, args.steps), stages=True)
        print(json.dumps({"metric": "attention chain, stream-ordered, S=2048", "chain_us": round(trimmed(t)[0], 2),
                          "stage_us": [round(trimmed([v[i] for v in st])[0], 2) for i in range(3)], "tiles": list(layer.tiles()),
                          "attention_gflop": round(4.0 * seq * seq * 128 * heads / 2 / 1e9, 2)}))
        layer.destroy()
        return
    if args.profile_chain == "conv":
        g = torch.Generator(device="cuda").manual_seed(4)
        rows = []
        # the two pairs of the benchmark set, then the two deep layers of the reference's table
        # (src/ml-bench/volta_conv2d/resnet_results.csv: 256 and 512 channels), whose few tiles the chain cuts into runs
        for n, hh, ww, cc in ((32, 56, 56, 64), (32, 28, 28, 128), (32, 14, 14, 256), (32, 7, 7, 512)):
            xc = (torch.rand((n, hh, ww, cc), device="cuda", generator=g) * 2 - 1).half()
            ws = [(torch.randn((cc, 3, 3, cc), device="cuda", generator=g) * (2.0 / (9 * cc)) ** 0.5).half() for _ in range(2)]
            ys = [torch.empty((n, hh, ww, cc), dtype=torch.float16, device="cuda") for _ in range(2)]
            torch.cuda.synchronize()
            ch = api.ConvChain(n, hh, ww, cc, [w.data_ptr() for w in ws], api.SYNC.STREAM)
            ch.run(xc.data_ptr(), [t.data_ptr() for t in ys], runs=args.warmup)
            t, per = ch.run(xc.data_ptr(), [t.data_ptr() for t in ys], runs=max(10, args.steps), layers=True)
            rows.append({"shape": [n, hh, ww, cc], "pair_us": round(trimmed(t)[0], 2),
                         "layer_us": [round(trimmed([v[i] for v in per])[0], 2) for i in range(2)], "tile": ch.tile(),
                         "gflop_per_layer": round(2.0 * n * hh * ww * cc * 9 * cc / 1e9, 2)})
            ch.destroy()
        print(json.dumps({"metric": "convolution pairs, stream-ordered", "rows": rows}))
        return

    B = args.batch
    if args.roofline_only:
        roof, stream_us, tiles = roofline_leg(B, args.warmup, max(10, args.steps))
        print(json.dumps({"metric": "dominant kernel only", "roofline": roof, "stream_ordered_us": round(stream_us, 2),
                          "tiles": list(tiles)}))
        return

    per_batch = []
    launcher = {}
    if not args.no_sweep:
        settle(max(BATCHES))
        # The reference's own loop (CuStage + CuSyncGemm objects wired by a plain C++ driver, invokeWaitKernel between the
        # two launches) next to the handle: the driver runs rounds of 20 steps of each in turn, in a process of its own
        # while this one is idle, and reports medians.
        exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cusync_amd", "bin", "mlp_stages")
        if not os.path.exists(exe):
            sys.exit("bench.py: %s is not built (make -C cusync_amd/drivers)" % exe)
        drv = subprocess.run([exe, "--batch", ",".join(str(b) for b in BATCHES), "--sync", "both", "--runs", "20", "--rounds", "3"],
                             capture_output=True, text=True, timeout=600)
        if drv.returncode != 0:
            sys.exit("bench.py: mlp_stages failed: " + drv.stderr[-2000:])
        for line in drv.stdout.splitlines():
            if line.startswith('{"batch"'):
                r = json.loads(line)
                launcher[(r["batch"], r["sync"])] = r
        for b in BATCHES:
            # all modes of this batch size alive together, one step each per round (10 untimed rounds, 20 timed):
            # stream-ordered, RowSync, TileSync, RowSync with both GEMMs in one launch (same stages and semaphores,
            # no wait, no second launch), and the same with copies of the weights whose rows are 256 bytes longer
            # (cusync_mlp_config.repack_weights: a column tile's k rows then spread over all memory channels)
            names = ["stream", "rowsync", "tilesync"]
            chains = [Chain(b, api.SYNC.STREAM), Chain(b, api.SYNC.ROW), Chain(b, api.SYNC.TILE)]
            tiles = chains[0].tiles
            # one launch needs one tile shape for both GEMMs: left to itself the handle gives GEMM2 the tile of GEMM1
            one_ok = tiles[0] == tiles[1] or args.tile2 < 0
            one_tiles = None
            if one_ok:
                names += ["rowsync_one_launch", "tilesync_one_launch"]
                chains += [Chain(b, api.SYNC.ROW, one_launch=True), Chain(b, api.SYNC.TILE, one_launch=True)]
                one_tiles = list(chains[-1].tiles)
            names += ["stream_rp", "rowsync_rp"]
            chains += [Chain(b, api.SYNC.STREAM, repack=True), Chain(b, api.SYNC.ROW, repack=True)]
            if one_ok:
                names.append("rowsync_one_launch_rp")
                chains.append(Chain(b, api.SYNC.ROW, one_launch=True, repack=True))
            times = interleaved(chains, 10, 20, split_first=True)
            # what a handle left to itself (one_launch = -1) runs under each policy: one launch or two
            default_one = {k: default_one_launch(b, sy) for k, sy in (("rowsync", api.SYNC.ROW), ("tilesync", api.SYNC.TILE))}
            for c in chains:
                c.close()
            t = dict(zip(names, times))
            g1, g2 = [v[1] for v in t["stream"]], [v[2] for v in t["stream"]]
            t["stream"] = [v[0] for v in t["stream"]]
            m = {k: trimmed(v) for k, v in t.items()}
            s_us = m["stream"][0]
            in_place = [k for k in ("rowsync", "tilesync", "rowsync_one_launch", "tilesync_one_launch") if k in m]
            best = min(m[k][0] for k in in_place)
            rp = [m[k][0] for k in ("stream_rp", "rowsync_rp", "rowsync_one_launch_rp") if k in m]
            per_batch.append({
                "B": b, "tiles": list(tiles),
                "stream_us": round(s_us, 2), "stream_std": round(m["stream"][1], 2),
                "gemm1_us": round(trimmed(g1)[0], 2), "gemm2_us": round(trimmed(g2)[0], 2),
                "rowsync_us": round(m["rowsync"][0], 2), "rowsync_std": round(m["rowsync"][1], 2),
                "rowsync_gain_pct": round(100 - m["rowsync"][0] / s_us * 100, 2),
                "tilesync_us": round(m["tilesync"][0], 2), "tilesync_std": round(m["tilesync"][1], 2),
                "tilesync_gain_pct": round(100 - m["tilesync"][0] / s_us * 100, 2),
                "rowsync_one_launch_us": round(m["rowsync_one_launch"][0], 2) if "rowsync_one_launch" in m else None,
                "tilesync_one_launch_us": round(m["tilesync_one_launch"][0], 2) if "tilesync_one_launch" in m else None,
                "one_launch_tiles": one_tiles,
                # the mode the handle picks by itself (cusync_mlp_config.one_launch = -1) and its time from the columns above
                "default_launches": {k: 1 if v else 2 for k, v in default_one.items()},
                "rowsync_default_us": round(m["rowsync_one_launch" if default_one["rowsync"] and "rowsync_one_launch" in m else "rowsync"][0], 2),
                "tilesync_default_us": round(m["tilesync_one_launch" if default_one["tilesync"] and "tilesync_one_launch" in m else "tilesync"][0], 2),
                # medians of 60 steps in the driver's process: the launcher objects' loop, and the handle beside it there
                "launcher_rowsync_us": launcher[(b, "rowsync")]["launcher_us"], "launcher_tilesync_us": launcher[(b, "tilesync")]["launcher_us"],
                "launcher_vs_handle_pct": {k: round(launcher[(b, k)]["launcher_us"] / launcher[(b, k)]["handle_us"] * 100 - 100, 2)
                                           for k in ("rowsync", "tilesync")},
                "best_policy": min(in_place, key=lambda k: m[k][0]),
                "best_gain_pct": round(100 - best / s_us * 100, 2),
                "repacked_weights": {"stream_us": round(m["stream_rp"][0], 2), "rowsync_us": round(m["rowsync_rp"][0], 2),
                                     "rowsync_one_launch_us": round(m["rowsync_one_launch_rp"][0], 2) if "rowsync_one_launch_rp" in m else None,
                                     "roofline_frac": round(ideal_us(b) / min(rp), 4)},
                "best_tflops": round(mlp_flops(b) / best / 1e6, 1),
                "bound": "mfma" if mlp_flops(b) / (PEAK_FP16_TFLOPS * 1e12) > mlp_bytes(b) / (PEAK_HBM_GBS * 1e9) else "hbm",
                "roofline_frac": round(ideal_us(b) / best, 4),
                # stream-ordered launches of these tiles at this batch, from the committed counter runs
                "mfma_busy_pct": (mfma_busy(tiles, b) or {}).get("mfma_busy_pct"),
            })

    # ---- the other chains of the benchmark set: self-attention and the convolution pair --------
    other = {}
    if not args.no_sweep:
        other["attention"] = []
        heads, e = 12, 12 * 128
        g = torch.Generator(device="cuda").manual_seed(4)
        wqkv = (torch.randn((HIDDEN, 3 * e), device="cuda", generator=g) * 0.02).half()
        wo = (torch.randn((e, HIDDEN), device="cuda", generator=g) * 0.02).half()
        for seq in (256, 512, 1024, 2048):
            x = x_all[:seq]
            qkv = torch.empty((seq, 3 * e), dtype=torch.float16, device="cuda")
            o = torch.empty((seq, e), dtype=torch.float16, device="cuda")
            y = torch.empty((seq, HIDDEN), dtype=torch.float16, device="cuda")
            torch.cuda.synchronize()
            row = {"S": seq}
            # all modes alive together, one step each per round (10 untimed rounds, 20 timed), like the GPT-3 sweep
            modes = (("stream", api.SYNC.STREAM), ("rowsync", api.SYNC.ROW), ("tilesync", api.SYNC.TILE), ("consecutivesync", api.SYNC.STRIDED))
            layers = [api.AttnLayer(seq, HIDDEN, heads, sync, wqkv.data_ptr(), wo.data_ptr()) for _, sync in modes]
            t, st = rounds(layers, lambda l: l.run(x.data_ptr(), qkv.data_ptr(), o.data_ptr(), y.data_ptr(), runs=1, stages=True))
            for (name, sync), layer, tt, ss in zip(modes, layers, t, st):
                if any(layer.stage_state(i).spin_timeouts for i in range(3)):
                    sys.exit("bench.py: attention chain waits timed out — results invalid")
                row[name + "_us"] = round(trimmed(tt)[0], 2)
                if sync == api.SYNC.STREAM:
                    row["stage_us"] = [round(trimmed([v[i] for v in ss])[0], 2) for i in range(3)]
                    row["tiles"] = list(layer.tiles())
                layer.destroy()
            best = min(row[k] for k in ("rowsync_us", "tilesync_us", "consecutivesync_us"))
            row["gain_pct"] = round(100 - best / row["stream_us"] * 100, 2)
            other["attention"].append(row)
        # LLaMA MLP shard (X[B,8192] x [W1|V][8192,2*2752] -> silu(g)*u in GEMM1's epilogue -> x W2[2752,8192])
        other["llama_mlp"] = []
        lh, li = 8192, 2752
        lw1 = (torch.randn((lh, 2 * li), device="cuda", generator=g) * 0.02).half()
        lw2 = (torch.randn((li, lh), device="cuda", generator=g) * 0.02).half()
        for b in BATCHES:      # the seven batch sizes of the GPT-3 sweep
            lx = (torch.rand((b, lh), device="cuda", generator=g) * 2 - 1).half()
            lhid = torch.empty((b, 2 * li), dtype=torch.float16, device="cuda")
            ly = torch.empty((b, lh), dtype=torch.float16, device="cuda")
            torch.cuda.synchronize()
            row = {"B": b}
            # rowsync_one_launch: both GEMMs in one launch (the handle gives GEMM2 the tile of GEMM1, which from 512 rows
            # on costs this chain more than the launch saves); *_repacked: W2's rows are 16 KiB, the handle's copies pad them
            modes = (("stream", api.SYNC.STREAM, {}), ("rowsync", api.SYNC.ROW, {}), ("tilesync", api.SYNC.TILE, {}),
                     ("stridedsync", api.SYNC.STRIDED, {}), ("rowsync_one_launch", api.SYNC.ROW, {"one_launch": True}),
                     ("stream_repacked", api.SYNC.STREAM, {"repack_weights": True}), ("rowsync_repacked", api.SYNC.ROW, {"repack_weights": True}))
            ms = [api.Mlp(api.MODEL.LLAMA, b, lh, li, sync, lw1.data_ptr(), lw2.data_ptr(), **kw) for _, sync, kw in modes]
            t, _ = rounds(ms, lambda m: (m.run(lx.data_ptr(), lhid.data_ptr(), ly.data_ptr(), runs=1), None))
            for (name, sync, kw), m, tt in zip(modes, ms, t):
                if m.stage_state(1).spin_timeouts:
                    sys.exit("bench.py: LLaMA consumer waits timed out — results invalid")
                row[name + "_us"] = round(trimmed(tt)[0], 2)
                if not kw.get("repack_weights"):
                    row[name + "_tiles"] = list(m.tiles())
                m.destroy()
            best = min(row[k] for k in ("rowsync_us", "tilesync_us", "stridedsync_us", "rowsync_one_launch_us"))
            row["gain_pct"] = round(100 - best / row["stream_us"] * 100, 2)
            row["best_tflops"] = round(2.0 * b * lh * 3 * li / best / 1e6, 1)
            other["llama_mlp"].append(row)
        other["conv_pair"] = []
        # the two pairs of the benchmark set, then the two deep layers of the reference's table
        # (src/ml-bench/volta_conv2d/resnet_results.csv: 256 and 512 channels), whose few tiles the chain cuts into runs
        for n, hh, ww, cc in ((32, 56, 56, 64), (32, 28, 28, 128), (32, 14, 14, 256), (32, 7, 7, 512)):
            xc = (torch.rand((n, hh, ww, cc), device="cuda", generator=g) * 2 - 1).half()
            ws = [(torch.randn((cc, 3, 3, cc), device="cuda", generator=g) * (2.0 / (9 * cc)) ** 0.5).half() for _ in range(2)]
            ys = [torch.empty((n, hh, ww, cc), dtype=torch.float16, device="cuda") for _ in range(2)]
            torch.cuda.synchronize()
            row = {"shape": [n, hh, ww, cc], "gflop": round(2 * 2.0 * n * hh * ww * cc * 9 * cc / 1e9, 2)}
            # *_one_launch: both layers in one launch, same semaphores (no wait kernel, no second launch)
            modes = (("stream", api.SYNC.STREAM, False), ("rowsync", api.SYNC.ROW, False), ("tilesync", api.SYNC.TILE, False),
                     ("rowsync_one_launch", api.SYNC.ROW, True), ("tilesync_one_launch", api.SYNC.TILE, True))
            chs = [api.ConvChain(n, hh, ww, cc, [w.data_ptr() for w in ws], sync, fused=fused) for _, sync, fused in modes]
            t, _ = rounds(chs, lambda ch: (ch.run(xc.data_ptr(), [v.data_ptr() for v in ys], runs=1), None))
            for (name, sync, fused), ch, tt in zip(modes, chs, t):
                if any(ch.stage_state(i).spin_timeouts for i in range(2)):
                    sys.exit("bench.py: convolution chain waits timed out — results invalid")
                row[name + "_us"] = round(trimmed(tt)[0], 2)
                row["tile"] = ch.tile()
                if name == "stream":
                    row["runs_per_tile"] = ch.split()
                ch.destroy()
            best = min(row[k] for k in ("rowsync_us", "tilesync_us", "rowsync_one_launch_us", "tilesync_one_launch_us"))
            row["gain_pct"] = round(100 - best / row["stream_us"] * 100, 2)
            other["conv_pair"].append(row)

        # cost of the synchronisation itself (src/examples/sync-overhead/sync-overhead.cu and a ping-pong)
        with_sync, without = api.sync_overhead_pair(1280, 128, warmup=10, iters=100)
        bare_with, bare_without = api.sync_overhead_bare(1280, 128, warmup=10, iters=100)
        other["sync_overhead"] = {
            # the example's own kernels: a bare flag per block, no fences, one stream (what its percentage measures)
            "bare_flags_with_us": round(bare_with, 2), "bare_flags_without_us": round(bare_without, 2),
            "bare_flags_overhead_pct": round((bare_with - bare_without) / bare_without * 100, 1),
            # the public CuStage tile/post/wait on two streams with the wait kernel: what a chain pays
            "pair_with_sync_us": round(with_sync, 2), "pair_without_sync_us": round(without, 2),
            "pair_overhead_pct": round((with_sync - without) / without * 100, 1),
            "handover_ns_same_xcd": round(api.sync_overhead_pingpong(8) / 2, 1),
            "handover_ns_other_xcd": round(api.sync_overhead_pingpong(1) / 2, 1),
        }

    # ---- the timed step: B = args.batch, CuSync against stream-ordered, interleaved ----------
    # Both policies and the stream-ordered pair are alive together and take turns, one step each per round: the
    # settling preamble (fixed, whatever --warmup says), then --warmup untimed rounds, then --steps timed rounds.
    # `value` is the better policy's mean; the gain is computed from steps that ran next to each other.
    settle(B)
    names = ["stream", "rowsync", "tilesync"]
    chains = [Chain(B, api.SYNC.STREAM), Chain(B, api.SYNC.ROW), Chain(B, api.SYNC.TILE)]
    tiles = chains[1].tiles
    if tiles[0] == tiles[1]:
        # the same stages and semaphores with both GEMMs in ONE launch: every workgroup works through the producer's
        # tiles it draws, then the consumer's, waiting on the tiles' semaphores in between (no second stream)
        names += ["rowsync_one_launch", "tilesync_one_launch"]
        chains += [Chain(B, api.SYNC.ROW, one_launch=True), Chain(B, api.SYNC.TILE, one_launch=True)]
    # settling on the chains that are timed (creating them left the device idle), then the --warmup rounds
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < MIN_WARM_S:
        for c in chains:
            c.step()
    for _ in range(args.warmup):
        for c in chains:
            c.step()
    torch.cuda.synchronize()
    step_times = {n: [] for n in names}
    wall = {n: 0.0 for n in names}
    for _ in range(args.steps):
        for n, c in zip(names, chains):
            t0 = time.perf_counter()
            step_times[n].append(c.step())        # returns after the step's last kernel has finished
            wall[n] += time.perf_counter() - t0
    for c in chains:
        c.close()
    policy = min((n for n in names if n != "stream"), key=lambda k: statistics.fmean(step_times[k]))
    ms_per_step = wall[policy] / args.steps * 1e3

    def spread(v):
        return {"mean": round(statistics.fmean(v), 2), "median": round(statistics.median(v), 2),
                "min": round(min(v), 2), "max": round(max(v), 2)}

    stream_mean = statistics.fmean(step_times["stream"])
    value = statistics.fmean(step_times[policy])

    # the kernels' own durations (stream-ordered, HIP events on the launching stream) for the roofline
    roof, _, _ = roofline_leg(B, 5, max(10, args.steps))
    # what the matrix pipes alone sustain on this machine (register operands, no LDS, no memory): the clock
    # drops under a device-wide MFMA load, further with random operands than with zeros
    zero_tf, zero_mhz = api.probe_mfma_rate(False)
    rand_tf, rand_mhz = api.probe_mfma_rate(True)
    roof["mfma_alone"] = {"zero_operands_tflops": round(zero_tf, 1), "zero_operands_mhz": round(zero_mhz),
                          "random_operands_tflops": round(rand_tf, 1), "random_operands_mhz": round(rand_mhz)}
    if roof["bound"] == "mfma":
        roof["mfma_alone"]["frac_of_random_operands_rate"] = round(roof["achieved"] / rand_tf, 4)

    # ---- the reference's own timed operands -------------------------------------------------
    # Its benchmark runs (--check false) fill the operands with constants, x = 0.05, w1 = 0.5, w2 = 0.01
    # (src/ml-bench/transformer/mlp.cu:283-290).  The instruction stream and the memory traffic are those of the
    # steps above; the multipliers of the matrix pipes see the same bits every clock, draw less, and the device holds
    # a higher clock under the big GEMMs.  `value` and `roofline` above are measured on random operands, which is what
    # a layer meets in use; this block says what the reference's protocol would have recorded on this device.
    reference_fill = None
    if not args.no_sweep:
        const = (torch.full_like(x_all, 0.05), torch.full_like(w1, 0.5), torch.full_like(w2, 0.01))
        torch.cuda.synchronize()
        rows = []
        for b in BATCHES:
            if b == B:
                settle(b)
            cs = [Chain(b, api.SYNC.STREAM, operands=const), Chain(b, api.SYNC.ROW, operands=const), Chain(b, api.SYNC.TILE, operands=const)]
            ts = interleaved(cs, 10, 20, split_first=True)
            for c in cs:
                c.close()
            g1, g2 = trimmed([v[1] for v in ts[0]])[0], trimmed([v[2] for v in ts[0]])[0]
            st, ro, ti = trimmed([v[0] for v in ts[0]])[0], trimmed(ts[1])[0], trimmed(ts[2])[0]
            rows.append({"B": b, "stream_us": round(st, 2), "rowsync_us": round(ro, 2), "tilesync_us": round(ti, 2),
                         "gemm1_us": round(g1, 2), "gemm2_us": round(g2, 2),
                         "best_gain_pct": round(100 - min(ro, ti) / st * 100, 2),
                         "roofline_frac": round(ideal_us(b) / min(ro, ti), 4)})
        big = rows[-1]
        reference_fill = {
            "operands": "x = 0.05, w1 = 0.5, w2 = 0.01 everywhere: the reference's timed runs (mlp.cu:283-290)",
            "gemm_frac_of_mfma_peak_at_B%d" % big["B"]: round(2.0 * big["B"] * HIDDEN * INNER / ((big["gemm1_us"] + big["gemm2_us"]) / 2 * 1e-6) / 1e12 / PEAK_FP16_TFLOPS, 4),
            "per_batch": rows,
        }
        del const

    out = {
        "metric": "GPT-3 MLP shard latency (us) + % gain vs kernel-boundary sync, B=1..2048",
        "value": round(value, 2),
        "unit": "us",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 (fp32 accumulate)", "data": "synthetic",
        "config": {"workload": "GPT-3 175B MLP 1/8 shard, B=%d: X[B,12288] x W1[12288,6144] +GeLU -> x W2[6144,12288]" % B,
                   "policy": policy, "tiles": list(tiles), "device": dev["arch"], "cus": dev["cus"]},
        # the same two GEMMs stream-ordered, timed in the same rounds as `value` (one step of each per round)
        "stream_ordered_us": round(stream_mean, 2),
        "gain_pct": round(100 - value / stream_mean * 100, 2),
        "gain_pct_median": round(100 - statistics.median(step_times[policy]) / statistics.median(step_times["stream"]) * 100, 2),
        "step_us": spread(step_times[policy]),
        "stream_step_us": spread(step_times["stream"]),
        "other_policy_step_us": {k: spread(v) for k, v in step_times.items() if k not in ("stream", policy)},
        "tflops": round(mlp_flops(B) / value / 1e6, 1),
        "roofline": roof,
        "per_batch": per_batch,
        "other_chains": other,
    }
    if reference_fill:
        out["reference_fill"] = reference_fill
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(x_host, w1_host, w2_host)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
