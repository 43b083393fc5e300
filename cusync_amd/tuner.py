"""Per-batch tuner for the MLP chains on one MI355X.

Takes the place of the hand-kept table of the reference (src/ml-bench/transformer/tile_sizes_db.py:4-15,
consumed by eval_mlp.py:141-213): for every batch size it times candidate tile shapes and k-slice counts
stream-ordered, then the CuSync policies with the option bits that are safe for the winning shapes, and
writes the result in the reference's schema:

    <name> = { M: {"TileSizes": [[BM, BN, BK, WaveM, WaveN, BK], [...]], "NumStages": [s1, s2],
                   "baseline": {"split_ks": [k1, k2]}, "rowsync": {"split_ks": [...]},
                   "tilesync": {"split_ks": [...], "AvoidCustomOrder": b, "AvoidWaitKernel": b,
                                "ReorderTileLoads": b, "NoAtomicAdd": b}}, ... }

plus, per entry, the tile ids of this library ("TileIds") and the measured latencies ("us").

    python -m cusync_amd.tuner --model gpt3 --batches 1,16,64,256,512,1024,2048 --out cusync_amd/tile_sizes_db.py
    python -m cusync_amd.tuner --model llama --out cusync_amd/tile_sizes_db.py        # "tilesync" is StridedSync there
    python -m cusync_amd.tuner --model attention --batches 256,512,1024,2048 --out cusync_amd/tile_sizes_db.py

(each call appends one table to the file).  The attention table follows the reference's gpt3_attention tables
(tile_sizes_db.py:364-392: {seqlen: {batch: entry}} with seqlen 0 = no key/value cache); its two tile shapes are
those of the QKV projection and the output projection, the fused attention kernel between them has one shape.
"""
import argparse
import pprint
import statistics
import sys
import time

from . import api

# tile id -> (wave grid M x N, pipeline stages)
WAVES = {api.TILE.T256x256x32: (4, 2, 4), api.TILE.T256x128x64: (2, 2, 2), api.TILE.T128x128x64: (2, 2, 2),
         api.TILE.T64x128x64: (1, 4, 2), api.TILE.T32x128x64: (1, 4, 2), api.TILE.T128x256x64: (2, 2, 2),
         api.TILE.T256x64x64: (4, 1, 2), api.TILE.T128x64x64: (2, 2, 2), api.TILE.T256x128x32: (2, 2, 3),
         api.TILE.T128x256x32: (2, 2, 3), api.TILE.T128x128x32: (2, 2, 3), api.TILE.T128x192x32: (2, 2, 3),
         api.TILE.T256x192x32: (4, 2, 4), api.TILE.D32x128x64: (1, 4, 4), api.TILE.D64x128x64: (1, 4, 3),
         api.TILE.D64x192x64: (2, 2, 4), api.TILE.T128x192x32_ALONE: (2, 2, 4), api.TILE.T256x384x32: (2, 4, 3),
         api.TILE.T256x192x64: (4, 2, 4), api.TILE.D128x192x64: (2, 2, 3)}

MIN_WARM_S = 0.025
SHAPES = {"gpt3": (api.MODEL.GPT3, 12288, 6144), "llama": (api.MODEL.LLAMA, 8192, 2752)}


def resident_share(tile, M, N, split):
    """Share of the device's workgroup slots a launch of this GEMM takes (1.0 = every slot)."""
    g = api.gemm_grid(tile, M, N, split)
    resident = api._lib.load().cusync_gemm_max_resident(tile)
    return min(g[0] * g[1] * g[2], resident) / float(resident)


def candidates(batch, n1, n2):
    """(tile, split) choices worth timing for a GEMM with `batch` rows."""
    if batch <= 32:
        tiles, splits = [api.TILE.D32x128x64, api.TILE.T32x128x64], [2, 4, 8, 16]
    elif batch <= 64:
        tiles, splits = [api.TILE.D64x192x64, api.TILE.D32x128x64, api.TILE.T64x128x64], [2, 4, 8, 16]
    elif batch <= 128:
        tiles, splits = [api.TILE.D64x192x64, api.TILE.T128x128x64, api.TILE.T128x128x32], [1, 2, 4, 8]
    elif batch <= 512:
        tiles, splits = [api.TILE.D64x192x64, api.TILE.D128x192x64, api.TILE.T128x192x32_ALONE, api.TILE.T256x192x64, api.TILE.T256x192x32, api.TILE.T128x192x32, api.TILE.T128x128x32], [1, 2, 4, 8]
    else:
        tiles, splits = [api.TILE.T256x192x64, api.TILE.T256x384x32, api.TILE.T256x192x32, api.TILE.T128x192x32, api.TILE.T128x256x32, api.TILE.T128x128x32], [1, 2]
    if n1 % 192 or n2 % 192:        # the LLaMA shard (5504 and 8192 columns): also the 256-wide tiles
        if batch > 512:
            tiles = tiles + [api.TILE.T256x256x32, api.TILE.T128x192x32_ALONE]
        elif batch > 32:
            tiles = tiles + [api.TILE.D64x128x64]
    # the register-staged tiles have no SwiGLU epilogue path worth timing against the direct-to-LDS ones
    return [(t, s) for t in tiles for s in splits], [(t, s) for t in tiles for s in splits]


def trimmed(times):
    t = sorted(times)
    return statistics.fmean(t[:max(1, len(t) - len(t) // 10)])


class Bench:
    def __init__(self, model, hidden, inner):
        import torch
        self.torch = torch
        self.model, self.hidden, self.inner = model, hidden, inner
        n1 = inner if model == api.MODEL.GPT3 else 2 * inner
        g = torch.Generator(device="cuda").manual_seed(2)
        self.w1 = (torch.randn((hidden, n1), device="cuda", generator=g) * 0.02).half()
        self.w2 = (torch.randn((inner, hidden), device="cuda", generator=g) * 0.02).half()
        self.n1 = n1

    def run(self, batch, sync, warm=15, timed=20, **kw):
        torch = self.torch
        x = (torch.rand((batch, self.hidden), device="cuda") * 2 - 1).half()
        h = torch.empty((batch, self.n1), dtype=torch.float16, device="cuda")
        y = torch.empty((batch, self.hidden), dtype=torch.float16, device="cuda")
        torch.cuda.synchronize()
        m = api.Mlp(self.model, batch, self.hidden, self.inner, sync, self.w1.data_ptr(), self.w2.data_ptr(), **kw)
        try:
            # after the idle gap a new handle leaves, the device runs big GEMMs up to a quarter slower from the 2nd to
            # about the 15th millisecond of load: warm up for at least MIN_WARM_S before anything is timed
            t0 = time.perf_counter()
            m.run(x.data_ptr(), h.data_ptr(), y.data_ptr(), runs=warm)
            while time.perf_counter() - t0 < MIN_WARM_S:
                m.run(x.data_ptr(), h.data_ptr(), y.data_ptr(), runs=5)
            out = m.run(x.data_ptr(), h.data_ptr(), y.data_ptr(), runs=timed, split=(sync == api.SYNC.STREAM))
            if m.stage_state(1).spin_timeouts:
                return None
        except api.CuSyncError:      # a candidate the library refuses (k-slices that do not fit this K)
            return None
        finally:
            m.destroy()
        return out

    def defaults(self, batch):
        """(tiles, k-slices) the library picks by itself for this batch."""
        m = api.Mlp(self.model, batch, self.hidden, self.inner, api.SYNC.STREAM, self.w1.data_ptr(), self.w2.data_ptr())
        try:
            return m.tiles(), m.splits()
        finally:
            m.destroy()


def tune_batch(bench, batch, log):
    c1, c2 = candidates(batch, bench.n1, bench.hidden)
    # the two GEMMs of the stream-ordered chain are independent choices: time each candidate once in a chain
    # whose other GEMM uses the first candidate, and read its own duration
    best1 = best2 = None
    bench.run(batch, api.SYNC.STREAM, warm=30, timed=1, tile1=c1[0][0], tile2=c2[0][0], split_k1=c1[0][1], split_k2=c2[0][1])   # clocks up
    for (t, s) in c1:
        r = bench.run(batch, api.SYNC.STREAM, tile1=t, tile2=c2[0][0], split_k1=s, split_k2=c2[0][1])
        if r is None:
            continue
        us = trimmed(r[1])
        log("B=%d GEMM1 tile %d split %d: %.1f us" % (batch, t, s, us))
        if best1 is None or us < best1[0]:
            best1 = (us, t, s)
    for (t, s) in c2:
        r = bench.run(batch, api.SYNC.STREAM, tile1=best1[1], tile2=t, split_k1=best1[2], split_k2=s)
        if r is None:
            continue
        us = trimmed(r[2])
        log("B=%d GEMM2 tile %d split %d: %.1f us" % (batch, t, s, us))
        if best2 is None or us < best2[0]:
            best2 = (us, t, s)
    # The fastest pair of kernels need not make the fastest chain under CuSync (a producer tile that fills its CUs
    # leaves the consumer nowhere to run): the library's own choice for this batch is timed as a chain too, and
    # the pair whose best mode is faster goes into the table.
    def chain(kw):
        stream = trimmed(bench.run(batch, api.SYNC.STREAM, timed=20, **kw)[0])
        row = trimmed(bench.run(batch, api.SYNC.ROW, timed=20, **kw))
        # TileSync with the option bits of the reference's table; AvoidCustomOrder is always safe here, AvoidWaitKernel
        # only when producer and consumer fit on the device together (nothing can then keep a producer workgroup off it)
        # (the LLaMA chain's tile policy is StridedSync, whose semaphores count to two: atomic adds, TB/mlp.cu:9-14, 109)
        llama = bench.model == api.MODEL.LLAMA
        mode = api.SYNC.STRIDED if llama else api.SYNC.TILE
        tile_opts = {"AvoidCustomOrder": False, "AvoidWaitKernel": False, "ReorderTileLoads": True, "NoAtomicAdd": not llama}
        base = api.OPT.REORDER_TILE_LOADS | (0 if llama else api.OPT.NO_ATOMIC_ADD)
        tile = trimmed(bench.run(batch, mode, timed=20, opts=base, **kw))
        t_aco = bench.run(batch, mode, timed=20, opts=base | api.OPT.AVOID_CUSTOM_ORDER, **kw)
        if t_aco is not None and trimmed(t_aco) < tile:
            tile, tile_opts["AvoidCustomOrder"] = trimmed(t_aco), True
        share = (resident_share(kw["tile1"], batch, bench.n1, kw["split_k1"]) +
                 resident_share(kw["tile2"], batch, bench.hidden, kw["split_k2"]))
        if share <= 1.0:       # both launches are resident together: no wait kernel is needed (CS/cusync.h:193-196, 205-206)
            o = base | api.OPT.AVOID_WAIT_KERNEL | (api.OPT.AVOID_CUSTOM_ORDER if tile_opts["AvoidCustomOrder"] else 0)
            t_awk = bench.run(batch, mode, timed=20, opts=o, **kw)
            if t_awk is not None and trimmed(t_awk) < tile:
                tile, tile_opts["AvoidWaitKernel"] = trimmed(t_awk), True
        return stream, row, tile, tile_opts

    tuned = dict(tile1=best1[1], tile2=best2[1], split_k1=best1[2], split_k2=best2[2])
    stream, row, tile, tile_opts = chain(tuned)
    log("B=%d chain of the fastest kernels: stream %.1f row %.1f tile %.1f %s" % (batch, stream, row, tile, tile_opts))
    dt, ds = bench.defaults(batch)
    dflt = dict(tile1=dt[0], tile2=dt[1], split_k1=ds[0], split_k2=ds[1])
    if dflt != tuned:
        d_stream, d_row, d_tile, d_opts = chain(dflt)
        log("B=%d chain of the library's choice %s: stream %.1f row %.1f tile %.1f" % (batch, dflt, d_stream, d_row, d_tile))
        if min(d_stream, d_row, d_tile) < min(stream, row, tile):
            stream, row, tile, tile_opts = d_stream, d_row, d_tile, d_opts
            g = bench.run(batch, api.SYNC.STREAM, **dflt)
            best1, best2 = (trimmed(g[1]), dt[0], ds[0]), (trimmed(g[2]), dt[1], ds[1])
    log("B=%d chain: stream %.1f row %.1f tile %.1f %s" % (batch, stream, row, tile, tile_opts))

    def sizes(t):
        bm, bn, bk = api.tile_shape(t)
        wm, wn, _ = WAVES[t]
        return [bm, bn, bk, bm // wm, bn // wn, bk]

    splits = [best1[2], best2[2]]
    return {
        "TileSizes": [sizes(best1[1]), sizes(best2[1])],
        "TileIds": [best1[1], best2[1]],
        "NumStages": [WAVES[best1[1]][2], WAVES[best2[1]][2]],
        "baseline": {"split_ks": splits},
        "rowsync": {"split_ks": splits},
        "tilesync": dict(split_ks=splits, **tile_opts),
        "us": {"baseline": round(stream, 1), "rowsync": round(row, 1), "tilesync": round(tile, 1),
               "gemm1": round(best1[0], 1), "gemm2": round(best2[0], 1)},
    }


def tune_attention(seq, log, hidden=12288, heads=12):
    """Tile shapes of the two projections and the key/value split of the attention chain at `seq` rows."""
    import torch
    e = heads * 128
    g = torch.Generator(device="cuda").manual_seed(4)
    wqkv = (torch.randn((hidden, 3 * e), device="cuda", generator=g) * 0.02).half()
    wo = (torch.randn((e, hidden), device="cuda", generator=g) * 0.02).half()
    x = (torch.rand((seq, hidden), device="cuda", generator=g) * 2 - 1).half()
    qkv = torch.empty((seq, 3 * e), dtype=torch.float16, device="cuda")
    o = torch.empty((seq, e), dtype=torch.float16, device="cuda")
    y = torch.empty((seq, hidden), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()

    def run(sync, **kw):
        layer = api.AttnLayer(seq, hidden, heads, sync, wqkv.data_ptr(), wo.data_ptr(), **kw)
        try:
            t0 = time.perf_counter()
            layer.run(x.data_ptr(), qkv.data_ptr(), o.data_ptr(), y.data_ptr(), runs=10)
            while time.perf_counter() - t0 < MIN_WARM_S:        # (see Bench.run)
                layer.run(x.data_ptr(), qkv.data_ptr(), o.data_ptr(), y.data_ptr(), runs=5)
            t, st = layer.run(x.data_ptr(), qkv.data_ptr(), o.data_ptr(), y.data_ptr(), runs=20, stages=True)
            return trimmed(t), [trimmed([v[i] for v in st]) for i in range(3)], layer.tiles()
        finally:
            layer.destroy()

    if seq <= 256:
        tiles = [api.TILE.D64x192x64, api.TILE.D128x192x64, api.TILE.T128x192x32_ALONE, api.TILE.T128x128x32]
    elif seq <= 1024:
        tiles = [api.TILE.T128x192x32_ALONE, api.TILE.T128x192x32, api.TILE.T256x192x64, api.TILE.T256x192x32, api.TILE.T128x128x32]
    else:
        tiles = [api.TILE.T128x192x32, api.TILE.T256x192x64, api.TILE.T256x384x32, api.TILE.T256x192x32, api.TILE.T128x192x32_ALONE]
    run(api.SYNC.STREAM)        # clocks up
    best1 = best3 = None
    for t in tiles:
        total, st, _ = run(api.SYNC.STREAM, tile1=t, tile3=tiles[0])
        log("S=%d QKV projection tile %d: %.1f us" % (seq, t, st[0]))
        if best1 is None or st[0] < best1[0]:
            best1 = (st[0], t)
    for t in tiles:
        total, st, _ = run(api.SYNC.STREAM, tile1=best1[1], tile3=t)
        log("S=%d output projection tile %d: %.1f us" % (seq, t, st[2]))
        if best3 is None or st[2] < best3[0]:
            best3 = (st[2], t)
    bestkv = None
    for kv in (0, 4, 8, 16):
        total, st, _ = run(api.SYNC.STREAM, tile1=best1[1], tile3=best3[1], kv_split_blocks=kv)
        log("S=%d attention with at most %d key/value blocks per workgroup: %.1f us" % (seq, kv, st[1]))
        if bestkv is None or st[1] < bestkv[0]:
            bestkv = (st[1], kv)
    kw = dict(tile1=best1[1], tile3=best3[1], kv_split_blocks=bestkv[1])
    us = {}
    for name, sync in (("baseline", api.SYNC.STREAM), ("rowsync", api.SYNC.ROW), ("tilesync", api.SYNC.TILE), ("consecutivesync", api.SYNC.STRIDED)):
        us[name] = round(run(sync, **kw)[0], 1)
    us.update(qkv=round(best1[0], 1), attention=round(bestkv[0], 1), out_proj=round(best3[0], 1))
    log("S=%d chain: %s" % (seq, us))

    def sizes(t):
        bm, bn, bk = api.tile_shape(t)
        wm, wn, _ = WAVES[t]
        return [bm, bn, bk, bm // wm, bn // wn, bk]

    entry = {"TileSizes": [sizes(best1[1]), sizes(best3[1])], "TileIds": [best1[1], best3[1]],
             "NumStages": [WAVES[best1[1]][2], WAVES[best3[1]][2]], "KVSplitBlocks": bestkv[1]}
    for key in ("baseline", "rowsync", "consecutivesync"):
        entry[key] = {"KVSplitBlocks": bestkv[1]}
    entry["tilesync"] = {"KVSplitBlocks": bestkv[1], "AvoidCustomOrder": False, "AvoidWaitKernel": False, "ReorderTileLoads": True, "NoAtomicAdd": True}
    entry["us"] = us
    return entry


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--model", choices=sorted(SHAPES) + ["attention"], default="gpt3")
    ap.add_argument("--batches", default="1,16,64,256,512,1024,2048")
    ap.add_argument("--out", default=None, help="file to write the table to (default: stdout)")
    args = ap.parse_args()
    log = lambda s: print(s, file=sys.stderr, flush=True)
    db = {}
    if args.model == "attention":
        db[0] = {}
        for s in sorted((int(v) for v in args.batches.split(",")), reverse=True):
            db[0][s] = tune_attention(s, log)
        name = "gpt3_attention_mi355x"
    else:
        model, hidden, inner = SHAPES[args.model]
        bench = Bench(model, hidden, inner)
        for b in sorted((int(v) for v in args.batches.split(",")), reverse=True):
            db[b] = tune_batch(bench, b, log)
        name = "%s_mlp_mi355x" % args.model
    text = ("# Written by `python -m cusync_amd.tuner --model %s`; schema of the reference's tile_sizes_db.py.\n"
            "# Dictionary of tile sizes for each M\n%s = %s\n" % (args.model, name, pprint.pformat(db, width=120, sort_dicts=False)))
    if args.out:
        with open(args.out, "a") as f:
            f.write(text)
    else:
        print(text)


if __name__ == "__main__":
    main()
