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
"""
import argparse
import pprint
import statistics
import sys

from . import api

# tile id -> (wave grid M x N, pipeline stages)
WAVES = {api.TILE.T256x256x32: (4, 2, 4), api.TILE.T256x128x64: (2, 2, 2), api.TILE.T128x128x64: (2, 2, 2),
         api.TILE.T64x128x64: (1, 4, 2), api.TILE.T32x128x64: (1, 4, 2), api.TILE.T128x256x64: (2, 2, 2),
         api.TILE.T256x64x64: (4, 1, 2), api.TILE.T128x64x64: (2, 2, 2), api.TILE.T256x128x32: (2, 2, 3),
         api.TILE.T128x256x32: (2, 2, 3), api.TILE.T128x128x32: (2, 2, 3), api.TILE.T128x192x32: (2, 2, 3),
         api.TILE.T256x192x32: (4, 2, 4), api.TILE.D32x128x64: (1, 4, 4), api.TILE.D64x128x64: (1, 4, 3),
         api.TILE.D64x192x64: (2, 2, 4), api.TILE.T128x192x32_ALONE: (2, 2, 4)}

SHAPES = {"gpt3": (api.MODEL.GPT3, 12288, 6144), "llama": (api.MODEL.LLAMA, 8192, 2752)}


def candidates(batch, n1, n2):
    """(tile, split) choices worth timing for a GEMM with `batch` rows."""
    if batch <= 32:
        tiles, splits = [api.TILE.D32x128x64, api.TILE.T32x128x64], [2, 4, 8]
    elif batch <= 64:
        tiles, splits = [api.TILE.D64x192x64, api.TILE.D32x128x64, api.TILE.T64x128x64], [2, 4, 8]
    elif batch <= 128:
        tiles, splits = [api.TILE.D64x192x64, api.TILE.T128x128x64, api.TILE.T128x128x32], [1, 2, 4, 8]
    elif batch <= 512:
        tiles, splits = [api.TILE.D64x192x64, api.TILE.T128x192x32_ALONE, api.TILE.T256x192x32, api.TILE.T128x192x32, api.TILE.T128x128x32], [1, 2, 4]
    else:
        tiles, splits = [api.TILE.T256x192x32, api.TILE.T128x192x32, api.TILE.T128x256x32, api.TILE.T128x128x32], [1, 2]
    ok = lambda t, n: n % 192 == 0 or t not in (api.TILE.T128x192x32, api.TILE.T256x192x32, api.TILE.D64x192x64, api.TILE.T128x192x32_ALONE)
    return [(t, s) for t in tiles for s in splits if ok(t, n1)], [(t, s) for t in tiles for s in splits if ok(t, n2)]


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
            m.run(x.data_ptr(), h.data_ptr(), y.data_ptr(), runs=warm)
            out = m.run(x.data_ptr(), h.data_ptr(), y.data_ptr(), runs=timed, split=(sync == api.SYNC.STREAM))
            if m.stage_state(1).spin_timeouts:
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
        us = trimmed(r[1])
        log("B=%d GEMM1 tile %d split %d: %.1f us" % (batch, t, s, us))
        if best1 is None or us < best1[0]:
            best1 = (us, t, s)
    for (t, s) in c2:
        r = bench.run(batch, api.SYNC.STREAM, tile1=best1[1], tile2=t, split_k1=best1[2], split_k2=s)
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
        tile_opts = {"AvoidCustomOrder": False, "AvoidWaitKernel": False, "ReorderTileLoads": True, "NoAtomicAdd": True}
        base = api.OPT.NO_ATOMIC_ADD | api.OPT.REORDER_TILE_LOADS
        tile = trimmed(bench.run(batch, api.SYNC.TILE, timed=20, opts=base, **kw))
        t_aco = bench.run(batch, api.SYNC.TILE, timed=20, opts=base | api.OPT.AVOID_CUSTOM_ORDER, **kw)
        if t_aco is not None and trimmed(t_aco) < tile:
            tile, tile_opts["AvoidCustomOrder"] = trimmed(t_aco), True
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--model", choices=sorted(SHAPES), default="gpt3")
    ap.add_argument("--batches", default="1,16,64,256,512,1024,2048")
    ap.add_argument("--out", default=None, help="file to write the table to (default: stdout)")
    args = ap.parse_args()
    model, hidden, inner = SHAPES[args.model]
    bench = Bench(model, hidden, inner)
    log = lambda s: print(s, file=sys.stderr, flush=True)
    db = {}
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
