"""The tile tables written by cusync_amd.tuner keep the schema of the reference's tile_sizes_db.py
(src/ml-bench/transformer/tile_sizes_db.py:4-15 for the MLPs, :364-392 for the attention chain; read by
eval_mlp.py:141-213), and a chain built from an entry computes what the oracle computes."""
import numpy as np
import pytest

import oracle as orc
from cusync_amd import api, tile_sizes_db


@pytest.mark.parametrize("name", ["gpt3_mlp_mi355x", "llama_mlp_mi355x"])
def test_schema_matches_the_reference_table(name):
    db = getattr(tile_sizes_db, name)
    assert set(db) >= {1, 16, 64, 256, 512, 1024, 2048}
    for m, e in db.items():
        assert len(e["TileSizes"]) == 2 and all(len(t) == 6 for t in e["TileSizes"])
        assert len(e["NumStages"]) == 2
        for key in ("baseline", "rowsync", "tilesync"):
            assert len(e[key]["split_ks"]) == 2 and all(k >= 1 for k in e[key]["split_ks"])
        assert set(e["tilesync"]) >= {"AvoidCustomOrder", "AvoidWaitKernel", "ReorderTileLoads", "NoAtomicAdd"}
        for (bm, bn, bk, wm, wn, wk) in e["TileSizes"]:
            assert bm % wm == 0 and bn % wn == 0 and wk == bk and (bm // wm) * (bn // wn) in (4, 8)   # four or eight wavefronts


def test_attention_table_schema():
    # {seqlen: {batch: entry}}, seqlen 0 = no key/value cache (tile_sizes_db.py:364-392)
    db = tile_sizes_db.gpt3_attention_mi355x
    assert set(db) == {0} and set(db[0]) >= {256, 512, 1024, 2048}
    for s, e in db[0].items():
        assert len(e["TileSizes"]) == 2 and len(e["TileIds"]) == 2 and len(e["NumStages"]) == 2
        for key in ("baseline", "rowsync", "tilesync", "consecutivesync"):
            assert e[key]["KVSplitBlocks"] >= 0
        assert set(e["tilesync"]) >= {"AvoidCustomOrder", "AvoidWaitKernel", "ReorderTileLoads"}


@pytest.mark.gpu
@pytest.mark.parametrize("model,batch", [("gpt3", 16), ("gpt3", 256), ("gpt3", 2048), ("llama", 1), ("llama", 64), ("llama", 512), ("llama", 2048)])
def test_chain_built_from_the_table_matches_the_oracle_in_every_mode(model, batch):
    # from_db takes tiles, k-slices and option bits from the entry (AvoidWaitKernel where the tuner found both launches
    # resident together); Y is checked against the oracle, and the modes against each other bit for bit
    import torch
    from util import assert_close, empty_dev, normal_f16, sample_rows, to_dev, to_host, uniform_f16
    print("table", model, batch, flush=True)
    llama = model == "llama"
    hidden, inner = (8192, 2752) if llama else (12288, 6144)
    db = tile_sizes_db.llama_mlp_mi355x if llama else tile_sizes_db.gpt3_mlp_mi355x
    w1h, w2h = normal_f16((hidden, 2 * inner if llama else inner), 2), normal_f16((inner, hidden), 3)
    w1, w2 = to_dev(w1h), to_dev(w2h)
    xh = uniform_f16((batch, hidden), 1)
    x, x_other = to_dev(xh), to_dev(uniform_f16((batch, hidden), 101))
    outs = []
    for sync in (api.SYNC.STREAM, api.SYNC.ROW, api.SYNC.STRIDED if llama else api.SYNC.TILE):
        h, y = empty_dev((batch, 2 * inner if llama else inner)), empty_dev((batch, hidden))
        m = api.Mlp.from_db(db[batch], api.MODEL.LLAMA if llama else api.MODEL.GPT3, batch, hidden, inner, sync, w1.data_ptr(), w2.data_ptr())
        for xin in (x_other, x):         # second pass: another input, intermediates refilled with NaN
            h.fill_(float("nan")); y.fill_(float("nan"))
            torch.cuda.synchronize()
            m.run(xin.data_ptr(), h.data_ptr(), y.data_ptr(), runs=1)
        assert m.stage_state(1).spin_timeouts == 0
        assert list(m.tiles()) == db[batch]["TileIds"]
        m.destroy()
        outs.append((to_host(h), to_host(y)))
    h, y = outs[0]
    rows = sample_rows(batch)
    xs = np.ascontiguousarray(xh[rows])
    if llama:
        hh = h.reshape(-1)[:batch * inner].reshape(batch, inner)
        assert_close(hh[rows], orc.gemm_swiglu(xs, w1h, inner), "silu(gate)*up rows")
    else:
        hh = h
        assert_close(hh[rows], orc.gemm(xs, w1h, orc.EPI_GELU), "H rows")
    assert_close(y[rows], orc.gemm(np.ascontiguousarray(hh[rows]), w2h), "Y rows")
    for other in outs[1:]:
        assert np.array_equal(y.view(np.uint16), other[1].view(np.uint16))


@pytest.mark.gpu
@pytest.mark.parametrize("seq", [256, 2048])
def test_attention_chain_built_from_the_table(seq):
    import torch
    from util import assert_close, empty_dev, normal_f16, sample_rows, to_dev, to_host, uniform_f16
    hidden, heads = 12288, 12
    e = heads * 128
    entry = tile_sizes_db.gpt3_attention_mi355x[0][seq]
    wqkv_h, wo_h = normal_f16((hidden, 3 * e), 2), normal_f16((e, hidden), 3)
    wqkv, wo = to_dev(wqkv_h), to_dev(wo_h)
    xh = uniform_f16((seq, hidden), 1)
    x = to_dev(xh)
    outs = []
    for key, sync in (("baseline", api.SYNC.STREAM), ("consecutivesync", api.SYNC.STRIDED)):
        qkv, o, y = empty_dev((seq, 3 * e), fill=float("nan")), empty_dev((seq, e), fill=float("nan")), empty_dev((seq, hidden), fill=float("nan"))
        torch.cuda.synchronize()
        layer = api.AttnLayer(seq, hidden, heads, sync, wqkv.data_ptr(), wo.data_ptr(), tile1=entry["TileIds"][0], tile3=entry["TileIds"][1],
                              kv_split_blocks=entry[key]["KVSplitBlocks"])
        layer.run(x.data_ptr(), qkv.data_ptr(), o.data_ptr(), y.data_ptr(), runs=1)
        assert all(layer.stage_state(i).spin_timeouts == 0 for i in range(3))
        assert list(layer.tiles()) == entry["TileIds"]
        layer.destroy()
        outs.append((to_host(qkv), to_host(o), to_host(y)))
    qkv, o, y = outs[0]
    rows = sample_rows(seq)
    assert_close(qkv[rows], orc.gemm(np.ascontiguousarray(xh[rows]), wqkv_h), "QKV rows")
    assert_close(o, orc.attention(qkv, heads, 128, True), "O")
    assert_close(y[rows], orc.gemm(np.ascontiguousarray(o[rows]), wo_h), "Y rows")
    assert np.array_equal(y.view(np.uint16), outs[1][2].view(np.uint16))
