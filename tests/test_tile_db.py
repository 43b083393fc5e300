"""The tile table written by cusync_amd.tuner keeps the schema of the reference's tile_sizes_db.py
(src/ml-bench/transformer/tile_sizes_db.py:4-15, read by eval_mlp.py:141-213)."""
import numpy as np
import pytest

from cusync_amd import api, tile_sizes_db


def test_schema_matches_the_reference_table():
    db = tile_sizes_db.gpt3_mlp_mi355x
    assert set(db) >= {1, 16, 64, 256, 512, 1024, 2048}
    for m, e in db.items():
        assert len(e["TileSizes"]) == 2 and all(len(t) == 6 for t in e["TileSizes"])
        assert len(e["NumStages"]) == 2
        for key in ("baseline", "rowsync", "tilesync"):
            assert len(e[key]["split_ks"]) == 2 and all(k >= 1 for k in e[key]["split_ks"])
        assert set(e["tilesync"]) >= {"AvoidCustomOrder", "AvoidWaitKernel", "ReorderTileLoads", "NoAtomicAdd"}
        for (bm, bn, bk, wm, wn, wk) in e["TileSizes"]:
            assert bm % wm == 0 and bn % wn == 0 and wk == bk and (bm // wm) * (bn // wn) in (4, 8)   # four or eight wavefronts


@pytest.mark.gpu
@pytest.mark.parametrize("batch", [16, 256, 2048])
def test_chain_built_from_the_table_is_bit_identical_across_modes(batch):
    import torch
    from util import empty_dev, normal_f16, to_dev, to_host, uniform_f16
    hidden, inner = 12288, 6144
    w1, w2 = to_dev(normal_f16((hidden, inner), 2)), to_dev(normal_f16((inner, hidden), 3))
    x = to_dev(uniform_f16((batch, hidden), 1))
    outs = []
    for sync in (api.SYNC.STREAM, api.SYNC.ROW, api.SYNC.TILE):
        h, y = empty_dev((batch, inner), fill=float("nan")), empty_dev((batch, hidden), fill=float("nan"))
        torch.cuda.synchronize()
        m = api.Mlp.from_db(tile_sizes_db.gpt3_mlp_mi355x[batch], api.MODEL.GPT3, batch, hidden, inner, sync, w1.data_ptr(), w2.data_ptr())
        m.run(x.data_ptr(), h.data_ptr(), y.data_ptr(), runs=2)
        assert m.stage_state(1).spin_timeouts == 0
        assert list(m.tiles()) == tile_sizes_db.gpt3_mlp_mi355x[batch]["TileIds"]
        m.destroy()
        outs.append(to_host(y))
    assert np.array_equal(outs[0].view(np.uint16), outs[1].view(np.uint16))
    assert np.array_equal(outs[0].view(np.uint16), outs[2].view(np.uint16))
