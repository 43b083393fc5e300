"""The command-line drivers (cusync_amd/drivers/*.cpp, plain host C++ on the C ABI) keep the options and
the START-/END- output protocol of the reference's drivers (src/ml-bench/transformer/mlp.cu:876-1120,
attention.cu:874-1075, src/ml-bench/volta_conv2d/resnet.cu:309-345, 754-827) and pass their own --check."""
import json
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu

BIN = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "cusync_amd", "bin")


def run(name, *args):
    exe = os.path.join(BIN, name)
    assert os.path.exists(exe), "driver not built: run make -C cusync_amd/drivers"
    p = subprocess.run([exe] + list(args), capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stdout[-2000:] + p.stderr[-2000:]
    return p.stdout


def between(out, start, end):
    lines = out.splitlines()
    i = next(k for k, l in enumerate(lines) if l.startswith(start))
    j = next(k for k, l in enumerate(lines) if l.startswith(end))
    return lines[i + 1:j], lines[j]


@pytest.mark.parametrize("model,batch,sync", [("gpt3", 64, "tilesync"), ("gpt3", 300, "rowsync"), ("llama", 128, "stridedsync")])
def test_mlp_driver(model, batch, sync):
    out = run("mlp", "--model", model, "--batch", str(batch), "--check", "true", "--sync", sync, "--runs", "5")
    base, _ = between(out, "START-BASELINE:", "END-BASELINE:")
    over, _ = between(out, "START-OVERLAPPED:", "END-OVERLAPPED:")
    rows = [json.loads(l) for l in base]
    assert len(rows) == 5 and all(r["Total"] > 0 and r["matmul1Time"] > 0 and r["matmul2Time"] > 0 for r in rows)
    assert len(over) == 5 and all(json.loads(l)["Total"] > 0 for l in over)
    assert "check: passed" in out


def test_mlp_driver_repacked_weights_one_launch():
    out = run("mlp", "--model", "gpt3", "--batch", "16", "--check", "true", "--sync", "rowsync", "--runs", "3",
              "--repack-weights", "true", "--one-launch", "true")
    over, _ = between(out, "START-OVERLAPPED:", "END-OVERLAPPED:")
    assert len(over) == 3 and "check: passed" in out


def test_mlp_driver_usage_error():
    p = subprocess.run([os.path.join(BIN, "mlp"), "--model", "bert"], capture_output=True, text=True, timeout=60)
    assert p.returncode != 0 and "usage" in p.stderr


@pytest.mark.parametrize("batch,seqlen", [(256, 0), (16, 512)])
def test_attention_driver(batch, seqlen):
    out = run("attention", "--model", "gpt3", "--batch", str(batch), "--seqlen", str(seqlen), "--check", "true", "--runs", "5")
    _, end = between(out, "START-BASELINE:", "END-BASELINE:")
    d = json.loads(re.search(r"\{.*\}", end).group(0))
    assert d["Total"] > 0 and d["matmul1Time"] > 0 and d["attentionTime"] > 0 and d["matmul4Time"] > 0
    _, end = between(out, "START-OVERLAPPED", "END-OVERLAPPED:")
    assert json.loads(re.search(r"\{.*\}", end).group(0))["Total"] > 0
    assert "check: passed" in out


@pytest.mark.parametrize("shape,layers,sync", [((4, 28, 28, 64), 2, "tilesync"), ((2, 14, 14, 128), 4, "rowsync")])
def test_resnet_driver(shape, layers, sync):
    n, h, w, c = shape
    out = run("resnet", "--n", str(n), "--h", str(h), "--w", str(w), "--c", str(c), "--layers", str(layers),
              "--iterations", "5", "--ref-check", "--sync", sync)
    _, end = between(out, "START-BASELINE:", "END-BASELINE:")
    assert end.count("Conv") == layers and "micro seconds" in end
    _, end = between(out, "START-OVERLAP:", "END-OVERLAP")
    assert float(re.search(r"Total: ([0-9.]+)", end).group(1)) > 0
    assert "check: passed" in out


@pytest.mark.parametrize("shape,extra", [((8, 14, 14, 256), ()), ((2, 7, 7, 512), ("--split_k_slices", "3")), ((2, 7, 7, 512), ("--split_k_slices", "1"))])
def test_resnet_driver_deep_layers(shape, extra):
    # 256 and 512 channels (resnet_results.csv): the chain cuts the tiles' steps into runs by itself, or as --split_k_slices says
    n, h, w, c = shape
    out = run("resnet", "--n", str(n), "--h", str(h), "--w", str(w), "--c", str(c), "--iterations", "5", "--ref-check", "--sync", "rowsync", *extra)
    _, end = between(out, "START-OVERLAP:", "END-OVERLAP")
    assert float(re.search(r"Total: ([0-9.]+)", end).group(1)) > 0
    assert "check: passed" in out


def test_mlp_stages_driver_against_oracle(tmp_path):
    """The reference's own loop (CuStage + CuSyncGemm objects, invokeWaitKernel, incrementIter) at 256 and 2048 rows,
    both policies, on inputs this test writes; the launchers' H and Y against the CPU oracle on sampled rows, and
    bit for bit against each other across policies."""
    import numpy as np
    import oracle as orc
    from util import assert_close, normal_f16, sample_rows, uniform_f16
    hidden, inner, batches = 12288, 6144, (256, 2048)
    x, w1, w2 = uniform_f16((max(batches), hidden), 1), normal_f16((hidden, inner), 2), normal_f16((inner, hidden), 3)
    for name, a in (("x", x), ("w1", w1), ("w2", w2)):
        a.tofile(tmp_path / (name + ".bin"))
    out = run("mlp_stages", "--batch", ",".join(str(b) for b in batches), "--sync", "both", "--runs", "5", "--check", "true",
              "--load", str(tmp_path), "--dump", str(tmp_path))
    assert out.count("check: passed") == 4
    rows = [json.loads(l) for l in out.splitlines() if l.startswith('{"batch"')]
    assert [(r["batch"], r["sync"]) for r in rows] == [(256, "rowsync"), (256, "tilesync"), (2048, "rowsync"), (2048, "tilesync")]
    for r in rows:
        assert r["runs"] == 5 and r["launcher_us"] > 0 and r["handle_us"] > 0
    for b in batches:
        got = {}
        for sync in ("rowsync", "tilesync"):
            h = np.fromfile(tmp_path / ("h_%d_%s.bin" % (b, sync)), dtype=np.float16).reshape(b, inner)
            y = np.fromfile(tmp_path / ("y_%d_%s.bin" % (b, sync)), dtype=np.float16).reshape(b, hidden)
            got[sync] = (h, y)
        sel = sample_rows(b)
        h, y = got["rowsync"]
        assert_close(h[sel], orc.gemm(np.ascontiguousarray(x[sel]), w1, orc.EPI_GELU), "H rows, %d" % b)
        assert_close(y[sel], orc.gemm(np.ascontiguousarray(h[sel]), w2), "Y rows, %d" % b)
        assert np.array_equal(got["tilesync"][0].view(np.uint16), h.view(np.uint16))
        assert np.array_equal(got["tilesync"][1].view(np.uint16), y.view(np.uint16))


def test_mlp_stages_driver_usage_error():
    p = subprocess.run([os.path.join(BIN, "mlp_stages"), "--batch", "0"], capture_output=True, text=True, timeout=60)
    assert p.returncode != 0 and "usage" in p.stderr
