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
