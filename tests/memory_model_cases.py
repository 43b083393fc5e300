"""Child process of test_gpu_memory_model.py: runs a fixed set of chains once each way the environment it was
started with says (CUSYNC_FORCE_ACQUIRE, CUSYNC_FORCE_RELEASE, CUSYNC_WAIT_KERNEL are read once per process by the
library) and writes a SHA-256 of every intermediate and output to the JSON file named on the command line.
The library's shortcuts around the plain release/acquire protocol (posts without a write-back after stores that
went through, waits without a cache invalidation over whole-line tiles, a host-side hold-back instead of the
wait kernel) may only change timing: the parent compares the digests of the processes with each other.

usage: python memory_model_cases.py out.json"""
import hashlib
import json
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

from cusync_amd import api  # noqa: E402
from util import empty_dev, normal_f16, to_dev, to_host, uniform_f16  # noqa: E402


def digest(t):
    return hashlib.sha256(np.ascontiguousarray(to_host(t)).view(np.uint16).tobytes()).hexdigest()


def mlp_case(out, name, model, batch, hidden, inner, sync, runs=3):
    import torch
    n1 = inner if model == api.MODEL.GPT3 else 2 * inner
    dw1, dw2 = to_dev(normal_f16((hidden, n1), 2)), to_dev(normal_f16((inner, hidden), 3))
    dx = [to_dev(uniform_f16((batch, hidden), 1)), to_dev(uniform_f16((batch, hidden), 101))]
    dh, dy = empty_dev((batch, n1), fill=float("nan")), empty_dev((batch, hidden), fill=float("nan"))
    torch.cuda.synchronize()
    mlp = api.Mlp(model, batch, hidden, inner, sync, dw1.data_ptr(), dw2.data_ptr())
    for r in range(runs):       # the last pass reads input 0; the ones before leave the other input's lines behind
        mlp.run(dx[(runs - 1 - r) % 2].data_ptr(), dh.data_ptr(), dy.data_ptr(), runs=1)
    for which in (0, 1):
        assert mlp.stage_state(which).spin_timeouts == 0
    out[name] = {"h": digest(dh), "y": digest(dy), "tiles": list(mlp.tiles() + mlp.splits())}
    mlp.destroy()


def attention_case(out, name, S, hidden, heads, sync, runs=3):
    import torch
    E = heads * 128
    dwqkv, dwo = to_dev(normal_f16((hidden, 3 * E), 21)), to_dev(normal_f16((E, hidden), 22))
    dx = [to_dev(uniform_f16((S, hidden), 1)), to_dev(uniform_f16((S, hidden), 101))]
    dqkv, do, dy = (empty_dev((S, 3 * E), fill=float("nan")), empty_dev((S, E), fill=float("nan")),
                    empty_dev((S, hidden), fill=float("nan")))
    torch.cuda.synchronize()
    layer = api.AttnLayer(S, hidden, heads, sync, dwqkv.data_ptr(), dwo.data_ptr())
    for r in range(runs):
        layer.run(dx[(runs - 1 - r) % 2].data_ptr(), dqkv.data_ptr(), do.data_ptr(), dy.data_ptr(), runs=1)
    for which in range(3):
        assert layer.stage_state(which).spin_timeouts == 0
    out[name] = {"qkv": digest(dqkv), "o": digest(do), "y": digest(dy)}
    layer.destroy()


def conv_case(out, name, N, H, W, Cc, layers, sync, runs=3):
    import torch
    rng = np.random.default_rng(31)
    dws = [to_dev((rng.standard_normal((Cc, 3, 3, Cc)) * np.sqrt(2.0 / (9 * Cc))).astype(np.float16)) for _ in range(layers)]
    dx = [to_dev(uniform_f16((N, H, W, Cc), 30)), to_dev(uniform_f16((N, H, W, Cc), 130))]
    dys = [empty_dev((N, H, W, Cc), fill=float("nan")) for _ in range(layers)]
    torch.cuda.synchronize()
    chain = api.ConvChain(N, H, W, Cc, [w.data_ptr() for w in dws], sync)
    for r in range(runs):
        chain.run(dx[(runs - 1 - r) % 2].data_ptr(), [y.data_ptr() for y in dys], runs=1)
    for which in range(layers):
        assert chain.stage_state(which).spin_timeouts == 0
    out[name] = {"y%d" % i: digest(y) for i, y in enumerate(dys)}
    chain.destroy()


def main(path):
    out = {}
    for batch in (256, 2048):
        for sync, tag in ((api.SYNC.ROW, "row"), (api.SYNC.TILE, "tile")):
            print("gpt3", batch, tag, flush=True)
            mlp_case(out, "gpt3_b%d_%s" % (batch, tag), api.MODEL.GPT3, batch, 12288, 6144, sync)
    print("llama 512 strided", flush=True)
    mlp_case(out, "llama_b512_strided", api.MODEL.LLAMA, 512, 8192, 2752, api.SYNC.STRIDED)
    for sync, tag in ((api.SYNC.ROW, "row"), (api.SYNC.STRIDED, "strided")):
        print("attention 1024", tag, flush=True)
        attention_case(out, "attention_s1024_%s" % tag, 1024, 12288, 12, sync)
    for sync, tag in ((api.SYNC.ROW, "row"), (api.SYNC.TILE, "tile")):
        print("conv 56x56x64", tag, flush=True)
        conv_case(out, "conv_56x56x64_%s" % tag, 32, 56, 56, 64, 2, sync)
    with open(path, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
    print("wrote", path, flush=True)


if __name__ == "__main__":
    main(sys.argv[1])
