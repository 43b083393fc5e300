"""What the library's kernels leave out of the plain release/acquire protocol must not change a bit of any result.

The shortcuts: a post after stores that were written through (sc1) is a relaxed add, with no write-back of the
XCD's L2; a wait over producer tiles that are whole 128-byte lines skips the cache invalidation; a producer launch
that fills the device is waited for on the host instead of by the wait kernel.  Each has a switch read once per
process (CUSYNC_FORCE_RELEASE, CUSYNC_FORCE_ACQUIRE, CUSYNC_WAIT_KERNEL), so the comparison runs child processes.
The second test runs one handle many times back to back over the same intermediate buffer with nothing of
torch's between the runs: a line of an earlier pass left in a cache would end up in a later pass's output."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from cusync_amd import api
from util import empty_dev, normal_f16, to_dev, to_host, uniform_f16

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
SWITCHES = ("CUSYNC_FORCE_ACQUIRE", "CUSYNC_FORCE_RELEASE", "CUSYNC_WAIT_KERNEL")


def run_child(tmp_path, name, env_extra):
    env = {k: v for k, v in os.environ.items() if k not in SWITCHES}
    env.update(env_extra)
    out = tmp_path / (name + ".json")
    print("child", name, env_extra, flush=True)
    r = subprocess.run([sys.executable, "-u", os.path.join(HERE, "memory_model_cases.py"), str(out)], env=env,
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=400, text=True)
    assert r.returncode == 0, "child %s failed:\n%s" % (name, r.stdout[-4000:])
    with open(out) as f:
        return json.load(f)


def test_protocol_shortcuts_change_no_bit(tmp_path):
    base = run_child(tmp_path, "default", {})
    assert len(base) == 9
    for name, env in (("acquire", {"CUSYNC_FORCE_ACQUIRE": "1"}),
                      ("release", {"CUSYNC_FORCE_RELEASE": "1"}),
                      ("wait_kernel", {"CUSYNC_WAIT_KERNEL": "1"}),
                      ("plain_protocol", {"CUSYNC_FORCE_ACQUIRE": "1", "CUSYNC_FORCE_RELEASE": "1", "CUSYNC_WAIT_KERNEL": "1"})):
        got = run_child(tmp_path, name, env)
        assert got.keys() == base.keys()
        for case in base:
            assert got[case] == base[case], "%s differs under %s: %r vs %r" % (case, env, got[case], base[case])


def _gpt3_reference(batch, dw1, dw2, dx):
    """H and Y of the stream-ordered chain for each input, from a handle of its own."""
    import torch
    ref = []
    mlp = api.Mlp(api.MODEL.GPT3, batch, 12288, 6144, api.SYNC.STREAM, dw1.data_ptr(), dw2.data_ptr())
    for x in dx:
        dh, dy = empty_dev((batch, 6144), fill=float("nan")), empty_dev((batch, 12288), fill=float("nan"))
        torch.cuda.synchronize()
        mlp.run(x.data_ptr(), dh.data_ptr(), dy.data_ptr(), runs=1)
        ref.append(to_host(dy).view(np.uint16))
    mlp.destroy()
    return ref


@pytest.mark.parametrize("batch,sync", [(256, api.SYNC.ROW), (256, api.SYNC.TILE), (2048, api.SYNC.ROW), (2048, api.SYNC.TILE)])
def test_gpt3_mlp_fifty_runs_back_to_back(batch, sync):
    import torch
    print("back to back", batch, sync, flush=True)
    RUNS = 50
    dw1, dw2 = to_dev(normal_f16((12288, 6144), 2)), to_dev(normal_f16((6144, 12288), 3))
    dx = [to_dev(uniform_f16((batch, 12288), 1)), to_dev(uniform_f16((batch, 12288), 101))]
    ref = _gpt3_reference(batch, dw1, dw2, dx)
    assert not np.array_equal(ref[0], ref[1])
    dh = empty_dev((batch, 6144), fill=float("nan"))
    dys = [empty_dev((batch, 12288), fill=float("nan")) for _ in range(RUNS)]       # one output per run, one intermediate for all
    torch.cuda.synchronize()
    mlp = api.Mlp(api.MODEL.GPT3, batch, 12288, 6144, sync, dw1.data_ptr(), dw2.data_ptr())
    for r in range(RUNS):       # nothing but the library's own launches and waits from here to the last run
        mlp.run(dx[r % 2].data_ptr(), dh.data_ptr(), dys[r].data_ptr(), runs=1)
    prod, cons = mlp.stage_state(0), mlp.stage_state(1)
    mlp.destroy()
    assert prod.spin_timeouts == 0 and cons.spin_timeouts == 0 and prod.kernel_executed == RUNS
    for r in range(RUNS):
        assert np.array_equal(to_host(dys[r]).view(np.uint16), ref[r % 2]), "run %d" % r


def test_attention_layer_fifty_runs_back_to_back():
    import torch
    S, hidden, heads, RUNS = 512, 12288, 12, 50
    E = heads * 128
    dwqkv, dwo = to_dev(normal_f16((hidden, 3 * E), 21)), to_dev(normal_f16((E, hidden), 22))
    dx = [to_dev(uniform_f16((S, hidden), 1)), to_dev(uniform_f16((S, hidden), 101))]
    ref = []
    layer = api.AttnLayer(S, hidden, heads, api.SYNC.STREAM, dwqkv.data_ptr(), dwo.data_ptr())
    for x in dx:
        dqkv, do, dy = empty_dev((S, 3 * E)), empty_dev((S, E)), empty_dev((S, hidden), fill=float("nan"))
        torch.cuda.synchronize()
        layer.run(x.data_ptr(), dqkv.data_ptr(), do.data_ptr(), dy.data_ptr(), runs=1)
        ref.append(to_host(dy).view(np.uint16))
    layer.destroy()
    for sync in (api.SYNC.ROW, api.SYNC.STRIDED):
        print("attention back to back", sync, flush=True)
        dqkv, do = empty_dev((S, 3 * E), fill=float("nan")), empty_dev((S, E), fill=float("nan"))
        dys = [empty_dev((S, hidden), fill=float("nan")) for _ in range(RUNS)]
        torch.cuda.synchronize()
        layer = api.AttnLayer(S, hidden, heads, sync, dwqkv.data_ptr(), dwo.data_ptr())
        for r in range(RUNS):
            layer.run(dx[r % 2].data_ptr(), dqkv.data_ptr(), do.data_ptr(), dys[r].data_ptr(), runs=1)
        states = [layer.stage_state(i) for i in range(3)]
        layer.destroy()
        assert all(st.spin_timeouts == 0 for st in states)
        for r in range(RUNS):
            assert np.array_equal(to_host(dys[r]).view(np.uint16), ref[r % 2]), "sync %d run %d" % (sync, r)
