"""Helpers shared by the GPU parity tests: seeded inputs in the distributions the
benchmark configs name (X ~ U[-1,1], W ~ N(0, 0.02)), device buffers via torch,
and row-sampled comparison against the CPU oracle."""
import numpy as np

REL_TOL = 1e-2   # fp16 results within rel 1e-2 / abs 1e-3 of an fp32-accumulate reference
ABS_TOL = 1e-3


def uniform_f16(shape, seed):
    return np.random.default_rng(seed).uniform(-1.0, 1.0, shape).astype(np.float32).astype(np.float16)


def normal_f16(shape, seed, std=0.02):
    return (np.random.default_rng(seed).standard_normal(shape, dtype=np.float32) * std).astype(np.float16)


def to_dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def empty_dev(shape, fill=None):
    import torch
    t = torch.empty(shape, dtype=torch.float16, device="cuda")
    if fill is not None:
        t.fill_(fill)
    return t


def to_host(t):
    return t.detach().cpu().numpy()


def assert_close(got, ref, what="", rel=REL_TOL, abs_=ABS_TOL):
    import oracle as orc
    bad, mx = orc.count_mismatch(np.ascontiguousarray(got), np.ascontiguousarray(ref), rel, abs_)
    assert bad == 0, "%s: %d of %d elements outside rel %g / abs %g (max abs err %g)" % (
        what, bad, got.size, rel, abs_, mx)


def sample_rows(M, block=128, seed=0):
    """Rows the oracle is evaluated on: the first and the last row, one row of every block of `block` rows
    (so that every row tile of every kernel, whose tiles are 32 to 256 rows tall, is looked at; the position
    inside the block varies with the block) and both neighbours of every 256-row tile boundary."""
    rows = {0, M - 1, M // 2}
    rng = np.random.default_rng(seed)
    for b0 in range(0, M, block):
        rows.add(int(b0 + rng.integers(0, min(block, M - b0))))
    for b in (31, 32, 63, 64, 127, 128):
        if b < M:
            rows.add(b)
    for b in range(256, M, 256):
        rows.add(b - 1)
        rows.add(b)
    return sorted(rows)
