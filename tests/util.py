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


def sample_rows(M, k=6, seed=0):
    """A few rows including the first, the last and tile-boundary neighbours."""
    rows = {0, M - 1, M // 2}
    for b in (31, 32, 127, 128, 255, 256):
        if b < M:
            rows.add(b)
    rng = np.random.default_rng(seed)
    while len(rows) < min(k, M):
        rows.add(int(rng.integers(0, M)))
    return sorted(rows)[:max(k, 3)] if M > 3 else sorted(rows)
