"""The sync-overhead experiment of the reference (src/examples/sync-overhead/sync-overhead.cu) and the
post -> wait hand-over latency between workgroups on the same and on different XCDs."""
import pytest

from cusync_amd import api

pytestmark = pytest.mark.gpu


def test_sync_overhead_pair_runs():
    # the example's grid: 80 * 2 * (1024 / 128) blocks of 128 threads (sync-overhead.cu:69-71).  The call itself
    # checks the consumer's output after each leg (out[i] == producer's last value + 1, as tests/simple-test.cu
    # checks a synced pair) and raises if an element differs or a wait gave up.
    with_sync, without = api.sync_overhead_pair(1280, 128, warmup=5, iters=30)
    print("pair: with sync %.1f us, without %.1f us, overhead %.1f %%" % (with_sync, without, (with_sync - without) / without * 100))
    assert 0 < without < 1e4 and 0 < with_sync < 1e4


@pytest.mark.parametrize("partner", [1, 7, 8, 9, 63])
def test_pingpong_terminates_with_sane_latency(partner):
    ns = api.sync_overhead_pingpong(partner, rounds=500)
    print("partner %d: %.0f ns per round trip" % (partner, ns))
    assert 100 < ns < 100000      # a round trip is two hand-overs through the coherent level of the memory system


@pytest.mark.parametrize("blocks,threads", [(1, 64), (7, 1024), (4096, 256)])
def test_sync_overhead_pair_checks_its_output(blocks, threads):
    # other grids than the example's: one block, blocks of the largest size, more blocks than stay resident
    with_sync, without = api.sync_overhead_pair(blocks, threads, warmup=2, iters=5)
    assert with_sync > 0 and without > 0


def test_pingpong_rejects_bad_arguments():
    with pytest.raises(api.CuSyncError):
        api.sync_overhead_pingpong(0)
    with pytest.raises(api.CuSyncError):
        api.sync_overhead_pingpong(64)


@pytest.mark.gpu
def test_mfma_rate_probe():
    """The matrix pipes alone: plausible rates and clocks, and zero operands are not slower than random ones."""
    zero_tf, zero_mhz = api.probe_mfma_rate(False, iters=1000, launches=5)
    rand_tf, rand_mhz = api.probe_mfma_rate(True, iters=1000, launches=5)
    print("MFMA alone: zeros %.0f TFLOP/s at %.0f MHz, random %.0f TFLOP/s at %.0f MHz" % (zero_tf, zero_mhz, rand_tf, rand_mhz), flush=True)
    for tf, mhz in ((zero_tf, zero_mhz), (rand_tf, rand_mhz)):
        assert 300.0 < tf < 2700.0            # cannot exceed the published dense rate
        assert 400.0 < mhz < 2700.0
    assert zero_tf > 0.9 * rand_tf


def test_sync_overhead_with_the_examples_own_kernels():
    # bare flag array, one stream (sync-overhead.cu:40-59, 84-101); the call checks the consumer's output itself
    print("sync overhead, bare flags", flush=True)
    with_flags, without = api.sync_overhead_bare(1280, 128, warmup=5, iters=30)
    print("bare flags: with %.1f us, without %.1f us" % (with_flags, without))
    assert 0 < without < 1e4 and 0 < with_flags < 1e4
    for blocks, threads in ((1, 64), (300, 1024)):
        api.sync_overhead_bare(blocks, threads, warmup=1, iters=3)
    with pytest.raises(api.CuSyncError):
        api.sync_overhead_bare(0, 128)
