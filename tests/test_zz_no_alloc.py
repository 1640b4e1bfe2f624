"""AHistSumNoAlloc (static work memory, no device allocation) against AHistSum, through the
C-ABI: two calls in a row on one GPU, the second with a smaller input, so that what the first
call left in the shared work memory would show."""
import numpy as np
import pytest

from hipmem import DeviceArray, free_device_bytes, synchronize
from test_gpu_hist_sum import arb, oracle_nodes, run_hist_sum  # noqa: F401

pytestmark = pytest.mark.gpu


def _case(seed, n, F, nodes, pair):
    rng = np.random.default_rng(seed)
    bins = rng.integers(0, 256, size=(n, F), dtype=np.uint8)
    g = (rng.random(n).astype(np.float32) * 2 - 1)
    h = rng.random(n).astype(np.float32) * 0.25 if pair else None
    cuts = np.sort(rng.integers(0, n + 1, size=nodes - 1))
    offs = np.concatenate([[0], cuts, [n]]).astype(np.uint32)
    return bins, g, h, offs


@pytest.mark.parametrize("pair", [True, False])
def test_no_alloc_equals_allocating_entry_point_twice(arb, oracle, pair):
    # the larger call first: 28 features, 8 nodes, then a smaller one with other shapes
    for seed, n, F, nodes, trick in [(1, 400000, 28, 8, True), (2, 9001, 13, 2, False), (3, 70000, 50, 4, True)]:
        bins, g, h, offs = _case(seed, n, F, nodes, pair)
        parents = None
        if trick:
            want = oracle_nodes(oracle, bins, g, h, offs, 30, 32)
            par = want[0::2] + want[1::2]
            Q4 = (F + 3) // 4 * 4
            pg = np.zeros((nodes // 2, Q4, 256), np.int64)
            ph = np.zeros_like(pg)
            pc = np.zeros((nodes // 2, Q4, 256), np.uint32)
            pg[:, :F], ph[:, :F], pc[:, :F] = par[..., 0], par[..., 1], par[..., 2]
            parents = (pg, ph, pc)
        ref = run_hist_sum(arb, bins, g, h, offs, 30, 32, trick=trick, parents=parents)
        status = DeviceArray(np.array([77], np.uint32))

        def entry(*a, **k):
            return arb.hist_sum_no_alloc(*a, status=status.ptr, **k)
        got = run_hist_sum(arb, bins, g, h, offs, 30, 32, trick=trick, parents=parents, entry=entry)
        assert int(status.get()[0]) == 0
        assert np.array_equal(got[0], ref[0])
        if pair:
            assert np.array_equal(got[1], ref[1])
        assert np.array_equal(got[2], ref[2])
        if trick:  # and both equal the checker
            assert np.array_equal(got[0][:, :F], want[..., 0])
            assert np.array_equal(got[2][:, :F].astype(np.int64), want[..., 2])


def test_no_alloc_leaves_the_free_device_memory_alone(arb):
    # after a first call of the same shape (one-time set-up: symbol address, LDS limits), further
    # calls neither take nor return device memory
    bins, g, h, offs = _case(5, 200000, 28, 4, True)
    Q, n = 7, len(g)
    d_bins = DeviceArray(np.ascontiguousarray(
        np.pad(bins, ((0, 0), (0, 0))).view(np.uint32).reshape(n, Q).T))
    d_g, d_h, d_off = DeviceArray(g), DeviceArray(h), DeviceArray(offs)
    out_g = DeviceArray(shape=(4, 28, 256), dtype=np.int64)
    out_h = DeviceArray(shape=(4, 28, 256), dtype=np.int64)
    out_c = DeviceArray(shape=(4, 28, 256), dtype=np.uint32)
    status = DeviceArray(np.array([0], np.uint32))

    def call():
        arb.hist_sum_no_alloc(out_g.ptr, out_h.ptr, out_c.ptr, d_g.ptr, d_h.ptr, d_off.ptr, d_bins.ptr, n, n, 28, 4,
                              30, 32, status=status.ptr)
        synchronize()
    call()
    first = out_c.get().copy()
    before = free_device_bytes()
    for _ in range(3):
        call()
        assert free_device_bytes() == before
    assert int(status.get()[0]) == 0
    assert np.array_equal(out_c.get(), first) and int(first[:, 0].sum()) == n


def test_no_alloc_reports_bad_offsets_in_the_status_word(arb):
    # every buffer has the size the call needs, so that the call is safe whatever it does:
    # 10 rows, 4 features (one quad), 2 nodes -> outputs of 2 * 4 * 256 cells
    bins = DeviceArray(shape=(64,), dtype=np.uint32)
    grad = DeviceArray(shape=(64,), dtype=np.float32)
    sum_g = DeviceArray(shape=(2, 4, 256), dtype=np.int64)
    count = DeviceArray(shape=(2, 4, 256), dtype=np.uint32)
    off = DeviceArray(np.array([0, 9, 4], np.uint32))   # runs backwards
    status = DeviceArray(np.array([0], np.uint32))
    arb.hist_sum_no_alloc(sum_g.ptr, None, count.ptr, grad.ptr, None, off.ptr, bins.ptr, 64, 10, 4, 2, 30,
                          status=status.ptr)
    synchronize()
    assert int(status.get()[0]) == 1
    assert int(count.get().sum()) == 9 * 4          # the good node was counted, the bad one skipped
