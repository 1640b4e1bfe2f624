"""AHistSum on the GPU: the reference's own histogram vectors (tests/cpp/test_hist_sum.cu, all
17 cases) and seeded random matrices against the CPU checker, through the C-ABI with device
pointers (tests/hipmem.py holds the device memory)."""
import numpy as np
import pytest

from conftest import check_hist_sum, hist_sum_inputs, load_golden
from hipmem import DeviceArray, synchronize

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def arb():
    import arboretum_amd
    if arboretum_amd.device_count() < 1:
        pytest.skip("needs an MI355X")
    return arboretum_amd


def pack_quads(bins):
    """Row-major uint8 [n][F] -> the library's device layout: int32 words [Q][stride], byte k of
    word q of a row = bin of feature 4 q + k.  Returns (tensor, stride)."""
    n, F = bins.shape
    Q = (F + 3) // 4
    stride = (n + 63) // 64 * 64
    padded = np.zeros((stride, Q * 4), np.uint8)
    padded[:n, :F] = bins
    words = padded.view(np.uint32).reshape(stride, Q)
    return DeviceArray(np.ascontiguousarray(words.T)), stride


def run_hist_sum(arb, bins, g, h, offsets, shift_g, shift_h=0, trick=False, parents=None, entry=None):
    """-> (sum_g, sum_h, count) as numpy [nodes][4Q][256]."""
    n, F = bins.shape
    Q = (F + 3) // 4
    nodes = len(offsets) - 1
    d_bins, stride = pack_quads(bins)
    d_g = DeviceArray(np.asarray(g, np.float32))
    d_h = None if h is None else DeviceArray(np.asarray(h, np.float32))
    d_off = DeviceArray(np.asarray(offsets, np.uint32))
    shape = (nodes, Q * 4, 256)
    out_g = DeviceArray(shape=shape, dtype=np.int64, fill_byte=0xA5)   # stale values would show
    out_h = DeviceArray(shape=shape, dtype=np.int64, fill_byte=0xA5)
    out_c = DeviceArray(shape=shape, dtype=np.uint32, fill_byte=0xA5)
    pg = ph = pc = None
    if trick:
        pg = DeviceArray(np.asarray(parents[0], np.int64))
        ph = DeviceArray(np.asarray(parents[1], np.int64))
        pc = DeviceArray(np.asarray(parents[2], np.uint32))
    synchronize()
    (entry or arb.hist_sum)(
        out_g.ptr, out_h.ptr if h is not None else None, out_c.ptr, d_g.ptr,
        None if d_h is None else d_h.ptr, d_off.ptr, d_bins.ptr, stride, n, F, nodes,
        shift_g, shift_h, use_trick=trick, parent_g=None if pg is None else pg.ptr,
        parent_h=None if ph is None or h is None else ph.ptr, parent_c=None if pc is None else pc.ptr)
    return out_g.get(), out_h.get(), out_c.get()


@pytest.mark.parametrize("case", load_golden("hist_sum.json"), ids=lambda c: c["name"])
def test_reference_hist_sum_vectors(arb, oracle, case):
    bins, g, offs = hist_sum_inputs(case)
    H = case["hist_size"]
    shift = oracle.lib().orc_fix_shift(float(g.max()))
    parents = None
    if case["trick"]:
        pg = np.zeros((len(offs) // 2, 4, 256), np.int64)
        pc = np.zeros((len(offs) // 2, 4, 256), np.uint32)
        pg[0, 0, :H] = np.array(case["parent_sum"]) * 2.0 ** shift
        pc[0, 0, :H] = case["parent_count"]
        parents = (pg, np.zeros_like(pg), pc)
    sg, _, sc = run_hist_sum(arb, bins, g, None, offs, shift, trick=case["trick"], parents=parents)
    check_hist_sum(case, sc[:, 0, :], sg[:, 0, :] * 2.0 ** -shift)


def oracle_nodes(oracle, bins, g, h, offs, shift_g, shift_h):
    n = bins.shape[0]
    rows = np.arange(n)
    out = []
    for k in range(len(offs) - 1):
        sel = (rows >= offs[k]) & (rows < offs[k + 1])
        out.append(oracle.hist_fixed_u8(bins, g, h, shift_g, shift_h, sel=sel))
    return np.stack(out)  # [nodes][F][256][3]


@pytest.mark.parametrize("n,F,nodes,pair,trick", [
    (1, 1, 1, True, False), (63, 3, 1, False, False), (4097, 28, 1, True, False), (50000, 28, 8, True, True),
    (50000, 28, 8, False, True), (30011, 50, 4, True, False), (30011, 50, 4, True, True), (20000, 5, 16, True, True),
    (300000, 28, 2, True, True), (20000, 130, 2, True, False)])
def test_random_against_the_checker(arb, oracle, n, F, nodes, pair, trick):
    rng = np.random.default_rng(n * 31 + F * 7 + nodes)
    bins = rng.integers(0, 256, size=(n, F), dtype=np.uint8)
    bins[:, 0] = 0                                   # every row in one cell
    if F > 2:
        bins[:, 2] = rng.choice([3, 250], size=n)    # two cells
    g = rng.normal(size=n).astype(np.float32)
    g /= max(1.0, float(np.abs(g).max()))
    h = rng.random(n).astype(np.float32) * 0.25 if pair else None
    cuts = np.sort(rng.integers(0, n + 1, size=nodes - 1))
    if nodes >= 4:
        cuts[1] = cuts[0]                            # an empty node
    offs = np.concatenate([[0], cuts, [n]]).astype(np.uint32)
    want = oracle_nodes(oracle, bins, g, h, offs, 30, 32)
    parents = None
    if trick:
        par = want[0::2] + want[1::2]                # [nodes/2][F][256][3]
        Q4 = (F + 3) // 4 * 4
        pg = np.zeros((nodes // 2, Q4, 256), np.int64)
        ph = np.zeros_like(pg)
        pc = np.zeros((nodes // 2, Q4, 256), np.uint32)
        pg[:, :F], ph[:, :F], pc[:, :F] = par[..., 0], par[..., 1], par[..., 2]
        parents = (pg, ph, pc)
    sg, sh_, sc = run_hist_sum(arb, bins, g, h, offs, 30, 32, trick=trick, parents=parents)
    assert np.array_equal(sg[:, :F], want[..., 0])
    if pair:
        assert np.array_equal(sh_[:, :F], want[..., 1])
    assert np.array_equal(sc[:, :F].astype(np.int64), want[..., 2])
    # padding features of the last quad hold bin 0 for every row (with the trick their derived
    # cells depend on the parents' padding, which this test leaves at zero)
    if F % 4 and not trick:
        assert np.array_equal(sc[:, F, 0].astype(np.int64), np.diff(offs.astype(np.int64)))


def test_argument_errors(arb):
    # buffers of the size a 10-row, 4-feature, 2-node call needs: safe whatever the call does
    bins = DeviceArray(shape=(64,), dtype=np.uint32)
    grad = DeviceArray(shape=(64,), dtype=np.float32)
    sum_g = DeviceArray(shape=(2, 4, 256), dtype=np.int64)
    count = DeviceArray(shape=(2, 4, 256), dtype=np.uint32)
    off = DeviceArray(np.array([0, 9, 4], np.uint32))   # runs backwards
    with pytest.raises(arb.ArboretumError, match="null pointer"):
        arb.hist_sum(sum_g.ptr, None, count.ptr, None, None, off.ptr, bins.ptr, 64, 10, 4, 2, 30)
    with pytest.raises(arb.ArboretumError, match="sibling pairs"):
        arb.hist_sum(sum_g.ptr, None, count.ptr, grad.ptr, None, off.ptr, bins.ptr, 64, 10, 4, 1, 30,
                     use_trick=True, parent_g=sum_g.ptr, parent_c=count.ptr)
    with pytest.raises(arb.ArboretumError, match="stride"):
        arb.hist_sum(sum_g.ptr, None, count.ptr, grad.ptr, None, off.ptr, bins.ptr, 5, 10, 4, 2, 30)
    # offsets that run backwards are refused, nothing is read out of range
    with pytest.raises(arb.ArboretumError, match="non-decreasing"):
        arb.hist_sum(sum_g.ptr, None, count.ptr, grad.ptr, None, off.ptr, bins.ptr, 64, 10, 4, 2, 30)
