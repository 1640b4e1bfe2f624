"""AHistSum on the GPU: the reference's own histogram vectors (tests/cpp/test_hist_sum.cu, all
17 cases) and seeded random matrices against the CPU checker, through the C-ABI with device
pointers (torch only holds the device memory)."""
import numpy as np
import pytest

from conftest import check_hist_sum, hist_sum_inputs, load_golden

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_dev():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("needs an MI355X")
    return torch


def pack_quads(torch, bins):
    """Row-major uint8 [n][F] -> the library's device layout: int32 words [Q][stride], byte k of
    word q of a row = bin of feature 4 q + k.  Returns (tensor, stride)."""
    n, F = bins.shape
    Q = (F + 3) // 4
    stride = (n + 63) // 64 * 64
    padded = np.zeros((stride, Q * 4), np.uint8)
    padded[:n, :F] = bins
    words = padded.view(np.uint32).reshape(stride, Q)
    return torch.from_numpy(np.ascontiguousarray(words.T).view(np.int32)).cuda(), stride


def run_hist_sum(torch, arb, bins, g, h, offsets, shift_g, shift_h=0, trick=False, parents=None, entry=None):
    """-> (sum_g, sum_h, count) as numpy [nodes][4Q][256]."""
    n, F = bins.shape
    Q = (F + 3) // 4
    nodes = len(offsets) - 1
    d_bins, stride = pack_quads(torch, bins)
    d_g = torch.from_numpy(np.ascontiguousarray(g, np.float32)).cuda()
    d_h = None if h is None else torch.from_numpy(np.ascontiguousarray(h, np.float32)).cuda()
    d_off = torch.from_numpy(np.asarray(offsets, np.uint32).view(np.int32)).cuda()
    cells = nodes * Q * 4 * 256
    out_g = torch.full((cells,), -7, dtype=torch.int64, device="cuda")
    out_h = torch.full((cells,), -7, dtype=torch.int64, device="cuda")
    out_c = torch.full((cells,), -7, dtype=torch.int32, device="cuda")
    pg = ph = pc = None
    if trick:
        pg = torch.from_numpy(np.ascontiguousarray(parents[0], np.int64)).cuda()
        ph = torch.from_numpy(np.ascontiguousarray(parents[1], np.int64)).cuda()
        pc = torch.from_numpy(np.ascontiguousarray(parents[2], np.uint32).view(np.int32)).cuda()
    torch.cuda.synchronize()
    (entry or arb.hist_sum)(
        out_g.data_ptr(), out_h.data_ptr() if h is not None else None, out_c.data_ptr(), d_g.data_ptr(),
        None if d_h is None else d_h.data_ptr(), d_off.data_ptr(), d_bins.data_ptr(), stride, n, F, nodes,
        shift_g, shift_h, use_trick=trick, parent_g=None if pg is None else pg.data_ptr(),
        parent_h=None if ph is None or h is None else ph.data_ptr(), parent_c=None if pc is None else pc.data_ptr())
    torch.cuda.synchronize()
    shape = (nodes, Q * 4, 256)
    return (out_g.cpu().numpy().reshape(shape), out_h.cpu().numpy().reshape(shape),
            out_c.cpu().numpy().view(np.uint32).reshape(shape))


@pytest.mark.parametrize("case", load_golden("hist_sum.json"), ids=lambda c: c["name"])
def test_reference_hist_sum_vectors(torch_dev, oracle, case):
    import arboretum_amd as arb
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
    sg, _, sc = run_hist_sum(torch_dev, arb, bins, g, None, offs, shift, trick=case["trick"], parents=parents)
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
def test_random_against_the_checker(torch_dev, oracle, n, F, nodes, pair, trick):
    import arboretum_amd as arb
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
    sg, sh_, sc = run_hist_sum(torch_dev, arb, bins, g, h, offs, 30, 32, trick=trick, parents=parents)
    assert np.array_equal(sg[:, :F], want[..., 0])
    if pair:
        assert np.array_equal(sh_[:, :F], want[..., 1])
    assert np.array_equal(sc[:, :F].astype(np.int64), want[..., 2])
    # padding features of the last quad hold bin 0 for every row (with the trick their derived
    # cells depend on the parents' padding, which this test leaves at zero)
    if F % 4 and not trick:
        assert np.array_equal(sc[:, F, 0].astype(np.int64), np.diff(offs.astype(np.int64)))


def test_argument_errors(torch_dev):
    import arboretum_amd as arb
    t = torch_dev.zeros(4096, dtype=torch_dev.int64, device="cuda")
    p = t.data_ptr()
    with pytest.raises(arb.ArboretumError, match="null pointer"):
        arb.hist_sum(p, p, p, None, None, p, p, 64, 10, 4, 1, 30)
    with pytest.raises(arb.ArboretumError, match="sibling pairs"):
        arb.hist_sum(p, None, p, p, None, p, p, 64, 10, 4, 3, 30, use_trick=True, parent_g=p, parent_c=p)
    with pytest.raises(arb.ArboretumError, match="stride"):
        arb.hist_sum(p, None, p, p, None, p, p, 5, 10, 4, 1, 30)
    # offsets that run backwards are refused, nothing is read out of range
    off = torch_dev.tensor([0, 9, 4], dtype=torch_dev.int32, device="cuda")
    with pytest.raises(arb.ArboretumError, match="non-decreasing"):
        arb.hist_sum(p, None, p, p, None, off.data_ptr(), p, 64, 10, 4, 2, 30)
