"""Matrices over caller-owned blocks of bin ids (ACreateFromQuantizedBlocks): nothing is copied, rows
are counted with 64 bits across blocks.  Small cases against the CPU checker, and a matrix of
2^32 rows (1024 descriptors of one 4 M-row block) whose trees must equal those of the block alone."""
import numpy as np
import pytest

from hipmem import PinnedArray

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def arb():
    import arboretum_amd
    if arboretum_amd.device_count() < 1:
        pytest.fail("no HIP device: the GPU tests must run on the GPU box")
    return arboretum_amd


def to_block(bins, block_rows):
    """Row-major uint8 [rows][F] (rows <= block_rows) -> a pinned block in the library's layout:
    32-bit words [Q][block_rows], byte k of word q = feature 4 q + k."""
    rows, F = bins.shape
    Q = (F + 3) // 4
    padded = np.zeros((block_rows, Q * 4), np.uint8)
    padded[:rows, :F] = bins
    blk = PinnedArray((Q, block_rows), np.uint32)
    blk.array[:] = padded.view(np.uint32).reshape(block_rows, Q).T
    return blk


def config(objective, depth, **tree):
    t = {"max_depth": depth, "eta": 0.3, "lambda": 1.0}
    t.update(tree)
    return {"objective": objective, "method": 1,
            "internals": {"hist_size": 255, "double_precision": True, "upload_features": False}, "tree": t}


@pytest.mark.parametrize("objective", [0, 1])
@pytest.mark.parametrize("rows,block_rows,F", [(300000, 65536, 28), (70000, 64, 5), (1000, 4096, 128)])
def test_block_matrix_matches_the_checker(arb, oracle, objective, rows, block_rows, F):
    rng = np.random.default_rng(rows + F)
    bins = rng.integers(0, 255, size=(rows, F), dtype=np.uint8)
    s = bins[:, 0].astype(np.float32) / 64 - (bins[:, 1] > 100) + 0.5 * rng.normal(size=rows)
    y = s.astype(np.float32) if objective == 0 else (s > 1).astype(np.float32)
    nblocks = (rows + block_rows - 1) // block_rows
    blocks = [to_block(bins[b * block_rows:(b + 1) * block_rows], block_rows) for b in range(nblocks)]
    data = arb.DMatrix.from_blocks([b.ptr for b in blocks], block_rows, rows, F, y=y)
    cfg = config(objective, 5)
    g = arb.Garden(cfg, data)
    ob = oracle.Booster(bins, y=y, config=cfg, binned=True)
    for r in range(3):
        g.grow_tree()
        ob.grow(1)
        to, tg = ob.tree(r), g.tree(r)
        for key in ("fid", "quantized", "threshold", "gain", "weights"):
            assert np.array_equal(to[key], tg[key]), (key, r)
        assert np.array_equal(ob.leaf(), g.leaves())
        assert np.array_equal(ob.yhat(), g.train_yhat())
    assert np.allclose(ob.predict(bins.astype(np.float32)), g.predict(data), atol=1e-6)
    # the same rows copied in (ACreateFromQuantized) give the same trees
    copied = arb.Garden(cfg, arb.DMatrix(bins, y=y, quantized=True))
    for r in range(3):
        copied.grow_tree()
        for key in ("fid", "quantized", "gain", "weights"):
            assert np.array_equal(copied.tree(r)[key], g.tree(r)[key])


def test_block_matrix_argument_errors(arb):
    blk = PinnedArray((1, 128), np.uint32)
    blk.array[:] = 0
    y = np.zeros(200, np.float32)
    with pytest.raises(arb.ArboretumError, match="multiple of 64"):
        arb.DMatrix.from_blocks([blk.ptr], 100, 100, 4)
    with pytest.raises(arb.ArboretumError, match="does not match"):
        arb.DMatrix.from_blocks([blk.ptr, blk.ptr], 128, 100, 4)
    with pytest.raises(arb.ArboretumError, match="does not match"):
        arb.DMatrix.from_blocks([blk.ptr], 128, 129, 4)
    data = arb.DMatrix.from_blocks([blk.ptr, blk.ptr], 128, 200, 4, y=y)
    resident = config(0, 2)
    resident["internals"]["upload_features"] = True
    with pytest.raises(arb.ArboretumError, match="upload_features"):
        arb.Garden(resident, data).grow_tree()


@pytest.mark.timeout(900)
@pytest.mark.parametrize("objective", [1])
def test_four_billion_rows(arb, objective):
    # 2^32 rows x 4 features: 1024 descriptors of ONE pinned block of 2^22 rows (16 MB), so the host
    # holds the targets only.  The matrix is the block repeated a power-of-two number of times:
    # every integer sum is 1024 times the block's, and with lambda = 0 and no minimum child weight
    # the gain arithmetic scales exactly (powers of two), so splits and leaf weights must be those
    # of the block alone, gains 1024 times larger, y_hat the block's repeated.
    block_rows, reps, F = 1 << 22, 1024, 4
    rows = block_rows * reps
    assert rows == 1 << 32
    rng = np.random.default_rng(7)
    bins = rng.integers(0, 255, size=(block_rows, F), dtype=np.uint8)
    s = bins[:, 0].astype(np.float32) / 64 - (bins[:, 1] > 100) + (bins[:, 2] % 7 == 0) + 0.5 * rng.normal(size=block_rows)
    yb = (s > 1.2).astype(np.float32)
    blk = to_block(bins, block_rows)
    cfg = config(objective, 3, min_child_weight=0.0, min_leaf_size=0)
    cfg["tree"]["lambda"] = 0.0
    base = arb.Garden(cfg, arb.DMatrix.from_blocks([blk.ptr], block_rows, block_rows, F, y=yb))
    base.grow_tree()
    base.grow_tree()
    base_yhat = base.train_yhat()
    print("block grown; building the targets of 2^32 rows", flush=True)
    y = np.tile(yb, reps)
    data = arb.DMatrix.from_blocks([blk.ptr] * reps, block_rows, rows, F, y=y)
    del y
    big = arb.Garden(cfg, data)
    print("growing on 2^32 rows", flush=True)
    big.grow_tree()
    big.synchronize()
    print("first tree grown", flush=True)
    big.grow_tree()
    big.synchronize()
    print("second tree grown", flush=True)
    for r in range(2):
        tb, tg = base.tree(r), big.tree(r)
        assert (tb["quantized"] >= 0).all(), "the block's tree is not full"
        for key in ("fid", "quantized", "threshold", "weights"):
            assert np.array_equal(tb[key], tg[key]), (key, r)
        assert np.array_equal(tb["gain"] * np.float32(reps), tg["gain"])
    assert big.rows_scanned_by_level()[0] == 2 * rows        # every row in both root histograms
    yhat = big.train_yhat()
    print("y_hat read back", flush=True)
    assert yhat.shape == (rows,)
    for rep in (0, 1, 511, 1023):
        assert np.array_equal(yhat[rep * block_rows:(rep + 1) * block_rows], base_yhat), rep
    del yhat
    leaves = big.leaves()
    assert np.array_equal(leaves[:block_rows], base.leaves())
    assert np.array_equal(leaves[-block_rows:], base.leaves())


@pytest.mark.timeout(900)
def test_one_histogram_cell_holds_more_than_2_32_rows(arb):
    # 1032 descriptors of one 4 M-row block = 2^32 + 2^25 rows; feature 3 is 0 in all but 1000 rows
    # of the block, so its cell (feature 3, bin 0) counts more than 2^32 rows, and with squared error
    # the count is the hessian: a 32-bit count would change the gain of 'feature 3 = 0 against the
    # rest', which the target makes the best split of the root.  Every integer sum is 1032 times the
    # block's, so the splits must be those of the block alone and the leaf weights equal up to the
    # rounding of G / H in another scale.
    block_rows, reps, F = 1 << 22, 1032, 4
    rows = block_rows * reps
    assert (1 << 32) < rows < (1 << 33)
    rng = np.random.default_rng(9)
    bins = rng.integers(0, 255, size=(block_rows, F), dtype=np.uint8)
    bins[:, 3] = 0
    flagged = rng.choice(block_rows, size=1000, replace=False)
    bins[flagged, 3] = 1
    yb = (bins[:, 0].astype(np.float32) / 128 + 0.1 * rng.normal(size=block_rows)).astype(np.float32)
    yb[flagged] += 400.0
    blk = to_block(bins, block_rows)
    # (one split level: below the root the gains of neighbouring bins lie within the rounding of
    # another scale, and 1032 is not a power of two)
    cfg = config(0, 1, min_child_weight=0.0, min_leaf_size=1)
    cfg["tree"]["lambda"] = 0.0
    base = arb.Garden(cfg, arb.DMatrix.from_blocks([blk.ptr], block_rows, block_rows, F, y=yb))
    base.grow_tree()
    tb = base.tree(0)
    assert (tb["fid"][0], tb["quantized"][0]) == (3, 0)
    print("block grown; building the targets of %d rows" % rows, flush=True)
    y = np.tile(yb, reps)
    data = arb.DMatrix.from_blocks([blk.ptr] * reps, block_rows, rows, F, y=y)
    del y
    big = arb.Garden(cfg, data)
    big.set_inspect(True)
    print("growing on %d rows" % rows, flush=True)
    big.grow_tree()
    big.synchronize()
    print("tree grown", flush=True)
    tg = big.tree(0)
    for key in ("fid", "quantized", "threshold"):
        assert np.array_equal(tb[key], tg[key]), key
    assert np.allclose(tb["weights"], tg["weights"], rtol=1e-5, atol=0)
    assert np.allclose(tb["gain"] * np.float32(reps), tg["gain"], rtol=1e-5, atol=0)
    h = big.level_hist(0)
    assert int(h[0, 3, 0, 2]) == reps * (block_rows - 1000) > (1 << 32)     # the cell's count, all 64 bits
    assert int(h[0, 3, 1, 2]) == reps * 1000
    assert int(h[0, 0, :, 2].sum()) == rows
    # the rows of the two leaves, from the prediction update: all of the block's copies alike
    yhat = big.train_yhat()
    base_yhat = base.train_yhat()
    for rep in (0, 517, reps - 1):
        assert np.allclose(yhat[rep * block_rows:(rep + 1) * block_rows], base_yhat, rtol=1e-5, atol=1e-6), rep
