"""The host-side plan checks (tests/plan_check.py) on plans built on the host from their definition:
they accept those, and reject copies corrupted by hand in the ways that matter (the GPU tests run
the same checks on the plans the library builds)."""
import numpy as np
import pytest

import plan_check as pc
from conftest import csr_from_lengths


def _scattered(seed=5, m=3000, n=70000):
    rng = np.random.default_rng(seed)
    lens = np.r_[np.minimum(rng.zipf(1.7, m - 3), 900), 0, 1500, 0]
    rp, col, _ = csr_from_lengths(lens, n, seed + 1, np.float64)
    return rp, col, n


@pytest.mark.parametrize("itemsize,width", [(8, 16384), (4, 32768)])
def test_sliced_plan_from_its_definition_passes(itemsize, width):
    rp, col, n = _scattered()
    plan = pc.sliced_plan_arrays(rp, col, n, width, 256, itemsize)
    pc.check_sliced(plan, rp, col, n, width, 256, itemsize)


def test_sliced_shares_of_tiles_across_slices():
    """Pass 1's workgroups as equal shares of the tiles: shares that reach over the start of a slice
    become two pieces, cuts near such a start move onto it, and the plan still passes."""
    rng = np.random.default_rng(5)
    m, n, width = 30000, 40000, 16384  # three slices
    lens = np.full(m, 12)
    rp = np.r_[0, np.cumsum(lens)].astype(np.int32)
    col = np.sort(rng.integers(0, n, (m, 12)), axis=1).reshape(-1).astype(np.int32)
    for shares in (1, 3, 7, 10, 40):
        plan = pc.sliced_plan_arrays(rp, col, n, width, 256, 8, shares=shares)
        pc.check_sliced(plan, rp, col, n, width, 256, 8)
        wgs, pieces = plan["wg_pieces"].reshape(-1, 8), plan["workgroups"].reshape(-1, 4)
        ntiles = int(pieces[:, 2].max())
        size = np.array([(pieces[a:b, 2] - pieces[a:b, 1]).sum() for a, b in wgs[:, :2]])
        assert size.sum() == ntiles
        if shares <= 10:  # shares of more than 64 tiles: none vanishes when its cuts move, and they stay alike
            assert wgs.shape[0] == shares and size.max() - size.min() <= 64
        else:
            assert wgs.shape[0] <= min(shares, ntiles // 32)
    assert (pc.sliced_plan_arrays(rp, col, n, width, 256, 8, shares=7)["wg_pieces"].reshape(-1, 8)[:, 1:2]
            - pc.sliced_plan_arrays(rp, col, n, width, 256, 8, shares=7)["wg_pieces"].reshape(-1, 8)[:, 0:1]).max() == 2
    # a cut 10 tiles behind the start of a slice moves onto it
    pieces, wgs = pc.split_tiles(np.array([0, 110, 400]), 4)  # cuts at 100, 200, 300
    assert pieces.reshape(-1, 4)[:, 1:3].tolist() == [[0, 110], [110, 200], [200, 300], [300, 400]]


def test_sliced_corruptions_are_rejected():
    rp, col, n = _scattered()
    good = pc.sliced_plan_arrays(rp, col, n, 16384, 256, 8)
    nslices = -(-n // 16384)

    def corrupt(name, fn):
        bad = {k: v.copy() for k, v in good.items()}
        fn(bad)
        with pytest.raises(pc.PlanError):
            pc.check_sliced(bad, rp, col, n, 16384, 256, 8)

    def dup_perm(p):  # one stored element placed twice, another not at all
        real = np.nonzero(p["perm"] >= 0)[0]
        p["perm"][real[10]] = p["perm"][real[11]]
    corrupt("perm", dup_perm)

    def swap_perm(p):  # still a permutation, but not the stable order
        real = np.nonzero(p["perm"] >= 0)[0]
        p["perm"][real[[20, 21]]] = p["perm"][real[[21, 20]]]
    corrupt("order", swap_perm)

    def range_off_by_one(p):
        r = p["ranges"].reshape(-1, nslices)
        b = int(np.nonzero(r[1:, 0] > r[:-1, 0])[0][1]) + 1
        r[b, 0] += 1
    corrupt("ranges", range_off_by_one)

    def step_base(p):
        p["steps"].reshape(-1, 4)[3, 0] += 1
    corrupt("steps", step_base)

    def step_count(p):  # a step that counts one entry fewer: a partial sum is never added
        st = p["steps"].reshape(-1, 4)
        j = int(np.nonzero((st[:, 3] >> 16) > 1)[0][0])
        st[j, 3] -= 1 << 16
    corrupt("step entries", step_count)

    def flag(p):
        p["cf"][5] ^= 0x8000
    corrupt("run flag", flag)

    def column(p):
        p["cf"][7] ^= 1
    corrupt("column", column)

    def tile_base(p):
        p["tile_words"][2] += 1
    corrupt("tile_base", tile_base)

    def partial_row(p):
        p["partial_rows"][4] ^= 3
    corrupt("partial row", partial_row)

    def workgroups(p):  # a tile no workgroup of pass 1 multiplies
        p["workgroups"].reshape(-1, 4)[0, 2] -= 1
    corrupt("workgroups", workgroups)

    def piece_taken_twice(p):  # two workgroups of pass 1 would write the same partial sums; another piece is left out
        p["wg_pieces"].reshape(-1, 8)[1] = p["wg_pieces"].reshape(-1, 8)[0]
    corrupt("every piece exactly once", piece_taken_twice)

    def stale_copy_of_the_first_piece(p):
        p["wg_pieces"].reshape(-1, 8)[2, 6] -= 1
    corrupt("copy of the first piece", stale_copy_of_the_first_piece)


def _banded(seed, m, n, half, dens, cut_rows=True):
    rng = np.random.default_rng(seed)
    rows, cols = [], []
    for r in range(m):
        c = r * (n - 1) // max(m - 1, 1)
        lo, hi = max(0, c - half), min(n, c + half + 1)
        k = 0 if rng.random() < 0.1 else max(1, rng.binomial(hi - lo, dens))
        if cut_rows and r % 97 == 0:
            k = hi - lo
        cs = np.sort(rng.choice(np.arange(lo, hi), size=min(k, hi - lo), replace=False))
        rows.append(cs.size)
        cols.append(cs)
    rp = np.zeros(m + 1, np.int32)
    np.cumsum(rows, out=rp[1:])
    return rp, np.concatenate(cols).astype(np.int32)


def _windows_moving_backwards(m=2048):
    """Block b's columns lie below block b-1's: a chain may not continue into such a block."""
    rng = np.random.default_rng(3)
    R, per = 256, 5
    rp = np.arange(m + 1, dtype=np.int32) * per
    base = (m // R - 1 - np.arange(m) // R) * 1000  # later blocks reach lower columns
    col = np.sort(base[:, None] + rng.integers(0, 900, (m, per)), axis=1).reshape(-1).astype(np.int32)
    return rp, col, int(col.max()) + 1


@pytest.mark.parametrize("itemsize", [8, 4])
def test_window_plan_from_its_definition_passes(itemsize):
    rp, col = _banded(11, 3000, 3000, 150, 0.05)
    for tiles_per_chain in (1 << 30, 40):
        plan = pc.window_plan_arrays(rp, col, 3000, 256, itemsize, tiles_per_chain)
        assert (plan["tile_words"].reshape(-1, 4)[:, 0] < 0).any(), "the matrix should have rows cut by tile starts"
        pc.check_window(plan, rp, col, 3000, 256, 1, itemsize)
    rp, col, n = _windows_moving_backwards()
    plan = pc.window_plan_arrays(rp, col, n, 256, itemsize)
    assert plan["workgroups"].size // 2 == 8, "every block must have begun a chain of its own"
    pc.check_window(plan, rp, col, n, 256, 1, itemsize)


def test_window_corruptions_are_rejected():
    # a chain that runs on into a block whose window starts below what the chain has fetched: the
    # block's columns were never put into the ring
    rp, col, n = _windows_moving_backwards()
    bad = pc.window_plan_arrays(rp, col, n, 256, 8, fresh_check=False)
    assert bad["workgroups"].size // 2 == 1
    with pytest.raises(pc.PlanError, match="holds column"):
        pc.check_window(bad, rp, col, n, 256, 1, 8)

    rp, col = _banded(13, 3000, 3000, 150, 0.05)
    good = pc.window_plan_arrays(rp, col, 3000, 256, 8, 40, in_place=False)

    def corrupt(fn, match=None):
        p = {k: v.copy() for k, v in good.items()}
        fn(p)
        with pytest.raises(pc.PlanError, match=match):
            pc.check_window(p, rp, col, 3000, 256, 1, 8)

    # a matrix whose values are read in place (no row of fewer than two stored elements): the words
    # that say where a tile's values lie
    rng = np.random.default_rng(17)
    lens = rng.integers(2, 40, 3000)
    rp2 = np.r_[0, np.cumsum(lens)].astype(np.int32)
    col2 = np.concatenate([np.sort(rng.choice(np.arange(max(0, r - 150), min(3000, r + 151)), k, replace=False))
                           for r, k in enumerate(lens)]).astype(np.int32)
    in_place = pc.window_plan_arrays(rp2, col2, 3000, 256, 8, 40)
    assert in_place["perm"] is None
    pc.check_window(in_place, rp2, col2, 3000, 256, 1, 8)

    def corrupt_in_place(fn, match):
        p = {k: None if v is None else v.copy() for k, v in in_place.items()}
        fn(p)
        with pytest.raises(pc.PlanError, match=match):
            pc.check_window(p, rp2, col2, 3000, 256, 1, 8)

    pc.check_window(pc.window_plan_arrays(rp2, col2, 3000, 256, 4, 40), rp2, col2, 3000, 256, 1, 4)

    def words_in_slot_order(p):  # fp64 in place: a lane's four words lie together, two slots from either half
        p["cf"] = p["cf"].reshape(-1, pc.TILE)[:, pc.halves_pos()].reshape(-1)
    corrupt_in_place(words_in_slot_order, "holds column|flag|a pad does not point")

    def first_value_off_by_one(p):
        p["tile_words"].reshape(-1, 4)[5, 2] += 1
    corrupt_in_place(first_value_off_by_one, "placed|out of order|another block")

    def one_value_fewer(p):
        p["tile_words"].reshape(-1, 4)[5, 3] -= 1
    corrupt_in_place(one_value_fewer, "placed")

    def one_value_more(p):  # the kernel would multiply the next tile's first value by the zero
        p["tile_words"].reshape(-1, 4)[5, 3] += 1
    corrupt_in_place(one_value_more, "placed|leaves 1 .. 256")

    def dup_perm(p):
        real = np.nonzero(p["perm"] >= 0)[0]
        p["perm"][real[10]] = p["perm"][real[11]]
    corrupt(dup_perm, "placed")

    def first_piece_above(p):  # the first fetch of the second chain starts 64 columns late
        ch = p["workgroups"].reshape(-1, 2)
        b = int(ch[1, 0])
        pcs = p["pieces"].reshape(-1, 4)
        pcs[p["blocks"].reshape(-1, 4)[b, 2], 0] += 64
    corrupt(first_piece_above, "holds column")

    def lds_slot(p):
        real = np.nonzero(pc.logical_order(p["perm"], 8) >= 0)[0]
        p["cf"][real[100]] ^= 2
    corrupt(lds_slot, "holds column")

    def flag(p):
        real = np.nonzero(pc.logical_order(p["perm"], 8) >= 0)[0]
        p["cf"][real[100]] ^= 0x8000
    corrupt(flag, "flag|fewer than two stored elements")

    def tile_rows(p):  # a tile that claims one row fewer: that row would never be written
        p["tile_words"].reshape(-1, 4)[3, 1] -= 1
    corrupt(tile_rows)

    def tile_first_row(p):
        p["tile_words"].reshape(-1, 4)[3, 0] += 1
    corrupt(tile_first_row)

    def chain_gap(p):
        p["workgroups"].reshape(-1, 2)[1, 0] += 1
    corrupt(chain_gap, "chains")

    def block_tiles(p):
        p["blocks"].reshape(-1, 4)[2, 1] -= 1
    corrupt(block_tiles)


def _stencil3d(nx, ny, nz, points=7):
    idx = np.arange(nx * ny * nz, dtype=np.int64)
    i, j, k = idx % nx, (idx // nx) % ny, idx // (nx * ny)
    keys = []
    for dk in (-1, 0, 1):
        for dj in (-1, 0, 1):
            for di in (-1, 0, 1):
                if points != 27 and abs(di) + abs(dj) + abs(dk) > 1:
                    continue
                ii, jj, kk = i + di, j + dj, k + dk
                ok = (ii >= 0) & (ii < nx) & (jj >= 0) & (jj < ny) & (kk >= 0) & (kk < nz)
                keys.append(idx[ok] * idx.size + (ii + nx * (jj + ny * kk))[ok])
    keys = np.unique(np.concatenate(keys))
    rp = np.zeros(idx.size + 1, np.int64)
    np.cumsum(np.bincount(keys // idx.size, minlength=idx.size), out=rp[1:])
    return rp.astype(np.int32), (keys % idx.size).astype(np.int32)


@pytest.mark.parametrize("points", [7, 27])
def test_stacked_planes_plan_from_its_definition_passes(points):
    # planes of 32 x 32 = 1024 points, 12 of them; blocks of 256 rows: four columns of blocks
    rp, col = _stencil3d(32, 32, 12, points)
    n = 32 * 32 * 12
    reach = 33 if points == 27 else 32
    for tiles_per_chain in (1 << 30, 30):
        plan = pc.window_plan_arrays(rp, col, n, 256, 8, tiles_per_chain, stack=(1024, -reach, reach))
        pc.check_window(plan, rp, col, n, 256, 3, 8)
        ch = plan["workgroups"].reshape(-1, 2)
        assert ch.shape[0] >= 4  # a chain never leaves its column of blocks
    # inside a chain every block but the first fetches one region only
    plan = pc.window_plan_arrays(rp, col, n, 256, 8, stack=(1024, -reach, reach))
    pcs = plan["pieces"].reshape(-1, 3, 4)
    fetched = (pcs[:, :, 1] > pcs[:, :, 0]).sum(axis=1)
    first = np.zeros(fetched.size, bool)
    first[plan["workgroups"].reshape(-1, 2)[:, 0]] = True
    # the first block of a chain is plane 0 here: nothing, or a few columns at the start of x, below it
    assert np.all(fetched[~first] <= 1) and np.all(fetched[first] >= 2)
    x_columns = (pcs[:, :, 1] - pcs[:, :, 0]).sum()
    assert x_columns < 1.5 * n  # x is fetched about once (rings per band: three times)


def test_stacked_planes_corruptions_are_rejected():
    rp, col = _stencil3d(32, 32, 12)
    n = 32 * 32 * 12
    bad = pc.window_plan_arrays(rp, col, n, 256, 8, stack=(1024, -32, 32), rotate=1)
    with pytest.raises(pc.PlanError, match="holds column"):
        pc.check_window(bad, rp, col, n, 256, 3, 8)
    good = pc.window_plan_arrays(rp, col, n, 256, 8, 30, stack=(1024, -32, 32))

    def corrupt(fn, match):
        p = {k: None if v is None else v.copy() for k, v in good.items()}
        fn(p)
        with pytest.raises(pc.PlanError, match=match):
            pc.check_window(p, rp, col, n, 256, 3, 8)

    def skip_a_region(p):  # a block in the middle of a chain does not fetch its new plane
        pcs = p["pieces"].reshape(-1, 3, 4)
        ch = p["workgroups"].reshape(-1, 2)
        b = int(ch[0, 0]) + 1
        k = int(np.argmax(pcs[b, :, 1] > pcs[b, :, 0]))
        pcs[b, k, 1] = pcs[b, k, 0]
    corrupt(skip_a_region, "holds column")

    def overlapping_regions(p):
        pcs = p["pieces"].reshape(-1, 4)
        pcs[pcs[:, 2] > 0, 2] -= 4
    corrupt(overlapping_regions, "rings overlap|holds column")

    def swap_two_blocks_tiles(p):  # the tables name another block's tiles
        blk = p["blocks"].reshape(-1, 4)
        info = p["tile_words"].reshape(-1, 4)
        t0, t1 = int(blk[0, 0]), int(blk[1, 0])
        info[t0, 0], info[t1, 0] = info[t1, 0], info[t0, 0]
    corrupt(swap_two_blocks_tiles, "block")
