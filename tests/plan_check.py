"""Host-side checks of a built sliced / window plan (the arrays asx_plan_export copies back).

The plan builders are GPU kernels; a wrong plan shows up in a product only if the input vector
happens to expose it.  These checks state, in numpy, what the kernels rely on:

* sliced: the stored elements regrouped by column slice in stable order (compared with the same
  regrouping done by numpy, slot by slot), run flags, partial-sum numbering, the ranges of every
  (row block, slice) pair, and that the steps of pass 2 enumerate every range exactly once, in
  order;
* window: every stored element placed once and in row order, run flags and tile words that make
  run k of a tile row (first row + k), and - by replaying the fetches of every chain on a model of
  the LDS rings - that the column of every slot is what its ring holds when its block is
  multiplied.

Every function raises PlanError with the first violation it finds.
"""
import numpy as np

TILE = 256
WINDOW_COLS = 16384
FETCH_COLS = 8192     # columns a block past the first of its chain may fetch
PAD_ROW = 0x7FFFFFFF
MIN_ROW_SLOTS = 2    # slots a row takes at least in a window plan
MAX_TILE_ROWS = 128  # so a tile of 256 slots holds at most this many rows


class PlanError(AssertionError):
    pass


def _need(cond, msg):
    if not cond:
        raise PlanError(msg)


def val_pos(itemsize):
    """Physical position inside a tile of logical element e = 4 * lane + j."""
    e = np.arange(TILE)
    if itemsize == 8:
        lane, j = e >> 2, e & 3
        return (j >> 1) * 128 + lane * 2 + (j & 1)
    return e


def halves_pos():
    """Where the column word of a tile's p-th slot lies in a plan that reads fp64 values in place:
    lane l holds slots 2l, 2l + 1, 128 + 2l, 128 + 2l + 1 and its four words lie together."""
    p = np.arange(TILE)
    return ((p & 127) >> 1) * 4 + (p >> 7) * 2 + (p & 1)


def logical_order(a, itemsize):
    """An array stored in the order the value loads deliver it -> slot order."""
    a = np.asarray(a).reshape(-1, TILE)
    return a[:, val_pos(itemsize)].reshape(-1)


def rows_of(rp, nnz):
    return np.repeat(np.arange(rp.size - 1, dtype=np.int64), np.diff(rp).astype(np.int64))[:nnz]


# ------------------------------------------------------------------------------------- sliced
def sliced_reference(rp, col, width, rows_per_wave):
    """The sliced plan's integer arrays as their definition gives them (numpy)."""
    rp = np.asarray(rp, np.int64)
    col = np.asarray(col, np.int64)
    m, nnz = rp.size - 1, col.size
    sl = col // width
    nslices = int(-(-int(max(col.max() + 1, 1)) // width)) if nnz else 0
    return _sliced_reference(rp, col, sl, m, nnz, width, rows_per_wave, nslices)


def _sliced_reference(rp, col, sl, m, nnz, width, rpw, nslices):
    order = np.argsort(sl, kind="stable")
    counts = np.bincount(sl, minlength=nslices).astype(np.int64)
    pstart = np.r_[0, np.cumsum(counts)]
    tiles = -(-counts // TILE)
    tile_off = np.r_[0, np.cumsum(tiles)]
    ntiles = int(tile_off[-1])
    slots = ntiles * TILE
    ssl = sl[order]
    q = np.arange(nnz) - pstart[ssl]
    d = tile_off[ssl] * TILE + q
    perm = np.full(slots, -1, np.int64)
    perm[d] = order
    row = np.full(slots, PAD_ROW, np.int64)
    row[d] = rows_of(rp, nnz)[order]
    head = np.ones(slots, bool)
    same = np.zeros(slots, bool)
    same[1:] = row[1:] == row[:-1]
    tile_start = (np.arange(slots) % TILE) == 0
    real = perm >= 0
    head[real] = (tile_start | ~same)[real]
    cf = np.full(slots, 0x8000, np.int64)
    cf[d] = (col[order] - ssl * width) | (head[d].astype(np.int64) << 15)
    hcount = np.cumsum(head)
    tile_base = np.r_[0, hcount[TILE - 1::TILE]][: ntiles + 1] if ntiles else np.zeros(1, np.int64)
    npartials = int(hcount[-1]) if slots else 0
    hd = np.nonzero(head)[0]
    prow_full = row[hd]
    cont = np.zeros(hd.size, bool)
    at_tile = (hd % TILE == 0) & (hd > 0)
    cont[at_tile] = row[hd[at_tile] - 1] == row[hd[at_tile]]
    prow = (prow_full % rpw) | (cont.astype(np.int64) << 15)
    nrb = -(-m // rpw)
    ranges = np.zeros((nrb + 1, nslices), np.int64)
    for s in range(nslices):
        lo, hi = int(tile_base[tile_off[s]]), int(tile_base[tile_off[s + 1]])
        ranges[:, s] = lo + np.searchsorted(prow_full[lo:hi], np.arange(nrb + 1) * rpw, side="left")
    return dict(perm=perm, cf=cf, tile_base=tile_base, prow=prow, prow_is_pad=prow_full == PAD_ROW, ranges=ranges,
                ntiles=ntiles, npartials=npartials, nslices=nslices, nrb=nrb, tile_off=tile_off)


def expand_steps(step_ptr, steps):
    """Entries of prow / partial that every step of pass 2 counts, step after step."""
    steps = np.asarray(steps, np.int64).reshape(-1, 4)
    w = steps[:, 3]
    f1, f2, total = w & 0xFF, (w >> 8) & 0xFF, w >> 16
    lane = np.arange(64)[None, :]
    base = np.where(lane >= f2[:, None], steps[:, 2:3], np.where(lane >= f1[:, None], steps[:, 1:2], steps[:, 0:1]))
    live = lane < total[:, None]
    return (base + lane)[live], np.repeat(np.arange(steps.shape[0]), total), f1, f2, total


def check_sliced(arrays, rp, col, n, width, rows_per_wave, itemsize):
    """arrays: name -> numpy array as Plan.export gives them (perm, cf, tile_words, workgroups,
    partial_rows, ranges, step_ptr, steps)."""
    rp = np.asarray(rp, np.int64)
    col = np.asarray(col, np.int64)
    m, nnz = rp.size - 1, col.size
    nslices = -(-n // width)
    ref = _sliced_reference(rp, col, col // width, m, nnz, width, rows_per_wave, nslices)
    slots = ref["ntiles"] * TILE
    perm = np.asarray(arrays["perm"], np.int64)
    _need(perm.size == slots, f"perm holds {perm.size} slots, expected {slots}")
    perm = logical_order(perm, itemsize)
    real = perm[perm >= 0]
    if real.size != nnz or not np.array_equal(np.sort(real), np.arange(nnz)):
        u, c = np.unique(real, return_counts=True)
        dup = u[c > 1]
        raise PlanError(f"perm is not a permutation of the stored elements: {real.size} placed of {nnz}"
                        + (f", element {int(dup[0])} placed {int(c[c > 1][0])} times" if dup.size else ""))
    bad = np.nonzero(perm != ref["perm"])[0]
    _need(bad.size == 0, f"slot {int(bad[0]) if bad.size else -1}: holds element {int(perm[bad[0]]) if bad.size else 0}, "
          f"the stable regrouping puts {int(ref['perm'][bad[0]]) if bad.size else 0} there")
    cf = np.asarray(arrays["cf"], np.int64)
    bad = np.nonzero(cf != ref["cf"])[0]
    if bad.size:
        d = int(bad[0])
        raise PlanError(f"slot {d}: column/flag word {int(cf[d]):#x}, expected {int(ref['cf'][d]):#x} "
                        f"(column in slice {int(ref['cf'][d]) & 0x7fff}, run start {int(ref['cf'][d]) >> 15})")
    tb = np.asarray(arrays["tile_words"], np.int64)
    _need(tb.size == ref["ntiles"] + 1, "tile_base size")
    _need(np.all(np.diff(tb) >= 1) if ref["ntiles"] else True, "tile_base must increase: every tile starts a run")
    bad = np.nonzero(tb != ref["tile_base"])[0]
    _need(bad.size == 0, f"tile {int(bad[0]) if bad.size else -1}: first partial sum differs from the count of run starts before it")
    prow = np.asarray(arrays["partial_rows"], np.int64)
    _need(prow.size == ref["npartials"], f"{prow.size} partial sums, expected {ref['npartials']}")
    keep = ~ref["prow_is_pad"]
    bad = np.nonzero((prow != ref["prow"]) & keep)[0]
    _need(bad.size == 0, f"partial sum {int(bad[0]) if bad.size else -1}: row word differs")
    ranges = np.asarray(arrays["ranges"], np.int64).reshape(ref["nrb"] + 1, nslices)
    _need(np.all(np.diff(ranges, axis=0) >= 0), "ranges of a slice must not decrease from one row block to the next")
    bad = np.argwhere(ranges != ref["ranges"])
    if bad.size:
        b, s = map(int, bad[0])
        raise PlanError(f"range start of row block {b} in slice {s} is {int(ranges[b, s])}, expected {int(ref['ranges'][b, s])}")
    # pass 1: every tile of every slice in exactly one piece, every piece inside one slice, every
    # piece worked off by exactly one workgroup
    wg = np.asarray(arrays["workgroups"], np.int64).reshape(-1, 4)
    _need(np.all(wg[:, 2] > wg[:, 1]), "a piece of pass 1 without tiles")
    wp = np.asarray(arrays["wg_pieces"], np.int64).reshape(-1, 8)
    _need(np.all(wp[:, 1] > wp[:, 0]) and np.all(wp[:, 0] >= 0) and np.all(wp[:, 1] <= wg.shape[0]), "a workgroup of pass 1 without pieces")
    _need(np.array_equal(wp[:, 4:8], wg[wp[:, 0]]), "a workgroup's copy of its first piece differs from the piece")
    taken = np.zeros(wg.shape[0] + 1, np.int64)
    np.add.at(taken, wp[:, 0], 1)
    np.add.at(taken, wp[:, 1], -1)
    _need(np.all(np.cumsum(taken)[:-1] == 1), "the workgroups of pass 1 do not take every piece exactly once")
    covered = np.zeros(ref["ntiles"] + 1, np.int64)
    np.add.at(covered, wg[:, 1], 1)
    np.add.at(covered, wg[:, 2], -1)
    _need(np.all(np.cumsum(covered)[:-1] == 1), "the pieces of pass 1 do not cover every tile exactly once")
    _need(np.all(ref["tile_off"][wg[:, 0]] <= wg[:, 1]) and np.all(wg[:, 2] <= ref["tile_off"][wg[:, 0] + 1]),
          "a piece's tiles leave its slice")
    check_sliced_steps(arrays["step_ptr"], arrays["steps"], ranges)


def check_sliced_steps(step_ptr, steps, ranges):
    """The steps of row block b enumerate ranges[b][s] .. ranges[b+1][s], s = 0, 1, ..., in order."""
    step_ptr = np.asarray(step_ptr, np.int64)
    nrb, nslices = ranges.shape[0] - 1, ranges.shape[1]
    _need(step_ptr.size == nrb + 1 and step_ptr[0] == 0 and np.all(np.diff(step_ptr) >= 0), "step_ptr must start at 0 and not decrease")
    entries, step_of, f1, f2, total = expand_steps(step_ptr, steps)
    nsteps = total.size
    _need(step_ptr[-1] == nsteps, f"step_ptr ends at {int(step_ptr[-1])}, there are {nsteps} steps")
    _need(np.all((total >= 1) & (total <= 64)), "a step holds 1 to 64 entries")
    _need(np.all((f1 >= 1) & (f1 <= f2) & (f2 <= 64)), "pieces of a step must start at increasing lanes")
    lens = (ranges[1:] - ranges[:-1]).reshape(-1)
    starts = ranges[:-1].reshape(-1)
    want = np.repeat(starts - np.r_[0, np.cumsum(lens)[:-1]], lens) + np.arange(int(lens.sum()))
    per_block = (ranges[1:] - ranges[:-1]).sum(axis=1)
    csum = np.r_[0, np.cumsum(total)]
    got_per_block = csum[step_ptr[1:]] - csum[step_ptr[:-1]]
    bad = np.nonzero(got_per_block != per_block)[0]
    _need(bad.size == 0, f"row block {int(bad[0]) if bad.size else -1}: its steps count "
          f"{int(got_per_block[bad[0]]) if bad.size else 0} partial sums, its ranges hold {int(per_block[bad[0]]) if bad.size else 0}")
    bad = np.nonzero(entries != want)[0]
    if bad.size:
        i = int(bad[0])
        raise PlanError(f"step {int(step_of[i])} reads partial sum {int(entries[i])} where the ranges continue with {int(want[i])}")


def pack_steps(ranges, pieces=3):
    """Steps of pass 2 from the ranges, the way the plan builder cuts them (a step is full at 64
    entries or `pieces` pieces).  Returns (step_ptr, steps x 4)."""
    nrb = ranges.shape[0] - 1
    step_ptr, out = [0], []
    for b in range(nrb):
        fill, base, first = 0, [], []
        for s in range(ranges.shape[1]):
            lo, ln = int(ranges[b, s]), int(ranges[b + 1, s] - ranges[b, s])
            while ln > 0:
                if len(base) == pieces or fill == 64:
                    out.append(_step_words(base, first, fill))
                    fill, base, first = 0, [], []
                take = min(ln, 64 - fill)
                base.append(lo - fill)
                first.append(fill)
                fill += take
                lo += take
                ln -= take
        if fill:
            out.append(_step_words(base, first, fill))
        step_ptr.append(len(out))
    return np.array(step_ptr, np.int32), np.array(out, np.int32).reshape(-1, 4)


def _step_words(base, first, fill):
    b = list(base) + [0] * (3 - len(base))
    f = list(first) + [64] * (3 - len(first))
    return [b[0], b[1], b[2], f[1] | f[2] << 8 | fill << 16]


def split_tiles(tile_off, shares):
    """Pass 1's work: `shares` equal shares of the tiles (no share below 32 tiles unless there is
    one only), a cut within 32 tiles of the start of a slice moved there, every share cut into
    pieces at the starts of slices.  Returns (pieces x 4, workgroups x 8) as a plan holds them."""
    tile_off = np.asarray(tile_off, np.int64)
    nt = int(tile_off[-1])
    shares = max(1, min(shares, nt // 32))
    cuts = [0]
    for k in range(1, shares + 1):
        c = nt * k // shares
        at = int(np.searchsorted(tile_off, c, side="left"))
        above = int(tile_off[at]) - c if at < tile_off.size else 32
        below = c - int(tile_off[at - 1]) if at > 0 else 32
        if above < 32 and above <= below:
            c += above
        elif below < 32:
            c -= below
        cuts.append(nt if k == shares else max(c, cuts[-1]))
    pieces, wgs = [], []
    for lo, hi in zip(cuts[:-1], cuts[1:]):
        if hi <= lo:
            continue
        first = len(pieces)
        a = lo
        while a < hi:
            sl = int(np.searchsorted(tile_off, a, side="right")) - 1
            z = min(hi, int(tile_off[sl + 1]))
            pieces.append([sl, a, z, 0])
            a = z
        wgs.append([first, len(pieces), 0, 0] + pieces[first])
    return np.array(pieces, np.int32).reshape(-1), np.array(wgs, np.int32).reshape(-1)


def sliced_plan_arrays(rp, col, n, width, rows_per_wave, itemsize, shares=None):
    """A whole sliced plan built on the host from its definition, in the layout Plan.export gives
    (one workgroup of pass 1 per slice that has tiles, or, with `shares`, that many equal shares
    of the tiles as the library's builder hands them out)."""
    rp = np.asarray(rp, np.int64)
    col = np.asarray(col, np.int64)
    nslices = -(-n // width)
    ref = _sliced_reference(rp, col, col // width, rp.size - 1, col.size, width, rows_per_wave, nslices)
    perm_phys = np.empty_like(ref["perm"]).reshape(-1, TILE)
    perm_phys[:, val_pos(itemsize)] = ref["perm"].reshape(-1, TILE)
    step_ptr, steps = pack_steps(ref["ranges"])
    to = ref["tile_off"]
    wg = [[s, to[s], to[s + 1], 0] for s in range(nslices) if to[s + 1] > to[s]]
    pieces, wgs = np.array(wg, np.int32).reshape(-1), np.array([[i, i + 1, 0, 0] + wg[i] for i in range(len(wg))], np.int32).reshape(-1)
    if shares:
        pieces, wgs = split_tiles(to, shares)
    return dict(perm=perm_phys.reshape(-1).astype(np.int32), cf=ref["cf"].astype(np.uint16),
                tile_words=ref["tile_base"].astype(np.int32), workgroups=pieces, wg_pieces=wgs,
                partial_rows=ref["prow"].astype(np.uint16), ranges=ref["ranges"].astype(np.int32).reshape(-1),
                step_ptr=step_ptr, steps=steps.reshape(-1))


# ------------------------------------------------------------------------------------- window
def check_window(arrays, rp, col, n, rows_per_block, nbands, itemsize):
    """arrays: perm (absent in a plan that reads A's values in place), cf, tile_words (tiles x 4),
    blocks (x 4), pieces (x 4), workgroups = chains (x 2)."""
    rp = np.asarray(rp, np.int64)
    col = np.asarray(col, np.int64)
    m, nnz = rp.size - 1, col.size
    R = rows_per_block
    info = np.asarray(arrays["tile_words"], np.int64).reshape(-1, 4)
    ntiles = info.shape[0]
    blocks = np.asarray(arrays["blocks"], np.int64).reshape(-1, 4)
    pieces = np.asarray(arrays["pieces"], np.int64).reshape(-1, 4)
    chains = np.asarray(arrays["workgroups"], np.int64).reshape(-1, 2)
    nblocks = blocks.shape[0]
    _need(nblocks == -(-m // R), f"{nblocks} blocks for {m} rows in blocks of {R}")
    # blocks tile the tiles, chains tile the blocks, blocks' pieces are consecutive
    _need(blocks[0, 0] == 0 and blocks[-1, 1] == ntiles and np.all(blocks[1:, 0] == blocks[:-1, 1]) and np.all(blocks[:, 1] > blocks[:, 0]),
          "the blocks' tile ranges must follow one another, cover every tile and hold at least one tile each")
    _need(blocks[0, 2] == 0 and blocks[-1, 3] == pieces.shape[0] and np.all(blocks[1:, 2] == blocks[:-1, 3]),
          "the blocks' piece ranges must follow one another")
    _need(np.all(blocks[:, 3] - blocks[:, 2] == nbands), f"every block lists one piece per band ({nbands})")
    _need(chains[0, 0] == 0 and chains[-1, 1] == nblocks and np.all(chains[1:, 0] == chains[:-1, 1]) and np.all(chains[:, 1] > chains[:, 0]),
          "the chains must follow one another and cover every block")
    _need(np.all(pieces[:, 0] % 4 == 0) and np.all(pieces[:, 2] % 4 == 0) and np.all(pieces[:, 3] % 4 == 0),
          "pieces start at, and rings are, multiples of 4 columns (16-byte units)")
    _need(np.all(pieces[:, 0] >= 0) and np.all(pieces[:, 1] <= n + 3), "a piece leaves the columns of x")
    _need(np.all(pieces[:, 1] >= pieces[:, 0]) and np.all(pieces[:, 1] - pieces[:, 0] <= pieces[:, 3]), "a piece is longer than its ring")
    if nbands == 1:
        _need(np.all(pieces[:, 2] == 0) and np.all(pieces[:, 3] == WINDOW_COLS), "one band: the ring is the whole window")
    # the rings (in any order within a block: stacked planes rotate them) are the same for every
    # block, apart and inside the window; what a block fetches fits the fetch registers (one window)
    rings = pieces[:, 2:4].reshape(-1, nbands, 2)
    rings = np.take_along_axis(rings, np.argsort(rings[:, :, 0], axis=1)[:, :, None], axis=1)
    ring = rings[0]
    _need(np.all(rings == ring[None]), "every block must use the same rings")
    _need(np.all(ring[1:, 0] >= ring[:-1, 0] + ring[:-1, 1]) and ring[-1, 0] + ring[-1, 1] <= WINDOW_COLS, "rings overlap or leave the LDS window")
    unit = 16 // itemsize * (64 if nbands > 1 else 1)  # several pieces: each starts a wave's 64 units
    fetched = (-(-(pieces[:, 1] - pieces[:, 0]) // unit) * unit).reshape(-1, nbands).sum(axis=1)
    _need(np.all(fetched <= WINDOW_COLS), "a block fetches more columns than the rings hold")
    later = np.ones(nblocks, bool)
    later[chains[:, 0]] = False  # a chain's first block takes as many rounds as it needs
    _need(np.all(fetched[later] <= FETCH_COLS), "a block past the first of its chain fetches more than one round of the fetch registers")

    # stored elements: each placed once; the blocks may be stored in another order than their rows'
    # (block i of the tables holds the rows of row block order[i]), the elements of one block in order
    slots = ntiles * TILE
    if arrays.get("perm") is None:
        # values read in place: slot e of a tile holds stored element (word 2) + e for e < (word 3)
        _need(np.all(rp[1:] - rp[:-1] >= MIN_ROW_SLOTS), "values can be read in place only where every row fills its slots")
        _need(np.all(info[:, 3] >= 1) and np.all(info[:, 3] <= TILE), "a tile's count of stored elements leaves 1 .. 256")
        _need(np.all(info[:, 2] >= 0) and np.all(info[:, 2] + info[:, 3] <= nnz), "a tile's stored elements leave the matrix")
        e = np.arange(TILE)[None, :]
        perm = np.where(e < info[:, 3:4], info[:, 2:3] + e, -1).reshape(-1)
    else:
        perm = np.asarray(arrays["perm"], np.int64)
        _need(perm.size == slots, f"perm holds {perm.size} slots for {ntiles} tiles")
        perm = logical_order(perm, itemsize)
    cf = np.asarray(arrays["cf"], np.int64)
    if arrays.get("perm") is None and itemsize == 8:
        cf = cf.reshape(-1, TILE)[:, halves_pos()].reshape(-1)  # into the order of the slots
    real = np.nonzero(perm >= 0)[0]
    src = perm[real]
    if src.size != nnz or not np.array_equal(np.sort(src), np.arange(nnz)):
        u, c = np.unique(src, return_counts=True)
        dup = u[c > 1]
        raise PlanError(f"stored elements are not placed once each: {src.size} placed of {nnz}"
                        + (f", element {int(dup[0])} placed {int(c[c > 1][0])} times" if dup.size else ""))
    erow = rows_of(rp, nnz)[src]  # row of the stored element in every occupied slot
    tile_of = real // TILE
    blk_of_tile = np.searchsorted(blocks[:, 1], np.arange(ntiles), side="right")
    order = (info[blocks[:, 0], 0] & 0x7FFFFFFF) // R
    _need(np.array_equal(np.sort(order), np.arange(nblocks)), "the stored blocks do not hold every block of rows once")
    _need(np.array_equal(order[blk_of_tile[tile_of]], erow // R), "a stored element sits in a tile of another block than its row's")
    same_block = blk_of_tile[tile_of][1:] == blk_of_tile[tile_of][:-1]
    _need(np.all(src[1:][same_block] > src[:-1][same_block]), "the stored elements of a block are out of order")
    # flags: first slot of a row, first slot of a tile; pads point at the zero and open runs of their
    # own, except the one that makes a row of fewer than MIN_ROW_SLOTS stored elements up to that many
    # slots (a tile then holds at most MAX_TILE_ROWS rows, all the kernel stages per tile)
    flag = cf >> 15
    pad = perm < 0
    _need(np.all((cf[pad] & 0x7FFF) == WINDOW_COLS), "a pad does not point at the zero behind the rings")
    first = info[:, 0] & 0x7FFFFFFF
    cont = (info[:, 0] >> 31) & 1
    limit = info[:, 1]
    _need(np.all(limit <= MAX_TILE_ROWS) and np.all(limit >= 0), f"a tile holds more than {MAX_TILE_ROWS} rows")
    row_of_element = rows_of(rp, nnz)
    want_flag = np.ones(slots, np.int64)
    want_flag[real] = ((src == rp[erow]) | (real % TILE == 0)).astype(np.int64)
    # where every row starts, from the tile words and the flags as they are: run k of a tile is row
    # first + k; the slot behind the start of a row of 0 or 1 stored elements continues its run
    hd0 = np.nonzero(flag)[0]
    ht0 = hd0 // TILE
    k0 = np.arange(hd0.size) - np.searchsorted(ht0, ht0, side="left")
    starts = (k0 < limit[ht0]) & ~((k0 == 0) & (cont[ht0] == 1))
    short = starts & (first[ht0] + k0 < m)
    short[short] = (rp[(first[ht0] + k0)[short] + 1] - rp[(first[ht0] + k0)[short]]) < MIN_ROW_SLOTS
    ext = hd0[short] + 1
    _need(np.all(ext % TILE != 0) and np.all(ext < slots), "a row of fewer than two stored elements starts in the last slot of a tile")
    _need(np.all(pad[ext]), "the slot behind a row of fewer than two stored elements holds a stored element")
    want_flag[ext] = 0
    bad = np.nonzero(flag != want_flag)[0]
    _need(bad.size == 0, f"slot {int(bad[0]) if bad.size else -1}: run-start flag {int(flag[bad[0]]) if bad.size else 0} is wrong")
    # tile words: run k of tile t is row first(t) + k for k < limit(t); later runs are padding
    hd = np.nonzero(flag)[0]
    ht = hd // TILE
    k = np.arange(hd.size) - np.searchsorted(ht, ht, side="left")
    is_row = k < limit[ht]
    hrow = first[ht] + k
    _need(np.all(perm[hd[~is_row]] < 0), "a run past a tile's row count holds stored elements")
    hr, hs = hrow[is_row], hd[is_row]
    _need(np.all(hr < m), "a tile's runs reach past the last row")
    empty = rp[hr + 1] == rp[hr]
    _need(np.all(perm[hs[empty]] < 0), "the slot of an empty row holds a stored element")
    ne = ~empty
    _need(np.all(perm[hs[ne]] >= 0) and np.array_equal(row_of_element[perm[hs[ne]]], hr[ne]), "run k of a tile is not row (first row + k)")
    starts_row = perm[hs[ne]] == rp[hr[ne]]
    kk, tt = k[is_row][ne], ht[is_row][ne]
    _need(np.all(starts_row | ((kk == 0) & (cont[tt] == 1))), "a run that continues a row must be the first of a tile marked so")
    _need(np.all(~((kk == 0) & (cont[tt] == 1)) | ~starts_row), "a tile marked as starting inside a row starts at a row start")
    # every row is written exactly once: by the run that starts it
    writes = np.zeros(m, np.int64)
    w_first = ~((k[is_row] == 0) & (cont[ht[is_row]] == 1))
    np.add.at(writes, hr[w_first], 1)
    bad = np.nonzero(writes != 1)[0]
    _need(bad.size == 0, f"row {int(bad[0]) if bad.size else -1} is written {int(writes[bad[0]]) if bad.size else 0} times")

    # columns: replay every chain's fetches on a model of the rings
    lds = cf & 0x7FFF
    ecol = np.full(slots, -1, np.int64)
    ecol[real] = col[src]
    for c0, c1 in chains:
        held = np.full(WINDOW_COLS, -1, np.int64)
        for b in range(int(c0), int(c1)):
            for fr, to, base, width in pieces[blocks[b, 2]:blocks[b, 3]]:
                cs = np.arange(fr, to)
                held[base + cs % width] = cs
            s0, s1 = int(blocks[b, 0]) * TILE, int(blocks[b, 1]) * TILE
            sel = np.nonzero(ecol[s0:s1] >= 0)[0] + s0
            bad = sel[held[lds[sel]] != ecol[sel]]
            if bad.size:
                d = int(bad[0])
                raise PlanError(f"block {b} (chain from block {int(c0)}): slot {d} reads LDS slot {int(lds[d])} for column "
                                f"{int(ecol[d])}, which holds column {int(held[lds[d]])} when the block is multiplied")


def window_plan_arrays(rp, col, n, rows_per_block, itemsize, tiles_per_chain=1 << 30, fresh_check=True, stack=None,
                       rotate=0, in_place=None):
    """A window plan built on the host from its definition, in the layout Plan.export gives: one
    band, or, with stack = (P, lowest, highest offset from the diagonal once the bands P below
    and above it are shifted onto it), three bands on stacked planes of P rows (square matrix, P a
    multiple of rows_per_block and a divisor of the number of rows).  fresh_check=False leaves out
    the rule that a block whose columns start below what its chain has fetched begins a new chain,
    rotate != 0 turns the regions of stacked planes the wrong way (the mistakes a replay of the
    rings must catch).  in_place (default: wherever every row has two stored elements or more)
    leaves perm out, as a plan does that reads A's values where they are."""
    rp = np.asarray(rp, np.int64)
    col = np.asarray(col, np.int64)
    m, nnz, R = rp.size - 1, col.size, rows_per_block
    nblocks = -(-m // R)
    lens = rp[1:] - rp[:-1]
    if in_place is None:
        in_place = bool(np.all(lens >= MIN_ROW_SLOTS))
    row_start = np.zeros(m, np.int64)
    btiles = np.zeros(nblocks, np.int64)
    for b in range(nblocks):
        pos = 0
        for r in range(b * R, min(m, (b + 1) * R)):
            ln = max(MIN_ROW_SLOTS, int(rp[r + 1] - rp[r]))
            if ln <= 16 and pos % TILE + ln > TILE:
                pos = (pos // TILE + 1) * TILE
            row_start[r] = pos
            pos += ln
        btiles[b] = -(-pos // TILE)
    if stack:
        P, ulo, uhi = stack
        assert m == n and m % P == 0 and P % R == 0
        per_plane, nplanes = P // R, m // P
        order = np.array([(i % nplanes) * per_plane + i // nplanes for i in range(nblocks)])
        unit = 64 * (16 // itemsize)
        size = -(-(R + (uhi - ulo) + 8 + 6) // unit) * unit
        assert 3 * size <= WINDOW_COLS
    else:
        order = np.arange(nblocks)
    stored_off = np.r_[0, np.cumsum(btiles[order])]
    tile_off = np.zeros(nblocks + 1, np.int64)
    tile_off[order] = stored_off[:-1]
    ntiles = int(stored_off[-1])
    slots = ntiles * TILE
    erow = rows_of(rp, nnz)
    o = row_start[erow] + (np.arange(nnz) - rp[erow])
    d = tile_off[erow // R] * TILE + o
    perm = np.full(slots, -1, np.int64)
    perm[d] = np.arange(nnz)
    cf = np.full(slots, 0x8000 | WINDOW_COLS, np.int64)
    short_rows = np.nonzero(lens < MIN_ROW_SLOTS)[0]
    cf[tile_off[short_rows // R] * TILE + row_start[short_rows] + 1] = WINDOW_COLS  # continues the row's run
    head = (np.arange(nnz) == rp[erow]) | (o % TILE == 0)
    if stack:
        off = col - erow
        band = np.where(off < ulo, 0, np.where(off > uhi, 2, 1))  # the bands lie P apart, further than they are wide
        q = erow // P + band - 1
        cf[d] = (((q + rotate) % 3) * size + col % size) | (head.astype(np.int64) << 15)
    else:
        cf[d] = (col % WINDOW_COLS) | (head.astype(np.int64) << 15)
    info = np.zeros((ntiles, 4), np.int64)
    for b in range(nblocks):
        r0, r1 = b * R, min(m, (b + 1) * R)
        rs = row_start[r0:r1]
        for t in range(int(tile_off[b]), int(tile_off[b] + btiles[b])):
            off = (t - tile_off[b]) * TILE
            a = r0 + int(np.searchsorted(rs, off, side="right")) - 1
            u = r0 + int(np.searchsorted(rs, off + TILE, side="left"))
            end = row_start[u - 1] + (rp[u] - rp[u - 1]) - off  # behind the last row's stored elements
            info[t] = (a | ((1 << 31) if row_start[a] != off else 0), u - a, rp[a] + (off - row_start[a]), min(end, TILE))
    blocks, pieces, chains = [], [], []
    chain_lo, chain_tiles = 0, 0
    if stack:
        held = [None, None, None]
        for i in range(nblocks):
            j, p = i // nplanes, i % nplanes
            if i != chain_lo and (p == 0 or chain_tiles >= tiles_per_chain):
                chains.append([chain_lo, i])
                chain_lo, chain_tiles, held = i, 0, [None, None, None]
            blocks.append([stored_off[i], stored_off[i + 1], len(pieces), len(pieces) + 3])
            for qq in (p - 1, p, p + 1):
                g = qq % 3
                fr = to = 0
                if held[g] != qq:
                    a = min(max(qq * P + j * R + ulo, 0), n)
                    z = min(max(qq * P + (j + 1) * R + uhi, 0), n)
                    fr = a & ~3
                    to = (z + 3) & ~3 if z > a else fr
                    held[g] = qq
                pieces.append([fr, to, g * size, size])
            chain_tiles += int(btiles[order[i]])
    else:
        have, low = -1, 0
        for b in range(nblocks):
            e0, e1 = int(rp[b * R]), int(rp[min(m, (b + 1) * R)])
            lo = hi = 0
            if e1 > e0:
                lo, hi = int(col[e0:e1].min()) & ~3, (int(col[e0:e1].max()) + 4) & ~3
            fresh = False
            if b != chain_lo:
                if fresh_check and hi > lo and have >= 0 and (lo < low or lo < max(have, hi) - WINDOW_COLS + 8):
                    fresh = True
                piece = 0 if hi <= lo else (hi - lo if have < 0 or lo >= have else max(have, hi) - have)
                if piece > FETCH_COLS:
                    fresh = True
                if chain_tiles >= tiles_per_chain:
                    fresh = True
            if fresh:
                chains.append([chain_lo, b])
                chain_lo, chain_tiles, have, low = b, 0, -1, 0
            fr = to = lo
            if hi > lo:
                if have < 0 or lo >= have:
                    fr, to, low = lo, hi, lo
                else:
                    fr, to = have, max(have, hi)
                have = to
            blocks.append([stored_off[b], stored_off[b + 1], len(pieces), len(pieces) + 1])
            pieces.append([fr, to, 0, WINDOW_COLS])
            chain_tiles += int(btiles[b])
    chains.append([chain_lo, nblocks])
    perm_phys = np.empty_like(perm).reshape(-1, TILE)
    perm_phys[:, val_pos(itemsize)] = perm.reshape(-1, TILE)
    if in_place and itemsize == 8:
        stored = np.empty_like(cf).reshape(-1, TILE)
        stored[:, halves_pos()] = cf.reshape(-1, TILE)
        cf = stored.reshape(-1)
    return dict(perm=None if in_place else perm_phys.reshape(-1).astype(np.int32), cf=cf.astype(np.uint16),
                tile_words=(info & 0xFFFFFFFF).astype(np.uint32).view(np.int32).reshape(-1),
                blocks=np.array(blocks, np.int32).reshape(-1), pieces=np.array(pieces, np.int32).reshape(-1),
                workgroups=np.array(chains, np.int32).reshape(-1))


def export_all(plan, names, value_dtype=None):
    held = [k for k in names if not (k == "perm" and plan.info("by_reference") == 1)]
    return {k: plan.export(k, value_dtype) for k in held}


SLICED_ARRAYS = ("perm", "cf", "tile_words", "workgroups", "wg_pieces", "partial_rows", "ranges", "step_ptr", "steps")
WINDOW_ARRAYS = ("perm", "cf", "tile_words", "blocks", "pieces", "workgroups")


def check_plan(plan, capi, rp, col, n, itemsize):
    """Exports a sliced or window plan and checks it."""
    if plan.alg == capi.SPMV_SLICED:
        check_sliced(export_all(plan, SLICED_ARRAYS), rp, col, n, plan.info("width"), plan.info("rows_per_wave"), itemsize)
    elif plan.alg == capi.SPMV_WINDOW:
        check_window(export_all(plan, WINDOW_ARRAYS), rp, col, n, plan.info("rows_per_block"), plan.info("bands"), itemsize)
    else:
        raise PlanError(f"plan of kernel {plan.alg} holds no regrouped copy")
