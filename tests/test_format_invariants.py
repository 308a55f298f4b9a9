"""Properties of the constructed format at wave = 64 (the production lane count), where the upstream
code (hard-wired to 32) cannot be run: the invariants upstream itself asserts, and the round trip
padded/interleaved arrays -> original COO."""
import numpy as np
import pytest

import cases
from alphasparse_amd import synthetic as S
import alphasparse_amd as A
from alphasparse_amd import _capi as K

SKELS = [("X1", {"slice": 64}), ("S5", {}), ("S1", {"m": 64}), ("S2", {"m": 64, "len": 1, "s": 3}), ("S3", {"n": 256, "s": 5}),
         ("S4", {"c": 16}), ("S6", {"m": 4, "len": 2, "c": 16}), ("S7", {"n": 256, "c": 32}), ("S8", {"b": 64})]


def _matrix(seed, wave):
    rng = np.random.default_rng(seed)
    lens = rng.integers(1, 70, 333)
    rows, cols, r, c, v, x = cases._steps(lens, 500, seed)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=wave)
    return m, r, c, v


@pytest.mark.parametrize("wave", [32, 64])
@pytest.mark.parametrize("skel,kw", SKELS, ids=[s[0] for s in SKELS])
def test_padding_invariants_and_round_trip(skel, kw, wave):
    from alphasparse_amd import skeletons as SK
    m, r, c, v = _matrix(11, wave)
    m.execute_strategy(K.COMPRESS_NONE)
    kw = dict(kw, wave=wave) if skel == "S5" else kw
    SK.apply_skeleton(m, 0, skel, **kw)
    d = m.dump()
    g = lambda k: d["sub0." + k]
    blb_begin = g("read_index[2].coo_begin_index_arr")[0].astype(np.int64)
    blb_wlb = g("read_index[2].index_arr")[0].astype(np.int64)
    blb_row = g("read_index[2].index_of_the_first_row_arr")[0].astype(np.int64)
    wlb_tlb = g("read_index[3].index_arr")[0].astype(np.int64)
    wlb_begin = g("read_index[3].coo_begin_index_arr")[0].astype(np.int64)
    wlb_size = g("read_index[3].coo_block_size_arr")[0].astype(np.int64)
    wlb_row = g("read_index[3].index_of_the_first_row_arr")[0].astype(np.int64)
    tlb_row = g("read_index[4].index_of_the_first_row_arr")[0].astype(np.int64)
    tlb_size = g("read_index[4].coo_block_size_arr")[0].astype(np.int64)
    pcol, scol = g("read_index[5].index_arr")[0].astype(np.int64), g("read_index[6].index_arr")[0].astype(np.int64)
    pval, sval = g("padding_val_arr"), g("staggered_padding_val_arr")
    # CSR offset arrays are monotone and end at the totals
    for a in (blb_begin, blb_wlb, wlb_tlb):
        assert np.all(np.diff(a) >= 0)
    assert blb_begin[-1] == len(pcol) == len(pval) == len(scol) == len(sval)
    assert blb_wlb[-1] == len(wlb_size) and wlb_tlb[-1] == len(tlb_row)
    got = []
    for b in range(len(blb_row)):
        for w in range(blb_wlb[b], blb_wlb[b + 1]):
            ntlb, s = wlb_tlb[w + 1] - wlb_tlb[w], tlb_size[w]
            assert ntlb % wave == 0                      # TLB count per WLB is a multiple of the wave
            assert wlb_size[w] == ntlb * s               # padded length = TLBs x TLB size
            base = blb_begin[b] + wlb_begin[w]
            seg_c, seg_v = pcol[base:base + wlb_size[w]], pval[base:base + wlb_size[w]]
            st_c, st_v = scol[base:base + wlb_size[w]], sval[base:base + wlb_size[w]]
            # un-interleave: dst[g*W*s + j*W + lane] = src[g*W*s + lane*s + j]
            un_c = st_c.reshape(-1, s, wave).transpose(0, 2, 1).reshape(-1)
            un_v = st_v.reshape(-1, s, wave).transpose(0, 2, 1).reshape(-1)
            assert np.array_equal(un_c, seg_c) and np.array_equal(un_v, seg_v)
            rows_of_tlb = blb_row[b] + wlb_row[w] + tlb_row[wlb_tlb[w]:wlb_tlb[w + 1]]
            rr = np.repeat(rows_of_tlb, s)
            keep = seg_v != 0
            got.append(np.stack([rr[keep], seg_c[keep], seg_v[keep]], 1))
    got = np.concatenate(got)
    keep = v != 0
    want = np.stack([r.astype(np.int64)[keep], c.astype(np.int64)[keep], v[keep].astype(np.float64)], 1)
    order = np.lexsort((got[:, 1], got[:, 0]))
    assert np.array_equal(got[order], want)   # stripping the zero padding reproduces the input COO


@pytest.mark.parametrize("wave", [32, 64])
def test_nnz_division_covers_every_element(wave):
    m, r, c, v = _matrix(12, wave)
    m.execute_strategy(K.COMPRESS_NONE)
    m.execute_strategy(K.COMPRESSED_THREAD_LEVEL_NNZ_DIV_DIRECT, 0, (5,))
    d = m.dump()
    first = d["sub0.read_index[4].index_of_the_first_row_arr"][0].astype(np.int64)
    count = d["sub0.read_index[4].row_number_of_block_arr"][0].astype(np.int64)
    rr = r.astype(np.int64)
    assert len(first) == -(-len(rr) // 5)
    assert np.array_equal(first, rr[::5])
    last = rr[np.minimum(np.arange(len(first)) * 5 + 4, len(rr) - 1)]
    assert np.array_equal(count, last - first + 1)
    # slots 5 and 6 alias the unpadded column array
    assert np.array_equal(d["sub0.read_index[5].index_arr"][0], d["sub0.read_index[1].index_arr"][0])


def test_coarse_sort_is_a_stable_bucket_permutation():
    m, r, c, v = _matrix(13, 64)
    lens = np.bincount(r.astype(np.int64))
    m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
    d = m.dump()
    perm = d["sorted_row_index"][0].astype(np.int64)          # new -> old
    assert sorted(perm.tolist()) == list(range(len(lens)))
    new_lens = lens[perm]
    assert np.all(np.diff(new_lens) <= 0)                       # longest rows first
    for L in np.unique(lens):                                   # original order kept inside a bucket
        assert np.all(np.diff(perm[new_lens == L]) > 0)
    nr = d["coo_row_index_cache"].astype(np.int64)
    assert np.array_equal(np.bincount(nr), new_lens)
    key_old = set(zip(r.astype(np.int64).tolist(), c.astype(np.int64).tolist()))
    key_new = set(zip(perm[nr].tolist(), d["coo_col_index_cache"].astype(np.int64).tolist()))
    assert key_old == key_new


def test_input_validation():
    m, r, c, v = _matrix(14, 64)
    assert m.check_sorted() and not m.has_empty_row()
    rows = 10
    m2 = A.Matrix.from_coo(rows, 10, [0, 0, 3, 2], [1, 0, 2, 2], [1.0, 2, 3, 4], K.FLOAT)
    assert not m2.check_sorted() and m2.has_empty_row()
    with pytest.raises(A.AlphaSparseError):
        A.Matrix.from_coo(4, 4, [0, 7], [0, 1], [1.0, 1.0], K.FLOAT)   # row outside the matrix
    with pytest.raises(A.AlphaSparseError):
        m.execute_strategy(K.COMPRESSED_ROW_PADDING_DIRECT, 0, (32, 1))  # not compressed yet


def test_coo_file_round_trip(tmp_path):
    rows, cols, r, c, v, _ = cases._steps([3, 1, 4, 1, 5, 9, 2, 6], 40, 3)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT)
    path = tmp_path / "m.mtx.coo"
    m.write_coo_file(path)
    first = open(path).readline().split()
    assert first[:2] == [str(rows), str(cols)]
    m2 = A.Matrix.from_coo_file(path, K.FLOAT)
    a, b = m.dump(), m2.dump()
    assert np.array_equal(a["coo_row_index_cache"], b["coo_row_index_cache"])
    assert np.array_equal(a["coo_col_index_cache"], b["coo_col_index_cache"])
    assert np.array_equal(a["coo_value_cache"], b["coo_value_cache"])


@pytest.mark.parametrize("slice_width", [32, 128, 1024])
def test_column_slice_division_and_x_slice_template(slice_width):
    """COMPRESSED_TBLOCK_LEVEL_COL_DIV_COL_SLICE: every BLB is one row piece inside one column slice, the pieces of
    a row are exactly its non-empty slices; the x-slice template regroups them by slice and stores
    slice-relative 16-bit columns that reproduce the original elements."""
    from alphasparse_amd import skeletons as SK
    m, r, c, v = _matrix(17, 64)
    m.execute_strategy(K.COMPRESS_NONE)
    tp = SK.apply_skeleton(m, 0, "X1", slice=slice_width)[0]
    assert A.template_is_supported(m, 0, tp)
    d = m.dump()
    g = lambda k: d["sub0." + k][0].astype(np.int64)
    blb_begin, blb_row = g("read_index[2].coo_begin_index_arr"), g("read_index[2].index_of_the_first_row_arr")
    pcol = g("read_index[5].index_arr")
    r, c = np.asarray(r, np.int64), np.asarray(c, np.int64)
    want = sorted(set(zip(r.tolist(), (c // slice_width).tolist())))
    got = [(int(blb_row[b]), int(pcol[blb_begin[b]] // slice_width)) for b in range(len(blb_row))]
    assert got == want
    for b in range(len(blb_row)):
        seg = pcol[blb_begin[b]:blb_begin[b + 1]]
        assert len(seg) % 64 == 0 and (seg // slice_width == seg[0] // slice_width).all()
    b = A.Builder(m)
    b.set_template(0, tp, compress=False)
    t = b.template_dump(0)
    arr = {k: np.asarray(a[0]).astype(np.int64) for k, a in t["arrays"].items()}
    assert t["arrays"]["col_index_arr"][1] == "UNSIGNED_SHORT"
    nzb, rows_of, gfb, gsl = (arr["block_nz_begin_offset"], arr["row_index_of_block_level_block"], arr["group_first_block"],
                              arr["group_slice"])
    assert gfb[0] == 0 and gfb[-1] == len(rows_of) and (np.diff(gfb) > 0).all() and (np.diff(gsl) >= 0).all()
    val = np.asarray(t["val_arr"][0] if isinstance(t["val_arr"], tuple) else t["val_arr"], np.float64)
    elems = []
    for grp in range(len(gsl)):
        for blb in range(gfb[grp], gfb[grp + 1]):
            for k in range(nzb[blb], nzb[blb + 1]):
                assert arr["col_index_arr"][k] < slice_width
                if val[k] != 0.0:
                    elems.append((int(rows_of[blb]), int(gsl[grp] * slice_width + arr["col_index_arr"][k]), float(val[k])))
    want = sorted((int(a), int(b_), float(np.float32(x))) for a, b_, x in zip(r, c, v) if np.float32(x) != 0)
    assert sorted(elems) == want


def _emulate_tile_template(t, slice_width, group, sub_rows, x, chunk=4):
    """y of the tile template's arrays, walking them the way its kernel does: trips, runs, lanes of 8 consecutive
    elements with one word each (bits 0-14 piece of the first element, bit 14+j element j starts a new piece,
    bit 22+j a sum emitted at element j is stored), 16-bit columns inside the slice, one LDS cell per piece of the
    run, written back at the end of the run to piece_target (a row of y, or of the scratch vector that the finish
    kernel moves to y through y_row_index).  A sum is emitted where a piece ends inside a lane and at the last lane
    of a stretch of lanes whose last elements share a piece; a flagged sum is STORED into the cell, the others are
    added: y comes out right only if every flagged piece gets that one sum."""
    arr = {k: np.asarray(a[0]).astype(np.int64) for k, a in t["arrays"].items()}
    val = np.asarray(t["val_arr"][0] if isinstance(t["val_arr"], tuple) else t["val_arr"], np.float64)
    own_rows = "run_row_group" in arr   # row ownership: cells are rows of the run's row group, kept across its runs
    rb = int(t["scalars"].get("row_block", 1))   # row blocks: an element is one value for each of rb neighbouring rows
    assert rb == 1 or own_rows
    gfr, nzb, word, yrow, lcol = (arr["group_first_run"], arr["run_nz_begin"], arr["lane_word"],
                                  arr["y_row_index"], arr["col_index_arr"])
    # the first column of the stretch of x a run reads: a slice of the format's grid, or (row ownership) a window
    # that starts at the row group's first column not yet covered, on a 16-byte boundary of x
    rs = arr["run_col_begin"] if own_rows else arr["run_slice"] * slice_width
    if own_rows:
        rrg = arr["run_row_group"]
        assert "run_slice" not in arr and (rs % chunk == 0).all()
        assert "piece_target" not in arr and "run_piece_begin" not in arr and len(rrg) == len(rs)
        # a trip is a whole number of row groups, a row group the runs of one trip that follow each other
        trip_of_run = np.repeat(np.arange(len(gfr) - 1), np.diff(gfr))
        for g in np.unique(rrg):
            runs = np.flatnonzero(rrg == g)
            assert (np.diff(runs) == 1).all() and len(set(trip_of_run[runs].tolist())) == 1
            assert (np.diff(rs[runs]) >= slice_width).all()      # window by window inside the group, none overlapping
        assert (np.diff(rrg) >= 0).all()
    else:
        rpb, target = arr["run_piece_begin"], arr["piece_target"]
    if "col_run_mask" in arr:
        # column-run form: per lane the first columns of up to four runs of consecutive columns and a byte whose
        # bit j says that element j opens the next run (a run beyond the fourth starts at column 0)
        starts, mask = lcol.reshape(-1, 4), arr["col_run_mask"]
        assert len(starts) == len(mask) and (mask & 1 == 0).all() and (mask < 256).all()
        lanes, run = np.arange(len(mask)), np.zeros(len(mask), np.int64)
        decoded = np.zeros((len(mask), 8), np.int64)
        decoded[:, 0] = starts[:, 0]
        for j in range(1, 8):
            opens = (mask >> j) & 1
            run += opens
            decoded[:, j] = np.where(opens == 1, np.where(run < 4, starts[lanes, np.minimum(run, 3)], 0), decoded[:, j - 1] + 1)
        lcol = decoded.reshape(-1)
    assert gfr[0] == 0 and gfr[-1] == len(rs) and (np.diff(gfr) > 0).all() and (np.diff(nzb) > 0).all()
    assert nzb[-1] * 512 * rb == len(lcol) * rb == len(val) == 8 * len(word) * rb and (lcol < slice_width).all()
    if not own_rows:
        assert rpb[0] == 0 and rpb[-1] == len(target) and (np.diff(rpb) > 0).all() and (np.diff(rpb) <= group).all()
    through_scratch = t["scalars"]["is_atom_add"] == 0 and not own_rows
    group_cells = {}
    # values are stored 16 bytes per lane and load: piece i of lane l of a wavefront step at (i * 64 + l)
    # (row blocks: the rb rows of a lane one after the other, each in its 16-byte pieces: val[q] = the values of row q)
    j, lane = np.meshgrid(np.arange(8), np.arange(64))
    steps = val.reshape(-1, 512 * rb)
    val_rows = []
    for q in range(rb):
        where = ((q * (8 // chunk) + j // chunk) * 64 + lane) * chunk + j % chunk    # [lane, j] -> place inside the step
        val_rows.append(steps[:, where.reshape(-1)].reshape(-1))
    val = val_rows[0]
    y = np.zeros(int(yrow.max()) + 1)
    flagged = plain = 0
    for run in range(len(rs)):
        k0, k1 = nzb[run] * 512, nzb[run + 1] * 512
        if own_rows:
            cells = group_cells.setdefault(int(rrg[run]), np.zeros(group))
        else:
            cells = np.zeros(rpb[run + 1] - rpb[run])
        touched = np.zeros(len(cells), np.int64)
        assert (rs[run] + lcol[k0:k1] < len(x)).all()            # padding included: the kernel reads x there
        prods = [vq[k0:k1] * x[rs[run] + lcol[k0:k1]] for vq in val_rows]
        for u in range(0, k1 - k0, 512):                         # one wavefront step
            w = word[(k0 + u) // 8:(k0 + u) // 8 + 64]
            first = w & 0x7fff
            new_piece = (w[:, None] >> (14 + np.arange(1, 8))[None, :]) & 1
            store = (w[:, None] >> (22 + np.arange(8))[None, :]) & 1
            final = first + rb * new_piece.sum(1)
            step = first[1:] - final[:-1]
            if own_rows:
                assert (step >= 0).all() and (first % rb == 0).all()   # a lane may skip rows that have no element in the slice
            else:
                assert ((step == 0) | (step == 1)).all()          # the next lane goes on with the piece or starts the next one
            carry = np.zeros(rb)                                 # the segmented sum over the lanes' last pieces
            for lane in range(64):
                cell, acc = first[lane], np.zeros(rb)

                def emit(j):
                    nonlocal flagged, plain
                    assert cell + rb <= len(cells)
                    if store[lane, j]:
                        assert touched[cell] == 0                # the only sum of this piece (in this run)
                        cells[cell:cell + rb] = cells[cell:cell + rb] + acc if own_rows else acc
                        touched[cell] = -1
                        flagged += 1
                    else:
                        assert touched[cell] >= 0
                        cells[cell:cell + rb] += acc
                        touched[cell] += 1
                        plain += 1
                for j in range(8):
                    if j and new_piece[lane, j - 1]:
                        emit(j - 1)
                        cell, acc = cell + rb, np.zeros(rb)
                    acc = acc + np.array([p[u + lane * 8 + j] for p in prods])
                if lane and final[lane - 1] == final[lane]:
                    acc = acc + carry
                if lane == 63 or final[lane + 1] != final[lane]:
                    emit(7)
                    carry = np.zeros(rb)
                else:
                    carry = acc
        if own_rows:
            continue
        assert (touched != 0).all()                              # every piece of the run got a sum
        rows_of_run = target[rpb[run]:rpb[run + 1]]
        np.add.at(y, yrow[rows_of_run] if through_scratch else rows_of_run, cells)
    if own_rows:
        # every row of every row group is stored once, rows without elements as zeros; a row group that holds no
        # element at all belongs to no run: its rows are... not written (there is none in a matrix without empty rows)
        y[:] = np.nan
        for g, cells in group_cells.items():
            live = min(group, sub_rows - g * group)
            y[yrow[g * group:g * group + live]] = cells[:live]
        assert not np.isnan(y).any()
    return y, flagged, plain


@pytest.mark.parametrize("slice_width,group,blb,sort", [(32, 16, 64, False), (128, 64, 100, True), (1024, 8, 17, False),
                                                          (64, 4096, 4096, True)])
def test_tile_division_and_tile_template(slice_width, group, blb, sort):
    """COMPRESSED_TBLOCK_LEVEL_COL_DIV_ROW_GROUP_COL_SLICE: the elements are a permutation of the input ordered by
    (slice, row group, row, column); every BLB lies inside one tile and holds at most `blb` elements; the tile
    template's packed words and run tables reproduce y = A x (also through the coarse-sort permutation)."""
    from alphasparse_amd import skeletons as SK
    rows, cols, r, c, v, x = cases._steps([3] * 40 + [20] * 24 + [90] * 8 + [1] * 30 + [300] * 3, 640, 21)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
    if sort:
        m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
    m.execute_strategy(K.COMPRESS_NONE)
    tp = SK.apply_skeleton(m, 0, "T1", slice=slice_width, group=group, b=blb)[0]
    assert tp == K.SHARED_MEMORY_TILE_TEMPLATE and A.template_is_supported(m, 0, tp)
    for other in (K.DIRECT_ATOM_TEMPLATE, K.SHARED_MEMORY_LONG_ROW_TEMPLATE, K.UNALIGNED_WARP_REDUCE_SAME_TLB_SIZE_TEMPLATE,
                  K.SHARED_MEMORY_X_SLICE_TEMPLATE):
        assert not A.template_is_supported(m, 0, other)
    d = m.dump()
    g = lambda k: d["sub0." + k][0].astype(np.int64)
    row, col = g("read_index[0].index_arr"), g("read_index[1].index_arr")
    begin, first, number = (g("read_index[2].coo_begin_index_arr"), g("read_index[2].index_of_the_first_row_arr"),
                            g("read_index[2].row_number_of_block_arr"))
    nrg = -(-rows // group)
    key = (col // slice_width) * nrg + row // group
    order = np.lexsort((col, row, key))
    assert np.array_equal(order, np.arange(len(row)))           # sorted by (tile, row, column)
    assert begin[0] == 0 and begin[-1] == len(row) and len(first) == len(begin) - 1
    for b in range(len(first)):
        k0, k1 = begin[b], begin[b + 1]
        assert 0 < k1 - k0 <= blb and len(set(key[k0:k1].tolist())) == 1
        assert first[b] == row[k0] and number[b] == row[k1 - 1] - row[k0] + 1
        # a BLB ends early only at the end of its tile
        assert k1 - k0 == blb or k1 == len(row) or key[k1] != key[k0]
    yref = np.zeros(rows)
    np.add.at(yref, np.asarray(r, np.int64), np.float32(v).astype(np.float64) * x[np.asarray(c, np.int64)])
    b = A.Builder(m)
    for compress in (False, True):
        b.set_template(0, tp, compress=compress)
        t = b.template_dump(0)
        if not compress:
            y, flagged, plain = _emulate_tile_template(t, slice_width, group, rows, x.astype(np.float64))
            assert np.allclose(y, yref, rtol=1e-12, atol=1e-12)
            assert flagged > 0 and plain > 0                     # both kinds of row sums occur
            assert t["arrays"]["col_index_arr"][1] == "UNSIGNED_SHORT" and t["arrays"]["lane_word"][1] == "UNSIGNED_INT"
    src = b.kernel_source()
    assert "as_wave_segmented_sum" in src and ("y_row_index[" in src) == sort


@pytest.mark.parametrize("vdt,chunk", [(K.FLOAT, 4), (K.DOUBLE, 2)], ids=["fp32", "fp64"])
@pytest.mark.parametrize("sort,runs", [(False, False), (True, False), (False, True), (True, True)],
                         ids=["plain", "sorted", "plain_runs", "sorted_runs"])
def test_tile_template_under_row_ownership(vdt, chunk, sort, runs):
    """set_row_ownership on a banded matrix of dense 3 x 3 blocks (many row groups, two or three slices each): the
    elements row group by row group and inside a group window by window of x, cells = rows of the group kept across
    its windows, lanes closed where a row of the group is missing from a window, no piece tables, no scratch, no atomics into y -- and the same y when the arrays
    are walked the way the kernel walks them, alone and on top of the column-run form.  Turned down where it does
    not fit: a few long rows (one row group for all CUs), a column band, another template."""
    from alphasparse_amd import skeletons as SK
    rows, cols, r, c, v, x = S.fem_blocks(1000, 27, 60, seed=5)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
    if sort:
        m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
    m.execute_strategy(K.COMPRESS_NONE)
    tp = SK.apply_skeleton(m, 0, "T1", slice=500, group=100, b=1000)[0]
    b = A.Builder(m)
    b.set_template(0, tp, compress=False)
    b.set_launch(0, thread_num_in_block=256)
    if runs:
        assert b.set_column_runs(0)
    before = b.template_dump(0)
    assert b.clears_y() == (not sort)                                    # atomics into y, or the scratch vector
    assert b.set_row_ownership(0) and not b.set_row_ownership(0)         # the second call finds the form in place
    t = b.template_dump(0)
    assert 0.95 * len(before["val_arr"]) <= len(t["val_arr"]) <= 1.05 * len(before["val_arr"])   # other runs, other padding
    assert ("col_run_mask" in t["arrays"]) == runs and "run_row_group" in t["arrays"]
    assert t["scalars"]["is_atom_add"] == 0 and not b.clears_y()
    assert b.get_launch(0)["thread_num_in_block"] == 256
    if not sort:
        # 100 rows and their band of +-180 columns fit one window of 500 columns, wherever the grid's slices fall:
        # one run and one copy of x per row group (the tiles of the format are two or three per row group)
        assert len(t["arrays"]["run_col_begin"][0]) == -(-rows // 100) < len(before["arrays"]["run_slice"][0])
    vv = np.float32(v).astype(np.float64) if vdt == K.FLOAT else v.astype(np.float64)
    yref = np.zeros(rows)
    np.add.at(yref, np.asarray(r, np.int64), vv * x[np.asarray(c, np.int64)])
    y, flagged, plain = _emulate_tile_template(t, 500, 100, rows, x.astype(np.float64), chunk=chunk)
    assert np.allclose(y, yref, rtol=1e-12, atol=1e-12) and flagged > 0
    src = b.kernel_source()
    assert "cur_group" in src and "piece_target" not in src and "_finish" not in src and ("y_row_index[" in src) == sort
    assert ("col_run_mask" in src) == runs
    # the column-run form on top of row ownership keeps the ownership
    if not runs:
        assert b.set_column_runs(0)
        t2 = b.template_dump(0)
        assert "run_row_group" in t2["arrays"] and "col_run_mask" in t2["arrays"]
        y2 = _emulate_tile_template(t2, 500, 100, rows, x.astype(np.float64), chunk=chunk)[0]
        assert np.allclose(y2, yref, rtol=1e-12, atol=1e-12)
    # a few long rows: one row group would have to feed every CU
    rows, cols, r, c, v, x = cases._steps([30000] * 6, 40000, 4)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
    m.execute_strategy(K.COMPRESS_NONE)
    b = A.Builder(m)
    b.set_template(0, SK.apply_skeleton(m, 0, "T1", slice=512, group=64, b=4096)[0])
    assert not b.set_row_ownership(0) and "run_row_group" not in b.template_dump(0)["arrays"]
    # a column band of the matrix shares its rows with the other bands
    rows, cols, r, c, v, x = S.fem_blocks(400, 9, 60, seed=5)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
    m.execute_node(K.DENSE_FIXED_COL_DIV, -1, scalars=(600,))
    m.execute_strategy(K.COMPRESS_NONE)
    for sub in range(m.info()["n_sub"]):
        tp = SK.apply_skeleton(m, sub, "T1", slice=500, group=64, b=1000)[0]
    b = A.Builder(m)
    b.set_template(0, tp)
    assert not b.set_row_ownership(0)
    # another template
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
    m.execute_strategy(K.COMPRESS_NONE)
    b = A.Builder(m)
    b.set_template(0, SK.apply_skeleton(m, 0, "S1", m=64)[0])
    assert not b.set_row_ownership(0)


@pytest.mark.parametrize("vdt,chunk", [(K.FLOAT, 4), (K.DOUBLE, 2)], ids=["fp32", "fp64"])
@pytest.mark.parametrize("runs", [False, True], ids=["plain", "runs"])
def test_tile_template_with_row_blocks(vdt, chunk, runs):
    """set_row_blocks on a matrix of dense 3 x 3 blocks under row ownership: the three rows of a block row hold the
    same columns and become one piece of the stream -- one set of columns and lane words, three values per element,
    a third of the stream's elements -- and walking the arrays the way the kernel does gives the same y.  Turned
    down where the row group's height is not a multiple of three, without row ownership, for blocks of another
    height, and where a row of a block differs from the others."""
    from alphasparse_amd import skeletons as SK
    rows, cols, r, c, v, x = S.fem_blocks(1000, 27, 60, seed=5)
    vv = np.float32(v).astype(np.float64) if vdt == K.FLOAT else v.astype(np.float64)
    yref = np.zeros(rows)
    np.add.at(yref, np.asarray(r, np.int64), vv * x[np.asarray(c, np.int64)])

    def build(matrix_rows=(rows, r, c, v), group=96):
        n, rr, cc, vals = matrix_rows
        m = A.Matrix.from_coo(n, cols, rr, cc, vals.astype(np.float64), vdt, wave=64)
        m.execute_strategy(K.COMPRESS_NONE)
        tp = SK.apply_skeleton(m, 0, "T1", slice=500, group=group, b=1000)[0]
        b = A.Builder(m)
        b.set_template(0, tp, compress=False)
        b.set_launch(0, thread_num_in_block=256)
        return b
    b = build()
    assert not b.set_row_blocks(0, 3)                                    # not before row ownership
    if runs:
        assert b.set_column_runs(0)
    assert b.set_row_ownership(0)
    before = b.template_dump(0)
    assert not b.set_row_blocks(0, 2) and not b.set_row_blocks(0, 4)     # 96 = 4 x 24, but the blocks are 3 rows high
    assert b.set_row_blocks(0, 3) and not b.set_row_blocks(0, 3)         # the second call finds the form in place
    t = b.template_dump(0)
    assert t["scalars"]["row_block"] == 3 and "run_row_group" in t["arrays"] and ("col_run_mask" in t["arrays"]) == runs
    assert len(t["val_arr"]) <= 1.25 * len(before["val_arr"])            # the same values; a run is padded to 512 elements of 3 values
    assert len(t["arrays"]["lane_word"][0]) * 2.5 <= len(before["arrays"]["lane_word"][0])   # a third of the lanes
    assert not b.clears_y() and b.get_launch(0)["thread_num_in_block"] == 256
    y, flagged, plain = _emulate_tile_template(t, 500, 96, rows, x.astype(np.float64), chunk=chunk)
    assert np.allclose(y, yref, rtol=1e-12, atol=1e-12) and flagged > 0
    src = b.kernel_source()
    assert "acc2" in src and "cell += 3u" in src and ("col_run_mask" in src) == runs
    if not runs:                                                         # the column-run form on top keeps the blocks
        assert b.set_column_runs(0)
        t2 = b.template_dump(0)
        assert t2["scalars"]["row_block"] == 3 and "col_run_mask" in t2["arrays"]
        y2 = _emulate_tile_template(t2, 500, 96, rows, x.astype(np.float64), chunk=chunk)[0]
        assert np.allclose(y2, yref, rtol=1e-12, atol=1e-12)
    # a row group height that the block does not divide
    b = build(group=100)
    assert b.set_row_ownership(0) and not b.set_row_blocks(0, 3)
    # one element taken out of one row: its block no longer holds the same columns in its three rows
    keep = np.ones(len(r), bool)
    keep[np.flatnonzero(np.asarray(r) == 301)[5]] = False
    b = build((rows, np.asarray(r)[keep], np.asarray(c)[keep], np.asarray(v)[keep]))
    assert b.set_row_ownership(0) and not b.set_row_blocks(0, 3)
    assert b.template_dump(0)["scalars"].get("row_block", 1) == 1        # nothing changed


def test_tile_template_stores_fp64_values_two_per_lane_and_load():
    """The same walk on an fp64 matrix: 16 bytes of values per lane and load are two doubles, so the values of a
    wavefront step are stored in four pieces per lane (chunk = 2)."""
    from alphasparse_amd import skeletons as SK
    rows, cols, r, c, v, x = cases._steps([3] * 40 + [20] * 24 + [90] * 8 + [1] * 30 + [300] * 3, 640, 23)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.DOUBLE, wave=64)
    m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
    m.execute_strategy(K.COMPRESS_NONE)
    tp = SK.apply_skeleton(m, 0, "T1", slice=128, group=64, b=100)[0]
    b = A.Builder(m)
    b.set_template(0, tp, compress=False)
    yref = np.zeros(rows)
    np.add.at(yref, np.asarray(r, np.int64), v.astype(np.float64) * x[np.asarray(c, np.int64)])
    y, flagged, plain = _emulate_tile_template(b.template_dump(0), 128, 64, rows, x.astype(np.float64), chunk=2)
    assert np.allclose(y, yref, rtol=1e-13, atol=1e-13) and flagged > 0
    with pytest.raises(AssertionError):
        y4 = _emulate_tile_template(b.template_dump(0), 128, 64, rows, x.astype(np.float64), chunk=4)[0]
        assert np.allclose(y4, yref, rtol=1e-13, atol=1e-13)     # the fp32 layout does not fit these arrays


@pytest.mark.parametrize("vdt,chunk", [(K.FLOAT, 4), (K.DOUBLE, 2)], ids=["fp32", "fp64"])
@pytest.mark.parametrize("sort", [False, True], ids=["plain", "sorted"])
def test_tile_template_in_column_run_form(vdt, chunk, sort):
    """set_column_runs on a matrix of dense 3 x 3 blocks: 4 run starts and one mask byte per lane instead of 8
    columns, no lane with a fifth run that is not padding, the element stream barely longer, and the same y when the
    arrays are walked the way the kernel walks them.  On a matrix with scattered columns the form is turned down
    and the template stays as it was."""
    from alphasparse_amd import skeletons as SK
    rows, cols, r, c, v, x = S.fem_blocks(400, 9, 60, seed=5)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
    if sort:
        m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
    m.execute_strategy(K.COMPRESS_NONE)
    tp = SK.apply_skeleton(m, 0, "T1", slice=500, group=64, b=1000)[0]    # 500: slices cut through the blocks
    b = A.Builder(m)
    b.set_template(0, tp, compress=False)
    b.set_launch(0, thread_num_in_block=512)
    before = b.template_dump(0)
    assert b.set_column_runs(0) and not b.set_column_runs(0)             # the second call finds the form in place
    t = b.template_dump(0)
    n_before, n = len(before["val_arr"]), len(t["val_arr"])
    assert n_before <= n <= 1.05 * n_before
    assert t["arrays"]["col_index_arr"][1] == "UNSIGNED_SHORT" and len(t["arrays"]["col_index_arr"][0]) == n // 2
    assert t["arrays"]["col_run_mask"][1] == "UNSIGNED_CHAR" and len(t["arrays"]["col_run_mask"][0]) == n // 8
    assert b.get_launch(0)["thread_num_in_block"] == 512                 # the launch setting is kept
    vv = np.float32(v).astype(np.float64) if vdt == K.FLOAT else v.astype(np.float64)
    yref = np.zeros(rows)
    np.add.at(yref, np.asarray(r, np.int64), vv * x[np.asarray(c, np.int64)])
    y, flagged, plain = _emulate_tile_template(t, 500, 64, rows, x.astype(np.float64), chunk=chunk)
    assert np.allclose(y, yref, rtol=1e-12, atol=1e-12)
    src = b.kernel_source()
    assert "col_run_mask" in src and "starts >>=" in src
    # scattered columns: every element is a run of its own, closing lanes after four would double the stream
    rows, cols, r, c, v, x = S.power_law(3000, max_len=400, mean_len=30.0, seed=2)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
    m.execute_strategy(K.COMPRESS_NONE)
    tp = SK.apply_skeleton(m, 0, "T1", slice=1024, group=512, b=4096)[0]
    b = A.Builder(m)
    b.set_template(0, tp)
    assert not b.set_column_runs(0) and "col_run_mask" not in b.template_dump(0)["arrays"]
    # another template: not applicable
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
    m.execute_strategy(K.COMPRESS_NONE)
    b = A.Builder(m)
    b.set_template(0, SK.apply_skeleton(m, 0, "S1", m=64)[0])
    assert not b.set_column_runs(0)


def test_formats_are_sized_for_the_device_they_are_told_about():
    """The tile and product-bin templates cut their element streams into one trip per workgroup the device holds:
    built for 128 compute units they have half the trips they have for 256, and a slice of x that needs more LDS
    than the device gives a workgroup is turned down.  The facts default to an MI355X and are read from the GPU at
    the first upload or search (here they are set by hand and put back)."""
    from alphasparse_amd import skeletons as SK
    rows, cols, r, c, v, x = S.power_law(200000, max_len=3000, mean_len=40.0, seed=4)
    trips = {}
    try:
        for cus in (256, 128):
            A.device_facts(cu_num=cus)
            for skel in ("T1", "T2"):
                m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
                m.execute_strategy(K.COMPRESS_NONE)
                b = A.Builder(m)
                b.set_template(0, SK.apply_skeleton(m, 0, skel, slice=16384, group=4096, b=8192)[0])
                trips[cus, skel] = b.describe(0)["group_num"]
        assert A.device_facts() == {"cu_num": 128, "lds_bytes": 163840, "xcd_num": 8, "l2_bytes_per_xcd": 4 << 20, "from_device": True}
        for skel in ("T1", "T2"):
            assert trips[256, skel] > 200 and abs(trips[128, skel] * 2 - trips[256, skel]) <= 0.1 * trips[256, skel], trips
        # 64 KB of LDS per workgroup: a 128 KB slice of x does not fit any more
        A.device_facts(lds_bytes=65536)
        m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
        m.execute_strategy(K.COMPRESS_NONE)
        tp = SK.apply_skeleton(m, 0, "T1", slice=32768, group=4096, b=8192)[0]
        assert not A.template_is_supported(m, 0, tp)
        with pytest.raises(K.AlphaSparseError):
            A.device_facts(lds_bytes=1000)
    finally:
        assert A.device_facts(reset=True) == {"cu_num": 256, "lds_bytes": 163840, "xcd_num": 8, "l2_bytes_per_xcd": 4 << 20,
                                              "from_device": False}


def _matrix_with_a_strip_of_zeros():
    """200 rows of 8 elements with values, then 100 rows of one explicit zero; sorted and cut at row length 2."""
    rng = np.random.default_rng(2)
    lens = np.r_[np.full(200, 8), np.full(100, 1)]
    r = np.repeat(np.arange(300), lens)
    c = np.concatenate([np.sort(rng.choice(300, n, replace=False)) for n in lens])
    v = np.where(r < 200, rng.uniform(0.5, 1.5, len(r)), 0.0)
    m = A.Matrix.from_coo(300, 300, r, c, v, K.DOUBLE, wave=64)
    m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
    m.execute_strategy(K.DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ, -1, (2, 2, 2, 0))
    m.execute_strategy(K.COMPRESS_NONE)
    assert m.info()["n_sub"] == 2
    return m, r, c, v, rng.uniform(-1, 1, 300)


def test_empty_template_takes_a_sub_matrix_of_zeros_and_has_no_kernel():
    """EMPTY_TEMPLATE (upstream empty_op.cc): no arrays, no kernel text beyond a comment, and the builder clears y
    because nobody else writes the rows of that sub-matrix.  A sub-matrix with a value is refused."""
    from alphasparse_amd import skeletons as SK
    m, r, c, v, x = _matrix_with_a_strip_of_zeros()
    for sub in (0, 1):
        SK.apply_skeleton(m, sub, "S1", m=64)
    assert A.template_is_supported(m, 1, K.EMPTY_TEMPLATE) and not A.template_is_supported(m, 0, K.EMPTY_TEMPLATE)
    b = A.Builder(m)
    b.set_template(0, K.DIRECT_ATOM_TEMPLATE_WARP_COMPRESS)
    b.set_template(1, K.EMPTY_TEMPLATE)
    src = b.kernel_source()
    assert "spmv_0(" in src and "spmv_1" not in src and "sub-matrix 1: no kernel" in src
    assert b.clears_y()
    b.compile()
    with pytest.raises(K.AlphaSparseError, match="not empty"):
        b.set_template(0, K.EMPTY_TEMPLATE)


def test_row_ownership_asks_for_a_cleared_y_when_a_row_group_holds_no_element():
    """Under row ownership the workgroup of a row group stores the group's rows at the end of its runs; a row group
    without elements has no run, so nobody stores its rows and y must be cleared first."""
    from alphasparse_amd import skeletons as SK
    rows, cols, r, c, v, x = S.fem_blocks(3000, 27, 400)
    for emptied, expect in (((750, 1000), 1), ((750, 999), 0), ((0, 0), 0)):
        keep = (np.asarray(r) < emptied[0]) | (np.asarray(r) >= emptied[1])
        m = A.Matrix.from_coo(rows, cols, r[keep], c[keep], v[keep].astype(np.float64), K.DOUBLE, wave=64)
        m.execute_strategy(K.COMPRESS_NONE)
        b = A.Builder(m)
        b.set_template(0, SK.apply_skeleton(m, 0, "T1", slice=4000, group=250, b=4096)[0])
        assert b.set_row_ownership(0)
        assert b.describe(0)["row_groups_without_elements"] == expect and b.clears_y() == bool(expect)


def _emulate_product_bin_template(t, slice_width, band_height, x, rows_of_y):
    """y of the product-bin template's arrays, walked the way its two kernels walk them: pass 1 writes
    val * x[slice base + column] of every element of every trip to the element's position in band order; pass 2 drops
    the products of each band into the band's slots (the j-th element of the row of rank r at first[j] + r), adds up
    every rank's slots and stores the sums to the band's rows of y.  Rows of y that the strip does not write stay NaN."""
    arr = {k: np.asarray(a[0]).astype(np.int64) for k, a in t["arrays"].items()}
    sc = t["scalars"]
    val = np.asarray(t["val_arr"][0] if isinstance(t["val_arr"], tuple) else t["val_arr"], np.float64)
    gs, gfu, ufb, shift, lcol = arr["group_slice"], arr["group_first_unit"], arr["unit_first_bin"], arr["bin_shift"], arr["col_index_arr"]
    bfu, bfc, yb, cnt, slot = (arr["band_first_unit"], arr["band_first_count"], arr["band_y_begin"], arr["band_slot_count"],
                               arr["slot_in_band"])
    flag, lcol = lcol >> 15, lcol & 0x7fff
    assert len(gfu) == len(gs) + 1 and gfu[0] == 0 and gfu[-1] * 256 == len(val) == len(lcol)
    assert (np.diff(gfu) > 0).all() and (np.diff(gs) >= 0).all() and (lcol < slice_width).all()
    nband = sc["band_num"]
    assert len(bfu) == len(bfc) == nband + 1 == len(yb) + 1 and bfu[0] == 0 and bfu[-1] * 256 == len(slot) == sc["product_len"]
    # a unit knows how many bins start before it; the first element of every slice opens one
    assert len(ufb) == gfu[-1] + 1 and ufb[-1] == len(shift) == flag.sum()
    assert (ufb[:-1] == np.concatenate([[0], np.cumsum(flag)])[:-1:256]).all()
    product = np.zeros(len(slot) + 256)
    written = np.zeros(len(slot) + 256, bool)
    for trip in range(len(gs)):
        k0, k1 = gfu[trip] * 256, gfu[trip + 1] * 256
        assert flag[k0] == 1 or (trip > 0 and gs[trip - 1] == gs[trip])      # a slice starts with a new bin
        xs = np.zeros(slice_width)
        part = x[gs[trip] * slice_width:(gs[trip] + 1) * slice_width]
        xs[:len(part)] = part
        bin0 = ufb[gfu[trip]] - 1 if ufb[gfu[trip]] else 0
        in_lds = shift[bin0:ufb[gfu[trip + 1]]]                              # the shifts the trip keeps in LDS
        assert 1 <= len(in_lds) <= sc["max_trip_bins"] <= 4096
        for u in range(gfu[trip], gfu[trip + 1]):                            # a wavefront step
            k = np.arange(u * 256, (u + 1) * 256)
            local = ufb[u] - bin0 - 1 + np.cumsum(flag[k])                   # flags up to and including the element
            assert (local >= 0).all()
            place = (k + in_lds[local]) & 0xffffffff
            assert not written[place[place < len(slot)]].any() and (val[k][place >= len(slot)] == 0).all()
            product[place] = val[k] * xs[lcol[k]]
            written[place] = True
    # padding of the first pass (value 0) lands behind the products
    assert (product[len(slot):] == 0).all()
    written, product = written[:len(slot) + 1], product[:len(slot) + 1]
    y = np.full(rows_of_y, np.nan)
    stored = np.zeros(rows_of_y, int)
    for g in range(nband):
        first = cnt[bfc[g]:bfc[g + 1]]                 # first[j]: slots of the elements 0..j-1 of all rows
        width = len(first) - 1
        assert width >= 1 and first[0] == 0 and (np.diff(first) >= 0).all() and (np.diff(first, 2) <= 0).all()
        assert width <= sc["max_width"] and first[-1] + 1 <= sc["max_slots"]
        k0, k1 = bfu[g] * 256, bfu[g + 1] * 256
        assert k1 - k0 >= first[-1] > k1 - k0 - 256 or (first[-1] == 0 and k1 == k0)
        slots = np.full(first[-1] + 1, np.nan)
        real_slot = slot[k0:k1][written[k0:k1]]
        assert (slot[k0:k1][~written[k0:k1]] == first[-1]).all()      # band padding: spare slot, never written
        assert sorted(real_slot) == list(range(first[-1]))            # every slot filled exactly once: no clear needed
        assert (product[k0:k1][~written[k0:k1]] == 0).all()
        slots[slot[k0:k1]] = product[k0:k1]
        live = first[1]

        def row_sum(r):
            return sum(slots[first[j] + r] for j in range(width) if r < first[j + 1] - first[j])
        if sc["dense_y"]:
            ye, rank = arr["band_y_end"], arr["rank_of_y_row"]
            assert yb[g] < ye[g] <= yb[g] + band_height and (g == 0 or ye[g - 1] <= yb[g])
            for p in range(yb[g], ye[g]):
                if rank[p] != 0xffff:
                    y[sc["y_base"] + p] = row_sum(rank[p]) if rank[p] < live else 0.0
                    stored[sc["y_base"] + p] += 1
        else:
            bfr, place = arr["band_first_row"], arr["y_row_of_rank"]
            assert live <= bfr[g + 1] - bfr[g] and (place[bfr[g]:bfr[g + 1]] < band_height).all()
            for r in range(bfr[g + 1] - bfr[g]):
                y[sc["y_base"] + yb[g] + place[bfr[g] + r]] = row_sum(r)
                stored[sc["y_base"] + yb[g] + place[bfr[g] + r]] += 1
    assert stored.max() == 1 and stored.sum() == sc["sub_rows"]
    return y


@pytest.mark.parametrize("slice_width,group,blb,sort", [(32, 16, 64, False), (128, 64, 100, True), (1024, 8, 17, False),
                                                          (64, 4096, 4096, True)])
def test_product_bin_template(slice_width, group, blb, sort):
    """SHARED_MEMORY_PRODUCT_BIN_TEMPLATE on the tile division: slices padded to whole 256-element units, trips cut
    inside slices, bands of `group` rows of y with their rows ranked by falling length; two passes reproduce y = A x."""
    from alphasparse_amd import skeletons as SK
    rows, cols, r, c, v, x = cases._steps([3] * 40 + [9] * 24 + [1] * 30 + [2] * 70 + [7] * 13, 640, 22)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
    if sort:
        m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
    m.execute_strategy(K.COMPRESS_NONE)
    tp = SK.apply_skeleton(m, 0, "T2", slice=slice_width, group=group, b=blb)[0]
    assert tp == K.SHARED_MEMORY_PRODUCT_BIN_TEMPLATE and A.template_is_supported(m, 0, tp)
    assert A.template_is_supported(m, 0, K.SHARED_MEMORY_TILE_TEMPLATE)
    assert not A.template_is_supported(m, 0, K.DIRECT_ATOM_TEMPLATE_WARP_COMPRESS)
    yref = np.zeros(rows)
    np.add.at(yref, np.asarray(r, np.int64), np.float32(v).astype(np.float64) * x[np.asarray(c, np.int64)])
    b = A.Builder(m)
    b.set_template(0, tp, compress=False)
    t = b.template_dump(0)
    assert t["scalars"]["dense_y"] == 1 and t["scalars"]["band_num"] == -(-rows // group)
    y = _emulate_product_bin_template(t, slice_width, group, x.astype(np.float64), rows)
    assert np.allclose(y, yref, rtol=1e-12, atol=1e-12)
    assert t["arrays"]["col_index_arr"][1] == "UNSIGNED_SHORT" and t["arrays"]["slot_in_band"][1] == "UNSIGNED_SHORT"
    assert t["arrays"]["rank_of_y_row"][1] == "UNSIGNED_SHORT"
    b.set_template(0, tp, compress=True)
    src = b.kernel_source()
    assert "spmv_0_finish" in src and "scratch_arr" in src and "rank_of_y_row[" in src
    assert not b.clears_y()     # the second pass stores every row of the strip


def _short_rows_with_a_few_longer(rows, seed, longer=50):
    rng = np.random.default_rng(seed)
    lens = rng.integers(1, 4, rows)
    lens[rng.choice(rows, longer, replace=False)] = rng.integers(5, 30, longer)
    r = np.repeat(np.arange(rows), lens)
    c = np.concatenate([np.sort(rng.choice(rows, n, replace=False)) for n in lens])
    return lens, r, c, rng.uniform(-1, 1, len(r)), rng.uniform(-1, 1, rows)


def test_product_bin_template_takes_sorted_rows_band_by_band():
    """Under a sort the product-bin template still takes the rows band by band of y (here 4096 rows of y each) and
    ranks them by falling length inside a band, whatever their place in the sorted strip: the ranks of a band are a
    permutation of its rows, a longer row never has a higher rank than a shorter one, and the two passes reproduce
    y = A x."""
    from alphasparse_amd import skeletons as SK
    rows = cols = 10000
    lens, r, c, v, x = _short_rows_with_a_few_longer(rows, 3)
    m = A.Matrix.from_coo(rows, cols, r, c, v, K.DOUBLE, wave=64)
    m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
    m.execute_strategy(K.COMPRESS_NONE)
    tp = SK.apply_skeleton(m, 0, "T2", slice=1024, group=4096, b=4096)[0]
    b = A.Builder(m)
    b.set_template(0, tp, compress=False)
    t = b.template_dump(0)
    assert t["scalars"]["band_num"] == 3 and t["scalars"]["dense_y"] == 1 and t["scalars"]["y_base"] == 0
    rank = np.asarray(t["arrays"]["rank_of_y_row"][0]).astype(np.int64)
    yb, ye = (np.asarray(t["arrays"][k][0]).astype(np.int64) for k in ("band_y_begin", "band_y_end"))
    assert list(yb) == [0, 4096, 8192] and list(ye) == [4096, 8192, 10000]
    for g in range(3):
        inside = rank[yb[g]:ye[g]]
        assert sorted(inside) == list(range(ye[g] - yb[g]))
        by_rank = lens[yb[g]:ye[g]][np.argsort(inside)]
        assert (np.diff(by_rank) <= 0).all()                          # longest first
        same = np.flatnonzero(np.diff(by_rank) == 0)
        assert (np.diff(np.argsort(inside))[same] > 0).all()          # rows of equal length in the order of y
    yref = np.zeros(rows)
    np.add.at(yref, r, v * x[c])
    y = _emulate_product_bin_template(t, 1024, 4096, x, rows)
    assert np.allclose(y, yref, rtol=1e-12, atol=1e-12)


def test_product_bin_template_cuts_bands_by_their_lds_slots_and_stores_by_rank_in_a_thin_strip():
    """A band ends where its elements would no longer fit its LDS slots (80 KB: 10239 fp64 elements), and a strip
    that holds few of the rows of y it spans (here the rows of 5 or more elements of a sorted matrix) keeps a 16-bit
    place in y per rank instead of a rank per row of y."""
    from alphasparse_amd import skeletons as SK
    rows = cols = 12000
    rng = np.random.default_rng(8)
    lens = np.full(rows, 7)
    r = np.repeat(np.arange(rows), lens)
    c = np.concatenate([np.sort(rng.choice(cols, n, replace=False)) for n in lens])
    v, x = rng.uniform(-1, 1, len(r)), rng.uniform(-1, 1, cols)
    m = A.Matrix.from_coo(rows, cols, r, c, v, K.DOUBLE, wave=64)
    m.execute_strategy(K.COMPRESS_NONE)
    tp = SK.apply_skeleton(m, 0, "T2", slice=4096, group=65536, b=4096)[0]
    b = A.Builder(m)
    b.set_template(0, tp, compress=False)
    t = b.template_dump(0)
    per_band = 10239 // 7
    assert t["scalars"]["band_num"] == -(-rows // per_band) and t["scalars"]["max_slots"] == per_band * 7 + 1
    yref = np.zeros(rows)
    np.add.at(yref, r, v * x[c])
    assert np.allclose(_emulate_product_bin_template(t, 4096, 65536, x, rows), yref, rtol=1e-12, atol=1e-12)
    # the thin strip
    rows = cols = 10000
    lens, r, c, v, x = _short_rows_with_a_few_longer(rows, 5, longer=200)
    m = A.Matrix.from_coo(rows, cols, r, c, v, K.DOUBLE, wave=64)
    m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
    m.execute_strategy(K.DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ, -1, (5, 5, 2, 0))
    m.execute_strategy(K.COMPRESS_NONE)
    assert m.info()["n_sub"] == 2                      # sorted: the 200 rows of 5 or more elements come first
    tp = SK.apply_skeleton(m, 0, "T2", slice=1024, group=2048, b=4096)[0]
    b = A.Builder(m)
    b.set_template(0, tp, compress=False)
    t = b.template_dump(0)
    assert t["scalars"]["sub_rows"] == 200
    assert t["scalars"]["dense_y"] == 0 and "y_row_of_rank" in t["arrays"] and "rank_of_y_row" not in t["arrays"]
    yref = np.zeros(rows)
    np.add.at(yref, r, v * x[c])
    y = _emulate_product_bin_template(t, 1024, 2048, x, rows)
    mine = lens >= 5
    assert np.isnan(y[~mine]).all() and np.allclose(y[mine], yref[mine], rtol=1e-12, atol=1e-12)
    b.set_template(0, tp, compress=True)
    assert "y_row_of_rank[" in b.kernel_source()


def test_relative_columns_of_the_ell_template():
    """set_relative_columns: the ELL template's columns become 16-bit differences to the TLB number (element k of
    TLB t at t + k * T); decoding them gives the 32-bit array back, except that far-away padding points at column t.
    A matrix with an element farther than 32767 columns from its row, or another template, is left alone."""
    from alphasparse_amd import skeletons as SK
    rows, cols, r, c, v, x = S.laplacian_5pt(300)                 # 90,000 rows: the +-300 band fits, row numbers do not
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
    m.execute_strategy(K.COMPRESS_NONE)
    tp = SK.apply_skeleton(m, 0, "S5")[0]
    b = A.Builder(m)
    b.set_template(0, tp)
    before = b.template_dump(0)
    wide = np.asarray(before["arrays"]["col_index_arr"][0]).astype(np.int64)
    assert before["arrays"]["col_index_arr"][1] == "UNSIGNED_INT"
    assert b.set_relative_columns(0) and b.set_relative_columns(0)
    after = b.template_dump(0)
    assert after["arrays"]["col_index_arr"][1] == "UNSIGNED_SHORT"
    narrow = np.asarray(after["arrays"]["col_index_arr"][0]).astype(np.int64)
    val = np.asarray(after["val_arr"][0] if isinstance(after["val_arr"], tuple) else after["val_arr"], np.float64)
    T = len(wide) // 5
    assert len(wide) == 5 * T == len(narrow)
    tlb = np.arange(len(wide)) % T
    decoded = tlb + np.where(narrow >= 32768, narrow - 65536, narrow)
    moved = decoded != wide
    assert (val[moved] == 0).all() and (decoded[moved] == np.minimum(tlb[moved], cols - 1)).all()
    assert (np.abs(wide[moved] - tlb[moved]) > 32767).all()
    assert moved.sum() < len(wide) // 100 and (decoded >= 0).all() and (decoded < cols).all()
    src = b.kernel_source()
    assert "(short)" in src and "unsigned short *__restrict__ col_index_arr" in src
    # random columns: not applicable, nothing changes
    rows, cols, r, c, v, x = S.uniform_rows(100000, 4, seed=3)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
    m.execute_strategy(K.COMPRESS_NONE)
    b = A.Builder(m)
    b.set_template(0, SK.apply_skeleton(m, 0, "S5")[0])
    assert not b.set_relative_columns(0) and b.template_dump(0)["arrays"]["col_index_arr"][1] == "UNSIGNED_INT"
    # another template: not applicable
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
    m.execute_strategy(K.COMPRESS_NONE)
    b = A.Builder(m)
    b.set_template(0, SK.apply_skeleton(m, 0, "S1", m=64)[0])
    assert not b.set_relative_columns(0)


def test_diagonal_columns_of_the_ell_template():
    """set_diagonal_columns: on a stencil every element moves to the slot of its diagonal, the column array shrinks to
    a dummy and slot k of TLB t means column t + diagonal_offset_k; the slots reproduce y = A x.  Matrices whose rows
    do not share their diagonals are left alone."""
    from alphasparse_amd import skeletons as SK
    rows, cols, r, c, v, x = S.laplacian_5pt(300)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
    m.execute_strategy(K.COMPRESS_NONE)
    b = A.Builder(m)
    b.set_template(0, SK.apply_skeleton(m, 0, "S5")[0])
    assert b.set_diagonal_columns(0) and b.set_diagonal_columns(0)
    t = b.template_dump(0)
    offs = [int(np.int64(np.uint64(t["scalars"]["diagonal_offset_%d" % k]))) for k in range(5)]
    assert offs == [-300, -1, 0, 1, 300] and len(t["arrays"]["col_index_arr"][0]) == 1
    val = np.asarray(t["val_arr"][0] if isinstance(t["val_arr"], tuple) else t["val_arr"], np.float64)
    T = len(val) // 5
    y = np.zeros(T)
    for k, off in enumerate(offs):
        col = np.clip(np.arange(T) + off, 0, cols - 1)
        y += val[k * T:(k + 1) * T] * x[col]
    yref = np.zeros(rows)
    np.add.at(yref, r, np.float32(v).astype(np.float64) * x[c])
    assert np.allclose(y[:rows], yref, rtol=1e-12, atol=1e-12) and (val[np.arange(len(val)) % T >= rows] == 0).all()
    src = b.kernel_source()
    assert "col_index_arr +" not in src and "(-300)" in src
    # 3x3 blocks at random block columns: the rows do not share five diagonals
    rows, cols, r, c, v, x = S.fem_blocks(300, 9, 100)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
    m.execute_strategy(K.COMPRESS_NONE)
    b = A.Builder(m)
    b.set_template(0, SK.apply_skeleton(m, 0, "S5")[0])
    before = b.template_dump(0)
    assert not b.set_diagonal_columns(0)
    after = b.template_dump(0)
    assert np.array_equal(before["arrays"]["col_index_arr"][0], after["arrays"]["col_index_arr"][0])
    assert before["arrays"]["col_index_arr"][1] == after["arrays"]["col_index_arr"][1]


def test_remove_empty_rows_and_sort_through_the_map():
    """remove_empty_rows renumbers the rows that hold elements in order and keeps the map to y; a coarse sort
    afterwards permutes compacted rows and its permutation goes through that map; templates write original rows."""
    from alphasparse_amd import skeletons as SK
    lens = np.array([3, 0, 0, 5, 1, 0, 2, 9, 0, 1, 0, 0, 4, 0], dtype=np.int64)
    rng = np.random.default_rng(3)
    cols = 40
    r = np.repeat(np.arange(len(lens)), lens)
    c = np.concatenate([np.sort(rng.choice(cols, n, replace=False)) for n in lens if n])
    v = rng.uniform(-1, 1, len(r))
    x = rng.uniform(-1, 1, cols)
    yref = np.zeros(len(lens))
    np.add.at(yref, r, np.float32(v).astype(np.float64) * x[c])
    kept = np.flatnonzero(lens)
    m = A.Matrix.from_coo(len(lens), cols, r, c, v, K.FLOAT, wave=64)
    assert m.has_empty_row()
    m.remove_empty_rows()
    info = m.info()
    assert info["rows"] == len(kept) and m.y_rows() == len(lens) and not info["is_sorted"]
    d = m.dump()
    assert np.array_equal(d["sorted_row_index"][0], kept)
    assert np.array_equal(kept[d["coo_row_index_cache"].astype(np.int64)], r)
    with pytest.raises(A.AlphaSparseError):
        m.remove_empty_rows()                                   # first operator only
    m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
    d = m.dump()
    perm = d["sorted_row_index"][0].astype(np.int64)
    assert sorted(perm.tolist()) == kept.tolist() and m.info()["rows"] == len(kept)
    assert (np.diff(lens[perm]) <= 0).all()                     # longest first
    assert sorted(perm[d["coo_row_index_cache"].astype(np.int64)].tolist()) == sorted(r.tolist())
    m.execute_strategy(K.COMPRESS_NONE)
    tp = SK.apply_skeleton(m, 0, "T1", slice=16, group=4, b=8)[0]
    b = A.Builder(m)
    b.set_template(0, tp, compress=False)
    assert b.rows == len(lens)
    y = _emulate_tile_template(b.template_dump(0), 16, 4, len(kept), x)[0]
    assert len(y) <= len(lens) and np.allclose(np.r_[y, np.zeros(len(lens) - len(y))], yref, rtol=1e-12, atol=1e-12)
    # a matrix without empty rows is left alone
    m2, _, _, _ = _matrix(17, 64)
    before = m2.info()["rows"]
    m2.remove_empty_rows()
    assert m2.info()["rows"] == before and "sorted_row_index" not in m2.dump()


def test_every_barrier_of_the_generated_kernels_waits_for_the_wavefronts_lds_operations():
    """Every workgroup barrier in the generated kernels is as_barrier(): the wait for the wavefront's outstanding LDS
    operations is written out in front of it.  (The compiler left that wait out on one path into a barrier of the
    fused tile + product-bin kernel -- the last iteration of the loop over a trip's runs -- and rows of the tile
    strip then lost the sums of a trip's last run now and then.)"""
    import os
    import sys
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
    import __graft_entry__ as G
    from alphasparse_amd import skeletons as SK
    mats = {"power_law": S.power_law(512, max_len=200, mean_len=12.0, seed=11), "uniform": S.uniform_rows(512, 40, seed=12)}
    with_lds = 0
    for mat, skel, kw in G.kernel_build_cases():
        rows, cols, r, c, v, _ = mats[mat]
        m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
        m.execute_strategy(K.COMPRESS_NONE)
        for template in SK.apply_skeleton(m, 0, skel, **kw):
            b = A.Builder(m)
            b.set_template(0, template)
            src = b.kernel_source()
            assert src.count("__syncthreads()") == 1 and "s_waitcnt lgkmcnt(0)" in src.split("__syncthreads()")[0].splitlines()[-1], K.TEMPLATE_NAMES[template]
            with_lds += "as_barrier();" in src
    assert with_lds >= 6


def test_tile_trips_fit_one_round_of_workgroups():
    """The tile template cuts its element stream into trips between BLBs; however the cuts fall, there are never more
    trips than workgroups the device holds at a time with the template's LDS need (one more would wait for a second
    round and the kernel would take nearly twice as long).  Cases 16, 99, 113 and 127 came out one to six trips above
    that before the share of a trip was raised until the trips fit."""
    from alphasparse_amd import skeletons as SK
    at_the_limit = 0
    try:
        for case in (16, 99, 113, 127, 0, 1, 3, 4, 5, 6, 7, 8):
            rng = np.random.default_rng(9000 + case)
            cus = int(rng.choice([8, 16, 24, 64]))
            A.device_facts(cu_num=cus)
            rows = int(rng.integers(2000, 30000))
            mult = int(rng.integers(1, 40))
            lens = np.minimum(rng.zipf(1.7, rows) * mult, 3000)
            rows, cols, r, c, v, x = cases._steps(lens, max(rows, int(lens.max())), 9000 + case)
            m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
            if rng.integers(2):
                m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
            m.execute_strategy(K.COMPRESS_NONE)
            slice_width, group = int(rng.choice([1024, 4096, 16384, 32768])), int(rng.choice([512, 2048, 4096, 6144]))
            blb = int(rng.choice([64, 256, 1024, 8192]))
            b = A.Builder(m)
            b.set_template(0, SK.apply_skeleton(m, 0, "T1", slice=slice_width, group=group, b=blb)[0])
            per_cu = max(1, 163840 // ((slice_width + group) * 4))
            trips = b.describe(0)["group_num"]
            assert 1 <= trips <= cus * per_cu, (case, trips, cus, per_cu)
            assert b.get_launch(0)["tblock_num"] == trips
            at_the_limit += trips > 0.9 * cus * per_cu
            b.close()
    finally:
        A.device_facts(reset=True)
    assert at_the_limit >= 6      # the cases do reach the limit
