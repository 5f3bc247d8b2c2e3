"""CPU: which list columns the short-list kernel may touch before it knows a sequence's length.

sparse_attn_kernel (csrc/sparse_attn.cuh) asks for the list entries of a wave's first tile
together with the kernel arguments, before the device-resident count of the sequence has arrived;
`list_capacity` (csrc/decode_attn.cuh) bounds the column it reads.  This file restates that
arithmetic for whole launches — every sequence, split, wave, tile and lane — and checks, for packed
(indptr) and padded (indptr + counts) tables with ragged lengths, that
  * no read leaves the index array (the last sequence of a packed table is shorter than the
    host's bound: reading n_list_host columns from its start would run past the array),
  * no read leaves the sequence's own segment,
  * every listed token is paired with its own entry.
The layout follows the reference's per-sequence segments of the index array
(kernels/include/decode/decode_attn.cuh:432-470, `indptr`)."""
import random

import pytest


def list_capacity(n_list_host, has_indptr, list_beg, list_end, row_cols):
    cap = n_list_host
    if has_indptr:
        cap = min(cap, list_end - list_beg)
    if row_cols > 0:
        cap = min(cap, row_cols - list_beg)
    return max(cap, 0)


def launch_reads(n_list_host, indptr, counts, row_cols, chunk, nw, rows_per_lane, max_splits, last_len=0):
    """(sequence, column read, token index) for every list read of a launch; the kernel's loop:
    t0 = (split * NW + wave) * TILE, step n_splits * NW * TILE, lane owns token t + own."""
    tile = 4 * rows_per_lane
    out = []
    for b in range(len(indptr) - 1):
        beg, end = indptr[b], indptr[b + 1]
        cap = list_capacity(n_list_host, True, beg, end, row_cols)
        n_list = counts[b] if counts is not None else end - beg
        n_list = max(0, min(n_list, cap))
        c1 = n_list + last_len
        n_splits = max(1, min(max_splits, -(-c1 // chunk)))
        for split in range(n_splits):
            for wave in range(nw):
                t0 = (split * nw + wave) * tile
                t = t0
                first = True
                while first or t < c1:      # the first fetch is unconditional
                    for own in range(tile):
                        pos = min(t + own, cap - 1)
                        if cap > 0:
                            out.append((b, beg + pos, t + own, n_list))
                    first = False
                    t += n_splits * nw * tile
    return out


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("padded", [False, True])
def test_reads_stay_inside_the_array_and_the_segment(seed, padded):
    rng = random.Random(seed)
    batch = rng.randint(1, 8)
    ks = [rng.choice([0, 1, 5, 31, 32, 33, 200, 700]) for _ in range(batch)]
    if batch > 1:
        ks[-1] = min(ks[-1], 5)                       # a short last sequence: the packed case that overran
        ks[0] = max(ks[0], 300)
    n_list_host = max(ks)
    if padded:
        width = n_list_host + rng.randint(0, 3)
        indptr = [i * width for i in range(batch + 1)]
        counts = ks
    else:
        indptr = [0]
        for k in ks:
            indptr.append(indptr[-1] + k)
        counts = None
    total = indptr[-1]                                # elements of a row (one row, or the row stride)
    for row_cols in (total, 0):
        for nw, rpl in ((8, 8), (4, 8), (4, 16), (8, 16)):
            chunk = nw * 4 * rpl
            max_splits = max(1, -(-(n_list_host + 16) // chunk))
            reads = launch_reads(n_list_host, indptr, counts, row_cols, chunk, nw, rpl, max_splits, last_len=3)
            for b, col, token, n_list in reads:
                assert 0 <= col < total, (b, col, total)
                assert indptr[b] <= col < indptr[b + 1], (b, col)
                if token < n_list:
                    assert col == indptr[b] + token, (b, col, token)


def test_the_host_bound_alone_would_leave_a_packed_array():
    """The case that motivated the segment clamp: packed lists, a last sequence shorter than the
    longest.  Clamping to n_list_host alone reads max(ks) columns from the last segment's start."""
    ks = [700, 3]
    indptr = [0, 700, 703]
    n_list_host = max(ks)
    worst_old = indptr[1] + min(31, n_list_host - 1)          # lane 31 of the first tile of sequence 1
    assert worst_old >= indptr[-1]
    cap = list_capacity(n_list_host, True, indptr[1], indptr[2], 0)
    assert indptr[1] + min(31, cap - 1) < indptr[-1]


def test_counts_beyond_the_segment_are_cut():
    """A device-resident count larger than the segment cannot pair a token with a column outside it."""
    reads = launch_reads(64, [0, 40, 80], [64, 64], 80, 128, 4, 8, 1)
    assert max(col for _, col, _, _ in reads) < 80
    assert all(n == 40 for _, _, _, n in reads)
