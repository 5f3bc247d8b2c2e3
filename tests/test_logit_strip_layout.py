"""CPU: the index arithmetic of the logit strip of the selection-layer kernel
(tidaldecode_amd/csrc/decode_attn.cuh: the strip writes of the two score paths and the reads of
emit_flush), restated lane by lane for every instantiated (head_dim, heads per KV row, waves, rows
per lane) and checked as sets: per waiting tile the 64 lanes of a wave write every (head, token)
cell of the tile exactly once, no two waves share a cell, and the flush reads exactly the cells
that were written and sends each to the token and head it was computed for.  The kernel orders the
writes before the reads with an LDS wait and a wave barrier; this test pins the other half, that
the two sides agree on where a logit lives."""
import re
from pathlib import Path

import pytest

SRC = Path(__file__).resolve().parents[1] / "tidaldecode_amd" / "csrc" / "decode_attn.cuh"


def instantiated_shapes():
    """(head_dim, qpg, waves, rows) of every TD_CASE line of the dispatch table"""
    text = SRC.read_text()
    shapes = [tuple(int(x) for x in m.groups())
              for m in re.finditer(r"^\s*TD_CASE\((\d+), (\d+), (\d+), (\d+)\)\s*$", text, re.M)]
    assert len(shapes) >= 17
    return shapes


def geometry(d, qpg, nw, u):
    lpr = d // 8
    tpi = 64 // lpr
    tile = u * tpi
    floats = 512 if nw == 16 else (3072 if qpg > 1 else 1024)   # EMIT_FLOATS of decode_attn.cuh
    tiles = floats // (qpg * tile)
    return lpr, tpi, tile, floats, tiles


def strip_writes(d, qpg, nw, u, wave, slot):
    """{strip index: (head, token offset in the tile)} written by the 64 lanes for one tile"""
    lpr, tpi, tile, floats, tiles = geometry(d, qpg, nw, u)
    mma = qpg > 1 and lpr == 16
    out = {}
    for lane in range(64):
        g, li = lane // lpr, lane % lpr
        if mma:
            copies = 16 // qpg
            head, c = li % qpg, li // qpg
            base = (wave * tiles + slot) * (qpg * tile)
            for u0 in range(0, u, copies):
                if u0 + c < u:
                    idx = base + head * tile + (u0 + c) * tpi + g
                    assert idx not in out, "two lanes write one cell"
                    out[idx] = (head, (u0 + c) * tpi + g)
        else:
            assert u <= lpr
            for j in range(qpg):
                if li < u:
                    idx = ((wave * tiles + slot) * qpg + j) * tile + li * tpi + g
                    assert idx not in out, "two lanes write one cell"
                    out[idx] = (j, li * tpi + g)
    return out


def strip_reads(d, qpg, nw, u, wave, n_waiting):
    """[(strip index, head, waiting tile, token offset)] read by emit_flush"""
    lpr, tpi, tile, floats, tiles = geometry(d, qpg, nw, u)
    tps = max(64 // tile, 1)
    out = []
    for lane in range(64):
        lt, ltok = lane // tile, lane % tile
        for n0 in range(0, n_waiting, tps):
            n = n0 + lt
            for j in range(qpg):
                if n < n_waiting:
                    out.append((((wave * tiles + n) * qpg + j) * tile + ltok, j, n, ltok))
    return out


@pytest.mark.parametrize("shape", instantiated_shapes(), ids=lambda s: "d%d_q%d_w%d_u%d" % s)
def test_strip_writes_and_reads_agree(shape):
    d, qpg, nw, u = shape
    lpr, tpi, tile, floats, tiles = geometry(d, qpg, nw, u)
    assert tile <= 64 and tiles >= 1 and tiles * qpg * tile <= floats
    owner = {}
    for wave in range(nw):
        written = {}
        for slot in range(tiles):
            w = strip_writes(d, qpg, nw, u, wave, slot)
            # every (head, token) cell of the tile, once
            assert sorted(w.values()) == [(j, t) for j in range(qpg) for t in range(tile)]
            for idx, cell in w.items():
                assert idx not in written and idx not in owner, "tiles or waves overlap"
                assert wave * floats <= idx < (wave + 1) * floats
                written[idx] = (slot,) + cell
        for idx in written:
            owner[idx] = wave
        for n_waiting in (1, tiles // 2 or 1, tiles):
            reads = strip_reads(d, qpg, nw, u, wave, n_waiting)
            seen = set()
            for idx, j, n, ltok in reads:
                assert written[idx] == (n, j, ltok), "a logit goes to another head or token"
                assert idx not in seen, "a cell is stored twice"
                seen.add(idx)
            assert seen == {i for i, c in written.items() if c[0] < n_waiting}


def _plan(batch, hq, hkv, d, rows, items):
    from tidaldecode_amd._lib import DecodePlan, lib

    p = DecodePlan(0, 0, 0, 0, -1, -1, 0, 0)  # sparse_waves -1: the streaming kernel, as with score output
    assert lib.td_decode_make_plan(batch, hq, hkv, d, rows, items, p) == 0
    return p


def emitted_tokens(n_items, chunk, max_splits, nw, u, d=128):
    """Every (token, split, wave, tile of that wave) whose logit the selection-layer kernel stores:
    the kernel's walk (tile t of the row belongs to split t mod splits, waves take interleaved
    tiles) followed through the strip (emit_push / emit_flush: first token of the oldest waiting
    tile, a fixed stride between a wave's tiles) down to the index `i` the store uses."""
    lpr, tpi, tile, floats, strip_tiles = geometry(d, 1, nw, u)
    n_splits = max(1, min(max_splits, -(-n_items // chunk)))
    step = n_splits * nw * tile
    out = []
    for split in range(n_splits):
        for wave in range(nw):
            waiting, first, n_tile = 0, 0, 0
            t = (split * nw + wave) * tile

            def flush():
                for n in range(waiting):
                    for ltok in range(tile):
                        i = first + n * step + ltok
                        if i < n_items:
                            out.append((i, split, wave, n_tile - waiting + n))

            while t < n_items:
                if waiting == 0:
                    first = t
                waiting += 1
                n_tile += 1
                if waiting == strip_tiles:
                    flush()
                    waiting = 0
                t += step
            flush()
    return out


@pytest.mark.parametrize("n", [1, 15, 16, 17, 1000, 4099, 32769, 33000, 102400])
@pytest.mark.parametrize("hq,hkv", [(32, 32), (40, 40)])
def test_every_logit_has_exactly_one_writer(n, hq, hkv):
    """The selection layer of one sequence of n tokens, one query head per head row (the case of
    the 33000-token logit observation): with the plan the library makes for it, every token's
    logit is stored by exactly one (split, wave, tile), none beyond the sequence -- two writers of
    one cell, say at a split edge or where the forced last page follows the listed pages, would be
    the one way a cell could receive a second value."""
    page = 16
    n_pages = -(-n // page)
    last_len = n - (n_pages - 1) * page
    items = (n_pages - 1) * page + last_len   # listed pages, all full, then the forced last page
    assert items == n
    p = _plan(1, hq, hkv, 128, 1, items)
    assert p.sparse_waves == 0 and p.chunk_tokens * p.max_splits >= items
    stored = emitted_tokens(items, p.chunk_tokens, p.max_splits, p.waves_per_block, p.tile_rows)
    tokens = sorted(i for i, *_ in stored)
    assert tokens == list(range(n))
    # the walk itself: token i of the list is entry i % page of page i // page, the forced last page
    # taking over exactly where the listed pages end (decode_page.cuh:326-329 of the reference)
    for i in (0, (n_pages - 1) * page - 1, (n_pages - 1) * page, n - 1):
        if 0 <= i < n:
            listed = i // page < n_pages - 1
            assert listed == (i < (n_pages - 1) * page)
