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
    floats = 512 if nw == 16 else 1024
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
