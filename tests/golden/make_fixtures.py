#!/usr/bin/env python3
"""Writes the golden fixtures of tests/golden/ from the CPU oracle (oracle/tidal_oracle.py).

The reference ships no golden vectors for the decode path (its tests use unseeded random input),
and its Python path cannot be imported in this environment (it needs transformers 4.45's
LlamaSdpaAttention), so the vectors come from this build's oracle AFTER that oracle has been
pinned by tests/test_oracle.py.  They freeze its behaviour and travel to the GPU box, where the
HIP path is compared against them.

    python tests/golden/make_fixtures.py

cfg0.npz      benchmark configuration 0: 32/32 heads, head_dim 128, 4096 tokens, top_k 256.
              Inputs are regenerated from seeds (selection layer seed 0, sparse layer seed 1) and
              rounded to fp16, so only outputs are stored.
small.npz     4 query / 2 KV heads, head_dim 64, 96 tokens, page size 4, top_k 16, fp16: inputs
              and outputs, including the paged pool and page table.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import tidal_oracle as orc  # noqa: E402


def draw(shape, seed, dtype=torch.float16):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g).to(dtype).float()


def cfg0_inputs(layer_seed):
    """q [32,128], k, v [4096,32,128]; one generator per layer, drawn in the order q, k, v"""
    g = torch.Generator().manual_seed(layer_seed)
    q = torch.randn((32, 128), generator=g).half().float()
    k = torch.randn((4096, 32, 128), generator=g).half().float()
    v = torch.randn((4096, 32, 128), generator=g).half().float()
    return q, k, v


def make_cfg0():
    out = {}
    q0, k0, v0 = cfg0_inputs(0)
    q1, k1, v1 = cfg0_inputs(1)
    for mode in ("per_head", "head_sum"):
        o_sel, idx, logits = orc.select_layer(q0, k0, v0, 256, mode)
        o_sp = orc.sparse_layer(q1, k1, v1, orc.mask_from_indices(idx, 32, 4096))
        out[f"{mode}_idx"] = idx.numpy().astype(np.int32)
        out[f"{mode}_o_sparse"] = o_sp.numpy()
        if mode == "head_sum":
            out["head_sum_scores"] = orc.head_sum_scores(logits, 1).numpy()
    out["o_select"] = o_sel.numpy()
    np.savez_compressed(os.path.join(HERE, "cfg0.npz"), **out)


def make_small():
    hq, hkv, d, n, page, k = 4, 2, 64, 96, 4, 16
    q_sel, q_sp = draw((hq, d), 10), draw((hq, d), 11)
    kk, vv = draw((n, hkv, d), 12), draw((n, hkv, d), 13)
    n_pages = n // page
    table = torch.randperm(n_pages + 3, generator=torch.Generator().manual_seed(14))[:n_pages]
    pool = np.zeros(orc.pool_shape(n_pages + 3, page, hkv, d), dtype=np.float32)
    orc.paged_append(pool, table.tolist(), n, kk.numpy(), vv.numpy())
    out = dict(q_select=q_sel.numpy(), q_sparse=q_sp.numpy(), k=kk.numpy(), v=vv.numpy(),
               pool=pool.astype(np.float16), page_table=table.numpy().astype(np.int32))
    for mode in ("per_head", "group_sum", "head_sum"):
        o_sel, idx, logits = orc.select_layer(q_sel, kk, vv, k, mode)
        out[f"{mode}_idx"] = idx.numpy().astype(np.int32)
        out[f"{mode}_slots"] = (table[idx // page] * page + idx % page).numpy().astype(np.int32)
        out[f"{mode}_o_sparse"] = orc.sparse_layer(q_sp, kk, vv,
                                                   orc.mask_from_indices(idx, hq, n)).numpy()
    out["o_select"] = o_sel.numpy()
    out["logits"] = logits.numpy()
    np.savez_compressed(os.path.join(HERE, "small.npz"), **out)


if __name__ == "__main__":
    make_cfg0()
    make_small()
    for f in ("cfg0.npz", "small.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
