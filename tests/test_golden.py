"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py).

CPU: the oracle still reproduces them (guards the oracle against silent change).
GPU: the HIP path -- selection layer with logits, score reduction, top-k, sparse layer -- reproduces
them: attention within 2e-3 max-abs (fp16), index lists bit-exact when computed from the same
scores, and equal to the fixture's lists up to elements whose scores tie with the threshold within
the fp32 evaluation error of the logits.
"""
import os
import sys

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
from make_fixtures import cfg0_inputs  # noqa: E402


def _load(name):
    return np.load(os.path.join(HERE, "golden", name))


def test_oracle_reproduces_small_fixture():
    from oracle import tidal_oracle as orc

    f = _load("small.npz")
    q_sel, q_sp = torch.from_numpy(f["q_select"]), torch.from_numpy(f["q_sparse"])
    k, v = torch.from_numpy(f["k"]), torch.from_numpy(f["v"])
    for mode in ("per_head", "group_sum", "head_sum"):
        o_sel, idx, logits = orc.select_layer(q_sel, k, v, 16, mode)
        assert np.array_equal(idx.numpy(), f[f"{mode}_idx"])
        o_sp = orc.sparse_layer(q_sp, k, v, orc.mask_from_indices(idx, 4, 96))
        assert np.abs(o_sp.numpy() - f[f"{mode}_o_sparse"]).max() < 1e-6
    assert np.abs(o_sel.numpy() - f["o_select"]).max() < 1e-6
    # the stored pool is the paged image of k, v
    got, _ = orc.paged_selected_attention(f["q_sparse"], f["pool"].astype(np.float32),
                                          f["per_head_slots"], 0, 0, kind="slots")
    assert np.abs(got - f["per_head_o_sparse"]).max() < 1e-5


def test_oracle_reproduces_cfg0_fixture():
    from oracle import tidal_oracle as orc

    f = _load("cfg0.npz")
    q0, k0, v0 = cfg0_inputs(0)
    q1, k1, v1 = cfg0_inputs(1)
    o_sel, idx, _ = orc.select_layer(q0, k0, v0, 256, "head_sum")
    assert np.array_equal(idx.numpy(), f["head_sum_idx"]) and idx.shape == (1, 256)
    o_sp = orc.sparse_layer(q1, k1, v1, orc.mask_from_indices(idx, 32, 4096))
    assert np.abs(o_sp.numpy() - f["head_sum_o_sparse"]).max() < 1e-6
    assert np.abs(o_sel.numpy() - f["o_select"]).max() < 1e-6


def _same_up_to_threshold_ties(got, want, scores, rel):
    """got/want: 1-D index arrays of one row; scores: the oracle's scores of that row.  Every
    element in one list but not the other must score within rel of the k-th score."""
    got, want = set(got.tolist()), set(want.tolist())
    if got == want:
        return True
    thr = np.sort(scores)[::-1][len(want) - 1]
    return all(abs(scores[i] - thr) <= rel * max(abs(thr), 1e-30) for i in got ^ want)


def _run_two_layers(cuda, dtype, q_sel, q_sp, pool, table, n, hq, hkv, d, page, k, mode):
    """selection layer + selection + sparse layer through the operator surface"""
    from tidaldecode_amd import _kernels

    w = _kernels.BatchDecodeWithPagedKVCachePyTorchWrapper(0)
    w.begin_forward(None, hq, hkv, d, page, torch.empty(0, dtype=dtype))
    n_pages = table.numel()
    last_len = (n - 1) % page + 1
    scores = torch.zeros((hq, n_pages * page), dtype=torch.float32, device=cuda)
    lse = torch.zeros((1, hq), dtype=torch.float32, device=cuda)
    o_sel = torch.empty((1, hq, d), dtype=dtype, device=cuda)
    w.forward(q_sel.to(dtype).to(cuda)[None], o_sel, pool, table[:-1][None].contiguous(), None,
              last_len, int(table[-1]), scores, lse=lse)
    rows = {"per_head": hq, "group_sum": hkv, "head_sum": 1}[mode]
    sel_scores = scores
    if mode != "per_head":
        sel_scores = _kernels.score_reduce(scores, lse.view(-1), hkv, n, mode)
    slots = torch.empty((rows, k), dtype=torch.int32, device=cuda)
    _kernels.topk_filtering(sel_scores[:, :n], None, None, slots, None, k, page_table=table,
                            page_size=page)
    pos = torch.empty((rows, k), dtype=torch.int32, device=cuda)
    _kernels.topk_filtering(sel_scores[:, :n], None, None, pos, None, k)
    o_sp = torch.empty((1, hq, d), dtype=dtype, device=cuda)
    w.forward(q_sp.to(dtype).to(cuda)[None], o_sp, pool, slots, None, 0, 0, None,
              index_kind="slots")
    torch.cuda.synchronize()
    return (o_sel[0].float().cpu(), o_sp[0].float().cpu(), pos.cpu(), slots.cpu(),
            sel_scores[:, :n].cpu())


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["per_head", "group_sum", "head_sum"])
def test_gpu_small_fixture(cuda, mode):
    from oracle import tidal_oracle as orc

    f = _load("small.npz")
    table = torch.from_numpy(f["page_table"]).to(cuda)
    o_sel, o_sp, pos, slots, gpu_scores = _run_two_layers(
        cuda, torch.float16, torch.from_numpy(f["q_select"]), torch.from_numpy(f["q_sparse"]),
        torch.from_numpy(f["pool"]).to(cuda), table, 96, 4, 2, 64, 4, 16, mode)
    assert np.abs(o_sel.numpy() - f["o_select"]).max() <= 2e-3
    # bit-exact from the same scores
    assert torch.equal(pos.long(), orc.stable_topk(gpu_scores, 16))
    assert np.array_equal(pos.numpy(), f[f"{mode}_idx"])
    assert np.array_equal(slots.numpy(), f[f"{mode}_slots"])
    assert np.abs(o_sp.numpy() - f[f"{mode}_o_sparse"]).max() <= 2e-3


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["per_head", "head_sum"])
def test_gpu_cfg0(cuda, mode):
    """benchmark configuration 0 on the GPU in fp16 against the fixture."""
    from oracle import tidal_oracle as orc

    f = _load("cfg0.npz")
    q0, k0, v0 = cfg0_inputs(0)
    q1, k1, v1 = cfg0_inputs(1)
    n, h, d, page, k = 4096, 32, 128, 16, 256
    n_pages = n // page
    table = torch.randperm(n_pages + 4, generator=torch.Generator().manual_seed(3))[:n_pages]

    def paged(kk, vv):
        pool = torch.zeros((n_pages + 4, 2, page, h, d), dtype=torch.float16)
        pool[table, 0] = kk.half().view(n_pages, page, h, d)
        pool[table, 1] = vv.half().view(n_pages, page, h, d)
        return pool.to(cuda)

    from tidaldecode_amd import _kernels
    table_d = table.to(torch.int32).to(cuda)
    # layer 1: selection on (q0, k0, v0); layer 2: sparse on fresh (q1, k1, v1) with those positions
    o_sel, _, pos, slots, gpu_scores = _run_two_layers(cuda, torch.float16, q0, q1, paged(k0, v0),
                                                       table_d, n, h, h, d, page, k, mode)
    assert np.abs(o_sel.numpy() - f["o_select"]).max() <= 2e-3
    assert torch.equal(pos.long(), orc.stable_topk(gpu_scores, k))  # bit-exact from same scores
    want_idx = f[f"{mode}_idx"]
    oracle_scores = (f["head_sum_scores"] if mode == "head_sum"
                     else orc.attn_logits(q0, k0).numpy())
    for r in range(want_idx.shape[0]):
        assert _same_up_to_threshold_ties(pos[r].numpy(), want_idx[r], oracle_scores[r], 2e-5), r
    # sparse layer over the FIXTURE's list (so that a threshold tie cannot leak into the output)
    w = _kernels.BatchDecodeWithPagedKVCachePyTorchWrapper(0)
    w.begin_forward(None, h, h, d, page, torch.empty(0, dtype=torch.float16))
    want_pos = torch.from_numpy(want_idx).long()
    want_slots = (table[want_pos // page] * page + want_pos % page).to(torch.int32).to(cuda)
    o = torch.empty((1, h, d), dtype=torch.float16, device=cuda)
    w.forward(q1.half().to(cuda)[None], o, paged(k1, v1), want_slots, None, 0, 0, None,
              index_kind="slots")
    torch.cuda.synchronize()
    assert np.abs(o[0].float().cpu().numpy() - f[f"{mode}_o_sparse"]).max() <= 2e-3
