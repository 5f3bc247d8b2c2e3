"""GPU parity: several sequences of different lengths decoding in lock step through
BatchInferenceController — selection layer (full attention + logits + top-k), then sparse layers
over the persisted lists, each ONE launch for the batch — against the CPU oracle run per sequence.
Index lists must equal the oracle's stable rule applied to the same scores, bit for bit; attention
outputs within max-abs 2e-3 (fp16) / 1e-2 (bf16)."""
import numpy as np
import pytest
import torch

from _util import ATOL, randn, rounded, tolerance_report

pytestmark = pytest.mark.gpu


def _rot(x, positions, dtype, theta):
    from oracle import tidal_oracle as orc

    return rounded(torch.from_numpy(orc.rope_closed_form(x.numpy(), np.asarray(positions), theta)).float(), dtype)


@pytest.mark.parametrize("hq,hkv,mode,dtype,page", [(8, 8, "per_head", torch.float16, 16),
                                                    (8, 2, "group_sum", torch.bfloat16, 16),
                                                    (8, 2, "per_head", torch.float16, 8),
                                                    (4, 4, "head_sum", torch.float16, 16),
                                                    (16, 4, "head_sum", torch.bfloat16, 4)])
def test_lockstep_decode_of_a_ragged_batch(cuda, hq, hkv, mode, dtype, page):
    from oracle import tidal_oracle as orc
    from tidaldecode_amd.utils import BatchInferenceController

    d, layers, budget, theta = 128, 3, 48, 1e4
    lens = [5, 130, 47, 64]
    steps = 20
    B = len(lens)
    ctl = BatchInferenceController(layers, hq, d, page, budget, 256, B + 1, dtype, cuda,
                                   num_kv_heads=hkv, select_mode=mode, page_order_seed=3)
    assert ctl.fused_step_ok
    ctl.add_sequences(lens)
    hist_k = [[randn((n, hkv, d), 100 * l + b, dtype) for b, n in enumerate(lens)] for l in range(layers)]
    hist_v = [[randn((n, hkv, d), 100 * l + b + 50, dtype) for b, n in enumerate(lens)] for l in range(layers)]
    for l in range(layers):
        for b in range(B):
            ctl.append_prompt(b, hist_k[l][b].to(dtype).to(cuda), hist_v[l][b].to(dtype).to(cuda), l)
    rows = ctl.index_rows
    for step in range(steps):
        ctl.begin_step()
        positions = [n - 1 for n in ctl.seq_lens]
        assert ctl.positions.tolist() == positions
        cos, sin = ctl.rope_table(1.0, theta)
        chosen = None
        for l in range(layers):
            seed = 1000 * step + 10 * l
            q, k, v = randn((B, hq, d), seed, dtype), randn((B, hkv, d), seed + 1, dtype), randn((B, hkv, d), seed + 2, dtype)
            q_rot, k_rot = _rot(q, positions, dtype, theta), _rot(k, positions, dtype, theta)
            for b in range(B):
                hist_k[l][b] = torch.cat([hist_k[l][b], k_rot[b: b + 1]])
                hist_v[l][b] = torch.cat([hist_v[l][b], v[b: b + 1]])
            qd, kd, vd = (t.to(dtype).to(cuda) for t in (q, k, v))
            if l == 0:
                o = ctl.attend_full(qd, l, True, fresh=(kd, vd, cos, sin))
                ctl.select()
                torch.cuda.synchronize()
                chosen = []
                for b in range(B):
                    n = ctl.seq_lens[b]
                    logits = orc.attn_logits(q_rot[b], hist_k[l][b])
                    assert tolerance_report(o[b], orc.softmax_pv(logits, hist_v[l][b])) <= ATOL[dtype], (step, b)
                    got_logits = ctl.qk_product[b * hq: (b + 1) * hq, :n].cpu()
                    assert (got_logits - logits).abs().max() <= 2e-2, (step, b)
                    assert torch.isinf(ctl.qk_product[b * hq: (b + 1) * hq, n:]).all()
                    scores = got_logits if mode == "per_head" else ctl.score_sum[b * rows: (b + 1) * rows, :n].cpu()
                    if mode != "per_head":   # the reduction itself, against the closed form
                        assert (scores - orc.head_sum_scores(got_logits, rows)).abs().max() <= 2e-6 * hq
                    kb = min(budget, n)
                    pos = orc.stable_topk(scores, kb)
                    table = torch.tensor(ctl._pages[b])
                    want_slots = table[pos // page] * page + pos % page
                    got_slots = ctl.topk_dindices_buffer[:, b * ctl.budget: b * ctl.budget + kb].cpu().long()
                    assert torch.equal(got_slots, want_slots), (step, b)
                    chosen.append(pos)
            else:
                if l == 1:   # the un-fused form: RoPE + append, then attention
                    ctl.rope_append(qd, kd, vd, l, 1.0, theta)
                    o = ctl.attend_sparse(qd, l)
                else:
                    o = ctl.attend_sparse(qd, l, fresh=(kd, vd, cos, sin))
                torch.cuda.synchronize()
                for b in range(B):
                    want = orc.sparse_layer_gather(q_rot[b], hist_k[l][b], hist_v[l][b], chosen[b])
                    assert tolerance_report(o[b], want) <= ATOL[dtype], (step, l, b)
    # the cache holds what the oracle appended, page by page
    for l in range(layers):
        for b in range(B):
            n = ctl.seq_lens[b]
            pages = torch.tensor(ctl._pages[b], device=cuda)
            got = ctl.buf_layer(l)[pages]                       # [pages, 2, P, H, D]
            got_k = got[:, 0].reshape(-1, hkv, d)[:n].float().cpu()
            assert (got_k - hist_k[l][b]).abs().max() <= 2.0 ** -6 * hist_k[l][b].abs().max()
            assert torch.equal(got[:, 1].reshape(-1, hkv, d)[:n].float().cpu(), hist_v[l][b])
    free_before = ctl.pool.num_free_blocks
    ctl.release()
    assert ctl.pool.num_free_blocks == free_before + sum(-(-n // page) for n in [x + steps for x in lens])
    assert ctl.batch == 0 and torch.isinf(ctl.qk_product).all()


def test_batch_controller_limits(cuda):
    from tidaldecode_amd.utils import BatchInferenceController

    ctl = BatchInferenceController(1, 4, 64, 4, 8, 16, 2, torch.float16, cuda)
    with pytest.raises(RuntimeError, match="max_batch"):
        ctl.add_sequences([3, 3, 3])
    with pytest.raises(ValueError):
        ctl.add_sequences([0])
    ctl.add_sequences([16])
    with pytest.raises(RuntimeError, match="max_seq_len"):
        ctl.begin_step()
    assert ctl.seq_lens == [16]
    with pytest.raises(RuntimeError, match="max_seq_len"):
        ctl.add_sequences([17])
    assert ctl.batch == 1 and ctl.pool.num_free_blocks == 4
