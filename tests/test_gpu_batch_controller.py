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
@pytest.mark.parametrize("stepping", ["host", "captured"])
def test_lockstep_decode_of_a_ragged_batch(cuda, hq, hkv, mode, dtype, page, stepping):
    _lockstep(cuda, hq, hkv, mode, dtype, page, stepping, [5, 130, 47, 64], 48, 20)


@pytest.mark.parametrize("stepping", ["host", "captured"])
@pytest.mark.parametrize("lens,budget,steps", [([1, 16, 17, 200, 31], 8, 18),     # from one token on
                                               ([200], 1000, 5),                   # budget above the length
                                               ([3, 3, 3, 3, 3, 3, 3, 90], 33, 35)])
def test_lockstep_decode_other_shapes(cuda, lens, budget, steps, stepping):
    _lockstep(cuda, 12, 4, "group_sum", torch.bfloat16, 8, stepping, lens, budget, steps)
    _lockstep(cuda, 4, 4, "per_head", torch.float16, 16, stepping, lens, budget, steps)


def test_lockstep_decode_with_logits_in_the_kv_dtype(cuda):
    """logits_dtype = the KV dtype: the buffer type of the reference (tidal/utils/controller.py:149).
    The selection is then the stable top-k of the ROUNDED logits, which is what the checks of
    _lockstep compare with (they rank the scores that the launch stored)."""
    _lockstep(cuda, 8, 2, "per_head", torch.float16, 16, "host", [5, 40, 200], 16, 6,
              logits_dtype=torch.float16)
    _lockstep(cuda, 4, 4, "per_head", torch.bfloat16, 8, "captured", [5, 40, 200], 16, 6,
              logits_dtype=torch.bfloat16)
    from tidaldecode_amd.utils import BatchInferenceController
    with pytest.raises(ValueError, match="float32 logits"):
        BatchInferenceController(1, 4, 128, 16, 8, 64, 2, torch.float16, cuda, num_kv_heads=2,
                                 select_mode="group_sum", logits_dtype=torch.float16)


def _lockstep(cuda, hq, hkv, mode, dtype, page, stepping, lens, budget, steps, logits_dtype=None):
    """stepping = "captured": pages are reserved ahead, the whole step (metadata advance on the
    device, RoPE table, the three layers, top-k) is captured once and replayed per token, with
    eager copies of the step's inputs and synchronisations between the replays."""
    from oracle import tidal_oracle as orc
    from tidaldecode_amd.utils import BatchInferenceController

    d, layers, theta = 128, 3, 1e4
    B = len(lens)
    ctl = BatchInferenceController(layers, hq, d, page, budget, 256, B + 1, dtype, cuda,
                                   num_kv_heads=hkv, select_mode=mode, page_order_seed=3,
                                   logits_dtype=logits_dtype)
    assert ctl.fused_step_ok and ctl.qk_product.dtype == (logits_dtype or torch.float32)
    ctl.add_sequences(lens)
    hist_k = [[randn((n, hkv, d), 100 * l + b, dtype) for b, n in enumerate(lens)] for l in range(layers)]
    hist_v = [[randn((n, hkv, d), 100 * l + b + 50, dtype) for b, n in enumerate(lens)] for l in range(layers)]
    for l in range(layers):
        for b in range(B):
            ctl.append_prompt(b, hist_k[l][b].to(dtype).to(cuda), hist_v[l][b].to(dtype).to(cuda), l)
    rows = ctl.index_rows

    def inputs(step):
        return [tuple(randn(shape, 1000 * step + 10 * l + i, dtype)
                      for i, shape in enumerate(((B, hq, d), (B, hkv, d), (B, hkv, d))))
                for l in range(layers)]

    def run_layers(dev_in):
        """the device work of one step after the metadata is current; returns the three outputs"""
        cos, sin = ctl.rope_table(1.0, theta)
        outs = []
        for l, (qd, kd, vd) in enumerate(dev_in):
            if l == 0:
                outs.append(ctl.attend_full(qd, l, True, fresh=(kd, vd, cos, sin)))
                ctl.select()
            elif l == 1:   # the un-fused form: RoPE + append, then attention
                ctl.rope_append(qd, kd, vd, l, 1.0, theta)
                outs.append(ctl.attend_sparse(qd, l))
            else:
                outs.append(ctl.attend_sparse(qd, l, fresh=(kd, vd, cos, sin)))
        return outs

    graph = static_in = static_out = None
    if stepping == "captured":
        ctl.reserve_ahead(steps)
        static_in = [tuple(t.to(dtype).to(cuda) for t in qkv) for qkv in inputs(0)]

        def body():
            ctl.advance_on_device()
            return run_layers(static_in)

        saved = ctl._meta.clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            body()                       # warm-up: plans, scratch, kernel loading
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        ctl._meta.copy_(saved)           # undo the warm-up's step on the device
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_out = body()

    for step in range(steps):
        host_in = inputs(step)
        if stepping == "captured":
            for dst, src in zip(static_in, host_in):
                for t_dst, t_src in zip(dst, src):
                    t_dst.copy_(t_src.to(dtype))
            ctl.note_step()
            graph.replay()
            torch.cuda.synchronize()
            outs = static_out
        else:
            ctl.begin_step()
            outs = run_layers([tuple(t.to(dtype).to(cuda) for t in qkv) for qkv in host_in])
            torch.cuda.synchronize()
        positions = [n - 1 for n in ctl.seq_lens]
        assert ctl.positions.tolist() == positions
        chosen = None
        for l in range(layers):
            q, k, v = host_in[l]
            q_rot, k_rot = _rot(q, positions, dtype, theta), _rot(k, positions, dtype, theta)
            for b in range(B):
                hist_k[l][b] = torch.cat([hist_k[l][b], k_rot[b: b + 1]])
                hist_v[l][b] = torch.cat([hist_v[l][b], v[b: b + 1]])
            o = outs[l]
            if l == 0:
                chosen = []
                for b in range(B):
                    n = ctl.seq_lens[b]
                    logits = orc.attn_logits(q_rot[b], hist_k[l][b])
                    assert tolerance_report(o[b], orc.softmax_pv(logits, hist_v[l][b])) <= ATOL[dtype], (step, b)
                    got_logits = ctl.qk_product[b * hq: (b + 1) * hq, :n].cpu()
                    tol = 2e-2
                    if logits_dtype is not None:   # stored in 16 bits: half a step of the type
                        tol += (2.0 ** -11 if logits_dtype == torch.float16 else 2.0 ** -8) * logits.abs()
                    assert ((got_logits - logits).abs() <= tol).all(), (step, b)
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


@pytest.mark.parametrize("hq,hkv,mode,dtype", [(8, 8, "per_head", torch.float16),
                                              (8, 2, "group_sum", torch.bfloat16)])
def test_sequences_join_and_leave_between_steps(cuda, hq, hkv, mode, dtype):
    """Sequences leave (release_sequences: the last ones move into the freed places) and join
    (add_sequences + append_prompt) between decode steps while the others go on: every active
    sequence's selection (bit-exact) and attention outputs follow its own oracle history."""
    from oracle import tidal_oracle as orc
    from tidaldecode_amd.utils import BatchInferenceController

    d, page, budget, layers, theta = 128, 16, 24, 2, 1e4
    ctl = BatchInferenceController(layers, hq, d, page, budget, 256, 5, dtype, cuda, num_kv_heads=hkv,
                                   select_mode=mode, page_order_seed=5)
    rows = ctl.index_rows
    seqs = []          # per place: {"id", "k": [per layer], "v": [per layer]}

    def join(ident, n):
        ctl.add_sequences([n])
        b = ctl.batch - 1
        ks = [randn((n, hkv, d), 1000 * ident + l, dtype) for l in range(layers)]
        vs = [randn((n, hkv, d), 1000 * ident + l + 50, dtype) for l in range(layers)]
        for l in range(layers):
            ctl.append_prompt(b, ks[l].to(dtype).to(cuda), vs[l].to(dtype).to(cuda), l)
        seqs.append({"id": ident, "k": ks, "v": vs})

    def leave(places):
        moved = ctl.release_sequences(places)
        keep = [s for i, s in enumerate(seqs) if i not in places]
        # the controller's promise: untouched sequences keep their index, movers fill the holes
        after = [None] * ctl.batch
        for i, s_ in enumerate(seqs):
            if i in places:
                continue
            after[moved.get(i, i)] = s_
        assert all(a is not None for a in after) and sorted(a["id"] for a in after) == sorted(k_["id"] for k_ in keep)
        seqs[:] = after

    def step(t):
        B = ctl.batch
        ctl.begin_step()
        cos, sin = ctl.rope_table(1.0, theta)
        positions = [n - 1 for n in ctl.seq_lens]
        outs, ins = [], []
        for l in range(layers):
            q, k, v = (randn(shape, 7000 * t + 10 * l + i, dtype)
                       for i, shape in enumerate(((B, hq, d), (B, hkv, d), (B, hkv, d))))
            ins.append((q, k, v))
            qd, kd, vd = (x.to(dtype).to(cuda) for x in (q, k, v))
            if l == 0:
                outs.append(ctl.attend_full(qd, l, True, fresh=(kd, vd, cos, sin)))
                ctl.select()
            else:
                outs.append(ctl.attend_sparse(qd, l, fresh=(kd, vd, cos, sin)))
        torch.cuda.synchronize()
        chosen = []
        for l in range(layers):
            q, k, v = ins[l]
            q_rot, k_rot = _rot(q, positions, dtype, theta), _rot(k, positions, dtype, theta)
            for b in range(B):
                s_ = seqs[b]
                s_["k"][l] = torch.cat([s_["k"][l], k_rot[b: b + 1]])
                s_["v"][l] = torch.cat([s_["v"][l], v[b: b + 1]])
                n = ctl.seq_lens[b]
                assert s_["k"][l].shape[0] == n
                if l == 0:
                    logits = orc.attn_logits(q_rot[b], s_["k"][l])
                    assert tolerance_report(outs[l][b], orc.softmax_pv(logits, s_["v"][l])) <= ATOL[dtype], (t, b)
                    got_logits = ctl.qk_product[b * hq: (b + 1) * hq, :n].cpu()
                    scores = got_logits if mode == "per_head" else ctl.score_sum[b * rows: (b + 1) * rows, :n].cpu()
                    kb = min(budget, n)
                    pos = orc.stable_topk(scores, kb)
                    table = torch.tensor(ctl._pages[b])
                    got = ctl.topk_dindices_buffer[:, b * ctl.budget: b * ctl.budget + kb].cpu().long()
                    assert torch.equal(got, table[pos // page] * page + pos % page), (t, b, s_["id"])
                    chosen.append(pos)
                else:
                    want = orc.sparse_layer_gather(q_rot[b], s_["k"][l], s_["v"][l], chosen[b])
                    assert tolerance_report(outs[l][b], want) <= ATOL[dtype], (t, l, b, s_["id"])

    for ident, n in ((0, 40), (1, 7), (2, 90), (3, 33)):
        join(ident, n)
    for t in range(3):
        step(t)
    free = ctl.pool.num_free_blocks
    held = len(ctl._pages[1])
    leave([1])                       # the last sequence (id 3) takes place 1
    assert [s_["id"] for s_ in seqs] == [0, 3, 2] and ctl.pool.num_free_blocks == free + held
    for t in range(3, 6):
        step(t)
    join(4, 21)                      # a newcomer mid-flight
    join(5, 1)
    for t in range(6, 9):
        step(t)
    leave([0, 4])                    # two at once, one of them the last: ids 0 and 5
    assert sorted(s_["id"] for s_ in seqs) == [2, 3, 4]
    for t in range(9, 12):
        step(t)
    with pytest.raises(IndexError):
        ctl.release_sequences([7])
    ctl.release_sequences(range(ctl.batch))
    assert ctl.batch == 0


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
