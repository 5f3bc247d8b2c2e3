"""CPU: the C-ABI library loads and exports what include/tidal_hip.h declares; argument checks
that run before any kernel launch; host-side bookkeeping (planner, KV pool, controller)."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "tidal_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(td_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from tidaldecode_amd import _lib

    names = _declared()
    assert len(names) >= 12
    assert sorted(_lib.SIGNATURES) == names  # the Python binding covers the header exactly
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), n
    assert _lib.lib.td_version() == 6
    assert isinstance(_lib.last_error(), str)


def test_every_declaration_cites_the_reference():
    text = open(os.path.join(ROOT, "include", "tidal_hip.h")).read()
    for name in ("td_rope_in_place", "td_append_kv", "td_decode_attn", "td_topk", "td_rms_norm",
                 "td_decode_make_plan"):
        head = text[: text.index(f"int {name}(")]
        comment = head[head.rindex("/*"):]
        assert re.search(r"\.(cu|cuh|h|py):\d+", comment), name


def _plan(batch, hq, hkv, d, rows, items, **preset):
    from tidaldecode_amd._lib import DecodePlan, lib

    p = DecodePlan(preset.get("chunk", 0), 0, preset.get("waves", 0), preset.get("rows", 0),
                   preset.get("merge", -1), preset.get("sparse_waves", 0),
                   preset.get("sparse_rows", 0), 0)
    rc = lib.td_decode_make_plan(batch, hq, hkv, d, rows, items, p)
    return rc, p


@pytest.mark.parametrize("hq,hkv,d,rows,items", [(32, 32, 128, 32, 2048), (32, 32, 128, 1, 2048),
                                                 (32, 8, 128, 8, 4096), (32, 8, 128, 32, 4096),
                                                 (40, 40, 128, 40, 102400), (32, 32, 64, 32, 17),
                                                 (32, 32, 256, 32, 0), (32, 8, 128, 1, 102400)])
def test_plan_covers_the_list(hq, hkv, d, rows, items):
    rc, p = _plan(1, hq, hkv, d, rows, items)
    assert rc == 0
    assert p.tile_rows in (2, 4)
    tile = p.waves_per_block * p.tile_rows * (64 // (d // 8))
    assert p.chunk_tokens % tile == 0 and p.chunk_tokens > 0
    assert 1 <= p.max_splits <= 64
    assert p.chunk_tokens * p.max_splits >= items
    assert (p.max_splits - 1) * p.chunk_tokens < max(items, 1)  # no empty trailing split
    assert p.workspace_bytes >= 65536 and p.fused_merge in (0, 1)


def test_plan_rejects_bad_geometry():
    from tidaldecode_amd import _lib

    for args in ((1, 32, 5, 128, 32, 100), (0, 32, 32, 128, 32, 100), (1, 32, 32, 128, 7, 100),
                 (1, 32, 32, 128, 32, -1)):
        rc, _ = _plan(*args)
        assert rc == _lib.TD_ERR_INVALID_ARG
        assert "td_decode_make_plan" in _lib.last_error()
    rc, _ = _plan(1, 32, 32, 48, 32, 100)
    assert rc == _lib.TD_ERR_UNSUPPORTED and "head_dim" in _lib.last_error()
    rc, p = _plan(1, 32, 8, 64, 8, 100)  # head_dim 64: no shared-row kernel, falls back to
    assert rc == 0 and p.max_splits >= 1  # one list walk per query head


def test_argument_checks_fire_before_any_launch():
    """NULL / range errors are reported without touching the GPU (none is present here)."""
    from tidaldecode_amd import _lib
    from tidaldecode_amd._lib import check, lib

    assert lib.td_decode_attn(None, None, None, None, None, 1, 32, 0.1, None, 0, 0, None, None, None,
                              0, None) == _lib.TD_ERR_INVALID_ARG
    assert lib.td_rope_table(None, 1, 128, 1.0, 1e4, None, None, None) == _lib.TD_ERR_INVALID_ARG
    assert lib.td_topk(None, 2, 0, 1, 1, 1, None, 0, None, 0, 0, None, 1, None, None, 1, None, 0, None) \
        == _lib.TD_ERR_INVALID_ARG
    assert lib.td_rope_in_place(None, None, 1, 1, 1, 128, 0, 1.0, 1e4, 0, None) \
        == _lib.TD_ERR_INVALID_ARG
    assert lib.td_rms_norm(None, None, None, 1, 1, 1e-5, 0, None) == _lib.TD_ERR_INVALID_ARG
    with pytest.raises(RuntimeError, match="NULL"):
        check(lib.td_score_reduce(None, 0, None, 32, 32, 1, 0, None, 0, None))


def test_python_surface_rejects_cpu_tensors_and_bad_shapes():
    from tidaldecode_amd import _kernels

    q = torch.zeros((1, 32, 128), dtype=torch.float16)
    with pytest.raises(RuntimeError, match="CUDA"):
        _kernels.apply_rope_in_place(q, q.clone(), 0, 1.0, 1e4)
    with pytest.raises(RuntimeError, match="CUDA"):
        _kernels.topk_filtering(torch.zeros((2, 8)), None, None,
                                torch.zeros((2, 4), dtype=torch.int32), None, 4)
    with pytest.raises(RuntimeError, match="Invalid layout"):
        _kernels.BatchDecodeWithPagedKVCachePyTorchWrapper(7)
    with pytest.raises(RuntimeError, match="CUDA"):
        _kernels.estimate_attn_score(q, torch.zeros((32, 4), dtype=torch.float16),
                                     torch.zeros((2, 2, 16, 32, 128), dtype=torch.float16),
                                     torch.zeros(1, dtype=torch.int32), None, 5, 0, 0)
    w = _kernels.BatchDecodeWithPagedKVCachePyTorchWrapper(0)
    with pytest.raises(RuntimeError, match="BeginForward"):
        w.forward(q, q, q, q, None, 1, 0, None)


def test_kv_pool_and_cache_bookkeeping():
    from tidaldecode_amd.utils import KvCache, TensorLayout
    from tidaldecode_amd.utils.decode_wrapper import _check_kv_layout

    assert (TensorLayout.NHD, TensorLayout.HND) == (0, 1)
    with pytest.raises(KeyError):
        _check_kv_layout("XYZ")
    with pytest.raises(ValueError):
        KvCache(2, 4, 8, 0, 16, torch.float16, torch.device("cpu"))
    c = KvCache(num_layers=2, num_heads=4, head_dim=8, max_seq_len=40, page_size=16,
                dtype=torch.float16, device=torch.device("cpu"))
    assert c.pool.capacity == 3 and c.pool.buf.shape == (2, 3, 2, 16, 4, 8)
    assert c.append_seq(0) == 0 and c.seqlen == 0
    assert c.append_seq(17) == 2 and c.seqlen == 17 and c.last_page_len == 1
    assert c.append_seq(15) == 0 and c.last_page_len == 16      # page exactly full
    assert c.append_seq(1) == 1 and c.last_page_len == 1 and len(c.indicies) == 3
    assert c.indices_device.tolist() == c.indicies == [0, 1, 2]
    assert c.buf_layer(1).shape == (3, 2, 16, 4, 8)
    with pytest.raises(KeyError):                               # pool exhausted
        c.append_seq(16)
    c.release()
    assert c.seqlen == 0 and c.pool.num_free_blocks == 3 and c.indicies == []
    hnd = KvCache(1, 4, 8, 32, 16, torch.float16, torch.device("cpu"), layout=TensorLayout.HND,
                  page_order_seed=5)
    assert hnd.pool.buf.shape == (1, 2, 2, 4, 16, 8)
    hnd.append_seq(32)
    assert sorted(hnd.indicies) == [0, 1]
    assert TensorLayout.FORMAT2STR == {0: "NHD", 1: "HND"}
    with pytest.raises(KeyError, match="Invalide kv_layout"):
        TensorLayout.parse("nhd")
    page = hnd.pool.alloc_block() if hnd.pool.num_free_blocks else None
    assert page is None                                         # both pages are held
    hnd.pool.free_block(hnd.indicies[0])
    with pytest.raises(AssertionError):                         # returning a page twice
        hnd.pool.free_block(hnd.indicies[0])


@pytest.mark.parametrize("scope", ["all", "exclude_last_page"])
def test_controller_budget_arithmetic(scope):
    from tidaldecode_amd.utils import InferenceController

    dev = torch.device("cpu")
    c = InferenceController(num_layers=2, num_heads=8, head_dim=64, page_size=16,
                            token_budget=100, max_seq_len=1000, dtype=torch.float16, device=dev,
                            num_kv_heads=2, select_mode="group_sum", select_scope=scope)
    assert c.index_rows == 2 and c.topk_dindices_buffer_full.shape == (2, 100)
    c.prepare_metadata(500)
    c.begin_forward(500)                 # prefill: no decode state
    assert c.kv_indices_with_last.numel() == 32 and int(c.kv_indptr_for_append[1]) == 32
    c.end_forward()
    c.prepare_metadata(1)
    c.begin_forward(1)
    assert c.kv_cache.seqlen == 501 and c.kv_cache.last_page_len == 5
    assert c.kv_indices_without_last.shape == (1, 31)
    if scope == "all":
        assert (c.num_candidates, c.num_selected) == (501, 100)
    else:
        assert (c.num_candidates, c.num_selected) == (31 * 16, 95)
    assert c.topk_dindices_buffer.shape == (2, c.num_selected)
    assert c.need_estimate()
    c.set_token_budget(10 ** 6)          # "unlimited" budget clamps to what the buffers hold
    c.begin_forward(1, updateTensor=False)
    assert c.num_selected <= 100
    c.end_forward()
    c.clean_states()
    assert c.kv_cache.seqlen == 0
    with pytest.raises(KeyError):
        InferenceController(2, 8, 64, 16, 100, 1000, torch.float16, dev, select_mode="nope")
    with pytest.raises(ValueError):
        InferenceController(2, 8, 64, 16, 100, 1000, torch.float16, dev, num_kv_heads=3)


def test_batch_controller_bookkeeping():
    """Page-table segments, per-step metadata and page accounting of the batched controller
    (host arithmetic only: no kernel runs)."""
    from tidaldecode_amd.utils import BatchInferenceController

    dev = torch.device("cpu")
    c = BatchInferenceController(2, 8, 64, 4, 16, 40, 3, torch.float16, dev, num_kv_heads=2,
                                 select_mode="group_sum", page_order_seed=1)
    assert c.pages_per_seq == 10 and c.pool.capacity == 30 and c.index_rows == 2
    assert c.topk_dindices_buffer.shape == (2, 3 * 16) and c.qk_product.shape == (24, 40)
    c.add_sequences([5, 9])
    assert c.batch == 2 and c.pool.num_free_blocks == 30 - 2 - 3
    assert c.page_table[0, :2].tolist() == c._pages[0] and c.page_table[1, :3].tolist() == c._pages[1]
    assert len(set(c._pages[0] + c._pages[1])) == 5
    for _ in range(4):                       # 5 -> 9 tokens (third page), 9 -> 13 (fourth page)
        c.begin_step()
    assert c.seq_lens == [9, 13] and [len(p) for p in c._pages] == [3, 4]
    from tidaldecode_amd import _lib
    meta = c._meta[:, :2].tolist()
    assert meta[_lib.TD_STEP_SEQ_LEN] == [9, 13] and meta[_lib.TD_STEP_COUNT] == [4, 4]
    assert meta[_lib.TD_STEP_PAGES_BEFORE_LAST] == [2, 3]
    assert meta[_lib.TD_STEP_LAST_PAGE_LEN] == [1, 1]
    assert meta[_lib.TD_STEP_LAST_PAGE_IDX] == [c._pages[0][-1], c._pages[1][-1]]
    assert meta[_lib.TD_STEP_DST_SLOT] == [c._pages[0][-1] * 4, c._pages[1][-1] * 4]
    assert meta[_lib.TD_STEP_POSITION] == [8, 12]
    assert meta[_lib.TD_STEP_N_SELECTED] == [9, 13]          # min(budget, n)
    assert c.positions.tolist() == [8, 12] and c.selected.tolist() == [9, 13]
    for _ in range(10):
        c.begin_step()
    assert c.selected.tolist() == [16, 16]                   # the budget caps the lists
    c.reserve_ahead(9)                       # pages beyond the one being filled change nothing
    assert c.seq_lens == [19, 23] and [len(p) for p in c._pages] == [7, 8]
    before = c._meta.clone()
    c._refresh()
    assert torch.equal(c._meta, before)
    with pytest.raises(RuntimeError, match="max_seq_len"):
        c.reserve_ahead(30)
    with pytest.raises(RuntimeError, match="max_batch"):
        c.add_sequences([4, 4])
    with pytest.raises(RuntimeError, match="max_seq_len"):   # a failed call keeps nothing
        c.add_sequences([41])
    assert c.batch == 2 and c.pool.num_free_blocks == 30 - 7 - 8
    c.release()
    assert c.batch == 0 and c.pool.num_free_blocks == 30


def test_split_partials_are_only_touched_through_the_coherent_accessors():
    """The split merge is ordered by device-scope write-through stores, a wait, a ticket and
    device-scope loads (the argument sits next to the code).  A plain load or store on the partial
    arrays would break it without failing any small test, so every use of ws_o / ws_ml in the
    kernels must go through store_coherent / load_coherent (or form the pointer those take)."""
    import re
    from pathlib import Path

    csrc = Path(__file__).resolve().parents[1] / "tidaldecode_amd" / "csrc"
    uses = 0
    for path in sorted(csrc.glob("*.cuh")) + sorted(csrc.glob("*.hip")):
        lines = path.read_text().splitlines()
        for no, line in enumerate(lines, 1):
            code = line.split("//")[0]
            if not re.search(r"\bws_(o|ml)\b", code):
                continue
            uses += 1
            ok = ("store_coherent(" in code or "load_coherent(" in code
                  or re.search(r"float\* ws_(o|ml);", code)                       # the field
                  or re.search(r"p\.ws_(o|ml) = reinterpret_cast<float\*>", code)  # host: carve the workspace
                  or re.search(r"float\* dst = p\.ws_o \+", code))               # pointer handed to store_coherent
            assert ok, f"{path.name}:{no}: {line.strip()}"
            if "float* dst = p.ws_o +" in code:
                following = " ".join(lines[no: no + 4])
                assert following.count("store_coherent(dst") == 4, f"{path.name}:{no}"
    assert uses >= 10
