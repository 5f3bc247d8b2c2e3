"""ctypes binding of ``libtidal_hip.so`` (declarations: ``include/tidal_hip.h``).

The library is the product: there is no fallback.  If it has not been built
(``make -C tidaldecode_amd/csrc`` or ``__graft_entry__.build()``) importing this module raises.
"""
import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_float, c_int32, c_int64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
# TIDAL_HIP_LIB selects another build of the same ABI (kernel experiments); default: in-tree build
LIB_PATH = os.environ.get("TIDAL_HIP_LIB") or os.path.join(_HERE, "libtidal_hip.so")

TD_OK, TD_ERR_INVALID_ARG, TD_ERR_UNSUPPORTED, TD_ERR_STATE, TD_ERR_HIP = range(5)
TD_F16, TD_BF16, TD_F32 = 0, 1, 2
TD_NHD, TD_HND = 0, 1
TD_IDX_PAGES, TD_IDX_SLOTS = 0, 1
TD_REDUCE_HEAD_SUM, TD_REDUCE_GROUP_SUM = 0, 1
TD_STATIC_SCRATCH_BYTES = 4 << 20  # scratch inside the library image (td_decode_attn_noalloc)
# words of the device-resident step state (td_step_advance)
(TD_STEP_SEQ_LEN, TD_STEP_PAGES_BEFORE_LAST, TD_STEP_LAST_PAGE_LEN, TD_STEP_LAST_PAGE_IDX,
 TD_STEP_DST_SLOT, TD_STEP_POSITION, TD_STEP_N_SELECTED, TD_STEP_COUNT, TD_STEP_WORDS) = range(9)


class PagedKV(Structure):
    """td_paged_kv"""

    _fields_ = [
        ("data", c_void_p),
        ("max_pages", c_int64),
        ("num_kv_heads", c_int32),
        ("head_dim", c_int32),
        ("page_size", c_int32),
        ("layout", c_int32),
        ("dtype", c_int32),
    ]


class IndexList(Structure):
    """td_index_list"""

    _fields_ = [
        ("idx", c_void_p),
        ("idx_rows", c_int32),
        ("idx_row_stride", c_int32),
        ("kind", c_int32),
        ("indptr", c_void_p),
        ("n_list_host", c_int32),
        ("last_page_len_arr", c_void_p),
        ("last_page_idx_arr", c_void_p),
        ("last_page_len", c_int32),
        ("last_page_idx", c_int32),
        ("count_arr", c_void_p),
    ]


class FreshToken(Structure):
    """td_fresh_token"""

    _fields_ = [
        ("k", c_void_p),
        ("v", c_void_p),
        ("cos", c_void_p),
        ("sin", c_void_p),
        ("dst_slot", c_void_p),
    ]


class DecodePlan(Structure):
    """td_decode_plan"""

    _fields_ = [
        ("chunk_tokens", c_int32),
        ("max_splits", c_int32),
        ("waves_per_block", c_int32),
        ("tile_rows", c_int32),
        ("fused_merge", c_int32),
        ("sparse_waves", c_int32),
        ("sparse_rows", c_int32),
        ("workspace_bytes", c_int64),
    ]


# name -> (restype, argtypes); one entry per function declared in include/tidal_hip.h
SIGNATURES = {
    "td_last_error": (c_char_p, []),
    "td_version": (c_int32, []),
    "td_num_cus": (c_int32, []),
    "td_last_decode_kernel": (c_char_p, []),
    "td_rope_in_place": (
        c_int32,
        [c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32, c_int64, c_float, c_float,
         c_int32, c_void_p],
    ),
    "td_append_kv": (
        c_int32,
        [POINTER(PagedKV), c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_int32,
         POINTER(PagedKV), c_void_p, c_void_p, c_int32, c_void_p],
    ),
    "td_rope_append_decode": (
        c_int32,
        [POINTER(PagedKV), c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_void_p, c_void_p,
         c_float, c_float, c_void_p],
    ),
    "td_decode_make_plan": (
        c_int32,
        [c_int32, c_int32, c_int32, c_int32, c_int32, c_int64, POINTER(DecodePlan)],
    ),
    "td_decode_attn": (
        c_int32,
        [POINTER(PagedKV), POINTER(IndexList), POINTER(DecodePlan), c_void_p, c_void_p, c_int32,
         c_int32, c_float, c_void_p, c_int32, c_int64, c_void_p, POINTER(FreshToken), c_void_p,
         c_int64, c_void_p],
    ),
    "td_decode_attn_noalloc": (
        c_int32,
        [POINTER(PagedKV), POINTER(IndexList), POINTER(DecodePlan), c_void_p, c_void_p, c_int32,
         c_int32, c_float, c_void_p, c_int32, c_int64, c_void_p, POINTER(FreshToken), c_void_p],
    ),
    "td_merge_states": (
        c_int32,
        [c_void_p, c_int32, c_void_p, c_int32, c_int32, c_int32, c_void_p, c_void_p, c_void_p],
    ),
    "td_argmax": (c_int32, [c_void_p, c_int32, c_int32, c_void_p, c_void_p]),
    "td_step_advance_batch": (
        c_int32, [c_void_p, c_int32, c_int32, c_void_p, c_int32, c_int32, c_int32, c_void_p]),
    "td_step_advance": (
        c_int32,
        [c_void_p, c_void_p, c_int32, c_int32, c_int32, c_void_p, c_void_p, c_int32, c_void_p],
    ),
    "td_rope_table": (
        c_int32,
        [c_void_p, c_int32, c_int32, c_float, c_float, c_void_p, c_void_p, c_void_p],
    ),
    "td_score_reduce": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_int32, c_int32, c_int32, c_int32, c_void_p, c_int64,
         c_void_p],
    ),
    "td_topk": (
        c_int32,
        [c_void_p, c_int32, c_int64, c_int32, c_int32, c_int32, c_void_p, c_int64, c_void_p,
         c_int64, c_int32, c_void_p, c_int32, c_void_p, c_void_p, c_int64, c_void_p, c_int64,
         c_void_p],
    ),
    "td_topk_bounded": (
        c_int32,
        [c_void_p, c_int32, c_int64, c_int32, c_int32, c_int32, c_void_p, c_int64, c_void_p,
         c_int64, c_int32, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
         c_int64, c_void_p],
    ),
    "td_topk_workspace_bytes": (c_int64, [c_int32]),
    "td_gather_probe": (
        c_int32,
        [POINTER(PagedKV), POINTER(IndexList), POINTER(DecodePlan), c_int32, c_int32, c_void_p,
         c_int64, c_void_p],
    ),
    "td_estimate_score": (
        c_int32,
        [POINTER(PagedKV), c_void_p, c_int32, c_int32, c_void_p, c_int32, c_void_p, c_int64,
         c_void_p],
    ),
    "td_prefill_attn": (
        c_int32,
        [POINTER(PagedKV), c_void_p, c_int32, c_int32, c_void_p, c_void_p, c_int32, c_int32,
         c_float, c_int32, c_void_p],
    ),
    "td_gemv": (
        c_int32,
        [c_void_p, c_int64, c_int32, c_int32, c_void_p, c_int32, c_void_p, c_float, c_void_p,
         c_int32, c_void_p, c_int32, c_void_p],
    ),
    "td_rms_norm": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_float, c_int32, c_void_p],
    ),
}


def _load():
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
            "(or `python -c 'import __graft_entry__ as g; g.build()'`). "
            "tidaldecode_amd has no fallback path."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the build is stale
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def last_error() -> str:
    msg = lib.td_last_error()
    return msg.decode("utf-8", "replace") if msg else ""


def check(rc: int) -> None:
    """Map a td_status to the exceptions the reference's bindings raise (TORCH_CHECK ->
    RuntimeError; tidal/ops/csrc/approx_attn.cu:144-150)."""
    if rc != TD_OK:
        raise RuntimeError(last_error() or f"libtidal_hip call failed with status {rc}")
