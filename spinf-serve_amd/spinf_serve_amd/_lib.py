"""ctypes binding of libspinf_tree.so (the C ABI declared in include/spinf_tree.h)."""

from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

SYMBOLS = (
    "spinf_last_error", "spinf_version", "spinf_tileplan_build", "spinf_tileplan_counts", "spinf_tileplan_export",
    "spinf_tileplan_schedule", "spinf_tileplan_free", "spinf_attn_heads_per_item", "spinf_tree_attn_fwd", "spinf_tree_attn_fwd_noalloc", "spinf_attn_exact_items", "spinf_gdn_fwd",
)


class AttnArgs(C.Structure):
    _fields_ = [
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("out", C.c_void_p),
        ("q_tok", C.c_int64), ("q_head", C.c_int64), ("k_tok", C.c_int64), ("k_head", C.c_int64),
        ("v_tok", C.c_int64), ("v_head", C.c_int64), ("o_tok", C.c_int64), ("o_head", C.c_int64),
        ("n", C.c_int64), ("hq", C.c_int32), ("hkv", C.c_int32), ("d", C.c_int32), ("scale", C.c_float), ("window", C.c_int32),
        ("art", C.c_void_p), ("end", C.c_void_p), ("pos", C.c_void_p),
        ("kv_idx", C.c_void_p), ("kv_bits", C.c_void_p), ("items", C.c_void_p), ("list_ptr", C.c_void_p),
        ("n_items", C.c_int64), ("variant", C.c_int32),
        ("row_of", C.c_void_p), ("kv_row0", C.c_void_p),
        ("grp", C.c_void_p), ("grp_mode", C.c_int32), ("ktile", C.c_int32), ("n_lists", C.c_int32), ("debug_expire", C.c_int32),
    ]


class GdnPreArgs(C.Structure):
    _fields_ = [
        ("y", C.c_void_p), ("y_tok", C.c_int64),
        ("conv", C.c_void_p), ("conv_w", C.c_void_p), ("a_log", C.c_void_p), ("dt_bias", C.c_void_p),
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("g", C.c_void_p), ("beta", C.c_void_p),
        ("T", C.c_int64), ("h", C.c_int32), ("hv", C.c_int32), ("dk", C.c_int32), ("dv", C.c_int32), ("normalize", C.c_int32),
    ]


class GdnGateArgs(C.Structure):
    _fields_ = [
        ("o", C.c_void_p), ("o_tok", C.c_int64), ("z", C.c_void_p), ("z_tok", C.c_int64), ("norm_w", C.c_void_p), ("eps", C.c_float),
        ("out", C.c_void_p), ("T", C.c_int64), ("hv", C.c_int32), ("dv", C.c_int32),
    ]


class LmArgs(C.Structure):
    _fields_ = [
        ("logits", C.c_void_p), ("ld", C.c_int64), ("dtype", C.c_int32),
        ("rows", C.c_int64), ("vocab", C.c_int64), ("softcap", C.c_float),
        ("cols", C.c_void_p), ("n_cols", C.c_int64),
        ("out", C.c_void_p), ("out_ld", C.c_int64),
    ]


class LmHeadArgs(C.Structure):
    _fields_ = [
        ("h", C.c_void_p), ("h_ld", C.c_int64),
        ("sel", C.c_void_p), ("rows", C.c_int64),
        ("w", C.c_void_p), ("w_ld", C.c_int64),
        ("vocab", C.c_int64), ("hidden", C.c_int64),
        ("softcap", C.c_float), ("logits_dtype", C.c_int32),
        ("cols", C.c_void_p), ("n_cols", C.c_int64),
        ("out", C.c_void_p), ("out_ld", C.c_int64),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_int64),
        ("h_rows", C.c_int64),
    ]


class XdecArgs(C.Structure):
    _fields_ = [
        ("q", C.c_void_p), ("q_g", C.c_int64), ("q_h", C.c_int64), ("q_q", C.c_int64),
        ("kp", C.c_void_p), ("vp", C.c_void_p), ("pos_p", C.c_void_p),
        ("kt", C.c_void_p), ("vt", C.c_void_p), ("pos_t", C.c_void_p), ("own_t", C.c_void_p),
        ("len_p", C.c_void_p), ("len_t", C.c_void_p),
        ("gk", C.c_void_p), ("gv", C.c_void_p),
        ("qpos", C.c_void_p), ("step", C.c_void_p),
        ("out", C.c_void_p),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_int64), ("nsplit", C.c_int32), ("tiles_per_split", C.c_int32),
        ("G", C.c_int32), ("H", C.c_int32), ("h", C.c_int32), ("Q", C.c_int32), ("S", C.c_int32), ("Lp", C.c_int32), ("Tt", C.c_int32),
        ("d", C.c_int32), ("beam", C.c_int32), ("window", C.c_int32),
        ("scale", C.c_float), ("softcap", C.c_float),
    ]


class GdnArgs(C.Structure):
    _fields_ = [
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("g", C.c_void_p), ("beta", C.c_void_p), ("o", C.c_void_p),
        ("q_tok", C.c_int64), ("v_tok", C.c_int64), ("g_tok", C.c_int64), ("o_tok", C.c_int64),
        ("h", C.c_int32), ("hv", C.c_int32), ("dk", C.c_int32), ("dv", C.c_int32), ("scale", C.c_float),
        ("cu", C.c_void_p), ("idx", C.c_void_p), ("n_seg", C.c_int64), ("max_len", C.c_int64),
        ("h0", C.c_void_p), ("h0_idx", C.c_void_p), ("ht", C.c_void_p), ("ht_idx", C.c_void_p),
        ("mode", C.c_int32),
    ]


def library_path() -> str:
    return os.environ.get("SPINF_TREE_LIB", os.path.join(_HERE, "libspinf_tree.so"))


def load_library():
    """-> the loaded library; raises RuntimeError when it has not been built (python __graft_entry__.py)."""
    global _LIB
    if _LIB is not None:
        return _LIB
    path = library_path()
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: build the HIP library first (python __graft_entry__.py); there is no fallback path")
    lib = C.CDLL(path)
    try:
        return _bind(lib, path)
    except AttributeError as e:   # a symbol of include/spinf_tree.h that this library does not export
        raise RuntimeError(f"{path} is of another version than this package ({e}): rebuild it (python __graft_entry__.py); there is no fallback path") from None


def _bind(lib, path):
    global _LIB
    lib.spinf_last_error.restype = C.c_char_p
    lib.spinf_version.restype = C.c_int
    lib.spinf_tileplan_build.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.POINTER(C.c_void_p)]
    lib.spinf_tileplan_build_groups.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int64, C.c_int32, C.POINTER(C.c_void_p)]
    lib.spinf_tileplan_build_ktile.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int64, C.c_int32, C.c_int32, C.POINTER(C.c_void_p)]
    lib.spinf_tileplan_counts.argtypes = [C.c_void_p, C.POINTER(C.c_int64)]
    lib.spinf_tileplan_export.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
    lib.spinf_tileplan_schedule.argtypes = [C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p]
    lib.spinf_gdn_plan_build.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_int32, C.c_int64, C.c_int32, C.c_int64, C.c_void_p, C.c_int64, C.POINTER(C.c_void_p)]
    lib.spinf_gdn_plan_counts.argtypes = [C.c_void_p, C.POINTER(C.c_int64)]
    lib.spinf_gdn_plan_export.argtypes = [C.c_void_p] * 15
    lib.spinf_gdn_plan_free.argtypes = [C.c_void_p]
    lib.spinf_gdn_plan_free.restype = None
    lib.spinf_tileplan_schedule_static.argtypes = [C.c_void_p, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p]
    lib.spinf_attn_ring_aborts.argtypes = [C.POINTER(C.c_int64)]
    lib.spinf_attn_heads_per_item.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.c_int32]
    lib.spinf_attn_heads_per_item.restype = C.c_int
    lib.spinf_tileplan_row0.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
    lib.spinf_tileplan_free.argtypes = [C.c_void_p]
    lib.spinf_tileplan_free.restype = None
    lib.spinf_tree_attn_fwd.argtypes = [C.POINTER(AttnArgs), C.c_void_p]
    lib.spinf_tree_attn_fwd_noalloc.argtypes = [C.POINTER(AttnArgs), C.c_void_p]
    lib.spinf_attn_exact_items.argtypes = [C.POINTER(C.c_int64)]
    lib.spinf_gdn_fwd.argtypes = [C.POINTER(GdnArgs), C.c_void_p]
    lib.spinf_gdn_prologue.argtypes = [C.POINTER(GdnPreArgs), C.c_void_p]
    lib.spinf_gdn_gate.argtypes = [C.POINTER(GdnGateArgs), C.c_void_p]
    lib.spinf_lm_logprobs.argtypes = [C.POINTER(LmArgs), C.c_void_p]
    lib.spinf_lm_head_workspace.argtypes = [C.POINTER(LmHeadArgs), C.POINTER(C.c_int64)]
    lib.spinf_diag_mfma_rate.argtypes = [C.c_int64, C.c_void_p, C.c_int64, C.POINTER(C.c_double), C.c_void_p]
    lib.spinf_lm_head_fwd.argtypes = [C.POINTER(LmHeadArgs), C.c_void_p]
    lib.spinf_diag_lds_order.argtypes = [C.c_int32, C.c_int32, C.c_void_p, C.c_void_p]
    lib.spinf_diag_mfma_hazard.argtypes = [C.c_int32, C.c_int32, C.c_void_p, C.c_void_p]
    lib.spinf_diag_mfma_valu.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p]
    lib.spinf_struct_sizes.argtypes = [C.POINTER(C.c_int64), C.c_int32]
    lib.spinf_diag_attn_stream.argtypes = [C.POINTER(AttnArgs), C.c_int32, C.c_int32, C.c_void_p, C.c_void_p]
    lib.spinf_xdecode_plan.argtypes = [C.POINTER(XdecArgs), C.POINTER(C.c_int32), C.POINTER(C.c_int64)]
    lib.spinf_xdecode_attn_fwd.argtypes = [C.POINTER(XdecArgs), C.c_void_p]
    lib.spinf_xdecode_tiles.argtypes = [C.POINTER(XdecArgs), C.POINTER(C.c_int32)]
    for name in ("spinf_struct_sizes", "spinf_diag_attn_stream", "spinf_diag_lds_order", "spinf_diag_mfma_hazard", "spinf_diag_mfma_valu", "spinf_diag_mfma_rate", "spinf_lm_head_workspace", "spinf_lm_head_fwd", "spinf_gdn_plan_build", "spinf_gdn_plan_counts", "spinf_gdn_plan_export", "spinf_tileplan_schedule_static", "spinf_attn_ring_aborts", "spinf_tileplan_build", "spinf_tileplan_build_groups", "spinf_tileplan_build_ktile", "spinf_tileplan_counts", "spinf_tileplan_export", "spinf_tileplan_schedule", "spinf_tileplan_row0", "spinf_tree_attn_fwd", "spinf_tree_attn_fwd_noalloc", "spinf_attn_exact_items", "spinf_gdn_fwd", "spinf_gdn_prologue", "spinf_gdn_gate", "spinf_lm_logprobs", "spinf_xdecode_plan", "spinf_xdecode_tiles", "spinf_xdecode_attn_fwd"):
        getattr(lib, name).restype = C.c_int
    # the argument blocks above mirror include/spinf_tree.h: a library built from another version of the header would read them wrongly
    mirrors = (AttnArgs, GdnArgs, GdnPreArgs, GdnGateArgs, LmArgs, LmHeadArgs, XdecArgs)
    sizes = (C.c_int64 * len(mirrors))()
    if lib.spinf_struct_sizes(sizes, len(mirrors)) != 0 or list(sizes) != [C.sizeof(m) for m in mirrors]:
        raise RuntimeError(f"{path}: argument blocks of {list(sizes)} bytes, this package's are {[C.sizeof(m) for m in mirrors]}: "
                           "the library and the package are of different versions (rebuild: python __graft_entry__.py); no fallback")
    _LIB = lib
    return lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = load_library().spinf_last_error().decode()
        raise (ValueError if code == -1 else RuntimeError)(f"{what}: {msg} (code {code})")
