"""ctypes binding of the C-ABI library (include/jacobiforcing.h).

The HIP library is the only implementation of the hot path this package has.  If it cannot be
loaded the package fails loudly — there is no CPU or eager-PyTorch fallback.
"""
from __future__ import annotations

import ctypes as C
import os
from pathlib import Path

_PKG = Path(__file__).resolve().parent
LIB_PATH = _PKG / "lib" / "libjacobiforcing.so"
SRC_DIR = _PKG / "csrc"
INCLUDE_DIR = _PKG.parent / "include"

JF_OK, JF_E_INVALID, JF_E_CAPACITY, JF_E_LAUNCH, JF_E_SHAPE = 0, -1, -2, -3, -4
JF_F32, JF_BF16 = 0, 1
JF_MB_INACTIVE, JF_MB_KEEP = -1, -2


class MbParams(C.Structure):
    _fields_ = [("n", C.c_int32), ("K", C.c_int32), ("spawn_threshold", C.c_int32), ("pool_size", C.c_int32),
                ("eos_id", C.c_int32), ("pad_id", C.c_int32), ("max_iter", C.c_int32), ("max_blocks", C.c_int32),
                ("lookahead_start_ratio", C.c_double)]


class MbDesc(C.Structure):
    _fields_ = [(k, C.c_int32) for k in
                ("B", "T", "done", "error", "iters", "kv_len", "ret_len", "next_token", "kv_src_row", "kv_copy_dst",
                 "kv_copy_len", "events", "accepted", "nspans", "rsv0", "rsv1")]


DESC_INTS = C.sizeof(MbDesc) // 4
DESC_FIELDS = [f[0] for f in MbDesc._fields_]


class MbLoop(C.Structure):
    """jf_mb_loop (include/jacobiforcing.h): the pointers of the loop around the step, filled once."""
    _fields_ = [("states", C.c_void_p), ("state_ints", C.c_int64), ("P", C.c_int32), ("order", C.c_int32),
                ("packed", C.c_void_p), ("packed_cap", C.c_int64), ("desc", C.c_void_p),
                ("input_ids", C.c_void_p), ("positions", C.c_void_p), ("row_prompt", C.c_void_p), ("row_len", C.c_void_p),
                ("row_cand", C.c_void_p), ("row_kv_len", C.c_void_p), ("valid_index", C.c_void_p),
                ("rows_cap", C.c_int32), ("t_cap", C.c_int32), ("t_align", C.c_int32), ("valid_align", C.c_int32),
                ("cand_rows", C.c_int32), ("flags", C.c_int32), ("pad_fill", C.c_int64),
                ("kv_len", C.c_void_p), ("mailbox", C.c_void_p),
                ("drv", C.c_void_p), ("drv_ints", C.c_int64), ("draws", C.c_void_p), ("draw_len", C.c_int32),
                ("max_seq_len", C.c_int32)]


# mailbox header slots / per-prompt driver record / driver block header (include/jacobiforcing.h)
MB_SEQ, MB_RTOT, MB_RMAIN, MB_TPAD, MB_TMAX, MB_NVALID, MB_NVALID_PAD, MB_NDONE, MB_MAXKV, MB_ERROR, MB_ACCEPTED, MB_NCALL_END = range(12)
MB_MAILBOX_HDR, MB_FIN_INTS = 16, 8
MB_PACKED_EXTRA = 65536            # JF_MB_PACKED_ENTRIES(positions) - positions: room for jf_mb_verify's per-chunk result slots
FIN_FIELDS = ["stop", "calls", "iters_total", "new_tokens", "ret_len", "next_token", "iters", "text_off"]
DRV_FIELDS = ["active", "stop", "calls", "iters_total", "new_tokens", "budget", "max_calls", "text_len", "cursor", "fin_ret_len",
              "fin_next", "fin_iters", "fin_off"]
DRV_HDR_INTS = 16
STOP_REASONS = {0: None, 1: "eos", 2: "max_new_tokens", 3: "max_calls", 4: "max_seq_len", 5: "max_seq_len"}
EVT_SPAWN, EVT_SWITCH, EVT_EARLY, EVT_CALL_END, EVT_STOPPED, EVT_FAST, EVT_SLOW_NEXT = 1, 2, 4, 8, 16, 32, 64


def mailbox_ints(P: int) -> int:
    return MB_MAILBOX_HDR + int(P) * (DESC_INTS + MB_FIN_INTS)


class EngineRow(C.Structure):
    _fields_ = [("acc_len", C.c_int32), ("n_new", C.c_int32), ("eos", C.c_int32), ("active_next", C.c_int32),
                ("n_pads", C.c_int32), ("rsv", C.c_int32 * 3)]


ENGINE_ROW_INTS = C.sizeof(EngineRow) // 4
MB_LOOP_PUBLISH_FENCE = 1        # jf_mb_loop.flags (JF_MB_LOOP_PUBLISH_FENCE)
ENGINE_FIELDS = ["acc_len", "n_new", "eos", "active_next", "n_pads", "rsv0", "rsv1", "rsv2"]   # int32 columns of a row record


class RsRow(C.Structure):
    _fields_ = [(k, C.c_int32) for k in ("n_committed", "eos", "reject_pos", "n_bonus_draws", "n_uniforms", "n_pads",
                                         "active_next", "rsv")]


class RsFilterRow(C.Structure):
    """jf_rs_filter_row (include/jacobiforcing.h): what top-k / top-p make of one row, as a function of (probability, id)."""
    _fields_ = [("sum", C.c_double), ("row_max", C.c_float), ("x_keep", C.c_float), ("cut1", C.c_uint32), ("tie1", C.c_int32),
                ("s1", C.c_float), ("cut2", C.c_uint32), ("tie2", C.c_int32), ("s2", C.c_float), ("flags", C.c_uint32),
                ("rsv", C.c_uint32)]


RS_FILTER_ROW_BYTES = C.sizeof(RsFilterRow)
RS_FILTER_FLAGS_WORD = RsFilterRow.flags.offset // 4
RS_FILT_TOPK, RS_FILT_TOPP = 1, 2
RS_ROW_INTS = C.sizeof(RsRow) // 4
RS_FIELDS = [f[0] for f in RsRow._fields_]


class OpRow(C.Structure):
    _fields_ = [(k, C.c_int32) for k in ("n_committed", "stop_hit", "reject_pos", "n_bonus_draws", "n_uniforms", "n_redraft",
                                         "redraft_base_lo", "redraft_base_hi")]


class SbDesc(C.Structure):
    _fields_ = [(k, C.c_int32) for k in ("raw", "num", "total", "done", "next_token", "kv_len", "next_len", "eos")]


SB_FIELDS = [f[0] for f in SbDesc._fields_]


class EngineLoop(C.Structure):
    """jf_engine_loop (include/jacobiforcing.h): the device arrays of the loop around jf_engine_step / jf_rs_step."""
    _fields_ = [("B", C.c_int32), ("L", C.c_int32), ("kind", C.c_int32), ("ring_cap", C.c_int32),
                ("rows", C.c_void_p), ("tokens", C.c_void_p), ("remaining", C.c_void_p), ("kv_start", C.c_void_p),
                ("positions", C.c_void_p), ("slot", C.c_void_p), ("ring", C.c_void_p), ("ring_len", C.c_void_p),
                ("cursors", C.c_void_p), ("n_cursors", C.c_int32), ("flags", C.c_int32), ("mailbox", C.c_void_p)]


EL_SEQ, EL_ERROR, EL_STEP_ERROR, EL_CURSORS, EL_HDR = 0, 1, 2, 4, 16
EL_KIND_GREEDY, EL_KIND_SAMPLING = 0, 1
OP_ROW_INTS = C.sizeof(OpRow) // 4
OP_FIELDS = [f[0] for f in OpRow._fields_]

_vp, _i32, _i64, _f32, _sz = C.c_void_p, C.c_int32, C.c_int64, C.c_float, C.c_size_t

_SIGNATURES = {
    "jf_version": (C.c_int, []),
    "jf_timing_arm": (C.c_int, [C.c_void_p, C.c_void_p]),
    "jf_last_error": (C.c_char_p, []),
    "jf_device_identity": (C.c_int, [C.c_int, C.c_char_p, _sz]),
    "jf_argmax_partial": (C.c_int, [_vp, C.c_int, _i64, _i64, _i64, _vp, _vp]),
    "jf_argmax_scatter": (C.c_int, [_vp, C.c_int, _i64, _i64, _i64, _vp, _vp, _vp]),
    "jf_argmax_decode": (C.c_int, [_vp, _i64, _vp, _vp]),
    "jf_argmax_rows": (C.c_int, [_vp, C.c_int, _i64, _i64, _i64, _vp, _vp, _vp]),
    "jf_accept_lengths": (C.c_int, [_vp, C.c_int, _vp, _i64, C.c_int, C.c_int, _vp, _vp, _vp]),
    "jf_mb_state_ints": (_i64, [C.POINTER(MbParams)]),
    "jf_mb_max_rows": (_i32, [C.POINTER(MbParams)]),
    "jf_mb_max_tokens": (_i32, [C.POINTER(MbParams)]),
    "jf_mb_begin": (C.c_int, [_vp, _i64, C.c_int, C.POINTER(MbParams), _vp, _vp, _vp, _vp]),
    "jf_mb_pack": (C.c_int, [_vp, _i64, C.c_int, _i32, _i64, _vp, _vp, _vp, _vp, _vp, _i32, _vp]),
    "jf_mb_step": (C.c_int, [_vp, _i64, C.c_int, _vp, _i64, _vp, _vp]),
    "jf_mb_verify": (C.c_int, [_vp, C.c_int, _i64, _i64, _i64, _vp, _vp, _i64, C.c_int, _vp, _i64, _i64, _i32, _vp,
                               C.POINTER(MbParams), _vp]),
    "jf_mb_read_ret": (C.c_int, [_vp, _i64, C.c_int, _vp, _i32, _vp]),
    "jf_mb_set_fast_path": (C.c_int, [C.c_int]),
    "jf_host_alloc": (C.c_int, [_sz, C.POINTER(C.c_void_p)]),
    "jf_host_free": (C.c_int, [_vp]),
    "jf_mailbox_wait": (C.c_int, [_vp, _i32, _i64, _vp]),
    "jf_mb_loop_begin": (C.c_int, [C.POINTER(MbLoop), _i32, C.POINTER(MbParams), _vp, _vp, _vp]),
    "jf_mb_loop_iterate": (C.c_int, [C.POINTER(MbLoop), _i32, _vp, C.c_int, _i64, _i64, _i64, C.c_int, _i32, _i32,
                                     C.POINTER(MbParams), C.c_int, _vp, _vp, _vp]),
    "jf_mb_loop_pack": (C.c_int, [C.POINTER(MbLoop), _i32, C.POINTER(MbParams), _vp]),
    "jf_kv_append": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32, _i64, _i64, _i64, _i32, _vp]),
    "jf_rope_kv_append": (C.c_int, [_vp, C.c_int, _i64, _i32, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp,
                                    _vp, _i64, _vp]),
    "jf_swiglu": (C.c_int, [_vp, C.c_int, _i64, _i64, _vp, _vp]),
    "jf_kv_commit": (C.c_int, [_vp, _vp, _vp, _vp, _i32, _vp, C.c_int, _i32, _i32, _i32, _i64, _i64, _i32, _vp]),
    "jf_engine_step": (C.c_int, [_vp, C.c_int, C.c_int, _vp, _i32, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp]),
    "jf_sb_step": (C.c_int, [_vp, C.c_int, _vp, _i32, _i32, _i32, _vp, _i32, _vp, _vp]),
    "jf_engine_loop_commit": (C.c_int, [C.POINTER(EngineLoop), _i32, _vp]),
    "jf_engine_fill": (C.c_int, [_vp, C.c_int, C.c_int, _vp, _vp, C.c_int, C.c_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "jf_rs_probs": (C.c_int, [_vp, C.c_int, _i64, _i64, _i64, _vp, _f32, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "jf_rs_filter_workspace_bytes": (_sz, [C.c_int, _i64, _i64]),
    "jf_rs_filter": (C.c_int, [_vp, C.c_int, _i64, _i64, _i64, _vp, _f32, _i32, C.c_double, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "jf_rs_filter_expand": (C.c_int, [_vp, C.c_int, _i64, _i64, _i64, _f32, _vp, _vp, _vp]),
    "jf_rs_workspace_bytes": (_sz, [_i64, _i64]),
    "jf_rs_step": (C.c_int, [_vp, C.c_int, _i64, _i64, _vp, C.c_int, C.c_int, _vp, _vp, _vp, _vp, _f32, _i32, _vp,
                             _vp, _i64, _vp, _vp, _i64, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _sz, _vp, _vp]),
    "jf_rs_step_workspace_bytes": (_sz, [_i64]),
    "jf_rs_onpolicy_step": (C.c_int, [_vp, C.c_int, _i64, _i64, _vp, C.c_int, _vp, _vp, _vp, _vp, C.c_float, _vp, C.c_int,
                                      _vp, _i64, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _sz, _vp, _vp]),
}
EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_LIB = None


class NativeLibraryError(RuntimeError):
    pass


def load(path: os.PathLike | None = None):
    """dlopen the library and attach signatures.  Raises NativeLibraryError when it is missing."""
    p = Path(path) if path is not None else Path(os.environ.get("JF_LIB", LIB_PATH))   # JF_LIB: kernel A/B builds (tools/)
    if not p.exists():
        raise NativeLibraryError(
            f"{p} not found: build the HIP extension first (python -c 'import __graft_entry__ as g; g.build()'). "
            "jacobiforcing_amd has no CPU / eager fallback for the Jacobi loop body.")
    try:
        lib = C.CDLL(str(p))
    except OSError as e:  # e.g. libamdhip64 missing
        raise NativeLibraryError(f"cannot load {p}: {e}") from e
    for name, (res, args) in _SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as e:
            raise NativeLibraryError(f"{p} does not export {name}") from e
        fn.restype = res
        fn.argtypes = args
    return lib


def lib():
    global _LIB
    if _LIB is None:
        _LIB = load()
    return _LIB


def check(rc: int, what: str = ""):
    """Map C-ABI return codes onto the exception types the reference raises."""
    if rc == JF_OK:
        return
    msg = lib().jf_last_error()
    msg = msg.decode() if isinstance(msg, (bytes, bytearray)) else str(msg)
    text = f"{what}: {msg}" if what else msg
    if rc == JF_E_INVALID:
        raise ValueError(text)
    raise RuntimeError(text)


def raise_state_error(code: int, what: str, aux: int = 0):
    if code == JF_E_INVALID:
        raise ValueError(f"{what}: invalid state inside the Jacobi state machine (shape/assert; see MB:482, MB:631, MB:667)")
    if code == JF_E_SHAPE:
        # what torch raises at MB:482 when a re-surfaced pseudo block (Q3, K >= 3) has k rows and the RA draft has B
        raise RuntimeError(f"{what}: The size of tensor a ({aux >> 16}) must match the size of tensor b ({aux & 0xFFFF}) at "
                           "non-singleton dimension 0 (draft rows vs candidate rows, MB:482)")
    if code == JF_E_CAPACITY:
        raise RuntimeError(f"{what}: fixed capacity exceeded inside the Jacobi state machine (raise max_blocks)")
    if code:
        raise RuntimeError(f"{what}: state machine error {code}")


# ---- libjf_layers.so (include/jf_layers.h): layer kernels of the models whose forward is not stock PyTorch ----------------------------
JL_F32, JL_BF16 = 0, 1
JL_VERSION = 124                 # include/jf_layers.h: a library of another version is not called (its signatures may differ)
JL_OUT_SAME, JL_OUT_F32 = 0, 2
JL_ACT_GELU_TANH, JL_ACT_CLAMPED_SWISH, JL_ACT_SILU, JL_ACT_GELU_ERF, JL_ACT_NONE = 0, 1, 2, 3, -1
JL_ROUTE_SIGMOID, JL_ROUTE_SOFTMAX_RENORM, JL_ROUTE_TOP_SOFTMAX = 0, 1, 2
JL_ROT_HALVES, JL_ROT_NEIGHBOURS = 0, 1
JL_MOE_UP_RELU2, JL_MOE_DOWN, JL_MOE_UP_PLAIN = 0, 1, 2


class AttnArgs(C.Structure):
    """jl_attn_args (include/jf_layers.h)."""
    _fields_ = [("q", _vp), ("gate", _vp), ("gate_ld", _i64), ("k_cache", _vp), ("v_cache", _vp), ("out", _vp),
                ("block_tables", _vp), ("tiles", _vp), ("rel", _vp), ("lut", _vp), ("talk", _vp),
                ("bt_stride", _i32), ("n_tiles", _i32), ("lut_len", _i32), ("page_size", _i32), ("H", _i32), ("G", _i32), ("D", _i32),
                ("Dv", _i32), ("window", _i32), ("keep_first", _i32), ("TQ", _i32), ("dtype", _i32), ("scale", _f32),
                ("splits", _i32), ("n_rows", _i32), ("scratch", _vp), ("q_pack", _vp), ("k_ld", _i64), ("v_ld", _i64), ("Gv", _i32),
                ("out_dtype", _i32), ("sink", _vp), ("gate_heads", _i32)]


class Addend(C.Structure):
    """jl_addend (include/jf_layers.h)."""
    _fields_ = [("y", _vp), ("dtype", _i32), ("count", _i32), ("scale", _vp)]


_LAYER_SIGNATURES = {
    "jl_version": (C.c_int, []),
    "jl_last_error": (C.c_char_p, []),
    "jl_embed_scale": (C.c_int, [_vp, C.c_int, _vp, _i64, _i32, _f32, _vp, _vp, _vp]),
    "jl_add_rmsnorm": (C.c_int, [_vp, _vp, C.c_int, _i32, _vp, _vp, _f32, _vp, C.c_int, _i64, _i32, _vp]),
    "jl_qk_norm_append": (C.c_int, [_vp, C.c_int, _i64, _i64, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _f32, _vp, _vp, _vp, _vp, _vp]),
    "jl_attn_window": (C.c_int, [C.POINTER(AttnArgs), _vp]),
    "jl_attn_scratch_floats": (_i64, [_i32, _i32, _i32, _i32, _i32]),
    "jl_attn_tile_rows": (C.c_int, [C.c_int, _i32, _i32, _i32, _i32, _i64, _i64]),
    "jl_attn_sweep": (C.c_int, [C.POINTER(AttnArgs), _vp]),
    "jl_attn_sweep_tile_rows": (C.c_int, [C.c_int, _i32, _i32, _i32, _i32, _i32, _i64, _i64, _i32]),
    "jl_attn_sweep_scratch_floats": (_i64, [_i32, _i32, _i32, _i32, _i32]),
    "jl_attn_sweep_wide_tile_rows": (C.c_int, [C.c_int, _i32, _i32, _i32, _i32, _i32, _i64, _i64, _i32]),
    "jl_norm_add": (C.c_int, [_vp, _vp, C.c_int, _vp, _f32, _vp, C.c_int, _i64, _i32, _vp]),
    "jl_polynorm": (C.c_int, [_vp, C.c_int, _i64, _i32, _vp, _f32, _vp, _vp]),
    "jl_causal_conv": (C.c_int, [_vp, _vp, C.c_int, _vp, _vp, _vp, _i64, _i32, _i32, _vp, _vp]),
    "jl_causal_conv_carry": (C.c_int, [_vp, _vp, _i32, _vp, _i32, _i32, _vp]),
    "jl_head_norm_append": (C.c_int, [_vp, C.c_int, _i64, _i64, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _f32, _f32, _i32,
                                      _vp, _vp, _i32, _vp, _vp, _vp, _i32, _vp, _vp, _vp]),
    "jl_scaled_add_norms": (C.c_int, [_vp, C.POINTER(Addend), _i32, _vp, _vp, _f32, _f32, _vp, _vp, _vp, C.c_int, _i64, _i32, _vp]),
    "jl_gated_act": (C.c_int, [_vp, C.c_int, _i64, _i64, _i32, _i32, _i32, _i32, _f32, _f32, _f32, _vp, _i64, _vp, _vp]),
    "jl_diff_combine": (C.c_int, [_vp, _vp, _i64, _i64, _i32, _i32, _f32, _f32, _f32, _vp, C.c_int, _vp]),
    "jl_latent_prep": (C.c_int, [_vp, C.c_int, _i64, _i64, _i32, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _f32, _vp, _vp, _vp, _i64, _vp, _vp,
                                 _vp, _i32, _vp]),
    "jl_latent_q_pack": (C.c_int, [_vp, _vp, _i64, C.c_int, _i64, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _vp, _i64, _vp, _i32, _vp]),
    "jl_depth_mix_norm": (C.c_int, [_vp, C.POINTER(Addend), _i32, _f32, _vp, _i64, _i32, _vp, _vp, _vp, _f32, _vp, C.c_int, _vp, _i64, _i32, _vp, _vp, _vp, _vp,
                                    _vp]),
    "jl_token_shift": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i32, _vp, C.c_int, _vp]),
    "jl_softcap": (C.c_int, [_vp, _i64, _f32, _vp]),
    "jl_short_conv": (C.c_int, [_vp, C.c_int, _i64, _i32, _vp, _vp, _vp, _i32, _i32, _vp, _i64, _i32, _i32, _i32, _vp, _vp]),
    "jl_delta_rule": (C.c_int, [_vp, C.c_int, _i64, _i32, _i32, _i32, _vp, C.c_int, _i64, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _i32, _i64, _i32, _i32,
                                _i32, _i32, _f32, _f32, _f32, _vp, _vp, _vp, _vp]),
    "jl_heads_gate": (C.c_int, [_vp, _vp, _i64, C.c_int, _i64, _i32, _i32, _vp, _vp]),
    "jl_retention": (C.c_int, [_vp, C.c_int, _i64, _i32, _i32, _i32, _i32, _vp, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _i64, _vp, _f32,
                               _vp, _vp, _i32, _vp]),
    "jl_retention_join": (C.c_int, [_vp, _i32, _vp, _i32, _i32, _i32, _vp, _vp, _vp, _vp]),
    "jl_moe_route": (C.c_int, [_vp, _vp, _i64, _i32, _i32, _f32, _vp, _vp, _i32, _f32, _vp]),
    "jl_moe_group": (C.c_int, [_vp, _i64, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _i32, _vp]),
    "jl_moe_tile_rows": (C.c_int, []),
    "jl_moe_gemm": (C.c_int, [_vp, _vp, C.c_int, _i32, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _i32, _vp, _vp, _vp]),
    "jl_moe_gemm_gated": (C.c_int, [_vp, _vp, C.c_int, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _i32, _i32, _f32, _f32, _f32, _vp, _vp]),
}
LAYER_SYMBOLS = tuple(_LAYER_SIGNATURES)
# which library a symbol lives in (jacobiforcing_amd/_build.py: LAYER_GROUPS); both carry their own jl_version / jl_last_error
_SEQ_SYMBOLS = ("jl_retention", "jl_retention_join", "jl_delta_rule", "jl_moe_route", "jl_moe_group", "jl_moe_tile_rows", "jl_moe_gemm", "jl_moe_gemm_gated")


class _LayerLibs:
    """The layer-kernel libraries behind one attribute namespace.  A library is loaded at the first use of one of its symbols:
    what is built is loaded; when there is none it is compiled (hipcc, about a minute for the attention kernels) — a fresh
    checkout's first call compiles only the library its model launches.  There is no CPU or eager fallback for these kernels."""

    def __init__(self):
        self._libs = {}
        self._last = None

    def _load(self, group: str):
        from . import _build
        env = {"layers": "JF_LAYERS_LIB", "layers_seq": "JF_LAYERS_SEQ_LIB"}[group]
        p = Path(os.environ.get(env, _build.layer_lib(group)))
        if not p.exists():
            if env in os.environ:
                raise NativeLibraryError(f"{p} not found")
            try:
                _build.build_layers(groups=[group])
            except Exception as e:
                raise NativeLibraryError(f"cannot build {p}: {e}") from e
        try:
            lib_ = C.CDLL(str(p))
        except OSError as e:
            raise NativeLibraryError(f"cannot load {p}: {e}") from e
        for name, (res, args) in _LAYER_SIGNATURES.items():
            if (name in _SEQ_SYMBOLS) != (group == "layers_seq") and name not in ("jl_version", "jl_last_error"):
                continue
            try:
                fn = getattr(lib_, name)
            except AttributeError as e:
                raise NativeLibraryError(f"{p} does not export {name}") from e
            fn.restype, fn.argtypes = res, args
        if int(lib_.jl_version()) != JL_VERSION:
            raise NativeLibraryError(f"{p} has version {int(lib_.jl_version())}, this package calls version {JL_VERSION}: build it again "
                                     "(python -c 'import __graft_entry__ as g; g.build()')")
        self._libs[group] = lib_
        return lib_

    def __getattr__(self, name: str):
        if name.startswith("_"):
            raise AttributeError(name)
        if name == "jl_last_error":                  # the message of the library that was called last
            return (self._last or self._libs.get("layers") or self._load("layers")).jl_last_error
        group = "layers_seq" if name in _SEQ_SYMBOLS else "layers"
        self._last = self._libs.get(group) or self._load(group)
        return getattr(self._last, name)


_LAYERS = None


def layers():
    global _LAYERS
    if _LAYERS is None:
        _LAYERS = _LayerLibs()
    if "layers" not in _LAYERS._libs:               # the attention / norm library is what every ragged family needs: load (or build) it now
        _LAYERS._load("layers")
    return _LAYERS


def check_layers(rc: int, what: str = ""):
    if rc == 0:
        return
    msg = layers().jl_last_error()
    msg = msg.decode() if isinstance(msg, (bytes, bytearray)) else str(msg)
    text = f"{what}: {msg}" if what else msg
    if rc == -1:
        raise ValueError(text)
    raise RuntimeError(text)
