"""ctypes binding of ``libtinyllm_hybrid.so``: the layer-list engine declared in ``include/tinyllm_hybrid.h``.

A library of its own (``make -C tiny-llm_amd/csrc hybrid``), so a checkout that serves only layer-list models builds only
this.  GPU-only like the rest of the extension: importing fails loudly when the library is missing; there is no CPU fallback.
"""

from __future__ import annotations

import ctypes
import os
from pathlib import Path

_LIB_NAME = "libtinyllm_hybrid.so"
_LIB_PATH = Path(__file__).resolve().parent / _LIB_NAME
CSRC = Path(__file__).resolve().parents[2] / "csrc"

if not _LIB_PATH.exists():
    raise ImportError(f"{_LIB_PATH} is missing: build it with `make -C {CSRC} hybrid` (hipcc, gfx950). There is no CPU fallback.")

_lib = ctypes.CDLL(str(_LIB_PATH), mode=os.RTLD_LOCAL if hasattr(os, "RTLD_LOCAL") else 0)

_vp, _i, _f, _sz, _l = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t, ctypes.c_long
_P = ctypes.POINTER

MIX_ATTENTION, MIX_DELTA, MIX_LINREC, MIX_LATENT = 0, 1, 2, 3
REC_CHANNEL, REC_EXPGATE, REC_FIXED = 0, 1, 2
NORM_RMS, NORM_DYT = 0, 1
FF_PLAIN, FF_GATED, FF_MOE = 0, 1, 2
ROUTER_SOFTMAX, ROUTER_SIGMOID = 0, 1
BLOCK_SEQUENTIAL, BLOCK_PARALLEL, BLOCK_POSTNORM, BLOCK_SANDWICH = 0, 1, 2, 3
VMIX_NONE, VMIX_FIRST, VMIX_BLEND = 0, 1, 2
HY_F32, HY_BF16 = 0, 2
FF_GELU_ERF, FF_GELU_TANH, FF_SILU, FF_RELU2 = 0, 1, 2, 3


class TlHybridLayer(ctypes.Structure):
    _fields_ = [("kind", _i), ("heads", _i), ("kv_heads", _i), ("dim", _i), ("vdim", _i), ("ff", _i), ("ff_act", _i),
                ("w_in_dev", _vp), ("w_out_dev", _vp), ("norm_dev", _vp), ("norm_offset", _f),
                ("rot_dims", _i), ("rot_base", _f), ("scale", _f), ("qk_unit_rms", _i), ("sink", _i), ("gated", _i),
                ("conv_taps", _i), ("conv_dev", _vp), ("a_log_dev", _vp), ("dt_bias_dev", _vp), ("out_norm_dev", _vp),
                ("unit_eps", _f),
                ("norm_kind", _i), ("norm_alpha", _f), ("norm2_alpha", _f), ("norm_bias_dev", _vp), ("norm2_bias_dev", _vp),
                ("norm2_dev", _vp), ("w_in2_dev", _vp), ("w_out2_dev", _vp), ("ls1_dev", _vp), ("ls2_dev", _vp), ("ff_kind", _i),
                ("experts", _i), ("identity", _i), ("top", _i), ("groups", _i), ("keep", _i), ("expert_ff", _i), ("shared_ff", _i),
                ("correction_dev", _vp),
                ("rec_kind", _i), ("gate_cap", _f), ("tau", _f), ("a_rank", _i), ("a2_dev", _vp), ("a2_bias_dev", _vp),
                ("i_bias_dev", _vp), ("f_bias_dev", _vp),
                ("q_rank", _i), ("kv_rank", _i), ("rot_dim", _i), ("kv_from", _i), ("dq_norm_dev", _vp), ("dkv_norm_dev", _vp),
                ("uq_dev", _vp), ("uk_t_dev", _vp), ("uv_dev", _vp),
                ("rot_factor", _f), ("rot_original", _f), ("rot_fast", _f), ("rot_slow", _f),
                ("qk_norm", _i), ("q_norm_dev", _vp), ("k_norm_dev", _vp), ("rot_half", _i), ("rot_scaling_kind", _i),
                ("talk_dev", _vp), ("sink_dev", _vp), ("chunk", _i), ("v_mix", _i), ("v_mix_lambda", _f),
                ("moe_router", _i), ("moe_gated", _i), ("moe_scale_input", _i), ("moe_shared_sg", _i),
                ("w_in_bias_dev", _vp), ("window", _i), ("qk_head_norm", _i), ("diff_maps", _i), ("diff_lambda", _f), ("diff_init", _f),
                ("decay_dev", _vp), ("post_norm_dev", _vp), ("post_norm2_dev", _vp),
                ("side_gate_dev", _vp), ("side_proj_dev", _vp), ("side_norm_dev", _vp), ("side_col0", _i)]


class TlHybridConfig(ctypes.Structure):
    _fields_ = [("dtype", _i), ("width", _i), ("vocab", _i), ("num_layers", _i), ("norm_eps", _f), ("residual_mult", _f),
                ("parallel_block", _i), ("loop_start", _i), ("loop_stop", _i), ("loop_times", _i),
                ("loop_in_dev", _vp), ("loop_step_dev", _vp), ("embed_dev", _vp), ("final_norm_dev", _vp),
                ("final_norm_offset", _f), ("head_dev", _vp),
                ("embed_scale", _f), ("final_norm_kind", _i), ("final_norm_alpha", _f), ("final_norm_bias_dev", _vp),
                ("page_size", _i), ("num_pages", _i), ("max_slots", _i), ("max_pages_per_seq", _i), ("max_rows", _i),
                ("logit_scale", _f), ("embed_norm_dev", _vp), ("side_embed_dev", _vp), ("side_cols", _i), ("side_dim", _i)]


class TlHybridStats(ctypes.Structure):
    _fields_ = [("pages_in_use", _i), ("pages_free", _i), ("peak_pages_in_use", _i),
                ("page_allocations", _l), ("reused_page_allocations", _l),
                ("steps", _l), ("rows", _l), ("slot_begins", _l), ("reused_slot_begins", _l),
                ("kv_bytes", _sz), ("state_bytes", _sz), ("workspace_bytes", _sz), ("layer_runs", _i),
                ("graph_captures", _l), ("graph_replays", _l)]


# every symbol declared in include/tinyllm_hybrid.h
SIGNATURES = {
    "tl_hybrid_last_error": (ctypes.c_char_p, []),
    "tl_hybrid_create": (_i, [_P(TlHybridConfig), _P(TlHybridLayer), _vp, _P(_vp)]),
    "tl_hybrid_destroy": (None, [_vp]),
    "tl_hybrid_synchronize": (_i, [_vp]),
    "tl_hybrid_begin": (_i, [_vp, _i]),
    "tl_hybrid_release": (_i, [_vp, _i]),
    "tl_hybrid_move": (_i, [_vp, _i, _i]),
    "tl_hybrid_context_len": (_i, [_vp, _i]),
    "tl_hybrid_step": (_i, [_vp, _i, _P(_i), _P(ctypes.c_int32), _P(_i), _i, _P(_i)]),
    "tl_hybrid_decode": (_i, [_vp, _i, _P(_i), _i, _i]),
    "tl_hybrid_set_token": (_i, [_vp, _i, ctypes.c_int32]),
    "tl_hybrid_read_pending": (_i, [_vp, _i, _P(_i), _P(ctypes.c_int32)]),
    "tl_hybrid_copy_logits": (_i, [_vp, _vp, _i]),
    "tl_hybrid_read_logits": (_i, [_vp, _P(_f), _i]),
    "tl_hybrid_read_argmax": (_i, [_vp, _i, _P(ctypes.c_int32)]),
    "tl_hybrid_set_trace": (_i, [_vp, _i]),
    "tl_hybrid_read_trace": (_i, [_vp, _i, _P(_f), _i]),
    "tl_hybrid_get_stats": (_i, [_vp, _P(TlHybridStats)]),
    "tl_hybrid_linear": (_i, [_i, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
}

for _name, (_res, _args) in SIGNATURES.items():
    _fn = getattr(_lib, _name)
    _fn.restype = _res
    _fn.argtypes = _args


def lib() -> ctypes.CDLL:
    return _lib


def library_path() -> str:
    return str(_LIB_PATH)


def check(status: int) -> None:
    """Raise RuntimeError(tl_hybrid_last_error()) for a non-zero status."""
    if status != 0:
        message = _lib.tl_hybrid_last_error()
        raise RuntimeError(message.decode() if message else f"tinyllm_hybrid error {status}")
