"""Layer-list engine: host mirror of include/tinyllm_hybrid.h.

``HybridEngine`` has the request-level surface of ``engine.DecodeEngine`` (begin / prefill / prefill_packed / decode /
set_token / read_pending / read_tokens / logits / move / release / stats / generate), so the schedulers and command lines
written against that surface (``engine.batch_generate_ids``, main.py, batch_main.py) drive either engine.  On top of it:
``step`` -- one packed pass over chunks of several slots, prompt portions beside single decode tokens, with the logits of any
rows -- which is what the engine's prefill and decode are made of.
"""

from __future__ import annotations

import ctypes
from typing import Any, Sequence

import torch

from .layer_list import LayerListConfig, pack_layer_list

__all__ = ["HybridEngine"]

_FF_ACT = {"gelu_erf": 0, "gelu_tanh": 1, "silu": 2, "relu2": 3}
_MIX = {"attention": 0, "delta": 1, "linrec": 2, "latent": 3}
_REC = {"channel": 0, "expgate": 1, "fixed": 2}
_NORM = {"rms": 0, "dyt": 1}
_FF_KIND = {"plain": 0, "gated": 1, "moe": 2}
_BLOCK = {"sequential": 0, "parallel": 1, "postnorm": 2, "sandwich": 3}
_VMIX = {"none": 0, "first": 1, "blend": 2}
_ROUTER = {"softmax": 0, "sigmoid": 1}


class HybridEngine:
    """Owns the packed weights, the paged K/V pools, the state slots and the captured decode graphs of one layer-list model."""

    supports_mixed_steps = True

    def __init__(self, model: Any, *, page_size: int = 64, num_pages: int = 512, max_batch: int = 1,
                 max_pages_per_seq: int | None = None, max_prefill_rows: int = 2048, dtype: torch.dtype | None = None,
                 device: str | torch.device = "cuda", **_ignored):
        """``model``: what ``loader.load_weights`` returns for a layer-list family (``.config`` a LayerListConfig, ``.tensors``
        name -> tensor, ``.dtype``).  ``dtype``: torch.bfloat16 (matrices, matrix-product inputs and K/V pages in bfloat16) or
        torch.float32 (everything in float32)."""
        import tiny_llm_ext_hybrid as ext  # GPU-only; fails loudly when the library is not built

        if not torch.cuda.is_available():
            raise RuntimeError("HybridEngine: the extension is GPU-only")
        self._ext, self._lib = ext, ext.lib()
        cfg: LayerListConfig = model.config
        dtype = dtype or getattr(model, "dtype", torch.bfloat16)
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("HybridEngine: dtype must be torch.bfloat16 or torch.float32")
        self.config, self.dtype, self.device = cfg, dtype, torch.device(device)
        self.page_size, self.max_batch, self.vocab_size = int(page_size), int(max_batch), cfg.vocab
        self.max_prefill_rows = max(int(max_prefill_rows), self.max_batch)
        self.num_hidden_layers = len(cfg.layers)
        self.has_recurrent_state = any(L.kind in ("delta", "linrec") for L in cfg.layers)
        for i, L in enumerate(cfg.layers):  # a size the configuration leaves to the tensors
            if L.a_rank < 0:
                L.a_rank = int(model.tensors[cfg.prefix(i) + "mix.a1"].shape[0])
        w = self._weights = pack_layer_list(cfg, model.tensors, dtype, self.device)
        layers = (ext.TlHybridLayer * len(cfg.layers))()
        for i, (L, t) in enumerate(zip(cfg.layers, w["layers"])):
            s = layers[i]
            s.kind = _MIX[L.kind]
            s.heads, s.kv_heads, s.dim, s.vdim, s.ff, s.ff_act = L.heads, L.kv_heads, L.dim, L.vdim, L.ff, _FF_ACT[L.ff_act]
            s.w_in_dev, s.w_out_dev, s.norm_dev, s.norm_offset = t["w_in"].data_ptr(), t["w_out"].data_ptr(), t["norm"].data_ptr(), cfg.norm_offset
            s.rot_dims, s.rot_base, s.scale = L.rot_dims, L.rot_base, L.scale
            s.qk_unit_rms, s.sink, s.gated = int(L.qk_unit_rms), int(L.sink), (2 if L.head_gate else 1) if L.gated else 0
            s.conv_taps, s.unit_eps = L.conv_taps, L.unit_eps
            if L.kind == "delta":
                s.conv_dev, s.a_log_dev, s.dt_bias_dev, s.out_norm_dev = (t["conv"].data_ptr(), t["a_log"].data_ptr(),
                                                                          t["dt_bias"].data_ptr(), t["out_norm"].data_ptr())
            ptr = lambda key: t[key].data_ptr() if key in t else None
            s.norm_kind, s.norm_alpha, s.norm2_alpha = _NORM[cfg.norm_kind], t.get("norm_alpha", 0.0), t.get("norm2_alpha", 0.0)
            s.norm_bias_dev, s.norm2_bias_dev, s.norm2_dev = ptr("norm_bias"), ptr("norm2_bias"), ptr("norm2")
            s.w_in2_dev, s.w_out2_dev, s.ls1_dev, s.ls2_dev = ptr("w_in2"), ptr("w_out2"), ptr("ls1"), ptr("ls2")
            s.ff_kind, s.experts, s.identity, s.top, s.groups, s.keep = _FF_KIND[L.ff_kind], L.experts, L.identity, L.top, L.groups, L.keep
            s.expert_ff, s.shared_ff, s.correction_dev = L.expert_ff, L.shared_ff, ptr("correction")
            s.kv_from = -1
            s.moe_router, s.moe_gated, s.moe_scale_input = _ROUTER[L.router], int(L.moe_gated), int(L.moe_scale_input)
            s.moe_shared_sg = int(L.moe_gated and L.moe_shared_sg)
            if L.kind == "attention":
                s.qk_norm, s.q_norm_dev, s.k_norm_dev, s.rot_half = int(L.qk_norm), ptr("q_norm"), ptr("k_norm"), int(L.rot_half)
                s.talk_dev, s.sink_dev, s.chunk = ptr("talk"), ptr("sink"), L.chunk
                s.v_mix, s.v_mix_lambda = _VMIX[L.v_mix], t.get("v_mix_lambda", 0.0)
                s.w_in_bias_dev, s.window, s.qk_head_norm = ptr("w_in_bias"), L.window, int(L.qk_head_norm)
                if L.diff is not None:
                    s.diff_maps, s.diff_lambda, s.diff_init = 1, t["diff_lambda"], L.diff
            if L.kind in ("attention", "linrec") and L.rot_scaling:
                s.rot_factor, s.rot_original, s.rot_fast, s.rot_slow = L.rot_scaling
                s.rot_scaling_kind = 1 if L.rot_scaling_kind == "wavelength" else 0
            s.post_norm_dev, s.post_norm2_dev = ptr("post_norm"), ptr("post_norm2")
            s.side_gate_dev, s.side_proj_dev, s.side_norm_dev, s.side_col0 = ptr("side_gate"), ptr("side_proj"), ptr("side_norm"), i * cfg.side_dim
            if L.kind == "linrec":
                s.rec_kind, s.gate_cap, s.tau, s.a_rank, s.out_norm_dev = _REC[L.rec_kind], L.gate_cap, L.tau, max(L.a_rank, 0), ptr("out_norm")
                s.decay_dev, s.rot_half = ptr("decay"), int(L.rot_half)
                s.a2_dev, s.a2_bias_dev, s.i_bias_dev, s.f_bias_dev = ptr("a2"), ptr("a2_bias"), ptr("i_bias"), ptr("f_bias")
            elif L.kind == "latent":
                s.q_rank, s.kv_rank, s.rot_dim, s.kv_from = L.q_rank, L.kv_rank, L.rot_dim, L.kv_from
                s.dq_norm_dev, s.dkv_norm_dev, s.uq_dev, s.uk_t_dev, s.uv_dev = ptr("dq_norm"), ptr("dkv_norm"), ptr("uq"), ptr("uk_t"), ptr("uv")
                if L.rot_scaling:
                    s.rot_factor, s.rot_original, s.rot_fast, s.rot_slow = L.rot_scaling
        c = ext.TlHybridConfig()
        c.dtype = ext.HY_BF16 if dtype == torch.bfloat16 else ext.HY_F32
        c.width, c.vocab, c.num_layers, c.norm_eps, c.residual_mult = cfg.width, cfg.vocab, len(cfg.layers), cfg.norm_eps, cfg.residual_mult
        c.parallel_block, c.embed_scale, c.logit_scale = _BLOCK[cfg.block], cfg.embed_scale, cfg.logit_scale
        c.final_norm_kind, c.final_norm_alpha = _NORM[cfg.norm_kind], w.get("final_norm_alpha", 0.0)
        c.final_norm_bias_dev = w["final_norm_bias"].data_ptr() if "final_norm_bias" in w else None
        if cfg.loop:
            c.loop_start, c.loop_stop, c.loop_times = cfg.loop
            c.loop_in_dev, c.loop_step_dev = (w["loop_in"].data_ptr() if "loop_in" in w else None), w["loop_step"].data_ptr()
        c.embed_dev, c.final_norm_dev, c.final_norm_offset, c.head_dev = w["embed"].data_ptr(), w["final_norm"].data_ptr(), cfg.norm_offset, w["head"].data_ptr()
        c.embed_norm_dev = w["embed_norm"].data_ptr() if "embed_norm" in w else None
        if cfg.side_dim:
            c.side_embed_dev, c.side_cols, c.side_dim = w["side_embed"].data_ptr(), w["side_embed"].shape[1], cfg.side_dim
        c.page_size, c.num_pages, c.max_slots = self.page_size, int(num_pages), self.max_batch
        c.max_pages_per_seq = int(max_pages_per_seq if max_pages_per_seq is not None else num_pages)
        c.max_rows = self.max_prefill_rows
        torch.cuda.synchronize()
        handle = ctypes.c_void_p()
        ext.check(self._lib.tl_hybrid_create(ctypes.byref(c), layers, None, ctypes.byref(handle)))
        self._h = handle
        self._produced: dict[int, list[int]] = {}

    @classmethod
    def from_model(cls, model: Any, **kwargs) -> "HybridEngine":
        return cls(model, **kwargs)

    def close(self) -> None:
        if getattr(self, "_h", None):
            self._lib.tl_hybrid_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # -- slots -------------------------------------------------------------------------------------------------------
    def begin(self, slot: int = 0) -> None:
        self._ext.check(self._lib.tl_hybrid_begin(self._h, slot))
        self._produced[slot] = []

    def release(self, slot: int = 0) -> None:
        self._ext.check(self._lib.tl_hybrid_release(self._h, slot))
        self._produced.pop(slot, None)

    def move(self, src: int, dst: int) -> None:
        self._ext.check(self._lib.tl_hybrid_move(self._h, src, dst))
        self._produced[dst] = self._produced.pop(src, [])

    def rewind(self, slot: int, n: int) -> None:
        raise RuntimeError("HybridEngine: a sequence cannot be rewound (recurrent state keeps no history)")

    def context_len(self, slot: int = 0) -> int:
        return self._lib.tl_hybrid_context_len(self._h, slot)

    def set_token(self, slot: int, token: int) -> None:
        self._ext.check(self._lib.tl_hybrid_set_token(self._h, slot, int(token)))

    def live_slots(self, upto: int | None = None) -> list[int]:
        return [s for s in range(upto if upto is not None else self.max_batch) if self.context_len(s) >= 0]

    # -- compute -----------------------------------------------------------------------------------------------------
    def step(self, entries: Sequence[tuple[int, Sequence[int], Sequence[int]]]) -> int:
        """One packed pass: ``entries`` = (slot, token ids, wanted places among these tokens) per sequence; a chunk of one token
        is a decode step.  Logits rows come in the order of the entries and of their wanted places (``logits`` /
        ``logits_host``); returns their number.  The last wanted row of a slot leaves its argmax as the slot's pending token."""
        n = len(entries)
        slots = (ctypes.c_int * n)(*[int(e[0]) for e in entries])
        lens = (ctypes.c_int * n)(*[len(e[1]) for e in entries])
        flat = [int(t) for e in entries for t in e[1]]
        want, row0 = [], 0
        for _, toks, places in entries:
            for p in places:
                if not 0 <= int(p) < len(toks):
                    raise ValueError("step: a wanted place lies outside its chunk")
                want.append(row0 + int(p))
            row0 += len(toks)
        tokens = (ctypes.c_int32 * max(1, len(flat)))(*flat)
        want_c = (ctypes.c_int * max(1, len(want)))(*want)
        self._ext.check(self._lib.tl_hybrid_step(self._h, n, slots, tokens, lens, len(want), want_c))
        self._rows = len(want)
        return len(want)

    def prefill(self, slot: int, tokens: Sequence[int], *, chunk: int | None = None, want_logits: bool = True) -> None:
        """Chunked prefill of one slot; the last chunk leaves the last row's logits and the first generated token."""
        tokens = [int(t) for t in tokens]
        if not tokens:
            raise ValueError("prefill needs at least one token")
        chunk = min(self.max_prefill_rows, chunk or self.max_prefill_rows)
        for start in range(0, len(tokens), chunk):
            part = tokens[start:start + chunk]
            last = start + chunk >= len(tokens)
            self.step([(slot, part, [len(part) - 1] if (last and want_logits) else [])])
        if want_logits:
            self._produced.setdefault(slot, []).append(self.read_pending_slots([slot])[0])

    def prefill_packed(self, chunks: Sequence[tuple[int, Sequence[int], bool]]) -> None:
        """Several slots' chunks in one pass: (slot, token ids, ends_prompt)."""
        self.step([(s, toks, [len(toks) - 1] if ends else []) for s, toks, ends in chunks])
        done = [s for s, _, ends in chunks if ends]
        for s, tok in zip(done, self.read_pending_slots(done)):
            self._produced.setdefault(s, []).append(tok)

    def decode(self, steps: int, batch: int | None = None, use_graph: bool = True, slots: Sequence[int] | None = None) -> None:
        """``steps`` greedy decode steps over the live slots of [0, batch) (or the slots listed), on the device."""
        slots = list(slots) if slots is not None else self.live_slots(batch or self.max_batch)
        if not slots:
            return
        arr = (ctypes.c_int * len(slots))(*slots)
        for _ in range(steps):  # one captured step per call: the ids of every step are kept for read_tokens
            self._ext.check(self._lib.tl_hybrid_decode(self._h, len(slots), arr, 1, int(use_graph)))
            for s, tok in zip(slots, self.read_pending_slots(slots)):
                self._produced.setdefault(s, []).append(tok)
        self._rows = len(slots)

    def decode_free_running(self, steps: int, slots: Sequence[int], use_graph: bool = True) -> None:
        """``steps`` decode steps enqueued back to back with no host round trip between them (throughput measurements)."""
        arr = (ctypes.c_int * len(slots))(*slots)
        self._ext.check(self._lib.tl_hybrid_decode(self._h, len(slots), arr, int(steps), int(use_graph)))
        self._rows = len(slots)

    def read_pending_slots(self, slots: Sequence[int]) -> list[int]:
        if not slots:
            return []
        arr = (ctypes.c_int * len(slots))(*[int(s) for s in slots])
        out = (ctypes.c_int32 * len(slots))()
        self._ext.check(self._lib.tl_hybrid_read_pending(self._h, len(slots), arr, out))
        return list(out)

    def read_pending(self, count: int | None = None) -> list[int]:
        """Pending token id of slots [0, count) (0 for idle slots); synchronises."""
        return self.read_pending_slots(list(range(count or self.max_batch)))

    def read_tokens(self, slot: int, count: int) -> list[int]:
        """The last ``count`` generated ids of ``slot``."""
        got = self._produced.get(slot, [])
        if count > len(got):
            raise RuntimeError("read_tokens: fewer tokens have been generated")
        return got[len(got) - count:]

    def logits(self, rows: int = 1) -> torch.Tensor:
        """A copy of the first ``rows`` rows of the latest logits, [rows, vocab] float32 on the device."""
        out = torch.empty((rows, self.vocab_size), dtype=torch.float32, device=self.device)
        torch.cuda.current_stream().synchronize()
        self._ext.check(self._lib.tl_hybrid_copy_logits(self._h, out.data_ptr(), rows))
        self.synchronize()
        return out

    def logits_host(self, rows: int):
        """The first ``rows`` rows of the latest logits as a numpy float32 array."""
        import numpy as np

        out = np.empty((rows, self.vocab_size), dtype=np.float32)
        if rows:
            self._ext.check(self._lib.tl_hybrid_read_logits(self._h, out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), rows))
        return out

    def argmax(self, rows: int) -> list[int]:
        out = (ctypes.c_int32 * max(1, rows))()
        self._ext.check(self._lib.tl_hybrid_read_argmax(self._h, rows, out))
        return list(out)[:rows]

    def synchronize(self) -> None:
        self._ext.check(self._lib.tl_hybrid_synchronize(self._h))

    # -- test aids ---------------------------------------------------------------------------------------------------
    def set_trace(self, on: bool) -> None:
        self._ext.check(self._lib.tl_hybrid_set_trace(self._h, int(on)))

    def read_trace(self, run: int, rows: int):
        """The residual stream after layer run ``run`` of the latest step, [rows, width] float32 (tracing on)."""
        import numpy as np

        out = np.empty((rows, self.config.width), dtype=np.float32)
        self._ext.check(self._lib.tl_hybrid_read_trace(self._h, run, out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), rows))
        return out

    def stats(self) -> dict:
        s = self._ext.TlHybridStats()
        self._ext.check(self._lib.tl_hybrid_get_stats(self._h, ctypes.byref(s)))
        return {name: getattr(s, name) for name, _ in s._fields_}

    # -- one request, like DecodeEngine.generate ------------------------------------------------------------------------
    def generate(self, prompt: Sequence[int], max_new_tokens: int, *, slot: int = 0, chunk: int | None = None) -> list[int]:
        self.begin(slot)
        try:
            self.prefill(slot, prompt, chunk=chunk)
            if max_new_tokens > 1:
                self.decode(max_new_tokens - 1, slots=[slot])
            return self.read_tokens(slot, max_new_tokens)
        finally:
            self.release(slot)
