"""Throughput of a layer-list model (the Fonapel family on the layer-list engine) beside the framework's closest existing
model, Qwen3 on the fused W4A16 engine, at equal layer sizes and with random weights:  `python bench.py --layer-list W[,W...]`.

Per width W (head width 128, W/128 query heads, a quarter of them K/V heads, feed-forward 3 W, 4 layers, vocabulary 32,768):
prefill of one prompt in one chunk, decode of 1 and of 4 sequences over that context.  Beside tokens/s every leg reports what
its roofline is made of -- the bytes a decode step must stream (weights once + K/V or state of every live sequence), the
multiply-adds of a prefill chunk -- and the fraction of 8 TB/s / 2.5 PFLOP/s (dense bf16) that the measured time amounts to.
The two models differ where the designs differ: bf16 matrices against 4-bit ones (4 x the bytes per decode step), two of
four mixers recurrent (no K/V to stream, a sequential recurrence in prefill), one fused in/out product pair per layer.

`--layer-list-family Zefapel` measures the Zefapel family instead, beside its closest existing model -- Fonapel, on the same
engine -- at equal width, head count, head width and matrix elements per layer: 4 layers (matrix memory + gated feed-forward,
gated linear attention + mixture of experts, latent attention + gated feed-forward, latent attention on the third layer's cache
+ mixture of experts).  Its roofline counts what the design needs, not what the engine computes: the experts a token takes (not
all of them), a latent cache row of kv_rank + rot_dim per token.

`--layer-list-family Lovulix` measures the Lovulix family beside Fonapel with attention layers only (the like kernels: the same projections,
attention over the same paged K/V, one more norm per branch), at equal width, heads, head width and matrix elements a token multiplies:
4 attention layers (16 heads at width 2048, a quarter of them K/V heads, scores mixed across heads, chunks of 8,192 positions, learned sinks,
values blended from the second layer on) with 8 gated experts of W / 2 (2 taken) beside a shared one of W.

`--layer-list-family Muduvik` measures the Muduvik family beside Zefapel with dense feed-forwards (the closest existing model: the same
sequential block with layer scales, latent attention over the same 192-wide cache rows, a linear recurrence over 128 x 128 states, the
same gated feed-forward of 2 W) and, for its attention layers, beside Fonapel's attention: 4 layers (retention, differential attention with
a window of 4,096 positions, latent attention, differential attention), a per-layer token input of 256 columns.
"""

from __future__ import annotations

import json
import random
import time

HBM_BYTES_PER_S = 8.0e12
BF16_FLOPS = 2.5e15


def lovulix_config(width: int, layers: int = 4, vocab: int = 32768, chunk: int = 8192) -> dict:
    heads = max(1, width // 128)
    kv = max(1, heads // 4)
    rot = {"base": 5e5, "dims": 64, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}
    mixer = {"heads": heads, "kv_heads": kv, "dim": 128, "vdim": 128, "mask": {"size": chunk}, "rot": rot, "scale": 128 ** -0.5, "v_mix": True}
    mlp = {"kind": "moe", "expert": {"ff": width // 2}, "router": {"experts": 8, "top": 2}, "shared": {"ff": width}}
    return {"architecture": "Lovulix", "layers": [{"type": "attention", "mixer": dict(mixer), "mlp": mlp} for _ in range(layers)], "logit_scale": 1.0,
            "norm": {"eps": 1e-5}, "vocab": vocab, "width": width}


def lovulix_costs(cfg: dict, ctx: int, dtype_bytes: int = 2) -> dict:
    """What the design needs: the matrix elements a token multiplies (the experts it takes), attention multiply-adds per (query, key) pair of
    one chunk, the bytes a decode step of b sequences streams (every matrix once, of the experts those b tokens can take; the keys and values of
    the query's own chunk)."""
    W, fixed, per_expert, taken, kv_per_tok, attn, chunk = cfg["width"], 0, [], [], 0, 0, 0
    for L in cfg["layers"]:
        m, mlp = L["mixer"], L["mlp"]
        H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        fixed += W * (H * D + G * D + G * V + H * V) + H * V * W
        kv_per_tok += G * (D + V)
        attn += H * (D + V + H)
        chunk = (m.get("mask") or {}).get("size", 0)
        if mlp:
            fixed += W * mlp["router"]["experts"] + (3 * W * mlp["shared"]["ff"] if mlp.get("shared") else 0)
            per_expert.append(3 * W * mlp["expert"]["ff"])
            taken.append((mlp["router"]["top"], mlp["router"]["experts"]))
    head = cfg["vocab"] * W
    seen = min(ctx, (ctx - 1) % chunk + 1) if chunk else ctx
    return {"matrix_elems": fixed + sum(pe * top for pe, (top, _) in zip(per_expert, taken)), "head_elems": head, "attn_macs_per_pair": attn, "chunk": chunk,
            "decode_bytes": lambda b: (fixed + head + sum(pe * min(n, b * top) for pe, (top, n) in zip(per_expert, taken))) * dtype_bytes
            + b * seen * kv_per_tok * dtype_bytes}


def muduvik_config(width: int, vocab: int = 32768, window: int = 4096, side: int = 256) -> dict:
    heads = max(1, width // 128)
    kv = max(1, heads // 4)
    dense = {"kind": "dense", "ff": 2 * width}
    rot = {"base": 1e6, "dims": 64, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}
    attn = {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv, "dim": 128, "vdim": 128, "mask": {"size": window}, "rot": rot, "scale": 128 ** -0.5,
                                           "diff": 0.5}, "mlp": dense}
    ret = {"type": "retention", "mixer": {"heads": heads, "dim": 128, "vdim": 128, "rot": {"base": 1e6, "dims": 64},
                                          "decay": [1.0 - 2.0 ** (-5 - 3 * h / max(1, heads - 1)) for h in range(heads)]}, "mlp": dense}
    lat = {"type": "latent_attention", "mixer": {"heads": heads, "dim": 128, "vdim": 128, "q_rank": max(64, width // 2), "kv_rank": 192, "scale": 128 ** -0.5},
           "mlp": dense}
    return {"architecture": "Muduvik", "layers": [ret, attn, lat, dict(attn)], "norm": {"eps": 1e-6}, "token_side": {"dim": side}, "vocab": vocab, "width": width}


def muduvik_costs(cfg: dict, ctx: int, dtype_bytes: int = 2) -> dict:
    """What the design needs: matrix elements a token multiplies, attention multiply-adds per (query, key) pair in the per-head form (two maps per
    head in differential attention), the pairs a window leaves, and the bytes a decode step of b sequences streams: every matrix once, the keys
    (two maps) and values inside the window, one latent row per cached token, the recurrent states read and written."""
    W, sd = cfg["width"], (cfg.get("token_side") or {}).get("dim", 0)
    fixed, state, windowed, causal = 0, 0, [], 0
    kv_bytes = lambda c: 0
    terms = []
    for L in cfg["layers"]:
        m, ff = L["mixer"], (L["mlp"] or {}).get("ff", 0)
        H, D, V = m["heads"], m["dim"], m["vdim"]
        if L["type"] == "retention":
            fixed += W * (2 * H * D + 2 * H * V) + H * V * W
            state += H * D * V
        elif L["type"] == "attention":
            G, win = m["kv_heads"], (m.get("mask") or {}).get("size", 0)
            fixed += W * (2 * H * D + 2 * G * D + G * V + H) + H * V * W
            windowed.append((H * 2 * (D + V), win))
            terms.append((G * (2 * D + V), win))
        else:
            C, Q = m["kv_rank"], m["q_rank"]
            fixed += W * Q + Q * H * D + W * C + H * (D + V) * C + H * V * W
            causal += H * (D + V)
            terms.append((C, 0))
        fixed += 3 * W * ff + 2 * W * sd
    head = cfg["vocab"] * W

    def attn_macs(n):  # multiply-adds of a causal prompt of n tokens
        full = n * (n + 1) / 2
        total = causal * full
        for macs, win in windowed:
            total += macs * (full if not win or win >= n else win * (win + 1) / 2 + (n - win) * win)
        return total

    return {"matrix_elems": fixed, "head_elems": head, "attn_macs": attn_macs,
            "decode_bytes": lambda b: (fixed + head) * dtype_bytes + b * (sum(per * (min(ctx, win) if win else ctx) for per, win in terms) * dtype_bytes + 2 * state * 4)}


def zefapel_dense_config(width: int, vocab: int = 32768) -> dict:
    """Zefapel with the gated feed-forward of 2 W on every layer (no experts): the closest existing model to Muduvik, layer for layer."""
    cfg = zefapel_config(width, vocab)
    for L in cfg["layers"]:
        L["mlp"] = {"kind": "dense", "ff": 2 * width}
    return cfg


def fonapel_config(width: int, layers: int = 4, vocab: int = 32768, order: str = "mixed") -> dict:
    heads = max(1, width // 128)
    kv = max(1, heads // 4)
    attn = {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv, "dim": 128, "vdim": 128, "rot": {"dims": 64, "base": 1e6}, "scale": 128 ** -0.5},
            "mlp": {"kind": "dense", "ff": 3 * width}}
    delta = {"type": "delta", "mixer": {"heads": heads, "kv_heads": heads, "dim": 128, "vdim": 128, "conv": 4}, "mlp": {"kind": "dense", "ff": 3 * width}}
    order = [attn] * 4 if order == "attention" else [delta, attn, attn, delta]
    return {"architecture": "Fonapel", "layers": [order[i % 4] for i in range(layers)], "norm": {"eps": 1e-5}, "residual_mult": 0.5, "vocab": vocab,
            "width": width}


def zefapel_config(width: int, vocab: int = 32768) -> dict:
    """Head width 128 like the other two; the latent cache row is 192 + 64 wide; gated feed-forward of 2 W (three matrices: as many
    elements as the 3 W two-matrix one beside it); 8 experts of W / 2 + 2 identity experts in 5 groups (3 kept), 2 taken, a shared one of W."""
    heads = max(1, width // 128)
    dense = {"kind": "dense", "ff": 2 * width}
    moe = {"kind": "moe", "expert": {"ff": width // 2}, "router": {"experts": 8, "identity": 2, "top": 2, "groups": {"count": 5, "keep": 3}},
           "shared": {"ff": width}}
    rot = {"base": 1e6, "dims": 64, "scaling": {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}}
    latent = {"heads": heads, "dim": 128, "vdim": 128, "rot_dim": 64, "q_rank": max(64, width // 2), "kv_rank": 192, "rot": rot, "scale": 192 ** -0.5}
    layers = [{"type": "mlstm", "mixer": {"heads": heads, "dim": 128, "vdim": 128, "gate_cap": 20.0}, "mlp": dense},
              {"type": "gla", "mixer": {"heads": heads, "dim": 128, "vdim": 128, "tau": 8.0}, "mlp": moe},
              {"type": "latent_attention", "mixer": dict(latent), "mlp": dense},
              {"type": "latent_attention", "mixer": dict(latent, kv_from=2), "mlp": moe}]
    return {"architecture": "Zefapel", "embedding": {"scale": 1.0}, "layers": layers, "norm": {"eps": 1e-6}, "vocab": vocab, "width": width}


def zefapel_costs(cfg: dict, ctx: int, dtype_bytes: int = 2) -> dict:
    """What the design needs: matrix elements a token multiplies (the experts it takes, not all), attention multiply-adds per
    (query, key) pair in the per-head form, the bytes a decode step of b sequences must stream (every matrix once, but of the
    experts only those b tokens can take; one latent row per cached token; the recurrent states read and written)."""
    W, fixed, per_expert, experts_taken, kv_per_tok, state, attn = cfg["width"], 0, [], [], 0, 0, 0
    for L in cfg["layers"]:
        m, mlp = L["mixer"], L["mlp"]
        H, D, V = m["heads"], m["dim"], m["vdim"]
        if L["type"] == "mlstm":
            fixed += W * (2 * H * D + 2 * H * V + 2 * H) + H * V * W
            state += H * D * (V + 1)
        elif L["type"] == "gla":
            fixed += W * (2 * H * D + 2 * H * V + 16) + 16 * H * D + H * V * W  # (synthetic weights: a decay projection pair of rank 16)
            state += H * D * V
        else:
            R, C, Q = m["rot_dim"], m["kv_rank"], m["q_rank"]
            fixed += W * Q + Q * H * (D + R) + H * (D + V) * C + 2 * H * V * W
            if "kv_from" not in m:
                fixed += W * (C + R)
                kv_per_tok += C + R
            attn += H * (D + R + V)
        if mlp and mlp["kind"] == "dense":
            fixed += 3 * W * mlp["ff"]
        elif mlp:
            r = mlp["router"]
            fixed += W * (r["experts"] + r.get("identity", 0)) + (2 * W * mlp["shared"]["ff"] + W if mlp.get("shared") else 0)
            per_expert.append(2 * W * mlp["expert"]["ff"])
            experts_taken.append((r["top"], r["experts"]))
    head = cfg["vocab"] * W
    active = fixed + sum(pe * top for pe, (top, _) in zip(per_expert, experts_taken))
    return {"matrix_elems": active, "head_elems": head, "attn_macs_per_pair": attn,
            "decode_bytes": lambda b: (fixed + head + sum(pe * min(n, b * top) for pe, (top, n) in zip(per_expert, experts_taken))) * dtype_bytes
            + b * (ctx * kv_per_tok * dtype_bytes + 2 * state * 4)}


def qwen3_config(width: int, layers: int = 4, vocab: int = 32768) -> dict:
    heads = max(1, width // 128)
    return dict(hidden_size=width, num_hidden_layers=layers, num_attention_heads=heads, num_key_value_heads=max(1, heads // 4), head_dim=128,
                intermediate_size=3 * width, vocab_size=vocab, rope_theta=1000000, rms_norm_eps=1e-6, max_position_embeddings=40960,
                tie_word_embeddings=False)


def fonapel_costs(cfg: dict, ctx: int, dtype_bytes: int = 2) -> dict:
    """Matrix elements (= multiply-adds per token), attention multiply-adds of a causal prompt, and the bytes a decode step streams."""
    W, params, kv_per_tok, state = cfg["width"], 0, 0, 0
    for L in cfg["layers"]:
        m, ff = L["mixer"], (L["mlp"] or {}).get("ff", 0)
        H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        if L["type"] == "attention":
            params += W * (H * D + G * D + G * V + H * V) + H * V * W
            kv_per_tok += G * (D + V)
        else:
            params += W * (2 * G * D + 2 * H * V + 2 * H) + H * V * W
            state += H * D * V
        params += 2 * W * ff
    attn_macs = sum(L["mixer"]["heads"] * (L["mixer"]["dim"] + L["mixer"]["vdim"]) for L in cfg["layers"] if L["type"] == "attention")
    head = cfg["vocab"] * W
    return {"matrix_elems": params, "head_elems": head, "attn_macs_per_pair": attn_macs,
            "decode_bytes": lambda b: (params + head) * dtype_bytes + b * (ctx * kv_per_tok * dtype_bytes + 2 * state * 4)}


def qwen3_costs(cfg: dict, ctx: int) -> dict:
    W, H, G, D, I = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["intermediate_size"]
    per_layer = W * (H * D + 2 * G * D) + H * D * W + 3 * W * I
    params = per_layer * cfg["num_hidden_layers"]
    head = cfg["vocab_size"] * W
    w4 = 0.5 + 4.0 / 128  # nibbles + bf16 scale and bias per group of 128
    return {"matrix_elems": params, "head_elems": head, "attn_macs_per_pair": cfg["num_hidden_layers"] * H * 2 * D,
            "decode_bytes": lambda b: (params + head) * w4 + b * ctx * cfg["num_hidden_layers"] * 2 * G * D * 2}


def _time(fn, sync, repeats: int) -> float:
    fn()
    sync()
    best = float("inf")
    for _ in range(repeats):
        t0 = time.perf_counter()
        fn()
        sync()
        best = min(best, time.perf_counter() - t0)
    return best


def measure(engine, prompt, decode_steps: int, batches=(1, 4), free_running=None) -> dict:
    """prefill seconds of `prompt` in one chunk and seconds per decode step at the batches given; the engine has max(batches) slots."""
    out = {}

    def prefill_once():
        engine.begin(0)
        engine.prefill(0, prompt, chunk=len(prompt))
        engine.synchronize()
        engine.release(0)

    out["prefill_s"] = _time(prefill_once, engine.synchronize, 3)
    for b in batches:
        for s in range(b):
            engine.begin(s)
            engine.prefill(s, prompt, chunk=len(prompt))
        run = (lambda: free_running(decode_steps, list(range(b)))) if free_running else (lambda: engine.decode(decode_steps, batch=b))
        run()  # captures the step
        engine.synchronize()
        t0 = time.perf_counter()
        run()
        engine.synchronize()
        out[f"decode_step_s_b{b}"] = (time.perf_counter() - t0) / decode_steps
        for s in range(b):
            engine.release(s)
    return out


def run_family_pair(widths, prompt_len: int = 2048, decode_steps: int = 64, seed: int = 0, device: str = "cuda", family: str = "Zefapel") -> dict:
    """Zefapel or Lovulix beside Fonapel (Lovulix: beside its attention layers only), all on the layer-list engine."""
    import torch

    from tiny_llm_hip.models import engine_for
    from tiny_llm_hip.synthetic import synthetic_layer_list

    rng = random.Random(seed)
    results = []
    for W in widths:
        prompt = [rng.randrange(1, 32768) for _ in range(prompt_len)]
        ctx = prompt_len + decode_steps
        page = 128
        pages = 4 * ((prompt_len + 3 * decode_steps) // page + 2)
        row = {"width": W, "prompt_len": prompt_len, "decode_steps": decode_steps}
        new = {"Zefapel": ("zefapel", zefapel_config(W), zefapel_costs), "Lovulix": ("lovulix", lovulix_config(W), lovulix_costs),
               "Muduvik": ("muduvik", muduvik_config(W), muduvik_costs)}[family]
        others = [("fonapel", fonapel_config(W, order="mixed" if family == "Zefapel" else "attention"), fonapel_costs)]
        if family == "Muduvik":
            others.insert(0, ("zefapel_dense", zefapel_dense_config(W), zefapel_costs))
        for key, cfg, costs in [new] + others:
            model = synthetic_layer_list(cfg, seed=seed, device=device)
            eng = engine_for(model, dtype=torch.bfloat16, page_size=page, num_pages=pages, max_batch=4, max_pages_per_seq=pages // 4, max_prefill_rows=prompt_len)
            try:
                got = measure(eng, prompt, decode_steps, free_running=eng.decode_free_running)
            finally:
                eng.close()
            del model
            row[key] = summarize(got, costs(cfg, ctx), prompt_len)
            torch.cuda.empty_cache()
        for other, _, _ in others:
            for leg in ("prefill", "decode_b1", "decode_b4"):
                a, b = row[new[0]][leg]["roofline_fraction"], row[other][leg]["roofline_fraction"]
                name = "times_as_far_from_roofline" if other == others[0][0] else f"times_as_far_from_roofline_{other}"
                row.setdefault(name, {})[leg] = round(b / a, 2) if a > 0 else None
        results.append(row)
    return {"bench": "layer_list_compare", "family": family, "beside": [o[0] for o in others] if len(others) > 1 else "Fonapel", "dtype": "bf16", "data": "synthetic",
            "roofline": {"hbm_bytes_per_s": HBM_BYTES_PER_S, "bf16_flops": BF16_FLOPS}, "results": results}


def run(widths, prompt_len: int = 2048, decode_steps: int = 64, seed: int = 0, device: str = "cuda") -> dict:
    import torch

    from tiny_llm_hip.engine import DecodeEngine
    from tiny_llm_hip.models import engine_for
    from tiny_llm_hip.synthetic import synthetic_layer_list, synthetic_qwen3

    rng = random.Random(seed)
    results = []
    for W in widths:
        prompt = [rng.randrange(1, 32768) for _ in range(prompt_len)]
        ctx = prompt_len + decode_steps
        page = 128
        pages = 4 * ((prompt_len + 3 * decode_steps) // page + 2)
        row = {"width": W, "prompt_len": prompt_len, "decode_steps": decode_steps}
        # the layer-list model
        fcfg = fonapel_config(W)
        model = synthetic_layer_list(fcfg, seed=seed, device=device)
        eng = engine_for(model, dtype=torch.bfloat16, page_size=page, num_pages=pages, max_batch=4, max_pages_per_seq=pages // 4, max_prefill_rows=prompt_len)
        try:
            got = measure(eng, prompt, decode_steps, free_running=eng.decode_free_running)
        finally:
            eng.close()
        del model
        fc = fonapel_costs(fcfg, ctx)
        row["fonapel"] = summarize(got, fc, prompt_len)
        # Qwen3 W4A16 at equal sizes
        qcfg = qwen3_config(W)
        qmodel = synthetic_qwen3(qcfg, seed=seed, sigma=0.02, device=device)
        qeng = DecodeEngine(qmodel, page_size=page, num_pages=pages, max_batch=4, max_pages_per_seq=pages // 4, max_prefill_rows=prompt_len)
        try:
            got = measure(qeng, prompt, decode_steps)
        finally:
            qeng.close()
        del qmodel
        row["qwen3_w4"] = summarize(got, qwen3_costs(qcfg, ctx), prompt_len)
        for leg in ("prefill", "decode_b1", "decode_b4"):
            a, b = row["fonapel"][leg]["roofline_fraction"], row["qwen3_w4"][leg]["roofline_fraction"]
            row.setdefault("times_as_far_from_roofline", {})[leg] = round(b / a, 2) if a > 0 else None
        results.append(row)
        torch.cuda.empty_cache()
    return {"bench": "layer_list_compare", "dtype": "bf16", "data": "synthetic", "roofline": {"hbm_bytes_per_s": HBM_BYTES_PER_S, "bf16_flops": BF16_FLOPS},
            "results": results}


def summarize(got: dict, costs: dict, prompt_len: int) -> dict:
    chunk = costs.get("chunk") or prompt_len  # a chunked mask: whole chunks and the prompt's last, partial one
    pairs = (prompt_len // chunk) * chunk * (chunk + 1) / 2 + (prompt_len % chunk) * (prompt_len % chunk + 1) / 2
    attn = costs["attn_macs"](prompt_len) if "attn_macs" in costs else costs["attn_macs_per_pair"] * pairs  # (a windowed design counts its own pairs)
    flops = 2.0 * (costs["matrix_elems"] * prompt_len + costs["head_elems"]) + 2.0 * attn
    out = {"prefill": {"tokens_per_s": round(prompt_len / got["prefill_s"], 1), "ms": round(got["prefill_s"] * 1e3, 3), "tflops": round(flops / got["prefill_s"] / 1e12, 1),
                       "roofline_fraction": round(flops / got["prefill_s"] / BF16_FLOPS, 4)}}
    for b in (1, 4):
        t = got[f"decode_step_s_b{b}"]
        bytes_ = costs["decode_bytes"](b)
        out[f"decode_b{b}"] = {"tokens_per_s": round(b / t, 1), "us_per_step": round(t * 1e6, 1), "gbytes_per_s": round(bytes_ / t / 1e9, 1),
                               "roofline_fraction": round(bytes_ / t / HBM_BYTES_PER_S, 4)}
    return out


def main(widths, prompt_len=2048, decode_steps=64, family="Fonapel") -> None:
    if family not in ("Fonapel", "Zefapel", "Lovulix", "Muduvik"):
        raise SystemExit(f"--layer-list-family: unknown family {family!r}")
    out = run(widths, prompt_len, decode_steps) if family == "Fonapel" else run_family_pair(widths, prompt_len, decode_steps, family=family)
    print(json.dumps(out), flush=True)
