"""Layer-list model descriptions: decoder-only models given as a list of layers, each a token mixer of some kind plus an
optional feed-forward, served by the layer-list engine (``hybrid_engine.HybridEngine``, include/tinyllm_hybrid.h).

A *family* turns a checkpoint's ``config.json`` into a ``LayerListConfig`` and names its tensors; ``FAMILIES`` is the
registry ``loader.load_weights`` and ``models.engine_for`` consult (key: config.json's ``architecture``).  The engine itself
knows mixer kinds and their options, not families.

Fonapel -- per layer, with h = norm(x) and one norm for both branches:

    x <- x + m * (mixer(h) + ff(h))            norm: x / sqrt(mean x^2 + eps) * (1 + w)
    ff(h) = W_down gelu_erf(W_up h)

    mixer "attention": grouped-query attention; rotary positions on the first rot.dims dimensions (adjacent pairs, angle
        p * base^(-2i/dims)); then q and k divided by their RMS over the head; scores q.k * scale, causal;
        weights exp(s_j) / (1 + sum_j exp(s_j)); heads * sigmoid(W_g h); W_o.
    mixer "delta": gated delta rule.  q, k (kv_heads x dim), v (heads x vdim) each pass a causal depthwise convolution
        of `conv` taps and SiLU; q, k -> unit vectors (x / sqrt(sum x^2 + 1e-6)), q * dim^-1/2;
        beta = sigmoid(W_b h); g = exp(-exp(A_log) * softplus(W_a h + dt_bias)); per head
        S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q;
        o / rms(o) * norm * silu(W_g h); W_o.

    loop {start, stop, times}: layers start..stop-1 run `times` times with the same weights and separate caches; each pass
        is entered through x <- W_in [x ; x0] + step[t] (x0 = the embedding output).

Zefapel -- x = embed[token] * embedding.scale; per layer, sequentially, with Dynamic Tanh norms dyt(x) = tanh(alpha x) w + b and
per-channel layer scales ls1 / ls2:

    x <- x + ls1 * W_o mixer(dyt1(x));   x <- x + ls2 * ff(dyt2(x))

    mixer "mlstm": q (* dim^-1/2), k, v per head; log gates i = cap tanh((W_i h + b_i) / cap), f = logsigmoid(cap tanh((W_f h + b_f) / cap));
        m' = max(f + m, i) (m starts at 0);  S <- e^(f+m-m') S + e^(i-m') k v^T;  n likewise with k;
        o = S^T q / (max(|n.q|, e^-m') + 1e-6);  o / rms(o) * norm * sigmoid(W_g h).
    mixer "gla": the same state with a decay per key channel, a = sigmoid(W_a2 W_a1 h + b)^(1/tau), no gates, no normaliser;
        rms_norm(o) * norm[vdim] * silu(W_g h).
    mixer "latent_attention": q = W_uq rms_norm(W_dq h); W_dkv h = [latent (kv_rank) | one rotated key part (rot_dim)], the latent
        RMS-normed; per head k = [W_uk c | rotated part], v = W_uv c, q = [plain (dim) | rotated (rot_dim)]; rotation of adjacent pairs with
        frequencies rescaled by rot.scaling (factor, original, fast, slow) and cos / sin times 0.1 ln(factor) + 1; causal softmax
        of q.k * scale; heads * sigmoid(W_g h).  Only [c | rotated part] is cached; "kv_from": j reads layer j's cache instead of
        projecting its own.
    ff "dense": W_down (silu(W_gate h) * W_up h).
    ff "moe": s = softmax(W_router h) over experts + identity experts; choice = s + correction; experts form groups.count runs of
        neighbours, the groups.keep groups with the largest choice stay; the `top` largest choices among them are taken with weight s
        (not renormalised); expert = W_down relu(W_up h)^2, identity expert = h; plus sigmoid(W_sg h) * shared expert.

Lovulix -- x = embed[token]; per layer the norm sits on what a branch RETURNS and the branches read the stream itself:

    x <- x + norm1(mixer(x));   x <- x + norm2(ff(x))          norm: y / sqrt(mean y^2 + eps) * w;  logits = head norm(x) * logit_scale

    mixer "attention": grouped-query attention.  q and k each pass an RMS norm over their whole projection (all heads at once, weights
        q.norm / k.norm); the first rot.dims dimensions of each head turn as pairs (i, i + dims/2) by p * f_i, f_i = base^(-2i/dims) rescaled by
        wavelength l = 2 pi / f (rot.scaling: kept where l < original/high, f / factor where l > original/low, blended linearly in
        original / l between); scores q.k * scale are mixed across heads, s_h <- sum_g talk[h, g] s_g; query i sees key j <= i of its own run of
        mask.size positions; weights exp(s_h) / (exp(sink_h) + sum exp); with v_mix every such layer but the first caches
        v <- (1 - vmix) v + vmix v_first (the first such layer's values of the same token); heads * sigmoid(W_g x); W_o.
    ff "moe": s = sigmoid(W_router x); the `top` largest s are taken; each contributes expert(s_e x) -- the score scales the expert's INPUT --
        with expert(u) = W_down (silu(W_gate u) * W_up u); plus a shared expert of the same form on x.

Muduvik -- x = rms_norm(embed[token]) * embed.norm; every sublayer has a norm on both sides and a per-channel scale, and a layer ends with a
per-layer token input:

    x <- x + ls1 * norm1b(mixer(norm1 x));   x <- x + ls2 * norm2b(ff(norm2 x));   x <- x + rms_norm(W_sp (gelu_tanh(W_sg x) * e)) * side.norm
    e = side.embed[token][i dim : (i + 1) dim] for layer i;   ff(h) = W_down (gelu_tanh(W_gate h) * W_up h);   norm: y / sqrt(mean y^2 + eps) * w

    mixer "attention": differential attention.  q, k (with biases) hold two maps per head, [map 1 | map 2]; each map is RMS-normed over dim with one
        [dim] weight, rotated on its first rot.dims dimensions (pairs (2i, 2i+1), frequencies rescaled by wavelength as in Lovulix), and is a softmax
        attention of its own over keys j with 0 <= i - j < mask.size and the head group's shared values; o = a1 - lambda a2 with
        lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff, o / rms(o) * (1 - diff), times one sigmoid gate per head; W_o.
    mixer "latent_attention": as Zefapel's without a rotated part and without a gate.
    mixer "retention": q, k, v per head, q and k rotated (pairs (i, i + dims/2)), k * dim^-1/2;  S <- decay_h S + k v^T;  o = S^T q;
        o / rms(o) * silu(W_g h); W_o.
    loop {start, stop, times}: as Fonapel's, entered by x <- x + step[t] alone.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable

import torch

__all__ = ["LayerSpec", "LayerListConfig", "FAMILIES", "fonapel_config", "zefapel_config", "lovulix_config", "muduvik_config", "pack_layer_list"]


@dataclass
class LayerSpec:
    kind: str                       # "attention" | "delta" | "linrec" | "latent"
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    ff: int = 0                     # 0: no feed-forward
    ff_act: str = "gelu_erf"
    # attention
    rot_dims: int = 0
    rot_base: float = 10000.0
    scale: float = 1.0
    qk_unit_rms: bool = False
    sink: bool = False
    gated: bool = False
    # delta
    conv_taps: int = 0
    unit_eps: float = 1e-6
    # feed-forward: "plain" W_down act(W_up h) | "gated" W_down (act(W_gate h) * W_up h) | "moe"
    ff_kind: str = "plain"
    experts: int = 0
    identity: int = 0               # identity experts behind the real ones in the router's output
    top: int = 0
    groups: int = 1
    keep: int = 1
    expert_ff: int = 0
    shared_ff: int = 0
    # linrec: "channel" (a decay per key channel, rank-`a_rank` projection pair, temperature tau) | "expgate" (capped exponential gates)
    rec_kind: str = "channel"
    gate_cap: float = 0.0
    tau: float = 1.0
    a_rank: int = 0
    # latent attention
    q_rank: int = 0
    kv_rank: int = 0
    rot_dim: int = 0
    kv_from: int = -1               # layer whose latent cache is read; -1: the layer's own
    rot_scaling: tuple[float, float, float, float] | None = None  # (factor, original, fast, slow)
    # attention, further options
    qk_norm: bool = False           # weighted RMS norm over the whole q / k projection before the rotation (tensors mix.q.norm / mix.k.norm)
    rot_half: bool = False          # rotation pairs (i, i + rot_dims/2) instead of (2i, 2i+1)
    rot_scaling_kind: str = "index" # "index": rot_scaling by dimension index | "wavelength": (factor, original, high, low) by wavelength
    talk: bool = False              # scores mixed across heads before the softmax (tensor mix.talk [heads, heads])
    learned_sink: bool = False      # the sink's logit is a tensor (mix.sink [heads]) instead of 0
    chunk: int = 0                  # > 0: chunked causal mask
    v_mix: str = "none"             # "first": keeps its values for later layers | "blend": v <- (1 - l) v + l v_first (tensor mix.vmix)
    # mixture of experts, further options
    router: str = "softmax"         # "softmax" | "sigmoid"
    moe_gated: bool = False         # experts W_down (act(W_gate h) * W_up h)
    moe_scale_input: bool = False   # the router's weight multiplies the expert's input
    moe_shared_sg: bool = True      # the shared expert is scaled by sigmoid of a scalar projection
    moe_correction: bool = True     # a selection-only correction vector (tensor mlp.correction)
    # attention, further options (2)
    bias: bool = False              # q, k, v carry biases (tensors mix.q.b / mix.k.b / mix.v.b)
    window: int = 0                 # > 0: sliding window (a query sees itself and the window - 1 keys before it)
    qk_head_norm: bool = False      # RMS norm per head (and map) over dim ahead of the rotation (tensors mix.q.norm / mix.k.norm [dim])
    diff: float | None = None       # differential attention: two maps per head, lambda from mix.lq1 / lk1 / lq2 / lk2 and this constant
    head_gate: bool = False         # gated: one gate number per head (tensor mix.g [heads, width])
    # linrec "fixed": a constant decay per head
    decay: tuple[float, ...] = ()
    out_norm_weight: bool = True    # linrec: the read-out's unit-RMS norm has a weight (tensor mix.norm)


@dataclass
class LayerListConfig:
    family: str
    width: int
    vocab: int
    norm_eps: float
    residual_mult: float
    layers: list[LayerSpec]
    norm_offset: float = 1.0        # norm weights stored around zero are applied as (1 + w)
    loop: tuple[int, int, int] | None = None  # (start, stop, times)
    norm_kind: str = "rms"          # "rms" | "dyt" (tanh(alpha x) w + b: tensors <name>, <name>.alpha, <name>.b)
    block: str = "parallel"         # "parallel": x += m (mixer(h) + ff(h)), one norm | "sequential": two norms, two residual sums
                                    # | "postnorm": x += m norm1(mixer(x)); x += m norm2(ff(x))
    layer_scale: bool = False       # sequential block: per-channel vectors ls1 / ls2 on the branches
    embed_scale: float = 1.0
    logit_scale: float = 1.0
    embed_norm: bool = False        # the embedding output passes the model's norm (tensor embed.norm)
    loop_projection: bool = True    # a loop pass is entered through loop.in [width, 2 width]; False: only loop.step is added
    side_dim: int = 0               # > 0: per-layer token input of this many columns a layer (tensors side.embed, <layer>.side.*)
    prefix: Callable[[int], str] = field(default=lambda i: f"l{i}.")

    @property
    def layer_runs(self) -> int:
        if not self.loop:
            return len(self.layers)
        start, stop, times = self.loop
        return len(self.layers) + (stop - start) * (times - 1)


def fonapel_config(config: dict) -> LayerListConfig:
    """config.json of a Fonapel checkpoint -> LayerListConfig.  Every size comes from the file."""
    for key in ("layers", "norm", "residual_mult", "vocab", "width"):
        if key not in config:
            raise ValueError(f"config.json lacks {key!r}")
    layers = []
    for i, entry in enumerate(config["layers"]):
        kind, mc, mlp = entry.get("type"), entry.get("mixer") or {}, entry.get("mlp")
        ff = 0
        if mlp is not None:
            if mlp.get("kind", "dense") != "dense":
                raise ValueError(f"layer {i}: unsupported mlp.kind={mlp.get('kind')!r} (dense only)")
            ff = int(mlp["ff"])
        common = dict(heads=int(mc["heads"]), kv_heads=int(mc["kv_heads"]), dim=int(mc["dim"]), vdim=int(mc["vdim"]), ff=ff)
        if kind == "attention":
            rot = mc.get("rot") or {}
            layers.append(LayerSpec(kind="attention", rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)),
                                    scale=float(mc["scale"]), qk_unit_rms=True, sink=True, gated=True, **common))
        elif kind == "delta":
            layers.append(LayerSpec(kind="delta", conv_taps=int(mc["conv"]), unit_eps=1e-6, **common))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
    loop = None
    lp = config.get("loop")
    if lp:
        loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"]))
        if not (0 <= loop[0] < loop[1] <= len(layers)) or loop[2] < 1:
            raise ValueError(f"loop {lp!r} does not fit {len(layers)} layers")
    return LayerListConfig(family="Fonapel", width=int(config["width"]), vocab=int(config["vocab"]),
                           norm_eps=float(config["norm"]["eps"]), residual_mult=float(config["residual_mult"]),
                           layers=layers, norm_offset=1.0, loop=loop)


def _fonapel_tensor_shapes(cfg: LayerListConfig) -> dict[str, tuple[int, ...]]:
    """Every tensor a Fonapel checkpoint must hold, with its shape (the loader checks the file against this)."""
    W = cfg.width
    want: dict[str, tuple[int, ...]] = {"embed": (cfg.vocab, W), "final.norm": (W,), "head": (cfg.vocab, W)}
    if cfg.loop:
        want["loop.in"] = (W, 2 * W)
        want["loop.step"] = (cfg.loop[2], W)
    for i, L in enumerate(cfg.layers):
        p = cfg.prefix(i)
        want[p + "norm1"] = (W,)
        hv = L.heads * L.vdim
        if L.kind == "attention":
            want.update({p + "mix.q": (L.heads * L.dim, W), p + "mix.k": (L.kv_heads * L.dim, W), p + "mix.v": (L.kv_heads * L.vdim, W),
                         p + "mix.g": (hv, W), p + "mix.o": (W, hv)})
        else:
            qk = L.kv_heads * L.dim
            want.update({p + "mix.q": (qk, W), p + "mix.k": (qk, W), p + "mix.v": (hv, W), p + "mix.g": (hv, W), p + "mix.o": (W, hv),
                         p + "mix.q.conv": (qk, L.conv_taps), p + "mix.k.conv": (qk, L.conv_taps), p + "mix.v.conv": (hv, L.conv_taps),
                         p + "mix.a": (L.heads, W), p + "mix.b": (L.heads, W), p + "mix.A_log": (L.heads,), p + "mix.dt_bias": (L.heads,),
                         p + "mix.norm": (L.vdim,)})
        if L.ff:
            want.update({p + "mlp.up": (L.ff, W), p + "mlp.down": (W, L.ff)})
    return want


def zefapel_config(config: dict) -> LayerListConfig:
    """config.json of a Zefapel checkpoint -> LayerListConfig.  Every size and every constant the file gives is read from it."""
    for key in ("layers", "norm", "embedding", "vocab", "width"):
        if key not in config:
            raise ValueError(f"config.json lacks {key!r}")
    layers = []
    for i, entry in enumerate(config["layers"]):
        kind, mc, mlp = entry.get("type"), entry.get("mixer") or {}, entry.get("mlp")
        ff: dict[str, Any] = {}
        if mlp is not None:
            if mlp.get("kind") == "dense":
                ff = dict(ff=int(mlp["ff"]), ff_kind="gated", ff_act="silu")
            elif mlp.get("kind") == "moe":
                r, shared = mlp["router"], mlp.get("shared")
                experts, expert_ff = int(r["experts"]), int(mlp["expert"]["ff"])
                shared_ff = int(shared["ff"]) if shared else 0
                groups = r.get("groups") or {"count": 1, "keep": 1}
                ff = dict(ff=shared_ff + experts * expert_ff, ff_kind="moe", ff_act="relu2", experts=experts, identity=int(r.get("identity", 0)),
                          top=int(r["top"]), groups=int(groups["count"]), keep=int(groups["keep"]), expert_ff=expert_ff, shared_ff=shared_ff)
                if (experts + ff["identity"]) % ff["groups"]:
                    raise ValueError(f"layer {i}: {experts} + {ff['identity']} router outputs do not form {ff['groups']} equal groups")
            else:
                raise ValueError(f"layer {i}: unsupported mlp.kind={mlp.get('kind')!r}")
        heads, dim, vdim = int(mc["heads"]), int(mc["dim"]), int(mc["vdim"])
        if kind == "mlstm":
            layers.append(LayerSpec(kind="linrec", rec_kind="expgate", heads=heads, kv_heads=heads, dim=dim, vdim=vdim, gate_cap=float(mc["gate_cap"]), **ff))
        elif kind == "gla":
            layers.append(LayerSpec(kind="linrec", rec_kind="channel", heads=heads, kv_heads=heads, dim=dim, vdim=vdim, tau=float(mc["tau"]),
                                    a_rank=-1, **ff))  # the rank is the first projection's row count: taken from the tensor
        elif kind == "latent_attention":
            rot, sc = mc.get("rot") or {}, None
            if rot.get("scaling"):
                g = rot["scaling"]
                sc = (float(g["factor"]), float(g["original"]), float(g["fast"]), float(g["slow"]))
            kv_from = int(mc["kv_from"]) if mc.get("kv_from") is not None else -1
            if kv_from >= i or kv_from < -1:
                raise ValueError(f"layer {i}: kv_from={kv_from} must name an earlier layer")
            layers.append(LayerSpec(kind="latent", heads=heads, kv_heads=1, dim=dim, vdim=vdim, q_rank=int(mc["q_rank"]), kv_rank=int(mc["kv_rank"]),
                                    rot_dim=int(mc["rot_dim"]), rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)),
                                    rot_scaling=sc, scale=float(mc["scale"]), gated=True, kv_from=kv_from, **ff))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
    return LayerListConfig(family="Zefapel", width=int(config["width"]), vocab=int(config["vocab"]), norm_eps=float(config["norm"]["eps"]),
                           residual_mult=1.0, layers=layers, norm_offset=0.0, norm_kind="dyt", block="sequential", layer_scale=True,
                           embed_scale=float(config["embedding"]["scale"]))


def lovulix_config(config: dict) -> LayerListConfig:
    """config.json of a Lovulix checkpoint -> LayerListConfig.  Every size and every constant the file gives is read from it."""
    for key in ("layers", "norm", "logit_scale", "vocab", "width"):
        if key not in config:
            raise ValueError(f"config.json lacks {key!r}")
    layers, first_mix = [], True
    for i, entry in enumerate(config["layers"]):
        kind, mc, mlp = entry.get("type"), entry.get("mixer") or {}, entry.get("mlp")
        if kind != "attention":
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        ff: dict[str, Any] = {}
        if mlp is not None:
            if mlp.get("kind", "moe") != "moe":
                raise ValueError(f"layer {i}: unsupported mlp.kind={mlp.get('kind')!r}")
            r, shared = mlp["router"], mlp.get("shared")
            experts, expert_ff = int(r["experts"]), int(mlp["expert"]["ff"])
            shared_ff = int(shared["ff"]) if shared else 0
            if not 1 <= int(r["top"]) <= experts:
                raise ValueError(f"layer {i}: top={r['top']} of {experts} experts")
            ff = dict(ff=shared_ff + experts * expert_ff, ff_kind="moe", ff_act="silu", experts=experts, top=int(r["top"]), expert_ff=expert_ff,
                      shared_ff=shared_ff, router="sigmoid", moe_gated=True, moe_scale_input=True, moe_shared_sg=False, moe_correction=False)
        rot, sc = mc.get("rot") or {}, None
        if rot.get("scaling"):
            g = rot["scaling"]
            sc = (float(g["factor"]), float(g["original"]), float(g["high"]), float(g["low"]))
        v_mix = "none"
        if mc.get("v_mix"):
            v_mix, first_mix = ("first" if first_mix else "blend"), False
        mask = mc.get("mask") or {}
        layers.append(LayerSpec(kind="attention", heads=int(mc["heads"]), kv_heads=int(mc["kv_heads"]), dim=int(mc["dim"]), vdim=int(mc["vdim"]),
                                rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)), rot_scaling=sc, rot_scaling_kind="wavelength",
                                rot_half=True, scale=float(mc["scale"]), qk_norm=True, sink=True, learned_sink=True, talk=True, gated=True,
                                chunk=int(mask.get("size", 0)), v_mix=v_mix, **ff))
    return LayerListConfig(family="Lovulix", width=int(config["width"]), vocab=int(config["vocab"]), norm_eps=float(config["norm"]["eps"]),
                           residual_mult=1.0, layers=layers, norm_offset=0.0, block="postnorm", logit_scale=float(config["logit_scale"]))


def _lovulix_tensor_shapes(cfg: LayerListConfig) -> dict[str, tuple[int, ...]]:
    """Every tensor a Lovulix checkpoint must hold, with its shape."""
    W = cfg.width
    want: dict[str, tuple[int, ...]] = {"embed": (cfg.vocab, W), "final.norm": (W,), "head": (cfg.vocab, W)}
    for i, L in enumerate(cfg.layers):
        p, m = cfg.prefix(i), cfg.prefix(i) + "mix."
        hv = L.heads * L.vdim
        want.update({p + "norm1": (W,), m + "q": (L.heads * L.dim, W), m + "k": (L.kv_heads * L.dim, W), m + "v": (L.kv_heads * L.vdim, W),
                     m + "q.norm": (L.heads * L.dim,), m + "k.norm": (L.kv_heads * L.dim,), m + "talk": (L.heads, L.heads), m + "sink": (L.heads,),
                     m + "g": (hv, W), m + "o": (W, hv)})
        if L.v_mix == "blend":  # (the first value-mixing layer's scalar is not read)
            want[m + "vmix"] = ()
        if L.ff:
            f = p + "mlp."
            want.update({p + "norm2": (W,), f + "router": (L.experts, W)})
            for name, n in [(f"e{e}.", L.expert_ff) for e in range(L.experts)] + ([("shared.", L.shared_ff)] if L.shared_ff else []):
                want.update({f + name + "gate": (n, W), f + name + "up": (n, W), f + name + "down": (W, n)})
    return want


def _rot(mc: dict) -> dict[str, Any]:
    """rot {base, dims, scaling {factor, low, high, original}} -> LayerSpec fields (frequencies rescaled by wavelength)."""
    rot = mc.get("rot") or {}
    sc = None
    if rot.get("scaling"):
        g = rot["scaling"]
        sc = (float(g["factor"]), float(g["original"]), float(g["high"]), float(g["low"]))
    return dict(rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)), rot_scaling=sc, rot_scaling_kind="wavelength")


def muduvik_config(config: dict) -> LayerListConfig:
    """config.json of a Muduvik checkpoint -> LayerListConfig.  Every size and every constant the file gives is read from it."""
    for key in ("layers", "norm", "vocab", "width"):
        if key not in config:
            raise ValueError(f"config.json lacks {key!r}")
    layers = []
    for i, entry in enumerate(config["layers"]):
        kind, mc, mlp = entry.get("type"), entry.get("mixer") or {}, entry.get("mlp")
        ff: dict[str, Any] = {}
        if mlp is not None:
            if mlp.get("kind", "dense") != "dense":
                raise ValueError(f"layer {i}: unsupported mlp.kind={mlp.get('kind')!r} (dense only)")
            ff = dict(ff=int(mlp["ff"]), ff_kind="gated", ff_act="gelu_tanh")
        heads, dim, vdim = int(mc["heads"]), int(mc["dim"]), int(mc["vdim"])
        if kind == "attention":
            kv_heads = int(mc.get("kv_heads", heads))
            if heads % kv_heads:
                raise ValueError(f"layer {i}: {heads} heads do not form {kv_heads} equal groups")
            layers.append(LayerSpec(kind="attention", heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=float(mc["scale"]), bias=True,
                                    qk_head_norm=True, diff=float(mc["diff"]), window=int((mc.get("mask") or {}).get("size", 0)), gated=True,
                                    head_gate=True, **_rot(mc), **ff))
        elif kind == "latent_attention":
            layers.append(LayerSpec(kind="latent", heads=heads, kv_heads=1, dim=dim, vdim=vdim, q_rank=int(mc["q_rank"]), kv_rank=int(mc["kv_rank"]),
                                    scale=float(mc["scale"]), gated=False, **ff))
        elif kind == "retention":
            decay = tuple(float(d) for d in mc["decay"])
            if len(decay) != heads:
                raise ValueError(f"layer {i}: {len(decay)} decays for {heads} heads")
            layers.append(LayerSpec(kind="linrec", rec_kind="fixed", heads=heads, kv_heads=heads, dim=dim, vdim=vdim, decay=decay, rot_half=True,
                                    out_norm_weight=False, **_rot(mc), **ff))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
    loop = None
    lp = config.get("loop")
    if lp:
        loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"]))
        if not (0 <= loop[0] < loop[1] <= len(layers)) or loop[2] < 1:
            raise ValueError(f"loop {lp!r} does not fit {len(layers)} layers")
    side = config.get("token_side") or {}
    return LayerListConfig(family="Muduvik", width=int(config["width"]), vocab=int(config["vocab"]), norm_eps=float(config["norm"]["eps"]),
                           residual_mult=1.0, layers=layers, norm_offset=0.0, loop=loop, block="sandwich", layer_scale=True, embed_norm=True,
                           loop_projection=False, side_dim=int(side.get("dim", 0)))


def _muduvik_tensor_shapes(cfg: LayerListConfig) -> dict[str, tuple[int, ...]]:
    """Every tensor a Muduvik checkpoint must hold, with its shape."""
    W, sd = cfg.width, cfg.side_dim
    want: dict[str, tuple[int, ...]] = {"embed": (cfg.vocab, W), "embed.norm": (W,), "final.norm": (W,), "head": (cfg.vocab, W)}
    if cfg.loop:
        want["loop.step"] = (cfg.loop[2], W)
    if sd:
        want["side.embed"] = (cfg.vocab, sd * len(cfg.layers))
    for i, L in enumerate(cfg.layers):
        p, m = cfg.prefix(i), cfg.prefix(i) + "mix."
        hv = L.heads * L.vdim
        want.update({p + "norm1": (W,), p + "norm1b": (W,), p + "ls1": (W,), m + "o": (W, hv)})
        if L.kind == "attention":
            nq, nk, nv = 2 * L.heads * L.dim, 2 * L.kv_heads * L.dim, L.kv_heads * L.vdim
            want.update({m + "q": (nq, W), m + "q.b": (nq,), m + "k": (nk, W), m + "k.b": (nk,), m + "v": (nv, W), m + "v.b": (nv,),
                         m + "q.norm": (L.dim,), m + "k.norm": (L.dim,), m + "lq1": (L.dim,), m + "lk1": (L.dim,), m + "lq2": (L.dim,),
                         m + "lk2": (L.dim,), m + "g": (L.heads, W)})
        elif L.kind == "latent":
            want.update({m + "dq": (L.q_rank, W), m + "dq.norm": (L.q_rank,), m + "uq": (L.heads * L.dim, L.q_rank), m + "dkv": (L.kv_rank, W),
                         m + "dkv.norm": (L.kv_rank,), m + "uk": (L.heads * L.dim, L.kv_rank), m + "uv": (hv, L.kv_rank)})
        else:
            hd = L.heads * L.dim
            want.update({m + "q": (hd, W), m + "k": (hd, W), m + "v": (hv, W), m + "g": (hv, W)})
        if L.ff:
            f = p + "mlp."
            want.update({p + "norm2": (W,), p + "norm2b": (W,), p + "ls2": (W,), f + "gate": (L.ff, W), f + "up": (L.ff, W), f + "down": (W, L.ff)})
        if sd:
            want.update({p + "side.gate": (sd, W), p + "side.proj": (W, sd), p + "side.norm": (W,)})
    return want


def _norm_shapes(cfg: LayerListConfig, name: str) -> dict[str, tuple[int, ...]]:
    if cfg.norm_kind == "dyt":
        return {name: (cfg.width,), name + ".b": (cfg.width,), name + ".alpha": ()}
    return {name: (cfg.width,)}


def _zefapel_tensor_shapes(cfg: LayerListConfig) -> dict[str, Any]:
    """Every tensor a Zefapel checkpoint must hold, with its shape; a dimension of -1 is read from the file (the decay's rank)."""
    W = cfg.width
    want: dict[str, Any] = {"embed": (cfg.vocab, W), "head": (cfg.vocab, W), **_norm_shapes(cfg, "final.norm")}
    for i, L in enumerate(cfg.layers):
        p, m = cfg.prefix(i), cfg.prefix(i) + "mix."
        want.update(_norm_shapes(cfg, p + "norm1"))
        want[p + "ls1"] = (W,)
        hv = L.heads * L.vdim
        want.update({m + "g": (hv, W), m + "o": (W, hv)})
        if L.kind == "linrec":
            want.update({m + "q": (L.heads * L.dim, W), m + "k": (L.heads * L.dim, W), m + "v": (hv, W)})
            if L.rec_kind == "expgate":
                want.update({m + "i": (L.heads, W), m + "i.b": (L.heads,), m + "f": (L.heads, W), m + "f.b": (L.heads,), m + "norm": (hv,)})
            else:
                want.update({m + "a1": (L.a_rank, W), m + "a2": (L.heads * L.dim, L.a_rank), m + "a2.b": (L.heads * L.dim,), m + "norm": (L.vdim,)})
        else:
            want.update({m + "dq": (L.q_rank, W), m + "dq.norm": (L.q_rank,), m + "uq": (L.heads * (L.dim + L.rot_dim), L.q_rank),
                         m + "uk": (L.heads * L.dim, L.kv_rank), m + "uv": (hv, L.kv_rank)})
            if L.kv_from < 0:
                want.update({m + "dkv": (L.kv_rank + L.rot_dim, W), m + "dkv.norm": (L.kv_rank,)})
        if L.ff:
            f = p + "mlp."
            want.update(_norm_shapes(cfg, p + "norm2"))
            want[p + "ls2"] = (W,)
            if L.ff_kind == "gated":
                want.update({f + "gate": (L.ff, W), f + "up": (L.ff, W), f + "down": (W, L.ff)})
            else:
                want.update({f + "router": (L.experts + L.identity, W), f + "correction": (L.experts + L.identity,)})
                for e in range(L.experts):
                    want.update({f + f"e{e}.up": (L.expert_ff, W), f + f"e{e}.down": (W, L.expert_ff)})
                if L.shared_ff:
                    want.update({f + "shared.up": (L.shared_ff, W), f + "shared.down": (W, L.shared_ff), f + "shared.sg": (1, W)})
    return want


# architecture name (config.json) -> (config reader, tensor table)
FAMILIES: dict[str, tuple[Callable[[dict], LayerListConfig], Callable[[LayerListConfig], dict]]] = {
    "Fonapel": (fonapel_config, _fonapel_tensor_shapes),
    "Zefapel": (zefapel_config, _zefapel_tensor_shapes),
    "Lovulix": (lovulix_config, _lovulix_tensor_shapes),
    "Muduvik": (muduvik_config, _muduvik_tensor_shapes),
}


def pack_layer_list(cfg: LayerListConfig, tensors: dict[str, torch.Tensor], dtype: torch.dtype, device: Any) -> dict:
    """The engine's weight layout from a family's named tensors: per layer one input matrix (every projection that reads the
    normed input, rows concatenated in the order include/tinyllm_hybrid.h lists per mixer kind) and one output matrix; in the
    parallel block the feed-forward's rows / columns are appended to them, in the sequential block it has a pair of its own
    (``w_in2`` / ``w_out2``).  Vectors in float32.  Matrices are cast to ``dtype`` (bfloat16 as stored, or float32)."""
    def mat(name):
        return tensors[name].to(device=device, dtype=dtype)

    def vec(name):
        return tensors[name].to(device=device, dtype=torch.float32).contiguous()

    def norm(entry, key, name):
        entry[key] = vec(name)
        if cfg.norm_kind == "dyt":
            entry[key + "_bias"], entry[key + "_alpha"] = vec(name + ".b"), float(tensors[name + ".alpha"].float())

    packed: dict[str, Any] = {"embed": mat("embed").contiguous(), "head": mat("head").contiguous(), "layers": []}
    norm(packed, "final_norm", "final.norm")
    if cfg.embed_norm:
        packed["embed_norm"] = vec("embed.norm")
    if cfg.side_dim:
        packed["side_embed"] = mat("side.embed").contiguous()
    if cfg.loop:
        if cfg.loop_projection:
            packed["loop_in"] = mat("loop.in").contiguous()
        packed["loop_step"] = vec("loop.step")
    for i, L in enumerate(cfg.layers):
        p = cfg.prefix(i)
        entry: dict[str, Any] = {}
        norm(entry, "norm", p + "norm1")
        if L.kind == "latent":
            rows = [mat(p + "mix.dq")] + ([mat(p + "mix.dkv")] if L.kv_from < 0 else []) + ([mat(p + "mix.g")] if L.gated else [])
            entry["dq_norm"], entry["uq"] = vec(p + "mix.dq.norm"), mat(p + "mix.uq").contiguous()
            if L.kv_from < 0:
                entry["dkv_norm"] = vec(p + "mix.dkv.norm")
            # per head: W_uk transposed ([kv_rank, dim]: the key projection is applied to the query), W_uv as stored ([vdim, kv_rank])
            entry["uk_t"] = mat(p + "mix.uk").reshape(L.heads, L.dim, L.kv_rank).transpose(1, 2).contiguous()
            entry["uv"] = mat(p + "mix.uv").reshape(L.heads, L.vdim, L.kv_rank).contiguous()
        else:
            rows = [mat(p + "mix.q"), mat(p + "mix.k"), mat(p + "mix.v")]
            if L.kind != "attention" or L.gated:
                rows.append(mat(p + "mix.g"))
        if L.kind == "attention":
            if L.qk_norm or L.qk_head_norm:
                entry["q_norm"], entry["k_norm"] = vec(p + "mix.q.norm"), vec(p + "mix.k.norm")
            if L.bias:  # one vector over the mixer's rows of w_in: q | k | v biases, zeros behind them (the gate has none)
                b = torch.cat([vec(p + "mix.q.b"), vec(p + "mix.k.b"), vec(p + "mix.v.b")])
                entry["w_in_bias"] = torch.cat([b, torch.zeros(sum(r.shape[0] for r in rows) - b.numel(), device=device)]).contiguous()
            if L.diff is not None:  # one number for the layer, from four [dim] vectors, in float32
                t32 = lambda name: tensors[p + "mix." + name].to(torch.float32)
                entry["diff_lambda"] = float(torch.exp((t32("lq1") * t32("lk1")).sum()) - torch.exp((t32("lq2") * t32("lk2")).sum()) + torch.tensor(L.diff, dtype=torch.float32))
            if L.talk:
                entry["talk"] = vec(p + "mix.talk")
            if L.learned_sink:
                entry["sink"] = vec(p + "mix.sink")
            if L.v_mix == "blend":
                entry["v_mix_lambda"] = float(tensors[p + "mix.vmix"].float())
        if L.kind == "delta":
            rows += [mat(p + "mix.a"), mat(p + "mix.b")]
            entry["conv"] = torch.cat([vec(p + "mix.q.conv"), vec(p + "mix.k.conv"), vec(p + "mix.v.conv")], 0).contiguous()
            entry["a_log"], entry["dt_bias"], entry["out_norm"] = vec(p + "mix.A_log"), vec(p + "mix.dt_bias"), vec(p + "mix.norm")
        elif L.kind == "linrec":
            if L.out_norm_weight:
                entry["out_norm"] = vec(p + "mix.norm")
            if L.rec_kind == "fixed":
                entry["decay"] = torch.tensor(L.decay, dtype=torch.float32, device=device)
            elif L.rec_kind == "expgate":
                rows += [mat(p + "mix.i"), mat(p + "mix.f")]
                entry["i_bias"], entry["f_bias"] = vec(p + "mix.i.b"), vec(p + "mix.f.b")
            else:
                rows.append(mat(p + "mix.a1"))
                entry["a2"], entry["a2_bias"] = mat(p + "mix.a2").contiguous(), vec(p + "mix.a2.b")
        out = [mat(p + "mix.o")]
        if L.ff:
            f = p + "mlp."
            if L.ff_kind == "plain":
                ff_rows, ff_out = [mat(f + "up")], [mat(f + "down")]
            elif L.ff_kind == "gated":
                ff_rows, ff_out = [mat(f + "gate"), mat(f + "up")], [mat(f + "down")]
            elif L.moe_gated:
                # gates (shared | experts) | ups (shared | experts) | router | [scalar shared gate] | zero rows up to a multiple of 8
                W = cfg.width
                names = (["shared."] if L.shared_ff else []) + [f"e{e}." for e in range(L.experts)]
                ff_rows = [mat(f + n + "gate") for n in names] + [mat(f + n + "up") for n in names] + [mat(f + "router")]
                if L.moe_shared_sg:
                    ff_rows.append(mat(f + "shared.sg") if L.shared_ff else torch.zeros(1, W, device=device, dtype=dtype))
                pad = -sum(r.shape[0] for r in ff_rows) % 8
                if pad:
                    ff_rows.append(torch.zeros(pad, W, device=device, dtype=dtype))
                ff_out = [mat(f + n + "down") for n in names]
                if L.moe_correction:
                    entry["correction"] = vec(f + "correction")
            else:
                W = cfg.width
                shared = [mat(f + "shared.up")] if L.shared_ff else []
                sg = mat(f + "shared.sg") if L.shared_ff else torch.zeros(1, W, device=device, dtype=dtype)
                ff_rows = shared + [mat(f + f"e{e}.up") for e in range(L.experts)] + [mat(f + "router"), sg]
                pad = -sum(r.shape[0] for r in ff_rows) % 8  # the engine's row count of this matrix is a multiple of 8
                if pad:
                    ff_rows.append(torch.zeros(pad, W, device=device, dtype=dtype))
                ff_out = ([mat(f + "shared.down")] if L.shared_ff else []) + [mat(f + f"e{e}.down") for e in range(L.experts)]
                entry["correction"] = vec(f + "correction")
            if cfg.block == "parallel":
                rows, out = rows + ff_rows, out + ff_out
            else:
                norm(entry, "norm2", p + "norm2")
                if cfg.block == "sandwich":
                    entry["post_norm2"] = vec(p + "norm2b")
                entry["w_in2"], entry["w_out2"] = torch.cat(ff_rows, 0).contiguous(), torch.cat(ff_out, 1).contiguous()
        if cfg.block == "sandwich":
            entry["post_norm"] = vec(p + "norm1b")
        if cfg.side_dim:
            entry["side_gate"], entry["side_proj"], entry["side_norm"] = mat(p + "side.gate").contiguous(), mat(p + "side.proj").contiguous(), vec(p + "side.norm")
        if cfg.layer_scale:
            entry["ls1"] = vec(p + "ls1")
            if L.ff:
                entry["ls2"] = vec(p + "ls2")
        entry["w_in"] = torch.cat(rows, 0).contiguous()
        entry["w_out"] = torch.cat(out, 1).contiguous()
        packed["layers"].append(entry)
    return packed
