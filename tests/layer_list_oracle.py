"""Plain float64 numpy restatement of the layer-list mechanisms, one function per mechanism, token by token where the
mechanism is a recurrence.  Shares nothing with the product: it works on a dict of named arrays and a plain config dict of a
family's checkpoint format (Fonapel first, Zefapel below), and always processes a whole sequence from position 0.  Test infrastructure only.
"""

from __future__ import annotations

import math

import numpy as np


def rms_norm(x, weight, eps, offset=0.0):
    """x / sqrt(mean x^2 + eps) * (offset + weight) over the last axis (weight None: no weight)."""
    y = x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    return y if weight is None else y * (offset + weight)


def rotate_pairs(z, positions, dims, base):
    """z [L, heads, dim]: dimensions (2i, 2i+1), i < dims/2, turn by positions * base^(-2i/dims); the rest pass."""
    out = z.copy()
    for i in range(dims // 2):
        ang = positions * base ** (-2.0 * i / dims)
        c, s = np.cos(ang)[:, None], np.sin(ang)[:, None]
        u, v = z[..., 2 * i], z[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def sink_attention(q, k, v, scale, sink=True):
    """q [L, H, D], k [L, G, D], v [L, G, V]; causal; weights exp(s) / (sink + sum exp(s)).  Row by row, key by key."""
    L, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((L, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        for i in range(L):
            s = (k[: i + 1, g] @ q[i, h]) * scale
            e = np.exp(s)
            out[i, h] = (e / ((1.0 if sink else 0.0) + e.sum())) @ v[: i + 1, g]
    return out


def short_conv_silu(z, w):
    """z [L, C], w [C, taps] (last column multiplies the current token); zeros before the start; then SiLU."""
    L, C = z.shape
    taps = w.shape[1]
    out = np.zeros_like(z)
    for t in range(L):
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                out[t] += w[:, j] * z[src]
    return out / (1.0 + np.exp(-out))


def gated_delta_rule(q, k, v, beta, g):
    """q, k [L, G, D] (already unit / scaled), v [L, H, V], beta, g [L, H].  Per head, token by token:
    S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q."""
    L, H, V = v.shape
    G, D = q.shape[1], q.shape[2]
    out = np.zeros((L, H, V))
    for h in range(H):
        kh = h // (H // G)
        S = np.zeros((D, V))
        for t in range(L):
            S = g[t, h] * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, kh])
            S = S + np.outer(k[t, kh], u)
            out[t, h] = S.T @ q[t, kh]
    return out


def gelu_erf(z):
    return 0.5 * z * (1.0 + np.vectorize(math.erf)(z / math.sqrt(2.0)))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.log1p(np.exp(-np.abs(z))) + np.maximum(z, 0.0)


def layer_runs(config):
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    runs = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        runs += [(i, t) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, None) for i in range(loop["stop"], n)]


def fonapel_forward(config, W, tokens, streams=None):
    """Logits [L, vocab] of a whole sequence; ``streams`` (a list) receives the residual stream after every layer run."""
    W = {k: np.asarray(v, dtype=np.float64) for k, v in W.items()}
    eps, m = config["norm"]["eps"], config["residual_mult"]
    L = len(tokens)
    pos = np.arange(L, dtype=np.float64)
    x0 = W["embed"][np.asarray(tokens)]
    x = x0
    for i, t in layer_runs(config):
        spec, p = config["layers"][i], f"l{i}."
        mc = spec["mixer"]
        if t is not None and i == config["loop"]["start"]:
            x = np.concatenate([x, x0], -1) @ W["loop.in"].T + W["loop.step"][t]
        h = rms_norm(x, W[p + "norm1"], eps, offset=1.0)
        H, G, D, V = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
        if spec["type"] == "attention":
            q = (h @ W[p + "mix.q"].T).reshape(L, H, D)
            k = (h @ W[p + "mix.k"].T).reshape(L, G, D)
            v = (h @ W[p + "mix.v"].T).reshape(L, G, V)
            rot = mc.get("rot") or {"dims": 0, "base": 1.0}
            q = rms_norm(rotate_pairs(q, pos, rot["dims"], rot["base"]), None, eps)
            k = rms_norm(rotate_pairs(k, pos, rot["dims"], rot["base"]), None, eps)
            o = sink_attention(q, k, v, mc["scale"]).reshape(L, H * V) * sigmoid(h @ W[p + "mix.g"].T)
        else:
            q = short_conv_silu(h @ W[p + "mix.q"].T, W[p + "mix.q.conv"]).reshape(L, G, D)
            k = short_conv_silu(h @ W[p + "mix.k"].T, W[p + "mix.k.conv"]).reshape(L, G, D)
            v = short_conv_silu(h @ W[p + "mix.v"].T, W[p + "mix.v.conv"]).reshape(L, H, V)
            q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * D ** -0.5
            k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
            beta = sigmoid(h @ W[p + "mix.b"].T)
            g = np.exp(-np.exp(W[p + "mix.A_log"]) * softplus(h @ W[p + "mix.a"].T + W[p + "mix.dt_bias"]))
            o = rms_norm(gated_delta_rule(q, k, v, beta, g), W[p + "mix.norm"], eps)
            o = o.reshape(L, H * V) * silu(h @ W[p + "mix.g"].T)
        y = o @ W[p + "mix.o"].T
        if spec.get("mlp"):
            y = y + gelu_erf(h @ W[p + "mlp.up"].T) @ W[p + "mlp.down"].T
        x = x + m * y
        if streams is not None:
            streams.append(x.copy())
    return rms_norm(x, W["final.norm"], eps, offset=1.0) @ W["head"].T


def make_fonapel_weights(config, seed=0, sigma=None):
    """Random bf16-representable weights by tensor name (float32 arrays) for a Fonapel config dict."""
    import torch

    gen = torch.Generator().manual_seed(seed)
    Wd, out = config["width"], {}

    def mat(rows, cols, scale=None):
        s = scale if scale is not None else (sigma if sigma is not None else cols ** -0.5)
        return (torch.randn(rows, cols, generator=gen) * s).to(torch.bfloat16).float().numpy()

    def vec(n, scale=0.1, shift=0.0):
        return (torch.randn(n, generator=gen) * scale + shift).to(torch.bfloat16).float().numpy()

    out["embed"], out["head"], out["final.norm"] = mat(config["vocab"], Wd, 1.0), mat(config["vocab"], Wd), vec(Wd)
    if config.get("loop"):
        out["loop.in"], out["loop.step"] = mat(Wd, 2 * Wd), mat(config["loop"]["times"], Wd, 0.1)
    for i, spec in enumerate(config["layers"]):
        p, mc = f"l{i}.", spec["mixer"]
        H, G, D, V = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
        out[p + "norm1"] = vec(Wd)
        if spec["type"] == "attention":
            out[p + "mix.q"], out[p + "mix.k"], out[p + "mix.v"] = mat(H * D, Wd), mat(G * D, Wd), mat(G * V, Wd)
        else:
            out[p + "mix.q"], out[p + "mix.k"], out[p + "mix.v"] = mat(G * D, Wd), mat(G * D, Wd), mat(H * V, Wd)
            for n, c in (("q", G * D), ("k", G * D), ("v", H * V)):
                out[p + f"mix.{n}.conv"] = mat(c, mc["conv"], 0.5)
            out[p + "mix.a"], out[p + "mix.b"] = mat(H, Wd), mat(H, Wd)
            out[p + "mix.A_log"], out[p + "mix.dt_bias"], out[p + "mix.norm"] = vec(H, 0.5), vec(H, 0.5), vec(V, 0.1, 1.0)
        out[p + "mix.g"], out[p + "mix.o"] = mat(H * V, Wd), mat(Wd, H * V)
        if spec.get("mlp"):
            out[p + "mlp.up"], out[p + "mlp.down"] = mat(spec["mlp"]["ff"], Wd), mat(Wd, spec["mlp"]["ff"])
    return out


def attention_layer(heads=4, kv_heads=2, dim=32, vdim=16, rot_dims=8, base=10000.0, scale=None, ff=64):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                                           "rot": {"dims": rot_dims, "base": base}, "scale": scale if scale is not None else dim ** -0.5},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def delta_layer(heads=4, kv_heads=2, dim=16, vdim=24, conv=3, ff=64):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def fonapel_config(layers, width=64, vocab=101, loop=None, eps=1e-5, residual_mult=0.5):
    cfg = {"architecture": "Fonapel", "layers": layers, "norm": {"eps": eps}, "residual_mult": residual_mult, "vocab": vocab, "width": width}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


# ---- Zefapel: sequential pre-norm layers (Dynamic Tanh norms, layer scale), mixers "mlstm" / "gla" / "latent_attention", dense or
# ---- mixture-of-experts feed-forward.  Same conventions: float64, whole sequences, one function per mechanism. -------------------

def dyt_norm(x, alpha, weight, bias):
    """tanh(alpha x) * weight + bias (no statistics of x)."""
    return np.tanh(alpha * x) * weight + bias


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def log_sigmoid(z):
    return -softplus(-z)


def scaled_frequencies(dims, base, scaling=None):
    """Rotation frequencies f_i = base^(-2i/dims), i < dims/2, and the factor on cos / sin.  With ``scaling`` (factor, original,
    fast, slow): dimensions that turn fewer than `slow` times over `original` positions are slowed by `factor`, those that turn
    more than `fast` times are kept, a linear ramp in between; cos and sin grow by 0.1 ln(factor) + 1."""
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    if not scaling:
        return f, 1.0

    def where(turns):
        return dims * math.log(scaling["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(where(scaling["fast"])), 0)
    hi = min(math.ceil(where(scaling["slow"])), dims - 1)
    ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / scaling["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(scaling["factor"]) + 1.0


def rotate_pairs_by(z, positions, freqs, mult=1.0):
    """z [L, ..., >= 2 len(freqs)]: the pair (2i, 2i+1) at position p turns by p * freqs[i]; cos and sin times ``mult``."""
    out = z.copy()
    for i, f in enumerate(freqs):
        shape = (-1,) + (1,) * (z.ndim - 2)
        c, s = (np.cos(positions * f) * mult).reshape(shape), (np.sin(positions * f) * mult).reshape(shape)
        u, v = z[..., 2 * i], z[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def matrix_memory(q, k, v, log_i, log_f):
    """mLSTM cell.  q, k [L, H, D] (q already scaled), v [L, H, V], log_i / log_f [L, H] (log input and forget gates).  Per head,
    with a running maximum m that starts at 0:  m' = max(f + m, i);  S <- e^(f + m - m') S + e^(i - m') k v^T;  n likewise with k;
    o = S^T q / (max(|n.q|, e^(-m')) + 1e-6)."""
    L, H, V = v.shape
    D = q.shape[2]
    out = np.zeros((L, H, V))
    for h in range(H):
        S, n, m = np.zeros((D, V)), np.zeros(D), 0.0
        for t in range(L):
            m_new = max(log_f[t, h] + m, log_i[t, h])
            a, b = math.exp(log_f[t, h] + m - m_new), math.exp(log_i[t, h] - m_new)
            S = a * S + b * np.outer(k[t, h], v[t, h])
            n = a * n + b * k[t, h]
            m = m_new
            out[t, h] = S.T @ q[t, h] / (max(abs(n @ q[t, h]), math.exp(-m)) + 1e-6)
    return out


def gated_linear_attention(q, k, v, alpha):
    """q, k, alpha [L, H, D], v [L, H, V].  Per head: S <- diag(alpha_t) S + k_t v_t^T;  o_t = S^T q_t."""
    L, H, V = v.shape
    D = q.shape[2]
    out = np.zeros((L, H, V))
    for h in range(H):
        S = np.zeros((D, V))
        for t in range(L):
            S = alpha[t, h][:, None] * S + np.outer(k[t, h], v[t, h])
            out[t, h] = S.T @ q[t, h]
    return out


def causal_softmax_attention(q, k, v, scale):
    """q [L, H, D], k [L, H, D], v [L, H, V]: row i sees keys j <= i; ordinary softmax."""
    L, H, _ = q.shape
    out = np.zeros((L, H, v.shape[2]))
    for h in range(H):
        for i in range(L):
            s = (k[: i + 1, h] @ q[i, h]) * scale
            e = np.exp(s - s.max())
            out[i, h] = (e / e.sum()) @ v[: i + 1, h]
    return out


def route(z, correction, top, groups, keep):
    """z [E] router logits.  Scores s = softmax(z); choice = s + correction; only experts of the `keep` groups (of `groups`
    equal runs of neighbours) with the largest group maximum of choice can be taken; the `top` largest choices win; weights are
    their s.  Returns {expert: weight}."""
    e = np.exp(z - z.max())
    s = e / e.sum()
    choice = s + correction
    E = len(z)
    per = E // groups
    gmax = [choice[g * per:(g + 1) * per].max() for g in range(groups)]
    kept = sorted(range(groups), key=lambda g: (-gmax[g], g))[:keep]
    allowed = [j for j in range(E) if j // per in kept]
    chosen = sorted(allowed, key=lambda j: (-choice[j], j))[:top]
    return {j: s[j] for j in chosen}


def relu2(z):
    return np.maximum(z, 0.0) ** 2


def zefapel_feed_forward(mlp, W, p, h):
    if mlp["kind"] == "dense":
        return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T
    r = mlp["router"]
    E, I = r["experts"], r.get("identity", 0)
    out = np.zeros_like(h)
    zs = h @ W[p + "router"].T
    for t in range(h.shape[0]):
        for j, w in route(zs[t], W[p + "correction"], r["top"], r["groups"]["count"], r["groups"]["keep"]).items():
            if j >= E:
                out[t] += w * h[t]
            else:
                out[t] += w * (relu2(h[t] @ W[p + f"e{j}.up"].T) @ W[p + f"e{j}.down"].T)
    if mlp.get("shared"):
        shared = relu2(h @ W[p + "shared.up"].T) @ W[p + "shared.down"].T
        out = out + shared * sigmoid(h @ W[p + "shared.sg"].T)
    return out


def zefapel_forward(config, W, tokens, streams=None):
    """Logits [L, vocab] of a whole sequence; ``streams`` (a list) receives the residual stream after every layer."""
    W = {k: np.asarray(v, dtype=np.float64) for k, v in W.items()}
    eps = config["norm"]["eps"]
    L = len(tokens)
    pos = np.arange(L, dtype=np.float64)
    x = W["embed"][np.asarray(tokens)] * config["embedding"]["scale"]
    latents = {}
    for i, spec in enumerate(config["layers"]):
        p, mc = f"l{i}.", spec["mixer"]
        h = dyt_norm(x, W[p + "norm1.alpha"], W[p + "norm1"], W[p + "norm1.b"])
        H, D, V = mc["heads"], mc["dim"], mc["vdim"]
        m = p + "mix."
        if spec["type"] == "mlstm":
            q = (h @ W[m + "q"].T).reshape(L, H, D) * D ** -0.5
            k = (h @ W[m + "k"].T).reshape(L, H, D)
            v = (h @ W[m + "v"].T).reshape(L, H, V)
            cap = mc["gate_cap"]
            li = cap * np.tanh((h @ W[m + "i"].T + W[m + "i.b"]) / cap)
            lf = log_sigmoid(cap * np.tanh((h @ W[m + "f"].T + W[m + "f.b"]) / cap))
            o = rms_norm(matrix_memory(q, k, v, li, lf), None, eps).reshape(L, H * V) * W[m + "norm"]
            o = o * sigmoid(h @ W[m + "g"].T)
        elif spec["type"] == "gla":
            q = (h @ W[m + "q"].T).reshape(L, H, D) * D ** -0.5
            k = (h @ W[m + "k"].T).reshape(L, H, D)
            v = (h @ W[m + "v"].T).reshape(L, H, V)
            z = (h @ W[m + "a1"].T) @ W[m + "a2"].T + W[m + "a2.b"]
            alpha = np.exp(log_sigmoid(z) / mc["tau"]).reshape(L, H, D)
            o = rms_norm(gated_linear_attention(q, k, v, alpha), W[m + "norm"], eps).reshape(L, H * V)
            o = o * silu(h @ W[m + "g"].T)
        elif spec["type"] == "latent_attention":
            R, C = mc["rot_dim"], mc["kv_rank"]
            freqs, mult = scaled_frequencies(mc["rot"]["dims"], mc["rot"]["base"], mc["rot"].get("scaling"))
            cq = rms_norm(h @ W[m + "dq"].T, W[m + "dq.norm"], eps)
            q = (cq @ W[m + "uq"].T).reshape(L, H, D + R)
            q_rot = rotate_pairs_by(q[..., D:], pos, freqs, mult)
            if "kv_from" in mc:
                c, k_rot = latents[mc["kv_from"]]
            else:
                dkv = h @ W[m + "dkv"].T
                c = rms_norm(dkv[:, :C], W[m + "dkv.norm"], eps)
                k_rot = rotate_pairs_by(dkv[:, C:], pos, freqs, mult)
                latents[i] = (c, k_rot)
            k_plain = (c @ W[m + "uk"].T).reshape(L, H, D)
            val = (c @ W[m + "uv"].T).reshape(L, H, V)
            qq = np.concatenate([q[..., :D], q_rot], -1)
            kk = np.concatenate([k_plain, np.broadcast_to(k_rot[:, None, :], (L, H, R))], -1)
            o = causal_softmax_attention(qq, kk, val, mc["scale"]).reshape(L, H * V) * sigmoid(h @ W[m + "g"].T)
        else:
            raise ValueError(spec["type"])
        x = x + W[p + "ls1"] * (o @ W[m + "o"].T)
        if spec.get("mlp"):
            h2 = dyt_norm(x, W[p + "norm2.alpha"], W[p + "norm2"], W[p + "norm2.b"])
            x = x + W[p + "ls2"] * zefapel_feed_forward(spec["mlp"], W, p + "mlp.", h2)
        if streams is not None:
            streams.append(x.copy())
    xf = dyt_norm(x, W["final.norm.alpha"], W["final.norm"], W["final.norm.b"])
    return xf @ W["head"].T


def make_zefapel_weights(config, seed=0):
    """Random bf16-representable weights by tensor name (float32 arrays) for a Zefapel config dict."""
    import torch

    gen = torch.Generator().manual_seed(seed)
    Wd, out = config["width"], {}

    def mat(rows, cols, scale=None):
        s = scale if scale is not None else cols ** -0.5
        return (torch.randn(rows, cols, generator=gen) * s).to(torch.bfloat16).float().numpy()

    def vec(n, scale=0.1, shift=0.0):
        return (torch.randn(n, generator=gen) * scale + shift).to(torch.bfloat16).float().numpy()

    def norm(name):
        out[name], out[name + ".b"] = vec(Wd, 0.1, 1.0), vec(Wd, 0.05)
        out[name + ".alpha"] = np.float32(vec(1, 0.1, 0.7)[0])

    out["embed"], out["head"] = mat(config["vocab"], Wd, 1.0), mat(config["vocab"], Wd)
    norm("final.norm")
    for i, spec in enumerate(config["layers"]):
        p, m, mc = f"l{i}.", f"l{i}.mix.", spec["mixer"]
        H, D, V = mc["heads"], mc["dim"], mc["vdim"]
        norm(p + "norm1")
        out[p + "ls1"] = vec(Wd, 0.2, 0.8)
        out[m + "g"], out[m + "o"] = mat(H * V, Wd), mat(Wd, H * V)
        if spec["type"] in ("mlstm", "gla"):
            out[m + "q"], out[m + "k"], out[m + "v"] = mat(H * D, Wd), mat(H * D, Wd), mat(H * V, Wd)
            if spec["type"] == "mlstm":
                out[m + "i"], out[m + "f"] = mat(H, Wd, 0.3), mat(H, Wd, 0.3)
                out[m + "i.b"], out[m + "f.b"], out[m + "norm"] = vec(H, 1.0, -1.0), vec(H, 1.0, 3.0), vec(H * V, 0.1, 1.0)
            else:
                r = mc.get("a_rank", 6)
                out[m + "a1"], out[m + "a2"], out[m + "a2.b"] = mat(r, Wd), mat(H * D, r), vec(H * D, 1.0, 1.0)
                out[m + "norm"] = vec(V, 0.1, 1.0)
        else:
            Q, C, R = mc["q_rank"], mc["kv_rank"], mc["rot_dim"]
            out[m + "dq"], out[m + "dq.norm"], out[m + "uq"] = mat(Q, Wd), vec(Q, 0.1, 1.0), mat(H * (D + R), Q)
            out[m + "uk"], out[m + "uv"] = mat(H * D, C), mat(H * V, C)
            if "kv_from" not in mc:
                out[m + "dkv"], out[m + "dkv.norm"] = mat(C + R, Wd), vec(C, 0.1, 1.0)
        mlp = spec.get("mlp")
        if mlp:
            f = p + "mlp."
            norm(p + "norm2")
            out[p + "ls2"] = vec(Wd, 0.2, 0.8)
            if mlp["kind"] == "dense":
                out[f + "gate"], out[f + "up"], out[f + "down"] = mat(mlp["ff"], Wd), mat(mlp["ff"], Wd), mat(Wd, mlp["ff"])
            else:
                r = mlp["router"]
                ET = r["experts"] + r.get("identity", 0)
                out[f + "router"], out[f + "correction"] = mat(ET, Wd, 2.0 * Wd ** -0.5), vec(ET, 0.1)
                for e in range(r["experts"]):
                    out[f + f"e{e}.up"], out[f + f"e{e}.down"] = mat(mlp["expert"]["ff"], Wd), mat(Wd, mlp["expert"]["ff"])
                if mlp.get("shared"):
                    s = mlp["shared"]["ff"]
                    out[f + "shared.up"], out[f + "shared.down"], out[f + "shared.sg"] = mat(s, Wd), mat(Wd, s), mat(1, Wd)
    return out


def dense_ff(ff=72):
    return {"kind": "dense", "ff": ff}


def moe_ff(experts=5, identity=1, top=2, groups=3, keep=2, ff=24, shared=40):
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "identity": identity, "top": top, "groups": {"count": groups, "keep": keep}}}
    if shared:
        mlp["shared"] = {"ff": shared}
    return mlp


def mlstm_layer(heads=3, dim=24, vdim=16, gate_cap=12.0, mlp=None):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": gate_cap}, "mlp": mlp}


def gla_layer(heads=2, dim=16, vdim=24, tau=8.0, a_rank=6, mlp=None):
    """(a_rank is not a key of the checkpoint format: readers take it from the tensor; the weight maker reads it here)"""
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "a_rank": a_rank}, "mlp": mlp}


def latent_layer(heads=4, dim=16, vdim=24, rot_dim=8, q_rank=20, kv_rank=40, base=5000.0, scale=0.2, scaling=(4.0, 64, 16.0, 2.0), kv_from=None, mlp=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling:
        rot["scaling"] = {"factor": scaling[0], "original": scaling[1], "fast": scaling[2], "slow": scaling[3]}
    mixer = {"heads": heads, "dim": dim, "vdim": vdim, "rot_dim": rot_dim, "q_rank": q_rank, "kv_rank": kv_rank, "rot": rot, "scale": scale}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


def zefapel_config(layers, width=64, vocab=101, eps=1e-5, embed_scale=0.7):
    return {"architecture": "Zefapel", "embedding": {"scale": embed_scale}, "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}


# ---- Lovulix: post-norm blocks x += norm1(mixer(x)); x += norm2(ff(x)) -------------------------------------------------------
# mixer: grouped-query attention with an RMS norm over the WHOLE q (and k) projection, rotation of the pairs (i, i + dims/2) with
# wavelength-dependent frequency rescaling, scores mixed across heads before the softmax, a chunked causal mask, a learned sink per
# head in the denominator, values blended with the first such layer's values, a sigmoid output gate.
# ff: experts chosen by the largest sigmoid(router) scores, the score multiplying the expert's INPUT, plus a shared expert.


def wavelength_scaled_frequencies(dims, base, scaling=None):
    """f_i = base^(-2i/dims), i < dims/2.  With ``scaling`` {factor, low, high, original}: by wavelength l = 2 pi / f, f stays where
    l < original/high, becomes f / factor where l > original/low, and between the two is blended with s = (original/l - low) / (high - low):
    (1 - s) f / factor + s f."""
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    if not scaling:
        return f
    out = f.copy()
    fac, lo, hi, orig = scaling["factor"], scaling["low"], scaling["high"], scaling["original"]
    for i, fi in enumerate(f):
        l = 2.0 * math.pi / fi
        if l < orig / hi:
            continue
        if l > orig / lo:
            out[i] = fi / fac
        else:
            s = (orig / l - lo) / (hi - lo)
            out[i] = (1.0 - s) * fi / fac + s * fi
    return out


def rotate_halves_by(z, positions, freqs):
    """z [L, heads, dim]: with n = len(freqs), the pair (i, i + n) at position p turns by p * freqs[i]; dimensions from 2 n on pass."""
    out = z.copy()
    n = len(freqs)
    for i, f in enumerate(freqs):
        c, s = np.cos(positions * f)[:, None], np.sin(positions * f)[:, None]
        u, v = z[..., i], z[..., i + n]
        out[..., i] = u * c - v * s
        out[..., i + n] = v * c + u * s
    return out


def talking_chunk_attention(q, k, v, scale, talk=None, sink=None, chunk=None):
    """q [L, H, D], k [L, G, D], v [L, G, V].  Query i sees key j <= i of its own chunk (floor(i / chunk) == floor(j / chunk); chunk None:
    every j <= i).  Scores q.k * scale of all heads are mixed per (i, j): s'_h = sum_g talk[h, g] s_g.  Weights exp(s'_h) / (exp(sink_h) + sum)
    (sink None: no extra term).  Head h reads the values of K/V head h // (H / G).  Row by row."""
    L, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((L, H, v.shape[2]))
    for i in range(L):
        lo = (i // chunk) * chunk if chunk else 0
        s = np.stack([(k[lo:i + 1, h // (H // G)] @ q[i, h]) * scale for h in range(H)])  # [H, keys]
        if talk is not None:
            s = talk @ s
        for h in range(H):
            e = np.exp(s[h])
            den = e.sum() + (math.exp(sink[h]) if sink is not None else 0.0)
            out[i, h] = (e / den) @ v[lo:i + 1, h // (H // G)]
    return out


def sigmoid_top_route(z, top):
    """Router logits z [E] -> {expert: weight}: the `top` largest sigmoid(z) (ties to the lower index), weight = the score itself."""
    s = sigmoid(z)
    return {j: s[j] for j in sorted(range(len(z)), key=lambda j: (-s[j], j))[:top]}


def gated_expert(W, p, h):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def lovulix_feed_forward(mlp, W, p, h):
    out = np.zeros_like(h)
    zs = h @ W[p + "router"].T
    for t in range(h.shape[0]):
        for j, w in sigmoid_top_route(zs[t], mlp["router"]["top"]).items():
            out[t] += gated_expert(W, p + f"e{j}.", w * h[t])
    if mlp.get("shared"):
        out = out + gated_expert(W, p + "shared.", h)
    return out


def lovulix_forward(config, W, tokens, streams=None):
    """Logits [L, vocab] of a whole sequence; ``streams`` (a list) receives the residual stream after every layer."""
    W = {k: np.asarray(v, dtype=np.float64) for k, v in W.items()}
    eps = config["norm"]["eps"]
    L = len(tokens)
    pos = np.arange(L, dtype=np.float64)
    x = W["embed"][np.asarray(tokens)]
    v_first = None
    for i, spec in enumerate(config["layers"]):
        p, m, mc = f"l{i}.", f"l{i}.mix.", spec["mixer"]
        if spec["type"] != "attention":
            raise ValueError(spec["type"])
        H, G, D, V = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
        q = rms_norm(x @ W[m + "q"].T, W[m + "q.norm"], eps).reshape(L, H, D)
        k = rms_norm(x @ W[m + "k"].T, W[m + "k.norm"], eps).reshape(L, G, D)
        v = (x @ W[m + "v"].T).reshape(L, G, V)
        rot = mc.get("rot")
        if rot and rot.get("dims", 0):
            f = wavelength_scaled_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
            q, k = rotate_halves_by(q, pos, f), rotate_halves_by(k, pos, f)
        if mc.get("v_mix"):
            if v_first is None:
                v_first = v
            else:
                lam = float(W[m + "vmix"])
                v = ((1.0 - lam) * v.reshape(L, G * V) + lam * v_first.reshape(L, -1)).reshape(L, G, V)  # (token by token, the values of all K/V heads side by side)
        mask = mc.get("mask") or {}
        o = talking_chunk_attention(q, k, v, mc["scale"], W[m + "talk"], W[m + "sink"], mask.get("size")).reshape(L, H * V)
        o = o * sigmoid(x @ W[m + "g"].T)
        x = x + rms_norm(o @ W[m + "o"].T, W[p + "norm1"], eps)
        if spec.get("mlp"):
            x = x + rms_norm(lovulix_feed_forward(spec["mlp"], W, p + "mlp.", x), W[p + "norm2"], eps)
        if streams is not None:
            streams.append(x.copy())
    return rms_norm(x, W["final.norm"], eps) @ W["head"].T * config["logit_scale"]


def make_lovulix_weights(config, seed=0):
    """Random bf16-representable weights by tensor name (float32 arrays) for a Lovulix config dict."""
    import torch

    gen = torch.Generator().manual_seed(seed)
    Wd, out = config["width"], {}

    def mat(rows, cols, scale=None):
        s = scale if scale is not None else cols ** -0.5
        return (torch.randn(rows, cols, generator=gen) * s).to(torch.bfloat16).float().numpy()

    def vec(n, scale=0.1, shift=0.0):
        return (torch.randn(n, generator=gen) * scale + shift).to(torch.bfloat16).float().numpy()

    out["embed"], out["head"], out["final.norm"] = mat(config["vocab"], Wd, 1.0), mat(config["vocab"], Wd), vec(Wd, 0.1, 1.0)
    for i, spec in enumerate(config["layers"]):
        p, m, mc = f"l{i}.", f"l{i}.mix.", spec["mixer"]
        H, G, D, V = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
        out[p + "norm1"] = vec(Wd, 0.1, 1.0)
        out[m + "q"], out[m + "k"], out[m + "v"] = mat(H * D, Wd), mat(G * D, Wd), mat(G * V, Wd)
        out[m + "q.norm"], out[m + "k.norm"] = vec(H * D, 0.2, 1.0), vec(G * D, 0.2, 1.0)
        out[m + "vmix"] = np.float32(vec(1, 0.1, 0.4)[0])
        out[m + "talk"] = (np.eye(H, dtype=np.float32) + mat(H, H, 0.3)).astype(np.float32)
        out[m + "talk"] = torch.from_numpy(out[m + "talk"]).to(torch.bfloat16).float().numpy()
        out[m + "sink"] = vec(H, 1.0, 0.5)
        out[m + "g"], out[m + "o"] = mat(H * V, Wd), mat(Wd, H * V)
        mlp = spec.get("mlp")
        if mlp:
            f = p + "mlp."
            out[p + "norm2"] = vec(Wd, 0.1, 1.0)
            out[f + "router"] = mat(mlp["router"]["experts"], Wd, 2.0 * Wd ** -0.5)
            names = [f"e{e}." for e in range(mlp["router"]["experts"])]
            sizes = [mlp["expert"]["ff"]] * len(names)
            if mlp.get("shared"):
                names.append("shared.")
                sizes.append(mlp["shared"]["ff"])
            for name, n in zip(names, sizes):
                out[f + name + "gate"], out[f + name + "up"], out[f + name + "down"] = mat(n, Wd), mat(n, Wd), mat(Wd, n)
    return out


def lovulix_moe(experts=6, top=2, ff=24, shared=40):
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        mlp["shared"] = {"ff": shared}
    return mlp


def lovulix_layer(heads=4, kv_heads=2, dim=16, vdim=24, rot_dims=8, base=5000.0, scaling=(8.0, 1.0, 4.0, 64), scale=0.3, chunk=16, v_mix=True,
                  mlp="default"):
    rot = {"base": base, "dims": rot_dims}
    if scaling:
        rot["scaling"] = {"factor": scaling[0], "low": scaling[1], "high": scaling[2], "original": scaling[3]}
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": rot, "scale": scale, "v_mix": v_mix}
    if chunk:
        mixer["mask"] = {"size": chunk}
    return {"type": "attention", "mixer": mixer, "mlp": lovulix_moe() if mlp == "default" else mlp}


def lovulix_config(layers, width=64, vocab=101, eps=1e-5, logit_scale=0.7):
    return {"architecture": "Lovulix", "layers": layers, "logit_scale": logit_scale, "norm": {"eps": eps}, "vocab": vocab, "width": width}


# ---- Muduvik: x = norm(embed[token]); layers with a norm before AND after each sublayer and per-channel layer scales; a per-layer token
# ---- input behind the feed-forward; a looped range entered by adding a per-pass vector.  Mixers: differential sliding-window attention,
# ---- latent attention without positions, retention.  Same conventions: float64, whole sequences, one function per mechanism. ---------

def window_softmax_attention(q, k, v, scale, window=None):
    """q [L, H, D], k [L, G, D], v [L, G', V] (head h reads key head h // (H/G) and value head h // (H/G')): query i sees keys j with
    0 <= i - j < window (None: every j <= i); ordinary softmax.  Row by row."""
    L, H, _ = q.shape
    G, Gv = k.shape[1], v.shape[1]
    out = np.zeros((L, H, v.shape[2]))
    for h in range(H):
        for i in range(L):
            lo = max(0, i - window + 1) if window else 0
            s = (k[lo:i + 1, h // (H // G)] @ q[i, h]) * scale
            e = np.exp(s - s.max())
            out[i, h] = (e / e.sum()) @ v[lo:i + 1, h // (H // Gv)]
    return out


def differential_combine(a1, a2, lam, diff, eps):
    """a1, a2 [L, H, V]: the two maps' read-outs.  o = a1 - lam a2, divided by its root mean square over V (eps inside the root), times (1 - diff)."""
    o = a1 - lam * a2
    return o / np.sqrt(np.mean(o * o, axis=-1, keepdims=True) + eps) * (1.0 - diff)


def differential_attention(W, m, mc, h, pos, eps):
    """The whole mixer on its input h [L, width] -> [L, width]: two maps per head over shared values, sliding window, per-head gate."""
    L = h.shape[0]
    H, G, D, V = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    q = (h @ W[m + "q"].T + W[m + "q.b"]).reshape(L, H, 2, D)
    k = (h @ W[m + "k"].T + W[m + "k.b"]).reshape(L, G, 2, D)
    v = (h @ W[m + "v"].T + W[m + "v.b"]).reshape(L, G, V)
    q, k = rms_norm(q, W[m + "q.norm"], eps), rms_norm(k, W[m + "k.norm"], eps)
    rot = mc.get("rot")
    if rot and rot.get("dims", 0):
        f = wavelength_scaled_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q = rotate_pairs_by(q.reshape(L, 2 * H, D), pos, f).reshape(L, H, 2, D)
        k = rotate_pairs_by(k.reshape(L, 2 * G, D), pos, f).reshape(L, G, 2, D)
    window = (mc.get("mask") or {}).get("size")
    a = [window_softmax_attention(q[:, :, j], k[:, :, j], v, mc["scale"], window) for j in (0, 1)]
    lam = math.exp(float(W[m + "lq1"] @ W[m + "lk1"])) - math.exp(float(W[m + "lq2"] @ W[m + "lk2"])) + mc["diff"]
    o = differential_combine(a[0], a[1], lam, mc["diff"], eps)
    o = o * sigmoid(h @ W[m + "g"].T)[:, :, None]
    return o.reshape(L, H * V) @ W[m + "o"].T


def latent_attention_plain(W, m, mc, h, eps):
    """Queries through a normed latent; keys and values are per-head projections of one normed latent per token; causal softmax; no positions."""
    L = h.shape[0]
    H, D, V = mc["heads"], mc["dim"], mc["vdim"]
    q = (rms_norm(h @ W[m + "dq"].T, W[m + "dq.norm"], eps) @ W[m + "uq"].T).reshape(L, H, D)
    c = rms_norm(h @ W[m + "dkv"].T, W[m + "dkv.norm"], eps)
    k, v = (c @ W[m + "uk"].T).reshape(L, H, D), (c @ W[m + "uv"].T).reshape(L, H, V)
    return causal_softmax_attention(q, k, v, mc["scale"]).reshape(L, H * V) @ W[m + "o"].T


def retention_states(q, k, v, decay):
    """q, k [L, H, D], v [L, H, V], decay [H].  Per head, token by token, from a zero state: S <- decay S + k v^T;  o = S^T q."""
    L, H, V = v.shape
    D = q.shape[2]
    out = np.zeros((L, H, V))
    for h in range(H):
        S = np.zeros((D, V))
        for t in range(L):
            S = decay[h] * S + np.outer(k[t, h], v[t, h])
            out[t, h] = S.T @ q[t, h]
    return out


def retention(W, m, mc, h, pos, eps):
    L = h.shape[0]
    H, D, V = mc["heads"], mc["dim"], mc["vdim"]
    q, k, v = (h @ W[m + "q"].T).reshape(L, H, D), (h @ W[m + "k"].T).reshape(L, H, D), (h @ W[m + "v"].T).reshape(L, H, V)
    rot = mc.get("rot")
    if rot and rot.get("dims", 0):
        f = wavelength_scaled_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q, k = rotate_halves_by(q, pos, f), rotate_halves_by(k, pos, f)
    o = retention_states(q, k * D ** -0.5, v, np.asarray(mc["decay"], dtype=np.float64))
    o = rms_norm(o, None, eps).reshape(L, H * V) * silu(h @ W[m + "g"].T)
    return o @ W[m + "o"].T


def token_side_input(W, p, x, side_rows, eps):
    """side_rows [L, dim]: the layer's part of the side embedding of each token.  y = W_proj (gelu_tanh(W_gate x) * e); returns rms_norm(y) * norm."""
    y = (gelu_tanh(x @ W[p + "side.gate"].T) * side_rows) @ W[p + "side.proj"].T
    return rms_norm(y, W[p + "side.norm"], eps)


def muduvik_layer_order(config):
    """(layer index, pass or None, first of its pass) for every layer run."""
    n, lp = len(config["layers"]), config.get("loop")
    if not lp:
        return [(i, None, False) for i in range(n)]
    runs = [(i, None, False) for i in range(lp["start"])]
    for t in range(lp["times"]):
        runs += [(i, t, i == lp["start"]) for i in range(lp["start"], lp["stop"])]
    return runs + [(i, None, False) for i in range(lp["stop"], n)]


def muduvik_forward(config, W, tokens, streams=None):
    """Logits [L, vocab] of a whole sequence; ``streams`` (a list) receives the residual stream after every layer run."""
    W = {k: np.asarray(v, dtype=np.float64) for k, v in W.items()}
    eps = config["norm"]["eps"]
    tokens = np.asarray(tokens)
    L = len(tokens)
    pos = np.arange(L, dtype=np.float64)
    x = rms_norm(W["embed"][tokens], W["embed.norm"], eps)
    sd = (config.get("token_side") or {}).get("dim", 0)
    for i, t, first in muduvik_layer_order(config):
        if first:
            x = x + W["loop.step"][t]
        spec = config["layers"][i]
        p, m, mc = f"l{i}.", f"l{i}.mix.", spec["mixer"]
        h = rms_norm(x, W[p + "norm1"], eps)
        if spec["type"] == "attention":
            y = differential_attention(W, m, mc, h, pos, eps)
        elif spec["type"] == "latent_attention":
            y = latent_attention_plain(W, m, mc, h, eps)
        elif spec["type"] == "retention":
            y = retention(W, m, mc, h, pos, eps)
        else:
            raise ValueError(spec["type"])
        x = x + rms_norm(y, W[p + "norm1b"], eps) * W[p + "ls1"]
        if spec.get("mlp"):
            h = rms_norm(x, W[p + "norm2"], eps)
            f = p + "mlp."
            y = (gelu_tanh(h @ W[f + "gate"].T) * (h @ W[f + "up"].T)) @ W[f + "down"].T
            x = x + rms_norm(y, W[p + "norm2b"], eps) * W[p + "ls2"]
        if sd:
            x = x + token_side_input(W, p, x, W["side.embed"][tokens][:, i * sd:(i + 1) * sd], eps)
        if streams is not None:
            streams.append(x.copy())
    return rms_norm(x, W["final.norm"], eps) @ W["head"].T


def make_muduvik_weights(config, seed=0):
    """Random bf16-representable weights by tensor name (float32 arrays) for a Muduvik config dict."""
    import torch

    gen = torch.Generator().manual_seed(seed)
    Wd, out = config["width"], {}

    def mat(rows, cols, scale=None):
        s = scale if scale is not None else cols ** -0.5
        return (torch.randn(rows, cols, generator=gen) * s).to(torch.bfloat16).float().numpy()

    def vec(n, scale=0.1, shift=0.0):
        return (torch.randn(n, generator=gen) * scale + shift).to(torch.bfloat16).float().numpy()

    n_layers, sd = len(config["layers"]), (config.get("token_side") or {}).get("dim", 0)
    out["embed"], out["head"] = mat(config["vocab"], Wd, 1.0), mat(config["vocab"], Wd)
    out["embed.norm"], out["final.norm"] = vec(Wd, 0.1, 1.0), vec(Wd, 0.1, 1.0)
    if config.get("loop"):
        out["loop.step"] = mat(config["loop"]["times"], Wd, 0.5)
    if sd:
        out["side.embed"] = mat(config["vocab"], sd * n_layers, 1.0)
    for i, spec in enumerate(config["layers"]):
        p, m, mc = f"l{i}.", f"l{i}.mix.", spec["mixer"]
        H, D, V = mc["heads"], mc["dim"], mc["vdim"]
        out[p + "norm1"], out[p + "norm1b"], out[p + "ls1"] = vec(Wd, 0.1, 1.0), vec(Wd, 0.1, 1.0), vec(Wd, 0.2, 0.6)
        out[m + "o"] = mat(Wd, H * V)
        if spec["type"] == "attention":
            G = mc["kv_heads"]
            out[m + "q"], out[m + "k"], out[m + "v"] = mat(2 * H * D, Wd), mat(2 * G * D, Wd), mat(G * V, Wd)
            out[m + "q.b"], out[m + "k.b"], out[m + "v.b"] = vec(2 * H * D, 0.3), vec(2 * G * D, 0.3), vec(G * V, 0.3)
            out[m + "q.norm"], out[m + "k.norm"] = vec(D, 0.2, 1.0), vec(D, 0.2, 1.0)
            for name in ("lq1", "lk1", "lq2", "lk2"):
                out[m + name] = vec(D, D ** -0.5)
            out[m + "g"] = mat(H, Wd)
        elif spec["type"] == "latent_attention":
            out[m + "dq"], out[m + "dq.norm"], out[m + "uq"] = mat(mc["q_rank"], Wd), vec(mc["q_rank"], 0.1, 1.0), mat(H * D, mc["q_rank"])
            out[m + "dkv"], out[m + "dkv.norm"] = mat(mc["kv_rank"], Wd), vec(mc["kv_rank"], 0.1, 1.0)
            out[m + "uk"], out[m + "uv"] = mat(H * D, mc["kv_rank"]), mat(H * V, mc["kv_rank"])
        else:
            out[m + "q"], out[m + "k"], out[m + "v"], out[m + "g"] = mat(H * D, Wd), mat(H * D, Wd), mat(H * V, Wd), mat(H * V, Wd)
        if spec.get("mlp"):
            f, n = p + "mlp.", spec["mlp"]["ff"]
            out[p + "norm2"], out[p + "norm2b"], out[p + "ls2"] = vec(Wd, 0.1, 1.0), vec(Wd, 0.1, 1.0), vec(Wd, 0.2, 0.6)
            out[f + "gate"], out[f + "up"], out[f + "down"] = mat(n, Wd), mat(n, Wd), mat(Wd, n)
        if sd:
            out[p + "side.gate"], out[p + "side.proj"], out[p + "side.norm"] = mat(sd, Wd), mat(Wd, sd), vec(Wd, 0.1, 0.5)
    return out


def muduvik_attention(heads=4, kv_heads=2, dim=16, vdim=24, rot_dims=8, base=5000.0, scaling=(8.0, 1.0, 4.0, 64), scale=0.3, window=20, diff=0.4, ff=48):
    rot = {"base": base, "dims": rot_dims}
    if scaling:
        rot["scaling"] = {"factor": scaling[0], "low": scaling[1], "high": scaling[2], "original": scaling[3]}
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": rot, "scale": scale, "diff": diff}
    if window:
        mixer["mask"] = {"size": window}
    return {"type": "attention", "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def muduvik_latent(heads=3, dim=16, vdim=24, q_rank=20, kv_rank=40, scale=0.2, ff=48):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def muduvik_retention(heads=3, dim=16, vdim=24, rot_dims=8, base=3000.0, decay=None, ff=0):
    decay = list(decay) if decay is not None else [1.0 - 2.0 ** (-3 - h) for h in range(heads)]
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "rot": {"base": base, "dims": rot_dims}, "decay": decay},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def muduvik_config(layers, width=64, vocab=101, eps=1e-5, loop=None, side=8):
    cfg = {"architecture": "Muduvik", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    if side:
        cfg["token_side"] = {"dim": side}
    return cfg
