"""CPU tier of the Muduvik family: the config reader, the tensor table, the engine's packed layout, the loader's checks, and the
float64 restatement (tests/layer_list_oracle.py) held against itself -- each mechanism against a second, differently written form."""

import json
import math

import numpy as np
import pytest
import torch

import layer_list_oracle as O
from tiny_llm_hip.layer_list import FAMILIES, pack_layer_list

CONFIG = O.muduvik_config([
    O.muduvik_retention(heads=3, dim=16, vdim=24, rot_dims=8, decay=[0.9, 0.95, 0.99], ff=32),
    O.muduvik_attention(heads=6, kv_heads=3, dim=12, vdim=8, rot_dims=12, scaling=None, window=7, diff=0.25),
    O.muduvik_latent(heads=2, dim=20, vdim=12, q_rank=10, kv_rank=28, scale=0.11, ff=0),
    O.muduvik_attention(heads=2, kv_heads=1, dim=8, vdim=24, rot_dims=4, window=0, ff=0),
], width=48, vocab=61, eps=2e-5, loop=(1, 3, 3), side=5)


def test_config_reader_takes_every_size_and_constant_from_the_file():
    read, table = FAMILIES["Muduvik"]
    cfg = read(CONFIG)
    assert (cfg.family, cfg.block, cfg.width, cfg.vocab, cfg.norm_eps, cfg.norm_offset, cfg.loop, cfg.side_dim) == ("Muduvik", "sandwich", 48, 61, 2e-5, 0.0, (1, 3, 3), 5)
    assert cfg.embed_norm and not cfg.loop_projection and cfg.layer_scale and cfg.layer_runs == 4 + 2 * 2
    r, a, l, b = cfg.layers
    assert (r.kind, r.rec_kind, r.heads, r.dim, r.vdim, r.rot_dims, r.rot_base, r.decay, r.rot_half, r.ff, r.ff_kind, r.ff_act) == \
        ("linrec", "fixed", 3, 16, 24, 8, 3000.0, (0.9, 0.95, 0.99), True, 32, "gated", "gelu_tanh")
    assert (a.kind, a.heads, a.kv_heads, a.dim, a.vdim, a.rot_dims, a.window, a.diff, a.scale, a.rot_scaling) == ("attention", 6, 3, 12, 8, 12, 7, 0.25, 0.3, None)
    assert a.bias and a.qk_head_norm and a.gated and a.head_gate and not a.rot_half and not a.sink
    assert (l.kind, l.heads, l.dim, l.vdim, l.q_rank, l.kv_rank, l.rot_dim, l.scale, l.gated, l.ff) == ("latent", 2, 20, 12, 10, 28, 0, 0.11, False, 0)
    assert (b.window, b.rot_scaling, b.rot_scaling_kind) == (0, (8.0, 64.0, 4.0, 1.0), "wavelength")
    names = table(cfg)
    assert names["l1.mix.q"] == (2 * 6 * 12, 48) and names["l1.mix.k.b"] == (2 * 3 * 12,) and names["l1.mix.v"] == (24, 48) and names["l1.mix.g"] == (6, 48)
    assert names["l1.mix.q.norm"] == (12,) and names["l1.mix.lk2"] == (12,) and names["l0.mix.g"] == (72, 48) and names["l2.mix.uq"] == (40, 10)
    assert names["side.embed"] == (61, 20) and names["l3.side.proj"] == (48, 5) and names["loop.step"] == (3, 48) and "loop.in" not in names
    assert "l2.norm2" not in names and "l2.mix.g" not in names and names["l0.norm2b"] == (48,) and names["embed.norm"] == (48,)
    assert set(names) == set(O.make_muduvik_weights(CONFIG))
    plain = {k: v for k, v in CONFIG.items() if k not in ("loop", "token_side")}
    cfg2 = read(plain)
    assert cfg2.loop is None and cfg2.side_dim == 0 and "side.embed" not in table(cfg2) and "loop.step" not in table(cfg2)
    for bad in ({**CONFIG, "layers": [dict(CONFIG["layers"][0], type="delta")]}, {k: v for k, v in CONFIG.items() if k != "norm"},
                {**CONFIG, "loop": {"start": 2, "stop": 5, "times": 2}},
                {**CONFIG, "layers": [O.muduvik_retention(heads=3, decay=[0.5, 0.6])]}):
        with pytest.raises(ValueError):
            read(bad)


def test_packed_layout():
    read, _ = FAMILIES["Muduvik"]
    cfg = read(CONFIG)
    W = O.make_muduvik_weights(CONFIG, seed=1)
    packed = pack_layer_list(cfg, {k: torch.from_numpy(np.asarray(v)) for k, v in W.items()}, torch.float32, "cpu")
    l0, l1, l2 = packed["layers"][:3]
    assert tuple(l1["w_in"].shape) == (144 + 72 + 24 + 6, 48) and tuple(l1["w_out"].shape) == (48, 48)
    np.testing.assert_array_equal(l1["w_in"][144:216].numpy(), W["l1.mix.k"])
    np.testing.assert_array_equal(l1["w_in"][240:].numpy(), W["l1.mix.g"])
    bias = l1["w_in_bias"].numpy()
    assert bias.shape == (246,) and not bias[240:].any()
    np.testing.assert_array_equal(bias[216:240], W["l1.mix.v.b"])
    lam = math.exp(float(W["l1.mix.lq1"] @ W["l1.mix.lk1"])) - math.exp(float(W["l1.mix.lq2"] @ W["l1.mix.lk2"])) + 0.25
    assert l1["diff_lambda"] == pytest.approx(lam, rel=1e-6)
    assert tuple(l0["w_in"].shape) == (48 + 48 + 72 + 72, 48) and "out_norm" not in l0 and l0["decay"].tolist() == pytest.approx([0.9, 0.95, 0.99])
    assert tuple(l0["w_in2"].shape) == (64, 48) and "post_norm2" in l0 and "ls2" in l0 and "post_norm2" not in l2 and "w_in2" not in l2
    assert tuple(l2["w_in"].shape) == (10 + 28, 48) and tuple(l2["uk_t"].shape) == (2, 28, 20) and tuple(l2["uv"].shape) == (2, 12, 28)
    assert tuple(packed["side_embed"].shape) == (61, 20) and tuple(l2["side_gate"].shape) == (5, 48) and "loop_in" not in packed
    np.testing.assert_array_equal(packed["embed_norm"].numpy(), W["embed.norm"])


def test_loader_checks_names_and_shapes(tmp_path):
    from safetensors.torch import save_file

    from tiny_llm_hip.loader import load_weights

    W = O.make_muduvik_weights(CONFIG, seed=2)
    (tmp_path / "config.json").write_text(json.dumps(CONFIG))

    def save(weights):
        save_file({k: torch.from_numpy(np.asarray(v, dtype=np.float32)).to(torch.bfloat16) for k, v in weights.items()}, str(tmp_path / "model.safetensors"))

    save(W)
    model = load_weights(str(tmp_path), dtype=torch.float32)
    assert model.family == "Muduvik" and model.config.layers[1].window == 7 and model.tensors["l1.mix.g"].shape == (6, 48)
    bad = dict(W)
    bad["l1.mix.q.norm"] = np.ones(13, dtype=np.float32)
    save(bad)
    with pytest.raises(ValueError, match="l1.mix.q.norm"):
        load_weights(str(tmp_path))
    save({k: v for k, v in W.items() if k != "l3.side.gate"})
    with pytest.raises(Exception, match="l3.side.gate"):
        load_weights(str(tmp_path))


# ---- the restatement against second forms -------------------------------------------------------------------------------------

def test_window_attention_against_a_dense_form():
    rng = np.random.default_rng(3)
    L, H, G, D, V, win = 23, 4, 2, 6, 5, 5
    q, k, v = rng.normal(size=(L, H, D)), rng.normal(size=(L, G, D)), rng.normal(size=(L, 1, V))
    got = O.window_softmax_attention(q, k, v, 0.4, win)
    for h in range(H):
        s = (q[:, h] @ k[:, h // 2].T) * 0.4
        i, j = np.indices((L, L))
        s[(j > i) | (i - j >= win)] = -np.inf
        p = np.exp(s - s.max(1, keepdims=True))
        np.testing.assert_allclose(got[:, h], (p / p.sum(1, keepdims=True)) @ v[:, 0], rtol=1e-10, atol=1e-12)
    # the window's edge: the key `win` back changes nothing, the key win - 1 back does
    v2 = v.copy()
    v2[10] += 1.0
    moved = np.abs(O.window_softmax_attention(q, k, v2, 0.4, win) - got).max(axis=(1, 2))
    assert moved[10 + win - 1] > 1e-3 and moved[10 + win] == 0.0 and moved[9] == 0.0
    np.testing.assert_allclose(O.window_softmax_attention(q, k, v, 0.4, None), O.window_softmax_attention(q, k, v, 0.4, L + 3))


def test_differential_combination():
    rng = np.random.default_rng(4)
    a1, a2 = rng.normal(size=(3, 2, 7)), rng.normal(size=(3, 2, 7))
    o = O.differential_combine(a1, a2, 0.8, 0.3, 0.0)
    np.testing.assert_allclose(np.sqrt((o ** 2).mean(-1)), 0.7)                   # unit RMS times (1 - diff)
    np.testing.assert_allclose(O.differential_combine(a1, a1, 1.0, 0.3, 1e-6), 0.0)  # equal maps with lambda 1 cancel
    np.testing.assert_allclose(O.differential_combine(2 * a1, 2 * a2, 0.8, 0.3, 0.0), o)


def test_retention_against_the_summed_form():
    rng = np.random.default_rng(5)
    L, H, D, V = 17, 2, 4, 3
    q, k, v, decay = rng.normal(size=(L, H, D)), rng.normal(size=(L, H, D)), rng.normal(size=(L, H, V)), np.array([0.8, 0.97])
    got = O.retention_states(q, k, v, decay)
    for h in range(H):
        for t in range(L):
            want = sum(decay[h] ** (t - j) * (q[t, h] @ k[j, h]) * v[j, h] for j in range(t + 1))
            np.testing.assert_allclose(got[t, h], want, rtol=1e-10, atol=1e-12)


def test_forward_is_causal_windowed_looped_and_reads_the_side_table():
    W = O.make_muduvik_weights(CONFIG, seed=6)
    toks = [int(t) for t in np.random.default_rng(7).integers(0, 61, 30)]
    streams = []
    base = O.muduvik_forward(CONFIG, W, toks, streams)
    assert len(streams) == 8 and base.shape == (30, 61)
    later = list(toks)
    later[20] = (toks[20] + 1) % 61
    moved = np.abs(O.muduvik_forward(CONFIG, W, later) - base).max(1)
    assert moved[:20].max() == 0.0 and moved[20:].min() > 0.0                       # (retention and the latent layer reach every later token)
    # the looped layers see another offset in every pass: with equal offsets... the passes still differ (their inputs do)
    W2 = dict(W)
    W2["loop.step"] = W["loop.step"] + np.array([[0.0], [0.5], [0.0]])
    assert np.abs(O.muduvik_forward(CONFIG, W2, toks) - base).max() > 1e-3
    # the side table: only the layer's own columns of the token's row are read
    W3 = dict(W)
    W3["side.embed"] = W["side.embed"].copy()
    W3["side.embed"][toks[5], 15:20] += 1.0                                          # layer 3's columns
    s3 = []
    O.muduvik_forward(CONFIG, W3, toks, s3)
    same = [np.array_equal(a[5], b[5]) for a, b in zip(streams, s3)]
    assert same == [True] * 7 + [False]
