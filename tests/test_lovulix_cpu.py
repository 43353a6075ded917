"""CPU tier of the Lovulix family: the config reader, the tensor table, the engine's packed layout, the loader's checks, and the
float64 restatement (tests/layer_list_oracle.py) held against itself -- each mechanism against a second, differently written form."""

import json
import math

import numpy as np
import pytest
import torch

import layer_list_oracle as O
from tiny_llm_hip.layer_list import FAMILIES, pack_layer_list

CONFIG = O.lovulix_config([
    O.lovulix_layer(v_mix=False, mlp=None),
    O.lovulix_layer(heads=6, kv_heads=3, dim=12, vdim=8, rot_dims=12, scaling=None, chunk=0, mlp=O.lovulix_moe(experts=5, top=3, ff=16, shared=0)),
    O.lovulix_layer(heads=6, kv_heads=2, dim=20, vdim=12, rot_dims=4, scale=0.11, chunk=7),
    O.lovulix_layer(heads=2, kv_heads=1, dim=8, vdim=24, rot_dims=0, v_mix=True, mlp=O.lovulix_moe(experts=2, top=1, ff=8, shared=24)),
], width=48, vocab=61, eps=2e-5, logit_scale=1.5)


def test_config_reader_takes_every_size_and_constant_from_the_file():
    read, table = FAMILIES["Lovulix"]
    cfg = read(CONFIG)
    assert (cfg.family, cfg.block, cfg.width, cfg.vocab, cfg.norm_eps, cfg.logit_scale, cfg.norm_offset) == ("Lovulix", "postnorm", 48, 61, 2e-5, 1.5, 0.0)
    a, b, c, d = cfg.layers
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.rot_dims, a.rot_base, a.scale, a.chunk, a.ff, a.v_mix) == (4, 2, 16, 24, 8, 5000.0, 0.3, 16, 0, "none")
    assert a.rot_scaling == (8.0, 64.0, 4.0, 1.0) and a.rot_scaling_kind == "wavelength" and a.rot_half and a.qk_norm and a.talk and a.learned_sink
    assert (b.rot_scaling, b.chunk, b.v_mix) == (None, 0, "first")           # the first layer that mixes values keeps them
    assert (b.experts, b.top, b.expert_ff, b.shared_ff, b.ff, b.router, b.moe_gated, b.moe_scale_input, b.moe_shared_sg) == (5, 3, 16, 0, 80, "sigmoid", True, True, False)
    assert (c.v_mix, c.chunk, c.scale, c.rot_dims) == ("blend", 7, 0.11, 4) and (d.v_mix, d.rot_dims, d.shared_ff, d.ff) == ("blend", 0, 24, 40)
    names = table(cfg)
    assert "l0.mix.vmix" not in names and "l1.mix.vmix" not in names and names["l2.mix.vmix"] == ()
    assert names["l2.mix.talk"] == (6, 6) and names["l2.mix.q.norm"] == (120,) and names["l2.mix.k.norm"] == (40,) and names["l3.mix.sink"] == (2,)
    assert "l0.norm2" not in names and names["l1.mlp.e4.gate"] == (16, 48) and "l1.mlp.shared.up" not in names and names["l3.mlp.shared.down"] == (48, 24)
    assert set(names) <= set(O.make_lovulix_weights(CONFIG))
    for bad in ({**CONFIG, "layers": [dict(CONFIG["layers"][0], type="delta")]}, {k: v for k, v in CONFIG.items() if k != "logit_scale"}):
        with pytest.raises(ValueError):
            read(bad)


def test_packed_layout():
    read, _ = FAMILIES["Lovulix"]
    cfg = read(CONFIG)
    W = O.make_lovulix_weights(CONFIG, seed=1)
    packed = pack_layer_list(cfg, {k: torch.from_numpy(np.asarray(v)) for k, v in W.items()}, torch.float32, "cpu")
    l1, l3 = packed["layers"][1], packed["layers"][3]
    assert tuple(l1["w_in"].shape) == (6 * 12 + 3 * 12 + 3 * 8 + 6 * 8, 48) and tuple(l1["w_out"].shape) == (48, 48)
    # gates | ups | router | zero rows up to a multiple of 8; one output matrix over every expert's columns
    assert tuple(l1["w_in2"].shape) == ((2 * 80 + 5 + 7) // 8 * 8, 48) and tuple(l1["w_out2"].shape) == (48, 80)
    np.testing.assert_array_equal(l1["w_in2"][16:32].numpy(), W["l1.mlp.e1.gate"])
    np.testing.assert_array_equal(l1["w_in2"][80 + 32:80 + 48].numpy(), W["l1.mlp.e2.up"])
    np.testing.assert_array_equal(l1["w_in2"][160:165].numpy(), W["l1.mlp.router"])
    assert not l1["w_in2"][165:].any()
    np.testing.assert_array_equal(l3["w_in2"][:24].numpy(), W["l3.mlp.shared.gate"])      # the shared expert leads gates, ups and output columns
    np.testing.assert_array_equal(l3["w_in2"][40 + 24:40 + 32].numpy(), W["l3.mlp.e0.up"])
    np.testing.assert_array_equal(l3["w_out2"][:, 24:32].numpy(), W["l3.mlp.e0.down"])
    assert "v_mix_lambda" not in l1 and packed["layers"][2]["v_mix_lambda"] == pytest.approx(float(W["l2.mix.vmix"]))
    assert l1["talk"].shape == (6, 6) and l1["sink"].dtype == torch.float32 and "correction" not in l1


def test_loader_checks_names_and_shapes(tmp_path):
    from safetensors.torch import save_file

    from tiny_llm_hip.loader import load_weights

    W = O.make_lovulix_weights(CONFIG, seed=2)
    (tmp_path / "config.json").write_text(json.dumps(CONFIG))

    def save(weights):
        save_file({k: torch.from_numpy(np.asarray(v, dtype=np.float32)).to(torch.bfloat16) for k, v in weights.items()}, str(tmp_path / "model.safetensors"))

    save(W)
    model = load_weights(str(tmp_path), dtype=torch.float32)
    assert model.family == "Lovulix" and model.config.layers[2].chunk == 7 and model.tensors["l2.mix.talk"].shape == (6, 6)
    bad = dict(W)
    bad["l2.mix.talk"] = W["l2.mix.talk"][:, :5]
    save(bad)
    with pytest.raises(ValueError, match="l2.mix.talk"):
        load_weights(str(tmp_path))
    save({k: v for k, v in W.items() if k != "l1.mlp.router"})
    with pytest.raises(Exception, match="l1.mlp.router"):
        load_weights(str(tmp_path))


# ---- the restatement against second forms -------------------------------------------------------------------------------------

def test_frequencies_by_wavelength():
    f = O.wavelength_scaled_frequencies(16, 100.0, {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 40})
    plain = np.array([100.0 ** (-2 * i / 16) for i in range(8)])
    lam = 2 * math.pi / plain
    assert lam[0] < 10 and f[0] == plain[0]                      # short waves stay
    assert lam[-1] > 40 and f[-1] == pytest.approx(plain[-1] / 4)  # long ones are slowed
    mid = [i for i in range(8) if 10 <= lam[i] <= 40]
    assert mid and all(plain[i] / 4 < f[i] < plain[i] for i in mid[1:-1] or mid)
    assert np.all(np.diff(f) < 0)
    np.testing.assert_array_equal(O.wavelength_scaled_frequencies(16, 100.0, None), plain)


def test_half_split_rotation_keeps_norms_and_relative_positions():
    rng = np.random.default_rng(0)
    f = O.wavelength_scaled_frequencies(8, 50.0)
    q, k = rng.standard_normal((1, 1, 12)), rng.standard_normal((1, 1, 12))
    a = O.rotate_halves_by(np.repeat(q, 9, 0), np.arange(9.0) + 5, f)
    b = O.rotate_halves_by(np.repeat(k, 9, 0), np.arange(9.0), f)
    np.testing.assert_allclose((a * a).sum(-1), (q * q).sum(-1).repeat(9, 0))
    np.testing.assert_array_equal(a[..., 8:], np.repeat(q, 9, 0)[..., 8:])   # dimensions from rot dims on pass
    dots = (a * b).sum(-1)[:, 0]
    np.testing.assert_allclose(dots, dots[0] * np.ones(9), rtol=1e-10)        # the product depends on the distance (5) alone
    one = O.rotate_halves_by(q, np.array([3.0]), f)[0, 0]
    assert one[1] == pytest.approx(q[0, 0, 1] * math.cos(3 * f[1]) - q[0, 0, 5] * math.sin(3 * f[1]))
    assert one[5] == pytest.approx(q[0, 0, 5] * math.cos(3 * f[1]) + q[0, 0, 1] * math.sin(3 * f[1]))


def test_attention_against_a_dense_form():
    rng = np.random.default_rng(1)
    L, H, G, D, V, C = 23, 6, 2, 5, 4, 8
    q, k, v = rng.standard_normal((L, H, D)), rng.standard_normal((L, G, D)), rng.standard_normal((L, G, V))
    talk, sink = rng.standard_normal((H, H)), rng.standard_normal(H)
    got = O.talking_chunk_attention(q, k, v, 0.4, talk, sink, C)
    kk, vv = np.repeat(k, H // G, 1), np.repeat(v, H // G, 1)
    s = np.einsum("ihd,jhd->hij", q, kk) * 0.4
    s = np.einsum("hg,gij->hij", talk, s)
    i, j = np.arange(L)[:, None], np.arange(L)[None, :]
    seen = (j <= i) & (i // C == j // C)
    e = np.where(seen[None], np.exp(s), 0.0)
    w = e / (e.sum(-1, keepdims=True) + np.exp(sink)[:, None, None])
    np.testing.assert_allclose(got, np.einsum("hij,jhv->ihv", w, vv), rtol=1e-10, atol=1e-12)
    # no mixing, no sink, no chunk: the plain causal softmax
    plain = O.talking_chunk_attention(q, k, v, 0.4)
    np.testing.assert_allclose(plain, O.causal_softmax_attention(q, kk, vv, 0.4), rtol=1e-10)
    np.testing.assert_allclose(O.talking_chunk_attention(q, k, v, 0.4, np.eye(H), np.zeros(H), None), O.sink_attention(q, k, v, 0.4), rtol=1e-10)


def test_expert_choice_and_input_scaling():
    z = np.array([0.3, -1.0, 2.0, 2.0, 0.1])
    assert list(O.sigmoid_top_route(z, 2)) == [2, 3] and list(O.sigmoid_top_route(z, 1)) == [2]       # ties go to the lower index
    assert O.sigmoid_top_route(z, 3)[0] == pytest.approx(1 / (1 + math.exp(-0.3)))                    # the weight is the score, not renormalised
    config = O.lovulix_config([O.lovulix_layer(mlp=O.lovulix_moe(experts=4, top=2, ff=8, shared=8))], width=16)
    W = {k: np.asarray(v, dtype=np.float64) for k, v in O.make_lovulix_weights(config, seed=3).items()}
    h = np.random.default_rng(2).standard_normal((5, 16))
    got = O.lovulix_feed_forward(config["layers"][0]["mlp"], W, "l0.mlp.", h)
    for t in range(5):
        s = 1 / (1 + np.exp(-(W["l0.mlp.router"] @ h[t])))
        want = O.gated_expert(W, "l0.mlp.shared.", h[t])
        for e in np.argsort(-s, kind="stable")[:2]:
            g, u = s[e] * (W[f"l0.mlp.e{e}.gate"] @ h[t]), s[e] * (W[f"l0.mlp.e{e}.up"] @ h[t])   # both projections are linear in the scaled input
            want = want + W[f"l0.mlp.e{e}.down"] @ (g / (1 + np.exp(-g)) * u)
        np.testing.assert_allclose(got[t], want, rtol=1e-10)


def test_forward_is_causal_chunked_and_blends_values():
    config = O.lovulix_config([O.lovulix_layer(chunk=8), O.lovulix_layer(chunk=8)], width=32, vocab=40)
    W = O.make_lovulix_weights(config, seed=4)
    toks = list(np.random.default_rng(3).integers(0, 40, 30))
    full = O.lovulix_forward(config, W, toks)
    np.testing.assert_allclose(O.lovulix_forward(config, W, toks[:19]), full[:19], rtol=1e-9, atol=1e-9)
    # a row depends on the tokens of its own chunk only: the same tokens at the same places in their chunk give the same rows
    np.testing.assert_allclose(O.lovulix_forward(config, W, toks[8:24])[:8], O.lovulix_forward(config, W, toks[8:16])[:8], rtol=1e-9, atol=1e-9)
    other = list(toks)
    other[15] = (toks[15] + 1) % 40
    changed = O.lovulix_forward(config, W, other)
    np.testing.assert_allclose(changed[16:], full[16:], rtol=1e-9, atol=1e-9)    # ... and not on the chunk before
    assert np.abs(changed[15] - full[15]).max() > 1e-3
    # the second layer's blend: with vmix = 0 nothing of the first layer's values arrives
    W0 = dict(W)
    W0["l1.mix.vmix"] = np.float32(0.0)
    assert np.abs(O.lovulix_forward(config, W0, toks) - full).max() > 1e-4
