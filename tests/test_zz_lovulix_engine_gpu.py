"""GPU tier: the Lovulix family on the layer-list engine against the plain float64 restatement in tests/layer_list_oracle.py, on
small made-up configurations with random (or crafted) weights: blocks with the norm on the branch's output; attention with a norm
over the whole q / k projection, half-split rotation pairs with wavelength-rescaled frequencies, scores mixed across heads, a
chunked mask, learned sinks, value mixing, an output gate; sigmoid-routed gated experts whose score scales their input.

float32 runs are held to a relative RMS error of 2e-4 per logits row, bfloat16 runs to 4e-2 (layer_list_engine_helpers.TOL).
"""

import json

import numpy as np
import pytest
import torch

import layer_list_oracle as O
from layer_list_engine_helpers import TOL, in_portions, make_engine, rel_err, tokens_for, whole

pytestmark = pytest.mark.gpu


def for_dtype(config, dtype):
    """bfloat16 runs of models with several layers take every expert: rounding can turn an expert choice whose scores are nearly equal, and
    with the norm on the branch's output the other expert's result is as large as the right one's; through the keys and values of later
    layers the row's successors follow.  The choice itself is held to the restatement in float32 everywhere and in bfloat16 on single layers."""
    if dtype == torch.float32:
        return config
    config = json.loads(json.dumps(config))
    for spec in config["layers"]:
        if spec.get("mlp"):
            spec["mlp"]["router"]["top"] = spec["mlp"]["router"]["experts"]
    return config


def close(got, want, dtype):
    """float32: every row within the tolerance.  bfloat16: a turned expert choice (see for_dtype) changes its row outright, so nine rows in
    ten must be within the tolerance and the whole within five times it; the float32 run of the same case is the sharp one."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    err = np.sqrt(((got - want) ** 2).mean(-1)) / np.sqrt((want ** 2).mean(-1))
    if dtype == torch.float32:
        return bool(err.max() < TOL[dtype])
    return bool((err < TOL[dtype]).mean() >= 0.9 and np.sqrt(((got - want) ** 2).mean() / (want ** 2).mean()) < 5 * TOL[dtype])

# four layers: values kept by the second and blended by the third and fourth; chunks of 16, 24, none and 5 positions
MIXED = O.lovulix_config([O.lovulix_layer(v_mix=False, mlp=O.lovulix_moe(experts=3, top=1, ff=16, shared=0)),
                          O.lovulix_layer(heads=6, kv_heads=2, dim=24, vdim=12, rot_dims=16, chunk=24),
                          O.lovulix_layer(heads=6, kv_heads=1, dim=8, vdim=24, rot_dims=8, scaling=None, chunk=0, mlp=None),
                          O.lovulix_layer(heads=3, kv_heads=3, dim=20, vdim=8, rot_dims=4, scale=0.15, chunk=5, mlp=O.lovulix_moe(experts=7, top=3, ff=8, shared=24))])

LAYERS = {
    "default": O.lovulix_layer(),
    "no_feed_forward": O.lovulix_layer(mlp=None),
    "no_chunks": O.lovulix_layer(chunk=0),
    "chunks_of_one": O.lovulix_layer(chunk=1),
    "chunks_across_pages": O.lovulix_layer(chunk=23),
    "plain_frequencies": O.lovulix_layer(scaling=None),
    "every_frequency_between": O.lovulix_layer(rot_dims=16, base=10.0, scaling=(3.0, 0.5, 40.0, 64)),
    "no_rotation": O.lovulix_layer(rot_dims=0),
    "one_kv_head": O.lovulix_layer(heads=4, kv_heads=1),
    "as_many_kv_heads": O.lovulix_layer(heads=3, kv_heads=3, dim=8, vdim=8, rot_dims=8),
    "one_head": O.lovulix_layer(heads=1, kv_heads=1, dim=32, vdim=40, rot_dims=32),
    "more_heads_than_waves": O.lovulix_layer(heads=20, kv_heads=5, dim=8, vdim=8, rot_dims=4),
    "eight_kv_heads": O.lovulix_layer(heads=16, kv_heads=8, dim=16, vdim=16, rot_dims=8),        # the value blocks of a prompt over two workgroups, of a decode step over four
    "sixteen_kv_heads_wide": O.lovulix_layer(heads=16, kv_heads=16, dim=72, vdim=72, rot_dims=32),  # the 128-wide tile, four workgroups of four blocks
    "head_group_beyond_the_tile_kernel": O.lovulix_layer(heads=24, kv_heads=1, dim=8, vdim=8, rot_dims=4),   # the row kernel, its waves taking the heads in two passes
    "odd_sizes": O.lovulix_layer(heads=6, kv_heads=2, dim=10, vdim=13, rot_dims=6, chunk=11, mlp=O.lovulix_moe(experts=5, top=2, ff=9, shared=11)),
    "wide_heads": O.lovulix_layer(heads=2, kv_heads=1, dim=136, vdim=130, rot_dims=64),
    "every_expert_taken": O.lovulix_layer(mlp=O.lovulix_moe(experts=3, top=3, ff=16, shared=8)),
    "one_expert_no_shared": O.lovulix_layer(mlp=O.lovulix_moe(experts=1, top=1, ff=24, shared=0)),
    "many_experts": O.lovulix_layer(mlp=O.lovulix_moe(experts=70, top=6, ff=8, shared=8)),
}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("layer", sorted(LAYERS))
def test_each_mechanism_alone(layer, dtype):
    config = O.lovulix_config([LAYERS[layer]])
    W = O.make_lovulix_weights(config, seed=1)
    toks = tokens_for(config, 37, seed=2)
    engine = make_engine(config, W, dtype)
    try:
        want = O.lovulix_forward(config, W, toks)
        assert close(whole(engine, toks), want, dtype)
        assert close(in_portions(engine, toks, [9, 1, 2]), want, dtype)
    finally:
        engine.close()


def test_width_and_vocabulary_that_are_no_multiples_of_8():
    config = O.lovulix_config([O.lovulix_layer(heads=3, kv_heads=1, dim=10, vdim=6, rot_dims=4, chunk=7, mlp=O.lovulix_moe(experts=3, top=2, ff=5, shared=7))], width=50, vocab=77)
    W = O.make_lovulix_weights(config, seed=40)
    toks = tokens_for(config, 33, seed=41)
    want = O.lovulix_forward(config, W, toks)
    engine = make_engine(config, W)
    try:
        assert rel_err(whole(engine, toks), want) < TOL[torch.float32]
        assert rel_err(in_portions(engine, toks, [4, 1, 1, 9]), want) < TOL[torch.float32]
    finally:
        engine.close()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_row_kernel_twin_of_the_tile_kernel(dtype, monkeypatch):
    """TL_HYBRID_ATTN_ROWS=1 sends every attention layer through the row kernels (a workgroup per row, a wave per head): the twin of the
    MFMA tile kernel gives the same logits, in prompts, portions and single tokens."""
    monkeypatch.setenv("TL_HYBRID_ATTN_ROWS", "1")
    config = for_dtype(MIXED, dtype)
    W = O.make_lovulix_weights(config, seed=42)
    toks = tokens_for(config, 70, seed=43)
    want = O.lovulix_forward(config, W, toks)
    engine = make_engine(config, W, dtype)
    try:
        assert close(whole(engine, toks), want, dtype)
        assert close(in_portions(engine, toks, [33, 1, 2, 1]), want, dtype)
    finally:
        engine.close()


def test_score_mixing_takes_rows_of_the_matrix_and_values_of_the_mixed_head():
    """A mixing matrix that is a permutation: head h's weights come from head perm[h]'s scores but still read head h's values; a
    transposed matrix or values taken from the scores' head would give another head's output."""
    config = O.lovulix_config([O.lovulix_layer(heads=4, kv_heads=4, dim=8, vdim=8, rot_dims=8, chunk=0, mlp=None)])
    W = O.make_lovulix_weights(config, seed=3)
    talk = np.zeros((4, 4), dtype=np.float32)
    for h, g in enumerate([2, 0, 3, 1]):
        talk[h, g] = 1.5
    W["l0.mix.talk"] = talk
    toks = tokens_for(config, 40, seed=4)
    want = O.lovulix_forward(config, W, toks)
    Wt = dict(W)
    Wt["l0.mix.talk"] = talk.T.copy()
    assert rel_err(O.lovulix_forward(config, Wt, toks), want) > 0.05
    engine = make_engine(config, W)
    try:
        assert rel_err(whole(engine, toks), want) < TOL[torch.float32]
        assert rel_err(in_portions(engine, toks, [1]), want) < TOL[torch.float32]
    finally:
        engine.close()


def test_stream_after_every_layer():
    W = O.make_lovulix_weights(MIXED, seed=5)
    toks = tokens_for(MIXED, 29, seed=6)
    streams = []
    want = O.lovulix_forward(MIXED, W, toks, streams)
    engine = make_engine(MIXED, W)
    try:
        assert engine.stats()["layer_runs"] == len(streams) == 4
        engine.set_trace(True)
        engine.begin(0)
        n = engine.step([(0, toks, list(range(len(toks))))])
        for run, ref in enumerate(streams):
            assert rel_err(engine.read_trace(run, len(toks)), ref) < 1e-5, f"layer {run}"
        assert rel_err(engine.logits_host(n), want) < TOL[torch.float32]
        engine.release(0)
    finally:
        engine.close()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_prefill_against_token_by_token(dtype):
    config = for_dtype(MIXED, dtype)
    W = O.make_lovulix_weights(config, seed=7)
    toks = tokens_for(config, 45, seed=8)
    want = O.lovulix_forward(config, W, toks)
    engine = make_engine(config, W, dtype)
    try:
        assert close(whole(engine, toks), want, dtype)
        assert close(in_portions(engine, toks, [1]), want, dtype)
        assert close(in_portions(engine, toks, [30, 1]), want, dtype)  # a prompt, then decoding
    finally:
        engine.close()


@pytest.mark.parametrize("sizes", [[2], [3, 2, 7], [16], [15, 17, 1], [24, 5, 2, 40], [70, 13], [64, 1, 63, 2]])
def test_portions_of_several_sizes(sizes):
    """Portions end inside pages (16 tokens) and inside chunks (16, 24 and 5 positions): chunks are counted from the sequence's start."""
    W = O.make_lovulix_weights(MIXED, seed=9)
    toks = tokens_for(MIXED, 150, seed=10)
    engine = make_engine(MIXED, W)
    try:
        assert rel_err(in_portions(engine, toks, sizes), O.lovulix_forward(MIXED, W, toks)) < TOL[torch.float32]
    finally:
        engine.close()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_unequal_requests_in_one_batch_against_each_alone(dtype):
    """Portions of some requests beside single tokens of others; every request's rows must equal its whole-sequence logits (the values
    kept for blending belong to the step's rows, whatever their sequence)."""
    config = for_dtype(MIXED, dtype)
    W = O.make_lovulix_weights(config, seed=11)
    prompts = [tokens_for(config, n, seed=10 + n) for n in (70, 9, 41, 25)]
    want = [O.lovulix_forward(config, W, p) for p in prompts]
    cuts = [[20, 1, 1, 30, 1, 1, 1, 15], [2, 1, 1, 1, 1, 1, 1, 1], [1, 17, 3, 19, 1], [25]]
    engine = make_engine(config, W, dtype)
    try:
        at = [0] * 4
        got = [[] for _ in prompts]
        for s in range(4):
            engine.begin(s)
        turn = 0
        while any(at[i] < len(prompts[i]) for i in range(4)):
            entries, who = [], []
            for i in range(4):
                if at[i] < len(prompts[i]):
                    n = cuts[i][turn] if turn < len(cuts[i]) else 1
                    if (turn + i) % 5 == 4 and entries:
                        continue  # a request may sit out a step
                    part = prompts[i][at[i]:at[i] + n]
                    entries.append((i, part, list(range(len(part)))))
                    who.append((i, len(part)))
                    at[i] += len(part)
            turn += 1
            if not entries:
                continue
            rows = engine.logits_host(engine.step(entries))
            r = 0
            for i, n in who:
                got[i].append(rows[r:r + n])
                r += n
        for i in range(4):
            assert close(np.concatenate(got[i], 0), want[i], dtype), f"request {i}"
    finally:
        engine.close()


def test_pages_and_slots_are_used_again():
    """6 pages of 16 tokens and 2 slots serve 6 requests in pairs: pages that held another request's keys and (blended) values are
    overwritten before they are read."""
    W = O.make_lovulix_weights(MIXED, seed=12)
    engine = make_engine(MIXED, W, page_size=16, num_pages=6, max_batch=2, max_prefill_rows=96)
    try:
        prompts = [tokens_for(MIXED, n, seed=20 + n) for n in (40, 33, 48, 17, 31, 47)]
        want = [O.lovulix_forward(MIXED, W, p) for p in prompts]
        for k in range(0, 6, 2):
            a, b = prompts[k], prompts[k + 1]
            engine.begin(0)
            engine.begin(1)
            ra = [engine.logits_host(engine.step([(0, a[:10], list(range(10)))]))]
            both = engine.logits_host(engine.step([(0, a[10:], list(range(len(a) - 10))), (1, b, list(range(len(b))))]))
            ra.append(both[:len(a) - 10])
            assert rel_err(np.concatenate(ra, 0), want[k]) < TOL[torch.float32]
            assert rel_err(both[len(a) - 10:], want[k + 1]) < TOL[torch.float32]
            engine.release(0)
            engine.release(1)
        st = engine.stats()
        assert st["reused_page_allocations"] > 0 and st["reused_slot_begins"] == 4 and st["pages_in_use"] == 0
        engine.begin(0)
        engine.step([(0, tokens_for(MIXED, 90, seed=1), [])])
        engine.begin(1)
        with pytest.raises(RuntimeError, match="exhausted"):
            engine.step([(1, tokens_for(MIXED, 10, seed=2), [])])
    finally:
        engine.close()


def _needle_model(chunk, kv_heads=1):
    """One attention layer whose query token B looks for key token A through ONE unrotated dimension that only these two tokens excite
    (so the match does not depend on distance): where A is among the keys B sees, the score of (B, A) towers over every other in every
    head, and a lost, shifted or doubled key -- or a mask that is one position off -- changes the logits at B by far more than the tolerance."""
    config = O.lovulix_config([O.lovulix_layer(heads=2, kv_heads=kv_heads, dim=16, vdim=16, rot_dims=8, scale=0.5, chunk=chunk, v_mix=False, mlp=None)], width=64, vocab=50)
    W = O.make_lovulix_weights(config, seed=15)
    A, B = 48, 49
    W["embed"][:, :2] = 0.0
    W["embed"][A] *= 0.05
    W["embed"][B] *= 0.05
    W["embed"][A, 0] = 8.0
    W["embed"][B, 1] = 8.0
    m = "l0.mix."
    for name, heads, channel in (("k", kv_heads, 0), ("q", 2, 1)):
        W[m + name][:, channel] = 0.0
        for h in range(heads):
            W[m + name][h * 16 + 8, :] = 0.0
            W[m + name][h * 16 + 8, channel] = 6.0        # dimension 8 of every head (not rotated) <- the channel only A (or only B) excites
    W[m + "q.norm"][:] = 1.0
    W[m + "k.norm"][:] = 1.0
    W[m + "v"][:, 0] += 1.0
    W[m + "sink"][:] = 0.0
    for k in W:
        W[k] = torch.from_numpy(np.asarray(W[k], dtype=np.float32)).to(torch.bfloat16).float().numpy()
    return config, W, A, B


def _needle_prompt(config, A, B, n, needle_at, seed):
    toks = tokens_for(config, n, seed=seed, avoid=(A, B))
    toks[needle_at] = A
    toks[-1] = B
    return toks


def _needle_case(config, W, A, B, n, needle_at, query, seen, **pool):
    toks = _needle_prompt(config, A, B, n, needle_at, 16)
    want = O.lovulix_forward(config, W, toks)[-1]
    other = list(toks)
    other[needle_at] = toks[needle_at - 1] if needle_at else toks[1]
    moved = rel_err(O.lovulix_forward(config, W, other)[-1][None], want[None])
    assert (moved > 0.2) if seen else (moved < 1e-9)   # the needle decides the answer exactly where the mask lets B see it
    engine = make_engine(config, W, **pool)
    try:
        engine.begin(0)
        if query == "prompt":
            cut = n - 40
            engine.step([(0, toks[:cut], [])])
            k = engine.step([(0, toks[cut:], [n - cut - 1])])
        else:
            engine.step([(0, toks[:-1], [])])
            k = engine.step([(0, toks[-1:], [0])])
        assert rel_err(engine.logits_host(k), want[None]) < TOL[torch.float32]
        engine.release(0)
    finally:
        engine.close()


@pytest.mark.parametrize("needle_at", [0, 3, 15, 16, 17, 31, 32, 63, 64, 250, 298])
@pytest.mark.parametrize("query", ["prompt", "decoded"])
def test_far_keys_and_page_borders(needle_at, query):
    """No chunks: the last token sees every key; the needle sits far back, at page borders (16) and key-tile borders (64)."""
    config, W, A, B = _needle_model(chunk=0)
    _needle_case(config, W, A, B, 300, needle_at, query, True, page_size=16, num_pages=24, max_batch=1)


@pytest.mark.parametrize("needle_at,seen", [(191, False), (192, True), (193, True), (207, True), (208, True), (254, True), (127, False), (0, False)])
@pytest.mark.parametrize("query", ["prompt", "decoded"])
def test_keys_just_inside_and_just_outside_a_chunk(needle_at, seen, query):
    """Chunks of 64 positions over pages of 16: the query at position 255 sees 192 .. 255 and nothing before."""
    config, W, A, B = _needle_model(chunk=64, kv_heads=2)
    _needle_case(config, W, A, B, 256, needle_at, query, seen, page_size=16, num_pages=24, max_batch=1)


@pytest.mark.parametrize("n,needle_at,seen", [(101, 99, False), (150, 99, False), (150, 100, True), (201, 199, False), (199, 100, True), (199, 99, False), (200, 101, True),
                                              (450, 399, False), (450, 400, True), (450, 447, True), (450, 448, True)])
@pytest.mark.parametrize("query", ["prompt", "decoded"])
def test_chunk_edges_that_are_no_page_or_tile_edges(n, needle_at, seen, query):
    """Chunks of 100 positions: their edges fall inside pages and inside the kernels' 64-key tiles; a query that is the first of its
    chunk (position 100, 200) sees only itself.  At 450 tokens a decoded token's key range is split over workgroups (64 keys each): most
    splits lie before the chunk and hold nothing but -- the first one -- the sink; the chunk starts inside one."""
    config, W, A, B = _needle_model(chunk=100)
    _needle_case(config, W, A, B, n, needle_at, query, seen, page_size=16, num_pages=30, max_batch=1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_first_tokens_and_heavy_sinks(dtype):
    """The first tokens of a sequence and of every chunk have few keys: there the sink takes most of the weight.  Sinks of +6 and -6
    make a forgotten, doubled or scaled sink show in every row."""
    config = O.lovulix_config([O.lovulix_layer(chunk=6), O.lovulix_layer(heads=2, kv_heads=2, chunk=0)])
    W = O.make_lovulix_weights(config, seed=20)
    W["l0.mix.sink"] = np.array([6.0, -6.0, 3.0, 0.0], dtype=np.float32)
    W["l1.mix.sink"] = np.array([5.0, -2.0], dtype=np.float32)
    toks = tokens_for(config, 14, seed=21)
    want = O.lovulix_forward(config, W, toks)
    W0 = dict(W)
    W0["l0.mix.sink"] = np.zeros(4, dtype=np.float32)
    assert rel_err(O.lovulix_forward(config, W0, toks), want) > 0.05
    engine = make_engine(config, W, dtype)
    try:
        assert close(whole(engine, toks), want, dtype)
        assert close(in_portions(engine, toks, [1]), want, dtype)
        assert close(whole(engine, toks[:1]), want[:1], dtype)
        assert close(in_portions(engine, toks, [5, 2, 1]), want, dtype)
    finally:
        engine.close()


def test_value_mixing_reaches_back_to_the_first_mixing_layer_only():
    """Layer 0 does not mix, layer 1 keeps its values, layers 2 and 3 blend with layer 1's (lambda 0.9 and 1: the own values vanish);
    rows of two sequences in one step keep their own values."""
    config = O.lovulix_config([O.lovulix_layer(v_mix=False), O.lovulix_layer(), O.lovulix_layer(heads=6, kv_heads=2, dim=8), O.lovulix_layer()])
    W = O.make_lovulix_weights(config, seed=22)
    W["l2.mix.vmix"], W["l3.mix.vmix"] = np.float32(0.90625), np.float32(1.0)
    a, b = tokens_for(config, 33, seed=23), tokens_for(config, 21, seed=24)
    wa, wb = O.lovulix_forward(config, W, a), O.lovulix_forward(config, W, b)
    engine = make_engine(config, W)
    try:
        engine.begin(0)
        engine.begin(1)
        r1 = engine.logits_host(engine.step([(0, a[:20], list(range(20))), (1, b[:5], list(range(5)))]))
        r2 = engine.logits_host(engine.step([(1, b[5:], list(range(16))), (0, a[20:], list(range(13)))]))
        assert rel_err(np.concatenate([r1[:20], r2[16:]], 0), wa) < TOL[torch.float32]
        assert rel_err(np.concatenate([r1[20:], r2[:16]], 0), wb) < TOL[torch.float32]
    finally:
        engine.close()


ODD = O.lovulix_config([O.lovulix_layer(heads=3, kv_heads=1, dim=24, vdim=40, rot_dims=10, base=777.0, scale=0.3, chunk=9, mlp=O.lovulix_moe(experts=7, top=4, ff=12, shared=20)),
                        O.lovulix_layer(heads=10, kv_heads=5, dim=6, vdim=8, rot_dims=6, scaling=(2.0, 2.0, 3.0, 30), chunk=0, mlp=None),
                        O.lovulix_layer(heads=1, kv_heads=1, dim=72, vdim=40, rot_dims=2, chunk=33, mlp=O.lovulix_moe(experts=2, top=2, ff=52, shared=0)),
                        O.lovulix_layer(heads=5, kv_heads=5, dim=10, vdim=8, rot_dims=0, chunk=2, v_mix=False)],
                       width=88, vocab=97, eps=1e-3, logit_scale=-1.25)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_other_sizes(dtype):
    """Sizes that are no multiples of 8, one head, heads * vdim != width, a layer without feed-forward, a negative logit scale, a large
    eps, values blended between layers of different head counts (equal total width)."""
    config = for_dtype(ODD, dtype)
    W = O.make_lovulix_weights(config, seed=24)
    toks = tokens_for(config, 41, seed=25)
    want = O.lovulix_forward(config, W, toks)
    engine = make_engine(config, W, dtype)
    try:
        assert close(whole(engine, toks), want, dtype)
        assert close(in_portions(engine, toks, [5, 1, 2, 9]), want, dtype)
    finally:
        engine.close()


WIDE = O.lovulix_config([O.lovulix_layer(heads=4, kv_heads=2, dim=32, vdim=32, rot_dims=32, chunk=128, mlp=O.lovulix_moe(experts=4, top=2, ff=64, shared=64)),
                         O.lovulix_layer(heads=8, kv_heads=2, dim=32, vdim=32, rot_dims=16, chunk=0, mlp=O.lovulix_moe(experts=8, top=1, ff=32, shared=0)),
                         O.lovulix_layer(heads=16, kv_heads=4, dim=16, vdim=16, rot_dims=16, chunk=64, mlp=None)], width=128, vocab=200)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_large_chunks_of_rows(dtype):
    """From 192 rows the bfloat16 products run on the 256-wide tile GEMM; the same prompt in small portions (64-wide tiles, row kernel)
    must give the same logits, with 4, 8 and 16 heads mixing their scores."""
    config = for_dtype(WIDE, dtype)
    W = O.make_lovulix_weights(config, seed=26)
    toks = tokens_for(config, 300, seed=27)
    want = O.lovulix_forward(config, W, toks)
    engine = make_engine(config, W, dtype, page_size=64, num_pages=8, max_batch=2)
    try:
        assert close(whole(engine, toks), want, dtype)
        assert close(in_portions(engine, toks, [250, 3, 40, 1]), want, dtype)
    finally:
        engine.close()


def test_long_greedy_decoding_on_the_device_and_graph_replays():
    """160 greedy steps through the captured decode step (across chunk and page borders); the ids are the float64 restatement's greedy
    choices, and replaying the graph gives what eager launches give."""
    W = O.make_lovulix_weights(MIXED, seed=28)
    prompt = tokens_for(MIXED, 21, seed=29)
    engine = make_engine(MIXED, W, page_size=16, num_pages=16, max_batch=2)
    try:
        ids = engine.generate(prompt, 161, slot=1)
        assert engine.stats()["graph_replays"] >= 160
        full = prompt + ids
        ref = O.lovulix_forward(MIXED, W, full[:-1])
        for k, tok in enumerate(ids):
            row = ref[len(prompt) - 1 + k]
            assert row[tok] >= row.max() - 1e-3 * np.abs(row).max(), f"generated token {k}"
        engine.begin(0)
        engine.prefill(0, prompt)
        engine.decode(40, slots=[0], use_graph=False)
        assert engine.read_tokens(0, 41) == ids[:41]
        engine.release(0)
    finally:
        engine.close()


@pytest.mark.parametrize("mixed", [True, False])
def test_greedy_generation_through_the_scheduler(mixed):
    """engine.batch_generate_ids (continuous batching: chunked prefill in a staging slot, adoption into decode slots, retirement):
    every request's ids are what the request alone generates."""
    from tiny_llm_hip.engine import batch_generate_ids

    W = O.make_lovulix_weights(MIXED, seed=30)
    prompts = [tokens_for(MIXED, n, seed=30 + n) for n in (5, 23, 40, 9, 31)]
    limits = [12, 7, 9, 15, 4]
    engine = make_engine(MIXED, W, page_size=16, num_pages=40, max_batch=4, max_prefill_rows=64)
    try:
        alone = [engine.generate(p, n, slot=0) for p, n in zip(prompts, limits)]
        done = dict(batch_generate_ids(engine, prompts, limits, batch_size=3, prefill_step=16, mixed_steps=mixed))
        assert sorted(done) == list(range(5))
        for i in range(5):
            assert done[i] == alone[i], f"request {i}"
        assert engine.stats()["pages_in_use"] == 0
    finally:
        engine.close()


def _save(tmp_path, config, W):
    from safetensors.torch import save_file

    tmp_path.mkdir(exist_ok=True)
    (tmp_path / "config.json").write_text(json.dumps(config))
    save_file({k: torch.from_numpy(np.asarray(v, dtype=np.float32)).to(torch.bfloat16) for k, v in W.items()}, str(tmp_path / "model.safetensors"))


def test_checkpoint_directory_through_loader_registry_and_command_line(tmp_path):
    W = O.make_lovulix_weights(MIXED, seed=31)
    _save(tmp_path, MIXED, W)
    from tiny_llm_hip import load
    from tiny_llm_hip.models import engine_for

    model, tokenizer = load(str(tmp_path))
    assert tokenizer is None and model.family == "Lovulix"
    prompt = tokens_for(MIXED, 11, seed=32)
    engine = engine_for(model, dtype=torch.float32, page_size=16, num_pages=8, max_batch=1, max_prefill_rows=32)
    try:
        want = engine.generate(prompt, 6)
    finally:
        engine.close()
    import main as cli

    out = cli.main(["--model", str(tmp_path), "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "6", "--dtype", "float32"])
    assert [int(t) for t in out.split()] == want
    out = cli.main(["--model", str(tmp_path), "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "6", "--dtype", "float32",
                    "--sampler-temp", "1e-4", "--sampler-top-k", "1"])
    assert [int(t) for t in out.split()] == want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_command_line(tmp_path, dtype):
    """bin/trace_run on a checkpoint directory: two requests share steps, one ends, and its slot and pages serve a third."""
    import subprocess
    import sys
    from pathlib import Path

    W = O.make_lovulix_weights(MIXED, seed=33)
    model_dir, out_dir = tmp_path / "model", tmp_path / "out"
    _save(model_dir, MIXED, W)
    long, short, third = (tokens_for(MIXED, n, seed=34 + n) for n in (150, 30, 50))
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": long[:100], "want": [0, 99]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": long[100:149], "want": []}, {"id": "y", "tokens": short[:29], "want": [28]}], "end": []},
             {"step": 2, "entries": [{"id": "y", "tokens": short[29:], "want": [0]}, {"id": "x", "tokens": long[149:], "want": [0]}], "end": ["x"]},
             {"step": 3, "entries": [], "end": []},
             {"step": 4, "entries": [{"id": "z", "tokens": third, "want": [49, 3]}, {"id": "y", "tokens": [5], "want": []}], "end": ["y", "z"]}]
    root = Path(__file__).resolve().parent.parent
    run = subprocess.run([sys.executable, str(root / "bin" / "trace_run"), "--model", str(model_dir), "--dtype", dtype, "--out", str(out_dir),
                          "--max-tokens", str(192 + 64), "--slots", "2"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                         capture_output=True, text=True, timeout=110)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [l for l in run.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(5)]
    ref_long, ref_short, ref_third = (O.lovulix_forward(MIXED, W, t) for t in (long, short, third))
    got = {i: np.fromfile(out_dir / f"{i}.f32", dtype="<f4").reshape(-1, MIXED["vocab"]) for i in (0, 1, 2, 4)}
    tol = TOL[torch.float32 if dtype == "float32" else torch.bfloat16]
    assert rel_err(got[0], ref_long[[0, 99]]) < tol
    assert rel_err(got[1], ref_short[[28]]) < tol
    assert rel_err(got[2], np.stack([ref_short[29], ref_long[149]])) < tol
    assert rel_err(got[4], ref_third[[49, 3]]) < tol
