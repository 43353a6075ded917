"""GPU tier: the Muduvik family on the layer-list engine against the plain float64 restatement in tests/layer_list_oracle.py, on
small made-up configurations with random (or crafted) weights: blocks with norms on both sides of a sublayer and layer scales, the
per-layer token input, the embedding norm, a loop entered by an offset alone; differential sliding-window attention (biases, a
norm per head and map, adjacent rotation pairs with wavelength-rescaled frequencies, one gate per head), latent attention without
positions or gate, retention (a constant decay per head, half-split rotation pairs).

float32 runs are held to a relative RMS error of 2e-4 per logits row, bfloat16 runs to 4e-2 (layer_list_engine_helpers.TOL).
"""

import json

import numpy as np
import pytest
import torch

import layer_list_oracle as O
from layer_list_engine_helpers import TOL, in_portions, make_engine, rel_err, tokens_for, whole

pytestmark = pytest.mark.gpu

# six layers, the first three looped twice: windows of 20, 37 and none; a retention layer with and without feed-forward
MIXED = O.muduvik_config([O.muduvik_retention(ff=0),
                          O.muduvik_attention(),
                          O.muduvik_latent(),
                          O.muduvik_attention(heads=6, kv_heads=2, dim=24, vdim=12, rot_dims=16, window=37, diff=0.7, ff=0),
                          O.muduvik_retention(heads=2, dim=32, vdim=16, rot_dims=32, decay=[0.97, 0.999], ff=40),
                          O.muduvik_attention(heads=3, kv_heads=3, dim=20, vdim=8, rot_dims=4, scale=0.15, window=0, scaling=None, diff=0.1)],
                         loop=(0, 3, 2))

LAYERS = {
    "attention": O.muduvik_attention(),
    "attention_no_feed_forward": O.muduvik_attention(ff=0),
    "attention_no_window": O.muduvik_attention(window=0),
    "attention_window_of_one": O.muduvik_attention(window=1),
    "attention_window_across_pages": O.muduvik_attention(window=23),
    "attention_plain_frequencies": O.muduvik_attention(scaling=None),
    "attention_every_frequency_between": O.muduvik_attention(rot_dims=16, base=10.0, scaling=(3.0, 0.5, 40.0, 64)),
    "attention_no_rotation": O.muduvik_attention(rot_dims=0),
    "attention_one_kv_head": O.muduvik_attention(heads=4, kv_heads=1),
    "attention_as_many_kv_heads": O.muduvik_attention(heads=3, kv_heads=3, dim=8, vdim=8, rot_dims=8),
    "attention_one_head": O.muduvik_attention(heads=1, kv_heads=1, dim=32, vdim=40, rot_dims=32),
    "attention_large_group": O.muduvik_attention(heads=20, kv_heads=1, dim=8, vdim=8, rot_dims=4),      # 20 heads of a group: two 16-head blocks a map
    "attention_many_kv_heads": O.muduvik_attention(heads=16, kv_heads=8, dim=16, vdim=16, rot_dims=8),
    "attention_odd_sizes": O.muduvik_attention(heads=6, kv_heads=2, dim=10, vdim=13, rot_dims=6, window=11, ff=9),
    "attention_wide_heads": O.muduvik_attention(heads=2, kv_heads=1, dim=136, vdim=130, rot_dims=64),
    "attention_widest_heads": O.muduvik_attention(heads=2, kv_heads=2, dim=264, vdim=72, rot_dims=8),   # beyond the tile kernel: the row kernel
    "attention_no_subtraction_constant": O.muduvik_attention(diff=0.0),
    "latent": O.muduvik_latent(),
    "latent_no_feed_forward": O.muduvik_latent(ff=0),
    "latent_one_head": O.muduvik_latent(heads=1, dim=24, vdim=8, q_rank=6, kv_rank=12),
    "latent_odd_sizes": O.muduvik_latent(heads=5, dim=10, vdim=9, q_rank=7, kv_rank=21, ff=13),
    "latent_wide": O.muduvik_latent(heads=2, dim=72, vdim=40, q_rank=48, kv_rank=136),
    "latent_widest": O.muduvik_latent(heads=2, dim=16, vdim=16, q_rank=16, kv_rank=264),               # a latent beyond the tile kernel
    "retention": O.muduvik_retention(),
    "retention_feed_forward": O.muduvik_retention(ff=24),
    "retention_no_rotation": O.muduvik_retention(rot_dims=0),
    "retention_whole_head_rotated": O.muduvik_retention(dim=16, rot_dims=16),
    "retention_one_head_no_decay": O.muduvik_retention(heads=1, dim=8, vdim=8, rot_dims=4, decay=[1.0]),
    "retention_fast_decay": O.muduvik_retention(heads=2, decay=[0.5, 0.25]),
    "retention_odd_sizes": O.muduvik_retention(heads=5, dim=10, vdim=13, rot_dims=6),
    "retention_wide": O.muduvik_retention(heads=2, dim=160, vdim=136, rot_dims=64),
    "retention_many_heads": O.muduvik_retention(heads=24, dim=8, vdim=8, rot_dims=8),
}


def close(got, want, dtype):
    return rel_err(got, want) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("layer", sorted(LAYERS))
def test_each_mechanism_alone(layer, dtype):
    config = O.muduvik_config([LAYERS[layer]])
    W = O.make_muduvik_weights(config, seed=3)
    toks = tokens_for(config, 53, seed=4)
    want = O.muduvik_forward(config, W, toks)
    engine = make_engine(config, W, dtype)
    try:
        assert close(whole(engine, toks), want, dtype)
        assert close(in_portions(engine, toks, [19, 1, 1, 6, 1]), want, dtype)
    finally:
        engine.close()


@pytest.mark.parametrize("side,loop", [(0, None), (5, None), (8, (0, 1, 1)), (3, (0, 3, 3)), (0, (1, 3, 2)), (12, (2, 3, 4))])
def test_token_input_and_loops(side, loop):
    """No token input, inputs of 3 to 12 columns a layer; no loop, a loop of one pass, the whole model looped, loops that start behind the
    first layer and end with the last: every pass has its own pages and state and its own offset."""
    config = O.muduvik_config([O.muduvik_retention(), O.muduvik_attention(window=9), O.muduvik_latent()], side=side, loop=loop)
    W = O.make_muduvik_weights(config, seed=40)
    toks = tokens_for(config, 38, seed=41)
    streams = []
    want = O.muduvik_forward(config, W, toks, streams)
    engine = make_engine(config, W)
    try:
        assert engine.stats()["layer_runs"] == len(streams)
        assert close(whole(engine, toks), want, torch.float32)
        assert close(in_portions(engine, toks, [7, 1, 2]), want, torch.float32)
    finally:
        engine.close()


def test_width_and_vocabulary_that_are_no_multiples_of_8():
    config = O.muduvik_config([O.muduvik_attention(ff=20), O.muduvik_retention(ff=10), O.muduvik_latent(ff=0)], width=52, vocab=77, side=3)
    W = O.make_muduvik_weights(config, seed=60)
    toks = tokens_for(config, 30, seed=61)
    want = O.muduvik_forward(config, W, toks)
    for dtype in (torch.float32, torch.bfloat16):
        engine = make_engine(config, W, dtype)
        try:
            assert close(whole(engine, toks), want, dtype)
            assert close(in_portions(engine, toks, [1]), want, dtype)
        finally:
            engine.close()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_row_kernel_twin_of_the_tile_kernel(dtype, monkeypatch):
    """TL_HYBRID_ATTN_ROWS=1 sends every attention through the row kernel (a wave per row and head): the twin of the matrix-core kernel,
    with the same window, shared values and float32 read-outs."""
    monkeypatch.setenv("TL_HYBRID_ATTN_ROWS", "1")
    W = O.make_muduvik_weights(MIXED, seed=62)
    toks = tokens_for(MIXED, 70, seed=63)
    want = O.muduvik_forward(MIXED, W, toks)
    engine = make_engine(MIXED, W, dtype)
    try:
        assert close(whole(engine, toks), want, dtype)
        assert close(in_portions(engine, toks, [33, 1]), want, dtype)
    finally:
        engine.close()


def test_stream_after_every_layer():
    W = O.make_muduvik_weights(MIXED, seed=5)
    toks = tokens_for(MIXED, 29, seed=6)
    streams = []
    want = O.muduvik_forward(MIXED, W, toks, streams)
    engine = make_engine(MIXED, W)
    try:
        assert engine.stats()["layer_runs"] == len(streams) == 9
        engine.set_trace(True)
        engine.begin(0)
        n = engine.step([(0, toks, list(range(len(toks))))])
        for run, ref in enumerate(streams):
            assert rel_err(engine.read_trace(run, len(toks)), ref) < 1e-5, f"layer run {run}"
        assert rel_err(engine.logits_host(n), want) < TOL[torch.float32]
        engine.release(0)
    finally:
        engine.close()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_prefill_against_token_by_token(dtype):
    W = O.make_muduvik_weights(MIXED, seed=7)
    toks = tokens_for(MIXED, 45, seed=8)
    want = O.muduvik_forward(MIXED, W, toks)
    engine = make_engine(MIXED, W, dtype)
    try:
        assert close(whole(engine, toks), want, dtype)
        assert close(in_portions(engine, toks, [1]), want, dtype)
        assert close(in_portions(engine, toks, [30, 1]), want, dtype)  # a prompt, then decoding
    finally:
        engine.close()


@pytest.mark.parametrize("sizes", [[2], [3, 2, 7], [16], [15, 17, 1], [24, 5, 2, 40], [70, 13], [64, 1, 63, 2]])
def test_portions_of_several_sizes(sizes):
    """Portions end inside pages (16 tokens) and inside windows (20 and 37 positions); the recurrent state is carried across every cut."""
    W = O.make_muduvik_weights(MIXED, seed=9)
    toks = tokens_for(MIXED, 150, seed=10)
    engine = make_engine(MIXED, W)
    try:
        assert rel_err(in_portions(engine, toks, sizes), O.muduvik_forward(MIXED, W, toks)) < TOL[torch.float32]
    finally:
        engine.close()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_unequal_requests_in_one_batch_against_each_alone(dtype):
    """Portions of some requests beside single tokens of others; every request's rows must equal its whole-sequence logits."""
    W = O.make_muduvik_weights(MIXED, seed=11)
    prompts = [tokens_for(MIXED, n, seed=10 + n) for n in (70, 9, 41, 25)]
    want = [O.muduvik_forward(MIXED, W, p) for p in prompts]
    cuts = [[20, 1, 1, 30, 1, 1, 1, 15], [2, 1, 1, 1, 1, 1, 1, 1], [1, 17, 3, 19, 1], [25]]
    engine = make_engine(MIXED, W, dtype)
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
    """6 pages of 16 tokens and 2 slots serve 6 requests in pairs: pages that held another request's keys are overwritten before they are
    read, and a slot's recurrent state starts at zero again."""
    W = O.make_muduvik_weights(MIXED, seed=12)
    engine = make_engine(MIXED, W, page_size=16, num_pages=6, max_batch=2, max_prefill_rows=96)
    try:
        prompts = [tokens_for(MIXED, n, seed=20 + n) for n in (40, 33, 48, 17, 31, 47)]
        want = [O.muduvik_forward(MIXED, W, p) for p in prompts]
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


# ---- one key that decides the answer ---------------------------------------------------------------------------------------------

def _quiet(W, A, B):
    W["embed"][:, :2] = 0.0
    W["embed"][A] *= 0.05
    W["embed"][B] *= 0.05
    W["embed"][A, 0] = 8.0
    W["embed"][B, 1] = 8.0


def _bf16(W):
    for k in W:
        W[k] = torch.from_numpy(np.asarray(W[k], dtype=np.float32)).to(torch.bfloat16).float().numpy()


def _needle_attention(window, kv_heads=1):
    """One attention layer whose query token B looks for key token A through ONE unrotated dimension of map 1 that only these two tokens
    excite (so the match does not depend on distance): where A is among the keys B sees, the score of (B, A) towers over every other in
    map 1 of every head, map 2 knows nothing of it, and a lost, shifted or doubled key -- or a window that is one position off -- changes
    the logits at B by far more than the tolerance."""
    config = O.muduvik_config([O.muduvik_attention(heads=2, kv_heads=kv_heads, dim=16, vdim=16, rot_dims=8, scale=0.5, window=window, diff=0.3, ff=0)],
                              width=64, vocab=50, side=0)
    W = O.make_muduvik_weights(config, seed=15)
    A, B = 48, 49
    _quiet(W, A, B)
    m = "l0.mix."
    for name, heads, channel in (("k", kv_heads, 0), ("q", 2, 1)):
        W[m + name][:, channel] = 0.0
        W[m + name + ".b"][:] = 0.0
        for h in range(heads):
            W[m + name][h * 32 + 8, :] = 0.0
            W[m + name][h * 32 + 8, channel] = 6.0        # dimension 8 of map 1 of every head (not rotated) <- the channel only A (or only B) excites
    W[m + "q.norm"][:] = 1.0
    W[m + "k.norm"][:] = 1.0
    W[m + "v"][:, 0] += 1.0
    _bf16(W)
    return config, W, A, B


def _needle_latent():
    """The same through the two stages of latent attention: latent 0 of the queries reads only B's channel, latent 0 of the keys only A's, and
    dimension 0 of every head reads only that latent."""
    config = O.muduvik_config([O.muduvik_latent(heads=2, dim=16, vdim=16, q_rank=12, kv_rank=24, scale=0.5, ff=0)], width=64, vocab=50, side=0)
    W = O.make_muduvik_weights(config, seed=16)
    A, B = 48, 49
    _quiet(W, A, B)
    m = "l0.mix."
    for down, up, channel in (("dkv", "uk", 0), ("dq", "uq", 1)):
        W[m + down][:, channel] = 0.0
        W[m + down][0, :] = 0.0
        W[m + down][0, channel] = 6.0
        W[m + down + ".norm"][:] = 1.0
        W[m + up][:, 0] = 0.0
        for h in range(2):
            W[m + up][h * 16, :] = 0.0
            W[m + up][h * 16, 0] = 3.0
    W[m + "uv"][:, 0] += 1.0
    _bf16(W)
    return config, W, A, B


def _needle_retention():
    """Retention keeps no history but its state: with decays of 1 and 0.999 the outer product that A left long ago still answers B's query
    (through one unrotated dimension), so a state that was lost, reset, or carried over from another sequence shows at B."""
    config = O.muduvik_config([O.muduvik_retention(heads=2, dim=16, vdim=16, rot_dims=8, decay=[1.0, 0.999], ff=0)], width=64, vocab=50, side=0)
    W = O.make_muduvik_weights(config, seed=17)
    A, B = 48, 49
    _quiet(W, A, B)
    m = "l0.mix."
    for name, channel in (("k", 0), ("q", 1)):
        W[m + name][:, channel] = 0.0
        for h in range(2):
            W[m + name][h * 16 + 12, :] = 0.0
            W[m + name][h * 16 + 12, channel] = 6.0
    W[m + "v"][:, 0] += 1.0
    _bf16(W)
    return config, W, A, B


def _needle_prompt(config, A, B, n, needle_at, seed):
    toks = tokens_for(config, n, seed=seed, avoid=(A, B))
    toks[needle_at] = A
    toks[-1] = B
    return toks


def _needle_case(config, W, A, B, n, needle_at, query, seen, **pool):
    toks = _needle_prompt(config, A, B, n, needle_at, 16)
    want = O.muduvik_forward(config, W, toks)[-1]
    other = list(toks)
    other[needle_at] = toks[needle_at - 1] if needle_at else toks[1]
    moved = rel_err(O.muduvik_forward(config, W, other)[-1][None], want[None])
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
@pytest.mark.parametrize("mixer", ["attention", "latent", "retention"])
def test_far_keys_and_page_borders(mixer, needle_at, query):
    """No window: the last token sees every key; the needle sits far back, at page borders (16) and key-tile borders (64).  At 300 tokens
    a decoded token's key range is split over workgroups."""
    config, W, A, B = {"attention": lambda: _needle_attention(0), "latent": _needle_latent, "retention": _needle_retention}[mixer]()
    _needle_case(config, W, A, B, 300, needle_at, query, True, page_size=16, num_pages=24, max_batch=1)


@pytest.mark.parametrize("needle_at,seen", [(191, False), (192, True), (193, True), (207, True), (208, True), (254, True), (127, False), (0, False)])
@pytest.mark.parametrize("query", ["prompt", "decoded"])
def test_keys_just_inside_and_just_outside_a_window(needle_at, seen, query):
    """A window of 64 positions over pages of 16: the query at position 255 sees 192 .. 255 and nothing before."""
    config, W, A, B = _needle_attention(64, kv_heads=2)
    _needle_case(config, W, A, B, 256, needle_at, query, seen, page_size=16, num_pages=24, max_batch=1)


@pytest.mark.parametrize("n,needle_at,seen", [(101, 0, False), (101, 1, True), (150, 49, False), (150, 50, True), (201, 100, False), (201, 101, True),
                                              (450, 349, False), (450, 350, True), (450, 383, True), (450, 384, True), (450, 448, True), (100, 0, True), (60, 0, True)])
@pytest.mark.parametrize("query", ["prompt", "decoded"])
def test_window_edges_that_are_no_page_or_tile_edges(n, needle_at, seen, query):
    """A window of 100 positions: its edge falls inside pages and inside the kernels' 64-key tiles, and moves with every query."""
    config, W, A, B = _needle_attention(100)
    _needle_case(config, W, A, B, n, needle_at, query, seen, page_size=16, num_pages=30, max_batch=1)


@pytest.mark.parametrize("n,needle_at,seen", [(700, 399, False), (700, 400, True), (700, 401, True), (700, 463, True), (700, 464, True), (700, 650, True), (320, 19, False),
                                              (320, 20, True), (280, 0, True)])
def test_wide_window_of_a_decoded_token_over_split_key_ranges(n, needle_at, seen):
    """A window of 300 positions in a long context: the decoded token's keys are split over workgroups, counted from the window's first key."""
    config, W, A, B = _needle_attention(300, kv_heads=2)
    _needle_case(config, W, A, B, n, needle_at, "decoded", seen, page_size=64, num_pages=12, max_batch=1, max_prefill_rows=1024)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_first_tokens(dtype):
    """The first tokens of a sequence have few keys and an empty state: single tokens and portions of two from position 0."""
    W = O.make_muduvik_weights(MIXED, seed=18)
    toks = tokens_for(MIXED, 12, seed=19)
    want = O.muduvik_forward(MIXED, W, toks)
    engine = make_engine(MIXED, W, dtype)
    try:
        assert close(in_portions(engine, toks, [1, 1, 1, 2, 2, 5]), want, dtype)
        assert close(in_portions(engine, toks, [2]), want, dtype)
        assert close(whole(engine, toks[:1]), want[:1], dtype)
    finally:
        engine.close()


def test_the_second_map_and_the_gate_of_a_head_are_its_own():
    """Map 2 of every head made equal to map 1, with lambda = 1: the maps cancel up to rounding, and what is left is noise scaled to unit RMS.
    With different maps the engine must subtract head h's second map from head h's first (not a neighbour's), and gate head h by row h."""
    config = O.muduvik_config([O.muduvik_attention(heads=4, kv_heads=2, dim=8, vdim=8, rot_dims=4, window=0, diff=0.5, ff=0)], side=0)
    W = O.make_muduvik_weights(config, seed=50)
    m = "l0.mix."
    W[m + "g"] *= 6.0                                   # gates far from 1/2, different from head to head
    W[m + "q"].reshape(4, 2, 8, -1)[2, 1] *= 3.0        # one head's second map stands out
    toks = tokens_for(config, 40, seed=51)
    want = O.muduvik_forward(config, W, toks)
    swapped = {k: v.copy() for k, v in W.items()}
    swapped[m + "g"] = W[m + "g"][[1, 0, 3, 2]]
    assert rel_err(O.muduvik_forward(config, swapped, toks), want) > 0.05
    engine = make_engine(config, W)
    try:
        assert close(whole(engine, toks), want, torch.float32)
    finally:
        engine.close()


ODD = O.muduvik_config([O.muduvik_latent(heads=1, dim=12, vdim=20, q_rank=9, kv_rank=15, ff=0),
                        O.muduvik_attention(heads=5, kv_heads=5, dim=6, vdim=10, rot_dims=2, window=3, diff=0.9, ff=23),
                        O.muduvik_retention(heads=1, dim=24, vdim=40, rot_dims=24, decay=[0.75], ff=11)], width=40, vocab=37, eps=1e-3, side=1, loop=(2, 3, 2))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_other_sizes(dtype):
    """Sizes that are no multiples of 8, one head, heads * vdim != width, a token input of one column, a large eps, a tiny window, a loop over the last layer."""
    W = O.make_muduvik_weights(ODD, seed=24)
    toks = tokens_for(ODD, 41, seed=25)
    want = O.muduvik_forward(ODD, W, toks)
    engine = make_engine(ODD, W, dtype)
    try:
        assert close(whole(engine, toks), want, dtype)
        assert close(in_portions(engine, toks, [5, 1, 2, 9]), want, dtype)
    finally:
        engine.close()


WIDE = O.muduvik_config([O.muduvik_retention(heads=4, dim=32, vdim=32, rot_dims=32, ff=128),
                         O.muduvik_attention(heads=4, kv_heads=2, dim=32, vdim=32, rot_dims=32, window=128, ff=256),
                         O.muduvik_latent(heads=8, dim=32, vdim=32, q_rank=64, kv_rank=64, ff=128),
                         O.muduvik_attention(heads=8, kv_heads=2, dim=16, vdim=64, rot_dims=16, window=70, ff=0)], width=128, vocab=200, side=64)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_large_chunks_of_rows(dtype):
    """From 192 rows the bfloat16 products run on the 256-wide tile GEMM (the projections' biases behind it); the same prompt in small
    portions (64-wide tiles, row kernel) must give the same logits."""
    W = O.make_muduvik_weights(WIDE, seed=26)
    toks = tokens_for(WIDE, 300, seed=27)
    want = O.muduvik_forward(WIDE, W, toks)
    engine = make_engine(WIDE, W, dtype, page_size=64, num_pages=8, max_batch=2)
    try:
        assert close(whole(engine, toks), want, dtype)
        assert close(in_portions(engine, toks, [250, 3, 40, 1]), want, dtype)
    finally:
        engine.close()


def test_long_greedy_decoding_on_the_device_and_graph_replays():
    """160 greedy steps through the captured decode step (across window and page borders); the ids are the float64 restatement's greedy
    choices, and replaying the graph gives what eager launches give."""
    W = O.make_muduvik_weights(MIXED, seed=28)
    prompt = tokens_for(MIXED, 21, seed=29)
    engine = make_engine(MIXED, W, page_size=16, num_pages=16, max_batch=2)
    try:
        ids = engine.generate(prompt, 161, slot=1)
        assert engine.stats()["graph_replays"] >= 160
        full = prompt + ids
        ref = O.muduvik_forward(MIXED, W, full[:-1])
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

    W = O.make_muduvik_weights(MIXED, seed=30)
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
    W = O.make_muduvik_weights(MIXED, seed=31)
    _save(tmp_path, MIXED, W)
    from tiny_llm_hip import load
    from tiny_llm_hip.models import engine_for

    model, tokenizer = load(str(tmp_path))
    assert tokenizer is None and model.family == "Muduvik"
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

    W = O.make_muduvik_weights(MIXED, seed=33)
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
    ref_long, ref_short, ref_third = (O.muduvik_forward(MIXED, W, t) for t in (long, short, third))
    got = {i: np.fromfile(out_dir / f"{i}.f32", dtype="<f4").reshape(-1, MIXED["vocab"]) for i in (0, 1, 2, 4)}
    tol = TOL[torch.float32 if dtype == "float32" else torch.bfloat16]
    assert rel_err(got[0], ref_long[[0, 99]]) < tol
    assert rel_err(got[1], ref_short[[28]]) < tol
    assert rel_err(got[2], np.stack([ref_short[29], ref_long[149]])) < tol
    assert rel_err(got[4], ref_third[[49, 3]]) < tol
