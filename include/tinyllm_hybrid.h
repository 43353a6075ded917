/*
 * tinyllm_hybrid.h — C ABI of the layer-list engine ("hybrid engine"): decoder-only models whose layers are
 * described one by one (a token mixer of some kind, an optional feed-forward, one shared pre-norm), with
 * unquantised bf16 or fp32 weights and a float32 residual stream.
 *
 * Where the Qwen3 engine (tinyllm_engine.h) is one fixed layer shape issued as 5 fused W4 kernels, this engine
 * walks a list of layer descriptions.  Mixer kinds so far:
 *
 *   TL_MIX_ATTENTION   grouped-query softmax attention over the paged K/V pool.  Options per layer: rotary
 *                      positions on the first rot_dims dimensions of each head (adjacent pairs), unit-RMS
 *                      normalisation of q and k after the rotation, a score scale, a "sink" (one is added to the
 *                      softmax denominator: a key of score 0 without a value), a sigmoid output gate.
 *                      Query/key width and value width of a head are independent.  Further options: a weighted RMS
 *                      norm over the WHOLE q (and k) projection before the rotation (qk_norm), rotation of the pairs
 *                      (i, i + rot_dims/2) instead of neighbours (rot_half), frequencies rescaled by wavelength
 *                      (rot_scaling_kind 1), scores mixed across query heads before the softmax (talk_dev), a learned
 *                      sink logit per head (sink_dev), a chunked causal mask (chunk: a query sees the keys of its own
 *                      run of `chunk` positions only), values blended with the values the first such layer computed for
 *                      the same token (v_mix).  Also: biases on the projections (w_in_bias_dev), an RMS norm per head with one [dim] weight
 *                      before the rotation (qk_head_norm), a sliding window (window: a query sees itself and the window - 1 keys
 *                      before it), one gate number per head (gated 2), and differential attention (diff_maps): every head has two
 *                      query / key maps [map 1 | map 2] over the same values, each an attention of its own; the read-outs combine
 *                      as a1 - lambda a2, are divided by their RMS over vdim and multiplied by 1 - diff_init.
 *   TL_MIX_DELTA       gated delta rule: a [key_dim, value_dim] float32 state per head that decays, is corrected
 *                      towards the new value along the new key and is read with the query; q/k/v pass a short
 *                      causal depthwise convolution + SiLU first.  The state and the convolution's last inputs
 *                      live in one state slot per sequence.
 *   TL_MIX_LINREC      linear recurrence with a decaying matrix state per head, S <- diag(a_t) S + b_t k_t v_t^T,
 *                      o_t = S^T q_t (q scaled by dim^-1/2).  rec_kind TL_REC_CHANNEL: a decay per key channel,
 *                      sigmoid(z)^(1/tau) with z from a low-rank pair of projections plus a bias, b = 1 (gated linear
 *                      attention); the read-out is RMS-normed per head with a [vdim] weight and gated by SiLU.
 *                      rec_kind TL_REC_EXPGATE: exponential input and forget gates per head, capped by
 *                      cap tanh(x / cap), with a running maximum m (starting at 0) that keeps them in range, and a
 *                      normaliser n_t = a n + b k: o / (max(|n.q|, e^-m) + 1e-6) (the matrix memory of xLSTM); the
 *                      read-out is unit-RMS per head, times a [heads*vdim] weight, gated by a sigmoid.
 *                      rec_kind TL_REC_FIXED: one constant decay per head (decay_dev), b = 1, no normaliser (retention); q and k
 *                      may carry rotary positions on their first rot_dims dimensions and k (not q) is scaled by dim^-1/2; the
 *                      read-out is unit-RMS per head without a weight (out_norm_dev NULL) and gated by SiLU.
 *                      State (and m) live in the state slot of the sequence.
 *   TL_MIX_LATENT      latent attention: queries through a normed low-rank latent; keys and values are per-head
 *                      projections (W_uk, W_uv) of ONE normed latent c [kv_rank] per token, plus one rotated key part
 *                      [rot_dim] shared by all heads; only (c | rotated part) is cached, one row per token.  The engine
 *                      runs it in absorbed form: q_h' = W_uk,h^T q_h, scores (q_h' . c + q_rot . k_rot) * scale, output
 *                      W_uv,h (sum_j p_j c_j) -- one K/V head of width kv_rank + rot_dim whose values are its leading
 *                      kv_rank columns.  Rotation frequencies may be rescaled (YaRN: rot_factor > 0).  kv_from >= 0: the
 *                      layer has no latent projection of its own and reads the pages of that earlier layer.
 *
 * Block forms: parallel_block 1 is x += m (mixer(h) + ff(h)) with one norm; 0 is the sequential pre-norm block
 * x += ls1 * mixer(norm1 x); x += ls2 * ff(norm2 x) with optional per-channel scales ls1 / ls2; 2 is the block with the norm on
 * the branch's OUTPUT, x += m norm1(mixer(x)); x += m norm2(ff(x)), whose sublayers read the stream itself; 3 has a norm on both sides
 * of every sublayer, x += m ls1 post1(mixer(norm1 x)); x += m ls2 post2(ff(norm2 x)).  A layer may end with a per-layer token input
 * (side_*): e = the layer's columns of a second embedding table, y = W_proj (gelu_tanh(W_gate x) * e), x += y / rms(y) * side_norm.
 * The embedding output may pass an RMS norm (embed_norm_dev).  Norms: RMS or
 * Dynamic Tanh (tanh(alpha x) w + b).  Feed-forward kinds: W_down act(W_up h), W_down (act(W_gate h) * W_up h), or a
 * mixture of experts (softmax or sigmoid router with a selection-only correction, groups of neighbouring experts, identity
 * experts, a shared expert with or without a scalar gate; experts W_down act(W_up h) or, with moe_gated, W_down (act(W_gate h) *
 * W_up h); the router's weight on the expert's output or, with moe_scale_input, on its input).
 *
 * A contiguous range of layers may be repeated ("loop"): each pass has its own K/V pages / state slots, and is
 * entered through a [width, 2 width] projection of the running stream beside the embedding output (loop_in_dev; NULL:
 * the stream passes as it is) plus a per-pass offset vector.
 *
 * One step function serves prefill, decode and any mixture: tl_hybrid_step takes chunks of token ids for several
 * sequence slots (a chunk of one token is a decode step), runs them as one packed batch of rows and returns the
 * logits of the rows asked for.  Row-wise work (norms, projections, feed-forward) runs once over the packed rows;
 * attention and the recurrences run per sequence from what earlier steps left in the pages and state slots.
 *
 * Float32 throughout: residual stream, norms, rotary angles, attention scores / weights, decays, gates of the
 * recurrence, recurrent state.  With dtype TL_BF16 the matrices, the activations entering a matrix product and
 * the K/V pages are bfloat16 (float32 accumulation); with TL_F32 everything is float32 (fp32 MFMA, no reduced mode).
 *
 * All functions return 0 / negative tl_status; message via tl_hybrid_last_error().  *_dev = device pointers.
 */
#ifndef TINYLLM_HYBRID_H
#define TINYLLM_HYBRID_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tl_hybrid tl_hybrid;

enum { TL_MIX_ATTENTION = 0, TL_MIX_DELTA = 1, TL_MIX_LINREC = 2, TL_MIX_LATENT = 3 };
enum { TL_REC_CHANNEL = 0, TL_REC_EXPGATE = 1, TL_REC_FIXED = 2 };
enum { TL_NORM_RMS = 0, TL_NORM_DYT = 1 };
enum { TL_FF_PLAIN = 0, TL_FF_GATED = 1, TL_FF_MOE = 2 };
enum { TL_ROUTER_SOFTMAX = 0, TL_ROUTER_SIGMOID = 1 };
enum { TL_BLOCK_SEQUENTIAL = 0, TL_BLOCK_PARALLEL = 1, TL_BLOCK_POSTNORM = 2, TL_BLOCK_SANDWICH = 3 };
enum { TL_VMIX_NONE = 0, TL_VMIX_FIRST = 1, TL_VMIX_BLEND = 2 };
enum { TL_ACT_GELU_ERF = 0, TL_ACT_GELU_TANH = 1, TL_ACT_SILU = 2, TL_ACT_RELU2 = 3 };
enum { TL_HY_F32 = 0, TL_HY_BF16 = 2 }; /* the values of tl_dtype in tinyllm_hip.h */

/* One layer.  Matrices are [out, in] row-major in the engine's dtype; vectors are float32.
 * w_in: every projection that reads the normed input, rows concatenated in this order:
 *   attention: q (heads*dim) | k (kv_heads*dim) | v (kv_heads*vdim) | gate (heads*vdim if gated 1, heads if gated 2) | up (ff, if ff > 0)
 *              with diff_maps: q (heads*2*dim, per head [map 1 | map 2]) | k (kv_heads*2*dim, likewise) | v | gate
 *   delta:     q (kv_heads*dim) | k (kv_heads*dim) | v (heads*vdim) | gate (heads*vdim) | a (heads) | b (heads) | up (ff)
 *   linrec:    q (heads*dim) | k (heads*dim) | v (heads*vdim) | gate (heads*vdim) | expgate: i (heads) | f (heads)
 *                                                                                    | channel: a1 (a_rank) | fixed: nothing
 *   latent:    dq (q_rank) | dkv (kv_rank + rot_dim, unless kv_from >= 0) | gate (heads*vdim, if gated)
 * w_out: [width, heads*vdim + ff]: the mixer's output projection beside the feed-forward's down projection, so
 *   one product yields mixer(h) + ff(h).
 * Sequential block (parallel_block 0): w_in / w_out hold the mixer's rows / columns only; the feed-forward reads
 *   norm2 through w_in2 and returns through w_out2:
 *   plain: up (ff)                   -> w_out2 [width, ff]
 *   gated: gate (ff) | up (ff)       -> w_out2 [width, ff]
 *   moe:   shared up (shared_ff) | expert 0 up (expert_ff) | expert 1 up ... | router (experts + identity) | shared gate (1) |
 *          zero rows up to a multiple of 8         -> w_out2 [width, shared_ff + experts * expert_ff]: shared down | expert 0 down | ...
 *   moe with moe_gated: shared gate (shared_ff) | expert 0 gate | ... | shared up (shared_ff) | expert 0 up | ... | router (experts + identity) |
 *          [scalar shared gate (1) if moe_shared_sg] | zero rows up to a multiple of 8         -> w_out2 as above */
typedef struct tl_hybrid_layer {
    int kind;
    int heads, kv_heads, dim, vdim;
    int ff;                 /* 0: no feed-forward */
    int ff_act;             /* 0 exact (erf) GELU, 1 tanh GELU, 2 SiLU */
    const void *w_in_dev, *w_out_dev;
    const float *norm_dev;  /* [width] pre-norm weight */
    float norm_offset;      /* weight is applied as (norm_offset + w): 1 for weights stored around zero */
    /* attention */
    int rot_dims;           /* 0: no rotary positions */
    float rot_base;
    float scale;
    int qk_unit_rms;        /* q and k divided by their RMS over dim after the rotation */
    int sink;               /* softmax denominator += 1 */
    int gated;              /* 1: output * sigmoid(gate), a gate per output channel; 2: one gate per head */
    /* delta */
    int conv_taps;
    const float *conv_dev;  /* [2*kv_heads*dim + heads*vdim, taps], last tap = current token */
    const float *a_log_dev, *dt_bias_dev; /* [heads] */
    const float *out_norm_dev;            /* [vdim] */
    float unit_eps;         /* q, k -> x / sqrt(sum x^2 + unit_eps) */
    /* norms and the sequential block */
    int norm_kind;          /* TL_NORM_RMS / TL_NORM_DYT, both norms of the layer */
    float norm_alpha, norm2_alpha;                /* Dynamic Tanh: the scalar inside the tanh */
    const float *norm_bias_dev, *norm2_bias_dev;  /* Dynamic Tanh: [width] */
    const float *norm2_dev;                       /* [width] the feed-forward's pre-norm (sequential block) */
    const void *w_in2_dev, *w_out2_dev;           /* the feed-forward's matrices (sequential block) */
    const float *ls1_dev, *ls2_dev;               /* [width] per-channel scale of the mixer's / feed-forward's result; NULL: none */
    int ff_kind;            /* TL_FF_* */
    /* mixture of experts (ff_kind TL_FF_MOE; ff = shared_ff + experts * expert_ff) */
    int experts, identity, top, groups, keep, expert_ff, shared_ff;
    const float *correction_dev;                  /* [experts + identity] added to the scores for the selection only */
    /* linear recurrence */
    int rec_kind;           /* TL_REC_* */
    float gate_cap, tau;
    int a_rank;             /* channel decay: rank of the projection pair */
    const void *a2_dev;     /* [heads*dim, a_rank] engine dtype */
    const float *a2_bias_dev;                     /* [heads*dim] */
    const float *i_bias_dev, *f_bias_dev;         /* [heads] */
    /* latent attention (out_norm_dev is not used; heads share one K/V head) */
    int q_rank, kv_rank, rot_dim, kv_from;        /* kv_from: layer index whose pages are read, -1: the layer's own */
    const float *dq_norm_dev, *dkv_norm_dev;      /* [q_rank], [kv_rank] */
    const void *uq_dev;     /* [heads*(dim + rot_dim), q_rank] */
    const void *uk_t_dev;   /* [heads, kv_rank, dim]: W_uk of every head transposed */
    const void *uv_dev;     /* [heads, vdim, kv_rank] */
    float rot_factor, rot_original, rot_fast, rot_slow; /* rot_factor <= 0: plain frequencies */
    /* attention, further options */
    int qk_norm;            /* 1: q and k each pass an RMS norm over their whole projection (all heads at once) with the weights below,
                               before the rotation */
    const float *q_norm_dev, *k_norm_dev; /* [heads*dim], [kv_heads*dim] */
    int rot_half;           /* 1: the rotation pairs dimension i with i + rot_dims/2; 0: 2i with 2i+1 */
    int rot_scaling_kind;   /* 0: by dimension index (rot_fast / rot_slow = turns over rot_original positions, cos and sin grow);
                               1: by wavelength l = 2 pi / f: f kept where l < rot_original / rot_fast, f / rot_factor where
                               l > rot_original / rot_slow, blended linearly in original / l between */
    const float *talk_dev;  /* [heads, heads]: score_h <- sum_g talk[h, g] score_g before the softmax; NULL: none */
    const float *sink_dev;  /* [heads]: with sink != 0 the denominator gains exp(sink_dev[h]) instead of 1; NULL: 1 */
    int chunk;              /* > 0: query i sees key j <= i only if i / chunk == j / chunk (positions of the sequence) */
    int v_mix;              /* TL_VMIX_FIRST: this layer's values are kept for the step's rows; TL_VMIX_BLEND: v <- (1 - l) v + l v_first
                               before they are cached */
    float v_mix_lambda;
    /* mixture of experts, further options */
    int moe_router;         /* TL_ROUTER_*: scores softmax(z) or sigmoid(z) */
    int moe_gated;          /* experts (and the shared one) are W_down (act(W_gate h) * W_up h) */
    int moe_scale_input;    /* the router's weight multiplies the expert's input: expert(w h) */
    int moe_shared_sg;      /* the shared expert is scaled by sigmoid of a scalar projection (its row follows the router's) */
    /* attention, further options (2) */
    const float *w_in_bias_dev; /* [the mixer's rows of w_in] added in the projection; NULL: none */
    int window;             /* > 0: query i sees key j <= i only if i - j < window */
    int qk_head_norm;       /* 1: every head (and map) of q and k passes an RMS norm over dim with the weights q_norm_dev / k_norm_dev [dim],
                               before the rotation */
    int diff_maps;          /* 1: differential attention (two maps per head, see above); the row's gate is applied after the combination */
    float diff_lambda, diff_init;
    /* linear recurrence with a constant decay per head (rec_kind TL_REC_FIXED; rotation by rot_dims / rot_base / rot_half / rot_factor ...) */
    const float *decay_dev; /* [heads] */
    /* the block with norms on both sides of a sublayer (TL_BLOCK_SANDWICH): RMS weights on the mixer's / feed-forward's result */
    const float *post_norm_dev, *post_norm2_dev; /* [width] */
    /* per-layer token input (all NULL / 0: none) */
    const void *side_gate_dev;  /* [side_dim, width] engine dtype */
    const void *side_proj_dev;  /* [width, side_dim] engine dtype */
    const float *side_norm_dev; /* [width], plain weight */
    int side_col0;              /* first of the layer's side_dim columns in the side embedding table */
} tl_hybrid_layer;

typedef struct tl_hybrid_config {
    int dtype;              /* TL_HY_BF16 or TL_HY_F32 */
    int width, vocab, num_layers;
    float norm_eps, residual_mult;
    int parallel_block;     /* TL_BLOCK_*: 1: x += m * (mixer(h) + ff(h)) with one norm; 0: x += m ls1 mixer(norm1 x), then x += m ls2 ff(norm2 x);
                               2: x += m norm1(mixer(x)), then x += m norm2(ff(x)) */
    int loop_start, loop_stop, loop_times; /* loop_times <= 1 or start == stop: no loop */
    const void *loop_in_dev;    /* [width, 2*width], stream first */
    const float *loop_step_dev; /* [loop_times, width] */
    const void *embed_dev;      /* [vocab, width] */
    const float *final_norm_dev;
    float final_norm_offset;
    const void *head_dev;       /* [vocab, width] */
    float embed_scale;          /* x = embed[token] * embed_scale (0 is read as 1) */
    int final_norm_kind;        /* TL_NORM_* */
    float final_norm_alpha;
    const float *final_norm_bias_dev;
    int page_size, num_pages, max_slots, max_pages_per_seq, max_rows;
    float logit_scale;          /* logits = head . norm(x) * logit_scale (0 is read as 1) */
    const float *embed_norm_dev; /* [width]: x = rms_norm(embed[token] * embed_scale) * (final_norm_offset + w); NULL: none */
    const void *side_embed_dev;  /* [vocab, side_cols] engine dtype: the table of the per-layer token inputs */
    int side_cols, side_dim;     /* columns of a table row; columns one layer reads */
} tl_hybrid_config;

typedef struct tl_hybrid_stats {
    int pages_in_use, pages_free, peak_pages_in_use;
    long page_allocations, reused_page_allocations;
    long steps, rows, slot_begins, reused_slot_begins;
    size_t kv_bytes, state_bytes, workspace_bytes;
    int layer_runs;
    long graph_captures, graph_replays;
} tl_hybrid_stats;

const char *tl_hybrid_last_error(void);

/* Weight memory is borrowed and must outlive the engine.  stream: the hipStream_t all work is issued on; NULL makes
 * the engine create and own one. */
int tl_hybrid_create(const tl_hybrid_config *cfg, const tl_hybrid_layer *layers, void *stream, tl_hybrid **out);
void tl_hybrid_destroy(tl_hybrid *e);
int tl_hybrid_synchronize(tl_hybrid *e);

/* begin: claim a free slot, context 0, recurrent state and convolution inputs zeroed.  release: pages back to the
 * free list; the slot may be claimed again. */
int tl_hybrid_begin(tl_hybrid *e, int slot);
int tl_hybrid_release(tl_hybrid *e, int slot);
int tl_hybrid_context_len(const tl_hybrid *e, int slot);
/* The sequence of the live slot `src` changes hands to the free slot `dst`: block-table row, context length and pending
 * token move, K/V pages stay; the recurrent state and convolution inputs of every delta layer run are copied. */
int tl_hybrid_move(tl_hybrid *e, int src, int dst);

/* One packed step.  tokens = the chunks back to back, lens[i] tokens for slots[i] (distinct, live) at positions
 * [context_i, context_i + lens[i]); sum(lens) <= max_rows.  want_rows[j] = index into the packed rows whose logits
 * are computed: row j of the logits buffer.  All-or-nothing: everything is checked and pages are reserved before
 * anything runs.  Enqueues only; the logits are read with tl_hybrid_copy_logits / tl_hybrid_read_argmax. */
int tl_hybrid_step(tl_hybrid *e, int n_seqs, const int *slots, const int32_t *tokens, const int *lens, int n_want,
                   const int *want_rows);

/* Greedy decode of the live slots listed: each slot's pending token (tl_hybrid_set_token, or the argmax of its last
 * wanted row) is fed as a one-token chunk; the argmax of its logits becomes the new pending token.  `steps` steps are
 * enqueued without host involvement between them (captured in a hipGraph per batch shape where use_graph != 0). */
int tl_hybrid_decode(tl_hybrid *e, int n_seqs, const int *slots, int steps, int use_graph);
int tl_hybrid_set_token(tl_hybrid *e, int slot, int32_t token);
/* Pending token of each listed slot after synchronising. */
int tl_hybrid_read_pending(tl_hybrid *e, int n, const int *slots, int32_t *out);

/* Stream-ordered copy of the first `rows` rows of the latest logits [rows, vocab] float32 to device or host memory;
 * the host form synchronises. */
int tl_hybrid_copy_logits(tl_hybrid *e, void *dst_dev, int rows);
int tl_hybrid_read_logits(tl_hybrid *e, float *dst_host, int rows);
/* argmax of the first `rows` logits rows; synchronises. */
int tl_hybrid_read_argmax(tl_hybrid *e, int rows, int32_t *out);

/* Test aid: the residual stream after layer run `run` of the latest step ([rows, width] float32) is kept when
 * tracing is on (one extra copy per layer run). */
int tl_hybrid_set_trace(tl_hybrid *e, int on);
int tl_hybrid_read_trace(tl_hybrid *e, int run, float *dst_host, int rows);

int tl_hybrid_get_stats(const tl_hybrid *e, tl_hybrid_stats *out);

/* Kernel-level entry points on caller buffers (tests, microbenchmarks).  dtype as in the config. */
int tl_hybrid_linear(int dtype, const void *a_dev, int lda, const void *w_dev, float *out_dev, int ldc, int M, int N, int K,
                     int force_kernel /* 0 by shape, 1 row kernel, 2 64-wide tile kernel, 3 256-wide tile GEMM (bfloat16) */, void *stream);

#ifdef __cplusplus
}
#endif
#endif
