// The layer-list engine (include/tinyllm_hybrid.h): host side.
//   * layer runs: the layer list unrolled over the loop passes; every run owns its K/V pages (attention) or state slots (delta)
//   * page pool + slots (page_pool.h), block table mirrored to the device when it changes
//   * one packed step function for prefill chunks, decode tokens and mixtures; a device-resident greedy decode loop on top of it,
//     captured in a hipGraph per slot list
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "../../include/tinyllm_hybrid.h"
#include "common.h"
#include "gemm8.h"
#include "hybrid_kernels.h"
#include "page_pool.h"

#define HY_HIP(call)                                                                                   \
    do {                                                                                               \
        hipError_t e__ = (call);                                                                       \
        if (e__ != hipSuccess) return ::tl::fail(TL_ERR_HIP, std::string(#call) + ": " + hipGetErrorString(e__)); \
    } while (0)
#define HY_TRY(call)              \
    do {                          \
        int s__ = (call);         \
        if (s__ != 0) return s__; \
    } while (0)

namespace tl {
int qmm3_num_cus() {  // gemm8.hip sizes its persistent grid by the CU count
    static int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        return n;
    }();
    return cus;
}
namespace hy {

struct Run {
    int layer = 0;
    int pass = -1;            // loop pass this run belongs to, -1 outside the loop
    bool enters_pass = false; // the loop-entry projection + pass offset come right before this run
    void *kpool = nullptr, *vpool = nullptr;      // attention: [pages, G, page, dim] / [pages, G, page, vdim] of the engine dtype
    float *state = nullptr, *conv_state = nullptr; // delta: [slots, H, vdim, dim] / [slots, taps-1, C]
                                                   // linrec: [slots, H, vdim (+1), dim] / the gates' running maximum [slots, H]
    // latent: kpool = [pages, page, kv_rank + rot_dim] (vpool unused); with kv_from the pages of an earlier run (not owned)
};

struct Meta {  // device int32 arrays of one step
    int32_t *tokens, *row_seq, *row_pos, *seq_row0, *seq_slot, *want_rows, *want_slot;
};

}  // namespace hy
}  // namespace tl

struct tl_hybrid {
    tl_hybrid_config cfg{};
    std::vector<tl_hybrid_layer> layers;
    std::vector<tl::hy::Run> runs;
    std::vector<float *> inv_freq;  // per layer (attention with rotary positions), device
    std::vector<float> rot_mult;    // per layer: factor on cos and sin (rescaled frequencies)
    float *f32a = nullptr, *gates = nullptr, *idw = nullptr;  // [R, max_c] scratch (conv output, latent queries, channel decays); [R, H, 3]; [R]
    void *da = nullptr, *db = nullptr;                         // D-typed scratch rows: latents / low-rank inputs / attention read-out; plain queries
    hipStream_t stream = nullptr;
    bool owns_stream = false;
    std::unique_ptr<tl::PagePool> pool;
    bool table_dirty = true;
    int32_t *table_dev = nullptr;
    // workspace
    float *part_acc = nullptr, *part_ml = nullptr;  // attention partials of split key ranges: [max_slots, heads, 64, vdim] / [..., 2]
    bool attn_rows_only = false;                    // TL_HYBRID_ATTN_ROWS=1: the one-wave-per-row attention everywhere (A/B twin of the tile kernel)
    float *x = nullptr, *x0 = nullptr, *proj = nullptr, *qbuf = nullptr, *obuf = nullptr, *logits = nullptr;
    unsigned long long *moe_mask = nullptr;  // which experts the rows of a small step take (SegSkip)
    float *y = nullptr;     // [R, width] a branch's result ahead of its norm (the block with the norm on the branch's output)
    float *vref = nullptr;  // [R, G * vdim] the values of the step's rows in the first value-mixing layer
    void *h = nullptr, *cat = nullptr, *cat2 = nullptr, *hsel = nullptr;
    int ld_proj = 0, ld_cat = 0;
    int32_t *meta_dev = nullptr, *meta_host = nullptr;  // step metadata (host side pinned)
    int32_t *dmeta_dev = nullptr;                        // decode-loop metadata (its own copy: captured graphs point into it)
    int32_t *ctx_dev = nullptr, *pending_dev = nullptr, *argmax_dev = nullptr;
    tl::hy::Meta meta{}, dmeta{};
    int last_rows = 0;
    // trace of the residual stream
    bool trace = false;
    float *trace_buf = nullptr;
    int trace_rows = 0;
    // decode graphs by slot list
    std::map<std::vector<int>, hipGraphExec_t> graphs;
    std::vector<int> dmeta_slots;  // the slot list dmeta currently describes
    tl_hybrid_stats stats{};
    std::vector<void *> allocs;
};

namespace tl {
namespace hy {

static size_t esize(int dtype) { return dtype == TL_HY_BF16 ? 2 : 4; }

static int attn_maps(const tl_hybrid_layer &L) { return L.diff_maps ? 2 : 1; }  // query / key maps per head
static int gate_cols(const tl_hybrid_layer &L) { return L.gated == 2 ? L.heads : (L.gated ? L.heads * L.vdim : 0); }
static int mixer_cols(const tl_hybrid_layer &L) {  // rows of w_in that belong to the mixer
    if (L.kind == TL_MIX_ATTENTION) return attn_maps(L) * (L.heads + L.kv_heads) * L.dim + L.kv_heads * L.vdim + gate_cols(L);
    if (L.kind == TL_MIX_LINREC)
        return 2 * L.heads * L.dim + 2 * L.heads * L.vdim + (L.rec_kind == TL_REC_EXPGATE ? 2 * L.heads : (L.rec_kind == TL_REC_CHANNEL ? L.a_rank : 0));
    if (L.kind == TL_MIX_LATENT) return L.q_rank + (L.kv_from < 0 ? L.kv_rank + L.rot_dim : 0) + (L.gated ? L.heads * L.vdim : 0);
    return 2 * L.kv_heads * L.dim + 2 * L.heads * L.vdim + 2 * L.heads;
}
static int ff_in_cols(const tl_hybrid_layer &L) {  // rows of the feed-forward's input matrix
    if (L.ff <= 0) return 0;
    if (L.ff_kind == TL_FF_GATED) return 2 * L.ff;
    if (L.ff_kind == TL_FF_MOE && L.moe_gated) return (2 * L.ff + L.experts + L.identity + (L.moe_shared_sg ? 1 : 0) + 7) / 8 * 8;
    if (L.ff_kind == TL_FF_MOE) return (L.shared_ff + L.experts * L.expert_ff + L.experts + L.identity + 1 + 7) / 8 * 8;
    return L.ff;
}
static int conv_channels(const tl_hybrid_layer &L) { return 2 * L.kv_heads * L.dim + L.heads * L.vdim; }
// floats of one sequence's recurrent state, and of what travels beside it (delta: the convolution's last inputs; expgate: the running maximum)
static size_t state_floats(const tl_hybrid_layer &L) {
    if (L.kind == TL_MIX_LINREC) return (size_t)L.heads * L.dim * (L.vdim + (L.rec_kind == TL_REC_EXPGATE ? 1 : 0));
    return (size_t)L.heads * L.dim * L.vdim;
}
static size_t aux_floats(const tl_hybrid_layer &L) {
    if (L.kind == TL_MIX_LINREC) return (size_t)L.heads;
    return (size_t)std::max(1, L.conv_taps - 1) * conv_channels(L);
}

template <typename T>
static int dev_alloc(tl_hybrid *e, T **p, size_t count, bool zero = false) {
    void *q = nullptr;
    HY_HIP(hipMalloc(&q, std::max<size_t>(count, 1) * sizeof(T)));
    e->allocs.push_back(q);
    *p = (T *)q;
    if (zero) HY_HIP(hipMemset(q, 0, std::max<size_t>(count, 1) * sizeof(T)));  // at creation only, never inside a captured region
    return TL_OK;
}

static Meta carve(int32_t *base, int R, int S) {
    Meta m;
    m.tokens = base;
    m.row_seq = base + R;
    m.row_pos = base + 2 * R;
    m.want_rows = base + 3 * R;
    m.want_slot = base + 4 * R;
    m.seq_row0 = base + 5 * R;
    m.seq_slot = base + 5 * R + S + 1;
    return m;
}
static size_t meta_ints(int R, int S) { return (size_t)5 * R + 2 * S + 2; }

// a Dynamic Tanh norm that may leave with the product completing a residual sum (epilogue 4 of the row and 64-wide tile kernels)
struct NormTail {
    const float *w = nullptr, *b = nullptr;
    float alpha = 0.f;
    void *out = nullptr;   // D rows of N
    bool done = false;     // set by linear_t when the product carried it
};

// out (+)= A . W^T by shape: a few rows stream the weights once per column (row kernel), more go through the MFMA tile kernel
template <typename D>
static int linear_t(const void *A, int lda, const void *W, float *out, int ldc, int M, int N, int K, int epi, float alpha, const float *bias,
                    int force, hipStream_t st, int batch = 1, long sa = 0, long sw = 0, long sc = 0, NormTail *tail = nullptr, const SegSkip *skip = nullptr) {
    using S = typename D::storage;
    if (M <= 0 || N <= 0 || batch <= 0) return TL_OK;
    const int vec_ok = (K % 8 == 0) && (lda % 8 == 0) && ((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0) && sa % 8 == 0 && sw % 8 == 0;
    const bool rows = force == 1 || (force == 0 && M <= 8);
    TL_REQUIRE(!rows || M <= 8, "hybrid linear: the row kernel takes at most 8 rows");
    if constexpr (sizeof(S) == 2) {
        // large bf16 products: the framework's LDS-DMA 256-wide tile GEMM with its float32 epilogues (gemm8.h); dense operands, whole 64-wide K steps
        const bool big = force == 3 || (force == 0 && M >= 192);
        if (big && batch == 1 && lda == K && ldc == N && gemm8_applicable(M, N, K) && (size_t)M * N * 4 < (1ull << 31) &&
            (epi != 3 || (uintptr_t)bias % 16 == 0)) {
            Gemm8Args g{};
            g.a = (const uint16_t *)A, g.w = (const uint16_t *)W, g.M = M, g.N = N, g.K = K, g.out_f32 = out, g.alpha = alpha;
            if (epi == 3) g.col_scale = bias;
            if (launch_gemm8_bf16(g, (epi == 1 || epi == 3) ? EPI_F32_AXPY : EPI_F32_STORE, st) == 0) {
                if (epi == 2) {
                    const size_t n = (size_t)M * N;
                    hipLaunchKernelGGL(add_rowvec_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, out, bias, N, M);
                    TL_CHECK_LAUNCH("hybrid linear bias");
                }
                return TL_OK;
            }
        }
        TL_REQUIRE(force != 3, "hybrid linear: the 256-wide tile GEMM does not take this shape");
    }
    const bool with_tail = tail && tail->out && epi == 3 && batch == 1 && ldc == N;
    const float *nw = with_tail ? tail->w : nullptr, *nb = with_tail ? tail->b : nullptr;
    const float nalpha = with_tail ? tail->alpha : 0.f;
    S *nout = with_tail ? (S *)tail->out : nullptr;
#define HY_GEMM(KERN, E) \
    hipLaunchKernelGGL((KERN<D, E>), grid, block, 0, st, (const S *)A, lda, (const S *)W, out, ldc, M, N, K, alpha, bias, vec_ok, sa, sw, sc, nw, nb, nalpha, nout)
#define HY_GEMM_ROWS(E) \
    hipLaunchKernelGGL((gemm_rows_kernel<D, E>), grid, block, 0, st, (const S *)A, lda, (const S *)W, out, ldc, M, N, K, alpha, bias, vec_ok, sa, sw, sc, nw, nb, nalpha, nout, sk)
    if (rows) {
        dim3 grid((N + 3) / 4, batch), block(256);
        const SegSkip sk = skip ? *skip : SegSkip{};
        if (epi == 0) HY_GEMM_ROWS(0);
        else if (epi == 1) HY_GEMM_ROWS(1);
        else if (epi == 2) HY_GEMM_ROWS(2);
        else if (!with_tail) HY_GEMM_ROWS(3);
        else HY_GEMM_ROWS(4);
    } else {
        dim3 grid(((M + 63) / 64) * ((N + 63) / 64), batch), block(256);
        if (epi == 0) HY_GEMM(gemm_tile_kernel, 0);
        else if (epi == 1) HY_GEMM(gemm_tile_kernel, 1);
        else if (epi == 2) HY_GEMM(gemm_tile_kernel, 2);
        else if (!with_tail) HY_GEMM(gemm_tile_kernel, 3);
        else HY_GEMM(gemm_tile_kernel, 4);
    }
#undef HY_GEMM
#undef HY_GEMM_ROWS
    if (with_tail) tail->done = true;
    TL_CHECK_LAUNCH("hybrid linear");
    return TL_OK;
}

static int launch_delta(const tl_hybrid *e, const tl_hybrid_layer &L, const Run &run, const Meta &m, int n_seqs, int ldp) {
    // LPC lanes per state column with RPT key rows each: key_dim <= LPC * RPT.  The token loop is a dependency chain whose cost per wave hardly
    // depends on RPT, so the fewest lanes per column that still give every SIMD a wave: 64 while the step's columns are at most the SIMDs, then 32, then
    // a DPP row of 16 (also for narrow keys)
    const long cols = (long)L.heads * L.vdim * n_seqs, simds = 4 * (long)qmm3_num_cus();
    int lpc = cols <= simds ? 64 : (cols <= 2 * simds ? 32 : 16);
    while (lpc > 16 && lpc >= 2 * L.dim) lpc /= 2;  // no more lanes than key rows
    int rpt = 1;
    while (lpc * rpt < L.dim) rpt *= 2;
    TL_REQUIRE(lpc * rpt <= 1024, "hybrid delta: key width above 1024 is not supported");
    dim3 grid(L.heads, n_seqs, (L.vdim + 256 / lpc - 1) / (256 / lpc)), block(256);
    const int C = conv_channels(L);
    const int a0 = 2 * L.kv_heads * L.dim + 2 * L.heads * L.vdim, b0 = a0 + L.heads;
#define HY_DELTA(RPT, LPC)                                                                                                                  \
    hipLaunchKernelGGL((delta_kernel<RPT, LPC>), grid, block, 0, e->stream, e->f32a, C, e->proj, ldp, a0, b0, L.a_log_dev, L.dt_bias_dev, \
                       L.unit_eps, m.seq_row0, m.seq_slot, run.state, e->obuf, L.heads, L.kv_heads, L.dim, L.vdim)
#define HY_DELTA_R(LPC)                          \
    switch (rpt) {                               \
        case 1: HY_DELTA(1, LPC); break;         \
        case 2: HY_DELTA(2, LPC); break;         \
        case 4: HY_DELTA(4, LPC); break;         \
        case 8: HY_DELTA(8, LPC); break;         \
        default: HY_DELTA(16, LPC); break;       \
    }
    if (lpc == 64) {
        HY_DELTA_R(64)
    } else if (lpc == 32) {
        switch (rpt) {
            case 32: HY_DELTA(32, 32); break;
            default: HY_DELTA_R(32)
        }
    } else {
        switch (rpt) {
            case 32: HY_DELTA(32, 16); break;
            case 64: HY_DELTA(64, 16); break;
            default: HY_DELTA_R(16)
        }
    }
#undef HY_DELTA_R
#undef HY_DELTA
    TL_CHECK_LAUNCH("hybrid delta");
    return TL_OK;
}

struct StepShape {
    int rows, n_seqs, max_len;         // packed rows, sequences, longest chunk
    int n_splits = 1, keys_per_split = 1 << 30;  // attention: the key range of a row split over workgroups (decode steps over long contexts)
};

// how a step's attention splits the keys: only steps of single tokens, from 256 keys on; one 64-key tile per split, doubled until at most 64
// splits (a decode step is a few rows: its time is the chain of tiles a workgroup walks, so the chain is kept short and the chip full)
static void plan_splits(StepShape &sh, int ctx_bound) {
    sh.n_splits = 1;
    sh.keys_per_split = 1 << 30;
    if (sh.max_len != 1 || ctx_bound <= 256) return;
    int kps = 64;
    while ((ctx_bound + kps - 1) / kps > 64) kps *= 2;
    int n = 1;
    while (n * kps < ctx_bound) n *= 2;
    sh.n_splits = n;
    sh.keys_per_split = kps;
}

// what the attention core needs beyond the layer's sizes (the defaults are plain causal attention into D rows)
struct AttnExtra {
    int window = 0;          // > 0: sliding window
    int vshare = 1;          // K/V heads in a row that read one value head
    int gate_per_head = 0;   // the gate holds one number per head
    float *out32 = nullptr;  // float32 read-out [rows, heads, vdim] instead of D rows
};

// a windowed layer's split of the keys: a decode step sees at most `window` keys, whatever the context
static StepShape window_shape(const StepShape &sh, int window) {
    StepShape w = sh;
    if (window > 0 && sh.n_splits > 1) {
        const long covered = (long)sh.n_splits * sh.keys_per_split;
        plan_splits(w, (int)std::min<long>(covered, window));
    }
    return w;
}

template <typename D, int DK4, int VT>
static int launch_attn_tile(tl_hybrid *e, const tl_hybrid_layer &L, const void *kpool, const void *vpool, int v_row, const Meta &m, const StepShape &sh,
                            const float *gate, int ldg, void *out, int ldo, const AttnExtra &x) {
    using S = typename D::storage;
    const tl_hybrid_config &c = e->cfg;
    const int HG = L.heads / L.kv_heads;
    int HGB = 1;
    while (HGB < HG && HGB < 16) HGB *= 2;
    const int n_hblk = (HG + HGB - 1) / HGB, TQ = 64 / HGB;
    const size_t lds_tiles = (size_t)64 * ((sizeof(S) == 2 ? (4 * DK4 + 8) / 2 : 4 * DK4 + 4) + (16 * VT + 4)) * 4;  // K tile (bf16 as stored, or float32) + V tile (float32)
    int page_shift = -1;
    for (int b = 0; b < 30; ++b)
        if ((1 << b) == c.page_size) page_shift = b;
    const int vec_ok = L.dim % 8 == 0 && L.vdim % 8 == 0 && v_row % 8 == 0;
    // chunks whose rows fit one 16-row MFMA tile (decode steps): the four waves share the keys of a tile instead of the rows
    const bool wsplit = sh.max_len * HGB <= 16;
    const size_t lds = std::max(lds_tiles, (size_t)(128 + 4 * 64 * 4 * VT) * 4);
    const bool ext = x.window > 0 || x.vshare != 1 || x.gate_per_head || x.out32;  // (plain causal attention keeps a kernel of its own)
    auto kern = ext ? (wsplit ? attn_tile_kernel<D, DK4, VT, true, true> : attn_tile_kernel<D, DK4, VT, false, true>)
                    : (wsplit ? attn_tile_kernel<D, DK4, VT, true, false> : attn_tile_kernel<D, DK4, VT, false, false>);
    (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    dim3 grid((sh.max_len + TQ - 1) / TQ, L.kv_heads * n_hblk, sh.n_seqs * sh.n_splits);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, e->stream, e->qbuf, (const S *)kpool, (const S *)vpool, m.seq_row0, m.seq_slot, m.row_pos,
                       e->table_dev, c.max_pages_per_seq, c.page_size, L.heads, L.kv_heads, L.dim, L.vdim, L.scale, L.sink, HGB, n_hblk, sh.keys_per_split,
                       sh.n_splits, gate, ldg, (S *)out, ldo, e->part_acc, e->part_ml, page_shift, vec_ok, v_row, x.window, x.vshare, x.gate_per_head, x.out32);
    TL_CHECK_LAUNCH("hybrid attention tile");
    if (sh.n_splits > 1) {
        hipLaunchKernelGGL((attn_merge_kernel<D>), dim3(sh.rows, L.heads), dim3(64), 0, e->stream, e->part_acc, e->part_ml, sh.n_splits, L.heads, L.vdim, gate,
                           ldg, (S *)out, ldo, x.gate_per_head, x.out32);
        TL_CHECK_LAUNCH("hybrid attention merge");
    }
    return TL_OK;
}

// the attention core over one K/V pool by head widths: the MFMA tile kernel where its templates reach, the row kernel beyond
template <typename D>
static int attention_core(tl_hybrid *e, const tl_hybrid_layer &L, const void *kpool, const void *vpool, int v_row, const Meta &m, const StepShape &sh0,
                          const float *gate, int ldg, void *out, int ldo, const AttnExtra &x = AttnExtra{}) {
    using S = typename D::storage;
    const tl_hybrid_config &c = e->cfg;
    const StepShape sh = window_shape(sh0, x.window);
    const int dk4 = (L.dim + 3) / 4, vt_n = (L.vdim + 15) / 16;
    // the two 64-wide tile templates serve widths that are multiples of 8 (whole 16-byte chunks); other widths beyond the 32-wide template
    // take the row kernel (the tile kernel faulted on a 136 / 130-wide head in float32, cause not found), and float32 pages take the 16-tile
    // value template for every width beyond 8 tiles
    const bool whole_chunks = L.dim % 8 == 0 && L.vdim % 8 == 0 && v_row % 8 == 0;
    const bool beyond_mid = dk4 > 32 || vt_n > 8;
    const bool ext = x.window > 0 || x.vshare != 1 || x.gate_per_head || x.out32;
    // (the 64-wide templates are built for plain causal attention only: with a window, shared values or float32 read-outs the 16-tile one gave
    // wrong rows in decode steps, so those options stay on the templates up to 128 x 128 and take the row kernel beyond)
    if (e->attn_rows_only || dk4 > 64 || vt_n > 16 || (beyond_mid && (!whole_chunks || ext))) {
        hipLaunchKernelGGL((attn_rows_kernel<D>), dim3(sh.rows, L.heads), dim3(64), (L.dim + 64) * sizeof(float), e->stream, e->qbuf, (const S *)kpool,
                           (const S *)vpool, m.row_seq, m.row_pos, m.seq_slot, e->table_dev, c.max_pages_per_seq, c.page_size, L.heads, L.kv_heads, L.dim,
                           L.vdim, L.scale, L.sink, gate, ldg, (S *)out, ldo, v_row, x.window, x.vshare, x.gate_per_head, x.out32);
        TL_CHECK_LAUNCH("hybrid attention");
        return TL_OK;
    }
    if (dk4 <= 16 && vt_n <= 4) return launch_attn_tile<D, 16, 4>(e, L, kpool, vpool, v_row, m, sh, gate, ldg, out, ldo, x);
    if (dk4 <= 32 && vt_n <= 8) return launch_attn_tile<D, 32, 8>(e, L, kpool, vpool, v_row, m, sh, gate, ldg, out, ldo, x);
    if (vt_n <= 12 && sizeof(S) == 2) return launch_attn_tile<D, 64, 12>(e, L, kpool, vpool, v_row, m, sh, gate, ldg, out, ldo, x);  // (a 192-wide latent beside a 64-wide rotated part)
    return launch_attn_tile<D, 64, 16>(e, L, kpool, vpool, v_row, m, sh, gate, ldg, out, ldo, x);
}

static size_t attn_talk_lds(int es, int DK4, int VT, int G, int HGB) {
    const size_t HP = (size_t)G * HGB, QP = es == 2 ? (4 * DK4 + 8) / 2 : 4 * DK4 + 4;
    return std::max(HP * HP + (size_t)G * 16 * QP + 4 * (size_t)(16 * (16 * VT + 4) + 16 * (16 * G + 4)), (size_t)128 + 4 * 64 * 4 * VT + 4 * 16 * (16 * VT + 4)) * sizeof(float);
}

template <typename D, int DK4, int VT, int NP>
static int launch_attn_talk_tile(tl_hybrid *e, const tl_hybrid_layer &L, const void *kpool, const void *vpool, const Meta &m, const StepShape &sh,
                                 const float *gate, int ldg, void *out, int ldo, int HGB) {
    using S = typename D::storage;
    const tl_hybrid_config &c = e->cfg;
    const int TQB = 16 / HGB;
    const size_t lds = attn_talk_lds((int)sizeof(S), DK4, VT, L.kv_heads, HGB);
    int page_shift = -1;
    for (int b = 0; b < 30; ++b)
        if ((1 << b) == c.page_size) page_shift = b;
    const int vec_ok = L.dim % 8 == 0 && L.vdim % 8 == 0;
    auto kern = attn_talk_tile_kernel<D, DK4, VT, NP>;
    (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    dim3 grid((sh.max_len + TQB - 1) / TQB, (L.kv_heads + NP - 1) / NP, sh.n_seqs * sh.n_splits);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, e->stream, e->qbuf, (const S *)kpool, (const S *)vpool, m.seq_row0, m.seq_slot, m.row_pos, e->table_dev,
                       c.max_pages_per_seq, c.page_size, L.heads, L.kv_heads, L.dim, L.vdim, L.scale, L.talk_dev, L.sink, L.sink_dev, L.chunk, HGB,
                       sh.keys_per_split, sh.n_splits, gate, ldg, (S *)out, ldo, e->part_acc, e->part_ml, page_shift, vec_ok);
    TL_CHECK_LAUNCH("hybrid attention tile (mixed heads)");
    if (sh.n_splits > 1) {
        hipLaunchKernelGGL((attn_merge_kernel<D>), dim3(sh.rows, L.heads), dim3(64), 0, e->stream, e->part_acc, e->part_ml, sh.n_splits, L.heads, L.vdim, gate,
                           ldg, (S *)out, ldo, 0, (float *)nullptr);
        TL_CHECK_LAUNCH("hybrid attention merge");
    }
    return TL_OK;
}

// attention whose scores are mixed across heads, whose mask is chunked or whose sinks are learned: every query head of a token in one workgroup.
// The MFMA tile kernel where its templates reach (head groups of at most 16, at most 64 padded heads, dim and vdim up to 128, its LDS within a CU's);
// the row kernel (a workgroup per row, a wave per head) beyond, and as the A/B twin (TL_HYBRID_ATTN_ROWS=1)
template <typename D>
static int attention_talk(tl_hybrid *e, const tl_hybrid_layer &L, const void *kpool, const void *vpool, const Meta &m, const StepShape &sh, const float *gate,
                          int ldg, void *out, int ldo) {
    using S = typename D::storage;
    const tl_hybrid_config &c = e->cfg;
    const int HG = L.heads / L.kv_heads, G = L.kv_heads, dk4 = (L.dim + 3) / 4, vt_n = (L.vdim + 15) / 16;
    int HGB = 1;
    while (HGB < HG) HGB *= 2;
    const bool narrow = dk4 <= 16 && vt_n <= 4, mid = dk4 <= 32 && vt_n <= 8;
    if (!e->attn_rows_only && HGB <= 16 && G * HGB <= 64 && (narrow || mid) &&
        attn_talk_lds((int)sizeof(S), narrow ? 16 : 32, narrow ? 4 : 8, G, HGB) <= 160 * 1024) {
        // blocks a workgroup weighs and multiplies: one for steps of single tokens (a short chain per workgroup, the K/V heads side by side), up to four for prompts
        const int np = sh.max_len == 1 ? (G > 4 ? 2 : 1) : (G >= 4 ? 4 : (G >= 2 ? 2 : 1));
#define HY_TALK(DK, VTT)                                                                                                   \
    switch (np) {                                                                                                          \
        case 1: return launch_attn_talk_tile<D, DK, VTT, 1>(e, L, kpool, vpool, m, sh, gate, ldg, out, ldo, HGB);          \
        case 2: return launch_attn_talk_tile<D, DK, VTT, 2>(e, L, kpool, vpool, m, sh, gate, ldg, out, ldo, HGB);          \
        default: return launch_attn_talk_tile<D, DK, VTT, 4>(e, L, kpool, vpool, m, sh, gate, ldg, out, ldo, HGB);         \
    }
        if (narrow) {
            HY_TALK(16, 4)
        }
        HY_TALK(32, 8)
#undef HY_TALK
    }
    const int nw = std::min(16, L.heads);
    const size_t lds = ((size_t)L.heads * L.dim + (size_t)L.heads * 64 + (size_t)nw * 64) * sizeof(float);
    TL_REQUIRE(lds <= 160 * 1024, "hybrid attention: heads * dim too large for the head-mixing kernel");
    auto kern = attn_talk_rows_kernel<D>;
    if (lds > 48 * 1024) (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(kern, dim3(sh.rows), dim3(64 * nw), lds, e->stream, e->qbuf, (const S *)kpool, (const S *)vpool, m.row_seq, m.row_pos, m.seq_slot,
                       e->table_dev, c.max_pages_per_seq, c.page_size, L.heads, L.kv_heads, L.dim, L.vdim, L.scale, L.talk_dev, L.sink, L.sink_dev, L.chunk, gate,
                       ldg, (S *)out, ldo);
    TL_CHECK_LAUNCH("hybrid attention (mixed heads)");
    return TL_OK;
}

static int launch_linrec(const tl_hybrid *e, const tl_hybrid_layer &L, const Run &run, const Meta &m, int n_seqs, int ldp) {
    const bool chan = L.rec_kind == TL_REC_CHANNEL;
    const int ones = L.rec_kind == TL_REC_EXPGATE ? 1 : 0, VE = L.vdim + ones;
    // lanes per state column: a wave while the step's columns are few (decode), a DPP row of 16 otherwise (or for narrow keys)
    const long cols = (long)L.heads * VE * n_seqs, simds = 4 * (long)qmm3_num_cus();
    int lpc = cols <= simds ? 64 : (cols <= 2 * simds + simds / 8 ? 32 : 16);
    while (lpc > 16 && lpc >= 2 * L.dim) lpc /= 2;  // no more lanes than key rows
    while (lpc < 64 && lpc * 16 < L.dim) lpc *= 2;  // at most 16 rows a lane
    int rpt = 1;
    while (lpc * rpt < L.dim) rpt *= 2;
    TL_REQUIRE(rpt <= 16, "hybrid linrec: key width above 1024 is not supported");
    dim3 grid(L.heads, n_seqs, (VE + 256 / lpc - 1) / (256 / lpc)), block(256);
    const int q0 = 0, k0 = L.heads * L.dim, v0 = 2 * L.heads * L.dim;
#define HY_LR(RPT, LPC, CHAN)                                                                                                                      \
    hipLaunchKernelGGL((linrec_kernel<RPT, LPC, CHAN>), grid, block, 0, e->stream, e->proj, ldp, q0, k0, v0, e->gates, e->f32a, m.seq_row0, m.seq_slot, \
                       run.state, e->obuf, L.heads, L.dim, L.vdim, ones)
#define HY_LR_R(LPC, CHAN)                    \
    switch (rpt) {                            \
        case 1: HY_LR(1, LPC, CHAN); break;   \
        case 2: HY_LR(2, LPC, CHAN); break;   \
        case 4: HY_LR(4, LPC, CHAN); break;   \
        case 8: HY_LR(8, LPC, CHAN); break;   \
        default: HY_LR(16, LPC, CHAN); break; \
    }
    if (lpc == 64) {
        if (chan) { HY_LR_R(64, true) } else { HY_LR_R(64, false) }
    } else if (lpc == 32) {
        if (chan) { HY_LR_R(32, true) } else { HY_LR_R(32, false) }
    } else {
        if (chan) { HY_LR_R(16, true) } else { HY_LR_R(16, false) }
    }
#undef HY_LR_R
#undef HY_LR
    TL_CHECK_LAUNCH("hybrid linrec");
    return TL_OK;
}

template <typename D>
static int norm_t(tl_hybrid *e, int kind, const float *w, const float *b, float alpha, float offset, void *out, const int32_t *rows_idx, int rows) {
    using S = typename D::storage;
    const tl_hybrid_config &c = e->cfg;
    // (a few rows: more threads per row, one pass of loads in flight instead of several in a row)
    if (kind == TL_NORM_DYT) hipLaunchKernelGGL((dyt_kernel<D>), dim3(rows), dim3(rows < 64 ? 1024 : 256), 0, e->stream, e->x, w, b, alpha, (S *)out, c.width, rows_idx);
    else hipLaunchKernelGGL((norm_kernel<D>), dim3(rows), dim3(rows < 64 ? 1024 : 256), 0, e->stream, e->x, w, offset, c.norm_eps, (S *)out, c.width, rows_idx);
    TL_CHECK_LAUNCH("hybrid norm");
    return TL_OK;
}

// the token mixer of one layer run: proj [rows, ldp] (every projection of the normed input) -> cat[:, 0 .. heads * vdim) as D rows of ldcat
template <typename D>
static int mixer_t(tl_hybrid *e, size_t ri, const Meta &m, const StepShape &sh, int ldp, int ldcat) {
    using S = typename D::storage;
    const Run &run = e->runs[ri];
    const tl_hybrid_layer &L = e->layers[run.layer];
    const tl_hybrid_config &c = e->cfg;
    hipStream_t st = e->stream;
    const int rows = sh.rows, n_seqs = sh.n_seqs, H = L.heads, HV = L.heads * L.vdim;
    if (L.kind == TL_MIX_ATTENTION) {
        const int G = L.kv_heads;
        if (L.diff_maps || L.qk_head_norm || L.window > 0 || L.gated == 2) {
            // q / k normed per head ahead of the rotation, maps side by side, a window on the keys, one gate per head
            const int M = attn_maps(L);
            hipLaunchKernelGGL((attn_prep_head_kernel<D>), dim3(rows, M * (H + G) + G), dim3(64), 0, st, e->proj, ldp, m.row_seq, m.row_pos, m.seq_slot, e->table_dev,
                               c.max_pages_per_seq, c.page_size, e->inv_freq[run.layer], L.rot_dims, L.rot_half, L.qk_head_norm, L.q_norm_dev, L.k_norm_dev, c.norm_eps,
                               H, G, M, L.dim, L.vdim, e->qbuf, (S *)run.kpool, (S *)run.vpool, L.w_in_bias_dev);
            TL_CHECK_LAUNCH("hybrid attention prep (per-head norm)");
            const float *gate = L.gated ? e->proj + (size_t)M * (H + G) * L.dim + (size_t)G * L.vdim : nullptr;
            AttnExtra x;
            x.window = L.window, x.vshare = M, x.gate_per_head = L.gated == 2;
            if (!L.diff_maps) return attention_core<D>(e, L, run.kpool, run.vpool, L.vdim, m, sh, gate, ldp, e->cat, ldcat, x);
            tl_hybrid_layer A = L;  // every map is a head of its own over M * G K/V heads; the read-outs stay float32 for the combination
            A.heads = M * H, A.kv_heads = M * G;
            x.out32 = e->obuf;
            HY_TRY(attention_core<D>(e, A, run.kpool, run.vpool, L.vdim, m, sh, nullptr, 0, nullptr, 0, x));
            hipLaunchKernelGGL((diff_combine_kernel<D>), dim3(rows, H), dim3(64), 0, st, e->obuf, L.diff_lambda, L.diff_init, c.norm_eps, gate, ldp, x.gate_per_head, H, G,
                               L.vdim, (S *)e->cat, ldcat);
            TL_CHECK_LAUNCH("hybrid differential combination");
            return TL_OK;
        }
        if (L.qk_norm || L.rot_half || L.v_mix != TL_VMIX_NONE)  // (options of the row-wise preparation; create checked that it covers the layer)
            hipLaunchKernelGGL((attn_prep_row_kernel<D>), dim3(rows), dim3(rows < 64 ? 1024 : 256), 0, st, e->proj, ldp, m.row_seq, m.row_pos, m.seq_slot, e->table_dev,
                               c.max_pages_per_seq, c.page_size, e->inv_freq[run.layer], L.rot_dims, L.rot_half, L.qk_norm, L.q_norm_dev, L.k_norm_dev,
                               c.norm_eps, H, G, L.dim, L.vdim, L.v_mix, L.v_mix_lambda, e->vref, e->qbuf, (S *)run.kpool, (S *)run.vpool);
        else
            hipLaunchKernelGGL((attn_prep_kernel<D>), dim3(rows, H + 2 * G), dim3(64), 0, st, e->proj, ldp, m.row_seq, m.row_pos, m.seq_slot,
                               e->table_dev, c.max_pages_per_seq, c.page_size, e->inv_freq[run.layer], L.rot_dims, L.qk_unit_rms, c.norm_eps, H, G, L.dim,
                               L.vdim, e->qbuf, (S *)run.kpool, (S *)run.vpool);
        TL_CHECK_LAUNCH("hybrid attention prep");
        const float *gate = L.gated ? e->proj + (size_t)(H + G) * L.dim + (size_t)G * L.vdim : nullptr;
        if (L.talk_dev || L.sink_dev || L.chunk > 0) return attention_talk<D>(e, L, run.kpool, run.vpool, m, sh, gate, ldp, e->cat, ldcat);
        return attention_core<D>(e, L, run.kpool, run.vpool, L.vdim, m, sh, gate, ldp, e->cat, ldcat);
    }
    if (L.kind == TL_MIX_LATENT) {
        // proj: dq (q_rank) | [dkv (kv_rank + rot_dim)] | gate (H * vdim)
        const int own = L.kv_from < 0, kv0 = L.q_rank, g0 = L.q_rank + (own ? L.kv_rank + L.rot_dim : 0), DT = L.kv_rank + L.rot_dim, DQ = L.dim + L.rot_dim;
        hipLaunchKernelGGL((rms_cols_kernel<D>), dim3(rows), dim3(rows < 64 ? 512 : 128), 0, st, e->proj, ldp, L.q_rank, L.dq_norm_dev, c.norm_eps, (S *)e->da, L.q_rank);
        TL_CHECK_LAUNCH("hybrid latent query norm");
        HY_TRY(linear_t<D>(e->da, L.q_rank, L.uq_dev, e->f32a, H * DQ, rows, H * DQ, L.q_rank, 0, 1.f, nullptr, 0, st));
        hipLaunchKernelGGL((latent_prep_kernel<D>), dim3(rows, H + 1), dim3(64), 0, st, e->f32a, H, L.dim, L.rot_dim, L.kv_rank, e->proj, ldp, kv0,
                           L.dkv_norm_dev, c.norm_eps, own, m.row_seq, m.row_pos, m.seq_slot, e->table_dev, c.max_pages_per_seq, c.page_size,
                           e->inv_freq[run.layer], L.rot_dims, e->rot_mult[run.layer], (S *)e->db, e->qbuf, (S *)run.kpool);
        TL_CHECK_LAUNCH("hybrid latent prep");
        // the keys' per-head projection moves onto the query: q_h' = W_uk,h^T q_h  -> qbuf[t, h, 0 .. kv_rank)
        HY_TRY(linear_t<D>(e->db, H * L.dim, L.uk_t_dev, e->qbuf, H * DT, rows, L.kv_rank, L.dim, 0, 1.f, nullptr, 0, st, H, L.dim, (long)L.kv_rank * L.dim, DT));
        tl_hybrid_layer A = L;  // one K/V head: keys [c | rotated part], values = the keys' leading kv_rank columns
        A.kv_heads = 1, A.dim = DT, A.vdim = L.kv_rank, A.sink = 0;
        HY_TRY(attention_core<D>(e, A, run.kpool, run.kpool, DT, m, sh, nullptr, 0, e->da, H * L.kv_rank));
        // ... and the values' onto the read-out: o_h = W_uv,h (sum_j p_j c_j)
        HY_TRY(linear_t<D>(e->da, H * L.kv_rank, L.uv_dev, e->obuf, HV, rows, L.vdim, L.kv_rank, 0, 1.f, nullptr, 0, st, H, L.kv_rank, (long)L.vdim * L.kv_rank, L.vdim));
        const size_t n = (size_t)rows * HV;
        hipLaunchKernelGGL((gate_mul_kernel<D>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, e->obuf, HV, e->proj + g0, ldp, HV, L.gated ? 0 : 2, (S *)e->cat, ldcat, rows);
        TL_CHECK_LAUNCH("hybrid latent gate");
        return TL_OK;
    }
    if (L.kind == TL_MIX_LINREC) {
        // proj: q (H dim) | k (H dim) | v (H vdim) | gate (H vdim) | i (H) | f (H)   or   ... | a1 (a_rank)
        const int g0 = 2 * H * L.dim + HV, x0 = g0 + HV;
        const bool chan = L.rec_kind == TL_REC_CHANNEL;
        if (L.rec_kind == TL_REC_FIXED) {  // rotation of q and k, k * dim^-1/2, the constant decays as this step's gates
            hipLaunchKernelGGL(fixed_decay_prep_kernel, dim3(rows, H), dim3(64), 0, st, e->proj, ldp, 0, H * L.dim, m.row_pos, e->inv_freq[run.layer], L.rot_dims,
                               L.rot_half, 1.f / sqrtf((float)L.dim), L.decay_dev, e->gates, H, L.dim);
            TL_CHECK_LAUNCH("hybrid constant decay prep");
            HY_TRY(launch_linrec(e, L, run, m, n_seqs, ldp));
            hipLaunchKernelGGL((linrec_out_kernel<D>), dim3(rows, H), dim3(64), 0, st, e->obuf, L.vdim, 0, e->gates, 1.f, L.out_norm_dev, 0, c.norm_eps, e->proj + g0, ldp,
                               1, H, L.vdim, (S *)e->cat, ldcat);
            TL_CHECK_LAUNCH("hybrid linrec out");
            return TL_OK;
        }
        if (chan) {
            const size_t na = (size_t)rows * L.a_rank, nd = (size_t)rows * H * L.dim;
            hipLaunchKernelGGL((cast_cols_kernel<D>), dim3((unsigned)((na + 255) / 256)), dim3(256), 0, st, e->proj, ldp, x0, L.a_rank, (S *)e->da, L.a_rank, rows);
            TL_CHECK_LAUNCH("hybrid decay input");
            HY_TRY(linear_t<D>(e->da, L.a_rank, L.a2_dev, e->f32a, H * L.dim, rows, H * L.dim, L.a_rank, 0, 1.f, nullptr, 0, st));
            hipLaunchKernelGGL(channel_decay_kernel, dim3((unsigned)((nd + 255) / 256)), dim3(256), 0, st, e->f32a, L.a2_bias_dev, H * L.dim, 1.f / L.tau, rows);
            TL_CHECK_LAUNCH("hybrid channel decay");
        } else {
            hipLaunchKernelGGL(expgate_scan_kernel, dim3(n_seqs, H), dim3(64), 0, st, e->proj, ldp, x0, x0 + H, L.i_bias_dev, L.f_bias_dev, L.gate_cap,
                               m.seq_row0, m.seq_slot, run.conv_state, e->gates, H);
            TL_CHECK_LAUNCH("hybrid gate scan");
        }
        HY_TRY(launch_linrec(e, L, run, m, n_seqs, ldp));
        hipLaunchKernelGGL((linrec_out_kernel<D>), dim3(rows, H), dim3(64), 0, st, e->obuf, L.vdim + (chan ? 0 : 1), chan ? 0 : 1, e->gates,
                           1.f / sqrtf((float)L.dim), L.out_norm_dev, chan ? 0 : L.vdim, c.norm_eps, e->proj + g0, ldp, chan ? 1 : 0, H, L.vdim, (S *)e->cat,
                           ldcat);
        TL_CHECK_LAUNCH("hybrid linrec out");
        return TL_OK;
    }
    const int C = conv_channels(L);
    const size_t n = (size_t)rows * C;
    hipLaunchKernelGGL(conv_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, e->proj, ldp, L.conv_dev, L.conv_taps, C, m.row_seq,
                       m.seq_row0, m.seq_slot, run.conv_state, e->f32a, rows);
    TL_CHECK_LAUNCH("hybrid conv");
    if (L.conv_taps > 1) {
        hipLaunchKernelGGL(conv_state_kernel, dim3((unsigned)(((size_t)n_seqs * C + 255) / 256)), dim3(256), 0, st, e->proj, ldp, L.conv_taps, C,
                           m.seq_row0, m.seq_slot, run.conv_state, n_seqs);
        TL_CHECK_LAUNCH("hybrid conv state");
    }
    HY_TRY(launch_delta(e, L, run, m, n_seqs, ldp));
    const float *gate = e->proj + (size_t)C;
    hipLaunchKernelGGL((delta_out_kernel<D>), dim3(rows, L.heads), dim3(64), 0, st, e->obuf, L.out_norm_dev, c.norm_eps, gate, ldp, L.heads,
                       L.vdim, (S *)e->cat, ldcat);
    TL_CHECK_LAUNCH("hybrid delta out");
    return TL_OK;
}

// the feed-forward's activation: proj columns up0 .. -> cat columns col0 .. col0 + L.ff
template <typename D>
static int ff_act_t(tl_hybrid *e, const tl_hybrid_layer &L, int rows, int ldp, int up0, int ldcat, int col0) {
    using S = typename D::storage;
    hipStream_t st = e->stream;
    if (L.ff_kind == TL_FF_MOE) {
        const dim3 grid(rows, rows >= 64 ? 1 : std::max(1, std::min(64, L.ff / 1024)));
        if (L.moe_gated) {  // gates | ups | router | [scalar shared gate] | padding
            const int ET = L.experts + L.identity, r0 = up0 + 2 * L.ff;
            hipLaunchKernelGGL((moe_gated_act_kernel<D>), grid, dim3(256), 0, st, e->proj, ldp, r0, L.moe_shared_sg ? r0 + ET : -1, up0, up0 + L.ff, L.experts,
                               L.identity, L.top, L.groups, L.keep, L.expert_ff, L.shared_ff, L.correction_dev, (S *)e->cat, ldcat, col0, e->idw, L.moe_router,
                               L.moe_scale_input, L.ff_act);
            TL_CHECK_LAUNCH("hybrid moe route (gated experts)");
            return TL_OK;
        }
        const int ET = L.experts + L.identity, r0 = up0 + L.ff;  // shared up | expert ups | router | shared gate | padding
        hipLaunchKernelGGL((moe_route_act_kernel<D>), grid, dim3(256), 0, st, e->proj, ldp, r0, r0 + ET, up0, up0 + L.shared_ff,
                           L.experts, L.identity, L.top, L.groups, L.keep, L.expert_ff, L.shared_ff, L.correction_dev, (S *)e->cat, ldcat, col0, e->idw, L.moe_router);
        TL_CHECK_LAUNCH("hybrid moe route");
        return TL_OK;
    }
    const size_t n = (size_t)rows * L.ff;
    if (L.ff_kind == TL_FF_GATED)
        hipLaunchKernelGGL((ff_gated_act_kernel<D>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, e->proj, ldp, up0, up0 + L.ff, L.ff, L.ff_act,
                           (S *)e->cat, ldcat, col0, rows);
    else
        hipLaunchKernelGGL((ff_act_kernel<D>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, e->proj, ldp, up0, L.ff, L.ff_act, (S *)e->cat, ldcat, col0,
                           rows);
    TL_CHECK_LAUNCH("hybrid ff act");
    return TL_OK;
}

// every layer run over the packed rows described by m
template <typename D>
static int forward_t(tl_hybrid *e, const Meta &m, const StepShape &sh) {
    const int rows = sh.rows;
    using S = typename D::storage;
    const tl_hybrid_config &c = e->cfg;
    hipStream_t st = e->stream;
    const int W = c.width;
    hipLaunchKernelGGL((embed_kernel<D>), dim3(rows), dim3(256), 0, st, m.tokens, (const S *)c.embed_dev, e->x0, e->x, W, c.vocab,
                       c.embed_scale != 0.f ? c.embed_scale : 1.f, c.embed_norm_dev, c.final_norm_offset, c.norm_eps);
    TL_CHECK_LAUNCH("hybrid embed");
    bool h_ready = false;  // e->h already holds this run's first norm (it left with the product that completed the previous residual sum)
    // the Dynamic Tanh norm that follows a residual sum: element-wise, so it can ride the completing product's epilogue
    auto tail_for = [&](const float *w, const float *b, float alpha) {
        NormTail t;
        if (w && b) t.w = w, t.b = b, t.alpha = alpha, t.out = e->h;
        return t;
    };
    for (size_t ri = 0; ri < e->runs.size(); ++ri) {
        const Run &run = e->runs[ri];
        const tl_hybrid_layer &L = e->layers[run.layer];
        // the first norm of the run after this one, if it is a Dynamic Tanh that reads the stream as this run leaves it
        NormTail next_first;
        if (c.parallel_block == TL_BLOCK_SEQUENTIAL && ri + 1 < e->runs.size() && !e->runs[ri + 1].enters_pass) {
            const tl_hybrid_layer &Nx = e->layers[e->runs[ri + 1].layer];
            if (Nx.norm_kind == TL_NORM_DYT) next_first = tail_for(Nx.norm_dev, Nx.norm_bias_dev, Nx.norm_alpha);
        }
        if (run.enters_pass && !c.loop_in_dev) {  // x <- x + step[pass]
            const size_t n = (size_t)rows * W;
            hipLaunchKernelGGL(add_rowvec_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, e->x, c.loop_step_dev + (size_t)run.pass * W, W, rows);
            TL_CHECK_LAUNCH("hybrid pass offset");
        } else if (run.enters_pass) {  // x <- W_in [x ; x0] + step[pass]
            hipLaunchKernelGGL((pack2_kernel<D>), dim3(rows), dim3(256), 0, st, e->x, e->x0, (S *)e->cat2, W);
            TL_CHECK_LAUNCH("hybrid pack2");
            HY_TRY(linear_t<D>(e->cat2, 2 * W, c.loop_in_dev, e->x, W, rows, W, 2 * W, 2, 1.f, c.loop_step_dev + (size_t)run.pass * W, 0, st));
        }
        const int nmix = mixer_cols(L), HV = L.heads * L.vdim;
        if (c.parallel_block == TL_BLOCK_POSTNORM) {
            // x += m norm1(W_o mixer(x));  x += m norm2(ff(x)): the sublayers read the stream itself, the norm sits on what they return
            const size_t n = (size_t)rows * W;
            if (!h_ready) {
                hipLaunchKernelGGL((cast_rows_kernel<D>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, e->x, (S *)e->h, n);
                TL_CHECK_LAUNCH("hybrid stream cast");
            }
            HY_TRY(linear_t<D>(e->h, W, L.w_in_dev, e->proj, nmix, rows, nmix, W, 0, 1.f, nullptr, 0, st));
            HY_TRY(mixer_t<D>(e, ri, m, sh, nmix, HV));
            HY_TRY(linear_t<D>(e->cat, HV, L.w_out_dev, e->y, W, rows, W, HV, 0, 1.f, nullptr, 0, st));
            hipLaunchKernelGGL((postnorm_add_kernel<D>), dim3(rows), dim3(rows < 64 ? 1024 : 256), 0, st, e->x, e->y, L.norm_dev, L.norm_offset, c.norm_eps,
                               c.residual_mult, (S *)e->h, W);
            TL_CHECK_LAUNCH("hybrid norm on the mixer's output");
            if (L.ff > 0) {
                const int nin2 = ff_in_cols(L);
                // a step of a few rows takes few experts: the router's rows first, then only the experts some row takes are streamed
                const bool few = rows <= 8 && L.ff_kind == TL_FF_MOE && L.moe_gated && L.experts <= 64 && L.top < L.experts && L.expert_ff % 8 == 0 && L.shared_ff % 8 == 0 && e->moe_mask;
                if (few) {
                    HY_TRY(linear_t<D>(e->h, W, (const S *)L.w_in2_dev + (size_t)2 * L.ff * W, e->proj + 2 * L.ff, nin2, rows, nin2 - 2 * L.ff, W, 0, 1.f, nullptr, 0, st));
                    hipLaunchKernelGGL(moe_taken_mask_kernel, dim3(1), dim3(256), 0, st, e->proj, nin2, 2 * L.ff, rows, L.experts, L.identity, L.top, L.groups, L.keep,
                                       L.correction_dev, L.moe_router, e->moe_mask);
                    TL_CHECK_LAUNCH("hybrid moe taken experts");
                    SegSkip in_skip, out_skip;
                    in_skip.mask = out_skip.mask = e->moe_mask;
                    in_skip.lead = out_skip.lead = L.shared_ff, in_skip.len = out_skip.len = L.expert_ff;
                    in_skip.period = L.ff, in_skip.limit = 2 * L.ff, out_skip.on_k = 1;
                    HY_TRY(linear_t<D>(e->h, W, L.w_in2_dev, e->proj, nin2, rows, 2 * L.ff, W, 0, 1.f, nullptr, 0, st, 1, 0, 0, 0, nullptr, &in_skip));
                    HY_TRY(ff_act_t<D>(e, L, rows, nin2, 0, L.ff, 0));
                    HY_TRY(linear_t<D>(e->cat, L.ff, L.w_out2_dev, e->y, W, rows, W, L.ff, 0, 1.f, nullptr, 0, st, 1, 0, 0, 0, nullptr, &out_skip));
                } else {
                    HY_TRY(linear_t<D>(e->h, W, L.w_in2_dev, e->proj, nin2, rows, nin2, W, 0, 1.f, nullptr, 0, st));
                    HY_TRY(ff_act_t<D>(e, L, rows, nin2, 0, L.ff, 0));
                    HY_TRY(linear_t<D>(e->cat, L.ff, L.w_out2_dev, e->y, W, rows, W, L.ff, 0, 1.f, nullptr, 0, st));
                }
                if (L.ff_kind == TL_FF_MOE && L.identity > 0) {  // identity experts return their input: weight * h joins the branch ahead of its norm
                    hipLaunchKernelGGL((identity_axpy_kernel<D>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, e->y, (const S *)e->h, e->idw,
                                       (const float *)nullptr, 1.f, W, rows);
                    TL_CHECK_LAUNCH("hybrid identity experts");
                }
                hipLaunchKernelGGL((postnorm_add_kernel<D>), dim3(rows), dim3(rows < 64 ? 1024 : 256), 0, st, e->x, e->y, L.norm2_dev, L.norm_offset, c.norm_eps,
                                   c.residual_mult, (S *)e->h, W);
                TL_CHECK_LAUNCH("hybrid norm on the feed-forward's output");
            }
            h_ready = true;
            if (e->trace && e->trace_buf && rows <= c.max_rows)
                HY_HIP(hipMemcpyAsync(e->trace_buf + ri * (size_t)c.max_rows * W, e->x, (size_t)rows * W * 4, hipMemcpyDeviceToDevice, st));
            continue;
        }
        if (!h_ready) HY_TRY(norm_t<D>(e, L.norm_kind, L.norm_dev, L.norm_bias_dev, L.norm_alpha, L.norm_offset, e->h, nullptr, rows));
        h_ready = false;
        if (c.parallel_block == TL_BLOCK_SANDWICH) {
            // x += m ls1 post1(W_o mixer(norm1 x));  x += m ls2 post2(ff(norm2 x));  x += side(x).  Each sum's kernel also writes what reads the new
            // stream next: the feed-forward's norm, the stream itself for the token input, or the next run's first norm.
            const tl_hybrid_layer *Nx = (ri + 1 < e->runs.size() && !e->runs[ri + 1].enters_pass) ? &e->layers[e->runs[ri + 1].layer] : nullptr;
            const bool side = L.side_gate_dev != nullptr;
            const int threads = rows < 64 ? 1024 : 256;
            // (biases: the per-head preparation of an attention layer adds them where it reads q, k and v; any other mixer gets them with the product)
            const bool prep_adds_bias = L.kind == TL_MIX_ATTENTION && (L.diff_maps || L.qk_head_norm || L.window > 0 || L.gated == 2);
            HY_TRY(linear_t<D>(e->h, W, L.w_in_dev, e->proj, nmix, rows, nmix, W, L.w_in_bias_dev && !prep_adds_bias ? 2 : 0, 1.f, L.w_in_bias_dev, 0, st));
            HY_TRY(mixer_t<D>(e, ri, m, sh, nmix, HV));
            HY_TRY(linear_t<D>(e->cat, HV, L.w_out_dev, e->y, W, rows, W, HV, 0, 1.f, nullptr, 0, st));
            {
                const int next = L.ff > 0 ? 2 : (side ? 1 : (Nx ? 2 : 0));
                const float *nw = L.ff > 0 ? L.norm2_dev : (Nx ? Nx->norm_dev : nullptr);
                hipLaunchKernelGGL((sandwich_add_kernel<D>), dim3(rows), dim3(threads), 0, st, e->x, e->y, L.post_norm_dev, L.norm_offset, c.norm_eps, c.residual_mult,
                                   L.ls1_dev, next, nw, L.ff > 0 ? L.norm_offset : (Nx ? Nx->norm_offset : 0.f), (S *)e->h, W);
                TL_CHECK_LAUNCH("hybrid norm on the mixer's output");
                h_ready = L.ff <= 0 && !side && next == 2;
            }
            if (L.ff > 0) {
                const int nin2 = ff_in_cols(L);
                HY_TRY(linear_t<D>(e->h, W, L.w_in2_dev, e->proj, nin2, rows, nin2, W, 0, 1.f, nullptr, 0, st));
                HY_TRY(ff_act_t<D>(e, L, rows, nin2, 0, L.ff, 0));
                HY_TRY(linear_t<D>(e->cat, L.ff, L.w_out2_dev, e->y, W, rows, W, L.ff, 0, 1.f, nullptr, 0, st));
                const int next = side ? 1 : (Nx ? 2 : 0);
                hipLaunchKernelGGL((sandwich_add_kernel<D>), dim3(rows), dim3(threads), 0, st, e->x, e->y, L.post_norm2_dev, L.norm_offset, c.norm_eps, c.residual_mult,
                                   L.ls2_dev, next, Nx ? Nx->norm_dev : nullptr, Nx ? Nx->norm_offset : 0.f, (S *)e->h, W);
                TL_CHECK_LAUNCH("hybrid norm on the feed-forward's output");
                h_ready = !side && next == 2;
            }
            if (side) {  // y = W_proj (gelu_tanh(W_gate x) * e);  x += y / rms(y) * side_norm
                const int sd = c.side_dim;
                HY_TRY(linear_t<D>(e->h, W, L.side_gate_dev, e->proj, sd, rows, sd, W, 0, 1.f, nullptr, 0, st));
                const size_t n = (size_t)rows * sd;
                hipLaunchKernelGGL((side_act_kernel<D>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, e->proj, sd, m.tokens, (const S *)c.side_embed_dev, c.side_cols,
                                   L.side_col0, sd, c.vocab, (S *)e->cat, sd, rows);
                TL_CHECK_LAUNCH("hybrid token input");
                HY_TRY(linear_t<D>(e->cat, sd, L.side_proj_dev, e->y, W, rows, W, sd, 0, 1.f, nullptr, 0, st));
                hipLaunchKernelGGL((sandwich_add_kernel<D>), dim3(rows), dim3(threads), 0, st, e->x, e->y, L.side_norm_dev, 0.f, c.norm_eps, 1.f, (const float *)nullptr,
                                   Nx ? 2 : 0, Nx ? Nx->norm_dev : nullptr, Nx ? Nx->norm_offset : 0.f, (S *)e->h, W);
                TL_CHECK_LAUNCH("hybrid norm on the token input");
                h_ready = Nx != nullptr;
            }
        } else if (c.parallel_block == TL_BLOCK_PARALLEL) {
            const int nin = nmix + L.ff, ldcat = HV + L.ff;  // dense rows: a layer's buffers are as wide as the layer needs
            HY_TRY(linear_t<D>(e->h, W, L.w_in_dev, e->proj, nin, rows, nin, W, 0, 1.f, nullptr, 0, st));
            HY_TRY(mixer_t<D>(e, ri, m, sh, nin, ldcat));
            if (L.ff > 0) HY_TRY(ff_act_t<D>(e, L, rows, nin, nmix, ldcat, HV));
            // x += m * ([mixer out ; ff act] . [W_o | W_down]^T)
            HY_TRY(linear_t<D>(e->cat, ldcat, L.w_out_dev, e->x, W, rows, W, HV + L.ff, 1, c.residual_mult, nullptr, 0, st));
        } else {
            // x += m ls1 * W_o mixer(norm1 x);  x += m ls2 * ff(norm2 x)
            HY_TRY(linear_t<D>(e->h, W, L.w_in_dev, e->proj, nmix, rows, nmix, W, 0, 1.f, nullptr, 0, st));
            HY_TRY(mixer_t<D>(e, ri, m, sh, nmix, HV));
            NormTail second = (L.ff > 0 && L.norm_kind == TL_NORM_DYT) ? tail_for(L.norm2_dev, L.norm2_bias_dev, L.norm2_alpha) : NormTail{};
            NormTail *after_mixer = L.ff > 0 ? &second : &next_first;
            HY_TRY(linear_t<D>(e->cat, HV, L.w_out_dev, e->x, W, rows, W, HV, L.ls1_dev ? 3 : 1, c.residual_mult, L.ls1_dev, 0, st, 1, 0, 0, 0, after_mixer));
            if (L.ff > 0) {
                if (!second.done) HY_TRY(norm_t<D>(e, L.norm_kind, L.norm2_dev, L.norm2_bias_dev, L.norm2_alpha, L.norm_offset, e->h, nullptr, rows));
                const int nin2 = ff_in_cols(L);
                HY_TRY(linear_t<D>(e->h, W, L.w_in2_dev, e->proj, nin2, rows, nin2, W, 0, 1.f, nullptr, 0, st));
                HY_TRY(ff_act_t<D>(e, L, rows, nin2, 0, L.ff, 0));
                if (L.ff_kind == TL_FF_MOE && L.identity > 0) {  // (before the experts' product: that one completes the sum and may carry the next norm, which overwrites h)
                    const size_t n = (size_t)rows * W;
                    hipLaunchKernelGGL((identity_axpy_kernel<D>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, e->x, (const S *)e->h, e->idw, L.ls2_dev,
                                       c.residual_mult, W, rows);
                    TL_CHECK_LAUNCH("hybrid identity experts");
                }
                HY_TRY(linear_t<D>(e->cat, L.ff, L.w_out2_dev, e->x, W, rows, W, L.ff, L.ls2_dev ? 3 : 1, c.residual_mult, L.ls2_dev, 0, st, 1, 0, 0, 0, &next_first));
            }
            h_ready = next_first.done;
        }
        if (e->trace && e->trace_buf && rows <= c.max_rows)
            HY_HIP(hipMemcpyAsync(e->trace_buf + ri * (size_t)c.max_rows * W, e->x, (size_t)rows * W * 4, hipMemcpyDeviceToDevice, st));
    }
    return TL_OK;
}

// final norm on the wanted rows, head product, argmax (and the slots' next input tokens)
template <typename D>
static int head_t(tl_hybrid *e, const Meta &m, int n_want, bool set_pending) {
    const tl_hybrid_config &c = e->cfg;
    if (n_want <= 0) return TL_OK;
    HY_TRY(norm_t<D>(e, c.final_norm_kind, c.final_norm_dev, c.final_norm_bias_dev, c.final_norm_alpha, c.final_norm_offset, e->hsel, m.want_rows, n_want));
    HY_TRY(linear_t<D>(e->hsel, c.width, c.head_dev, e->logits, c.vocab, n_want, c.vocab, c.width, 0, 1.f, nullptr, 0, e->stream));
    if (c.logit_scale != 0.f && c.logit_scale != 1.f) {
        const size_t n = (size_t)n_want * c.vocab;
        hipLaunchKernelGGL(scale_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, e->stream, e->logits, c.logit_scale, n);
        TL_CHECK_LAUNCH("hybrid logit scale");
    }
    hipLaunchKernelGGL(argmax_kernel, dim3(n_want), dim3(1024), 0, e->stream, e->logits, c.vocab, e->argmax_dev, set_pending ? m.want_slot : (const int32_t *)nullptr,
                       e->pending_dev);
    TL_CHECK_LAUNCH("hybrid argmax");
    return TL_OK;
}

static int forward(tl_hybrid *e, const Meta &m, const StepShape &sh) {
    return e->cfg.dtype == TL_HY_BF16 ? forward_t<BF16>(e, m, sh) : forward_t<F32>(e, m, sh);
}
static int head(tl_hybrid *e, const Meta &m, int n_want, bool set_pending) {
    return e->cfg.dtype == TL_HY_BF16 ? head_t<BF16>(e, m, n_want, set_pending) : head_t<F32>(e, m, n_want, set_pending);
}

static int sync_table(tl_hybrid *e) {
    if (!e->table_dirty) return TL_OK;
    const auto &t = e->pool->table();
    // the pageable source is consumed before the call returns (no pinned staging to keep alive)
    HY_HIP(hipMemcpyAsync(e->table_dev, t.data(), t.size() * 4, hipMemcpyHostToDevice, e->stream));
    HY_HIP(hipStreamSynchronize(e->stream));
    e->table_dirty = false;
    return TL_OK;
}

static int check_slots(tl_hybrid *e, int n_seqs, const int *slots) {
    TL_REQUIRE(n_seqs >= 1 && n_seqs <= e->cfg.max_slots, "hybrid: between 1 and max_slots sequences per step");
    std::vector<char> seen(e->cfg.max_slots, 0);
    for (int i = 0; i < n_seqs; ++i) {
        TL_REQUIRE(slots[i] >= 0 && slots[i] < e->cfg.max_slots, "hybrid: slot out of range");
        TL_REQUIRE(e->pool->live(slots[i]), "hybrid: slot holds no sequence");
        TL_REQUIRE(!seen[slots[i]], "hybrid: a slot appears twice in one step");
        seen[slots[i]] = 1;
    }
    return TL_OK;
}

// pages for `extra[i]` more tokens in slots[i]: all or nothing
static int reserve_all(tl_hybrid *e, int n_seqs, const int *slots, const int *extra) {
    long need = 0;
    for (int i = 0; i < n_seqs; ++i) {
        const int mi = e->pool->missing(slots[i], e->pool->context(slots[i]) + extra[i]);
        TL_REQUIRE(mi >= 0, "hybrid: sequence exceeds max_pages_per_seq * page_size tokens");
        need += mi;
    }
    TL_REQUIRE(need <= e->pool->free_pages(), "hybrid: KV page pool exhausted");
    for (int i = 0; i < n_seqs; ++i)
        if (e->pool->reserve(slots[i], e->pool->context(slots[i]) + extra[i])) e->table_dirty = true;
    return TL_OK;
}

}  // namespace hy
}  // namespace tl

using namespace tl;
using namespace tl::hy;

extern "C" const char *tl_last_error(void);
extern "C" const char *tl_hybrid_last_error(void) { return tl_last_error(); }

extern "C" int tl_hybrid_create(const tl_hybrid_config *cfg, const tl_hybrid_layer *layers, void *stream, tl_hybrid **out) {
    TL_REQUIRE(cfg && layers && out, "hybrid_create: null argument");
    const tl_hybrid_config &c = *cfg;
    TL_REQUIRE(c.dtype == TL_HY_BF16 || c.dtype == TL_HY_F32, "hybrid_create: dtype must be bfloat16 or float32");
    TL_REQUIRE(c.width > 0 && c.vocab > 0 && c.num_layers > 0, "hybrid_create: width, vocab and num_layers must be positive");
    TL_REQUIRE(c.parallel_block >= 0 && c.parallel_block <= 3,
               "hybrid_create: parallel_block is 0 (sequential), 1 (parallel), 2 (norm on the branch's output) or 3 (norms on both sides)");
    TL_REQUIRE(c.side_dim >= 0 && (c.side_dim == 0 || (c.side_embed_dev && c.side_cols >= c.side_dim)), "hybrid_create: a token-input table needs its width");
    TL_REQUIRE(c.final_norm_kind == TL_NORM_RMS || (c.final_norm_kind == TL_NORM_DYT && c.final_norm_bias_dev), "hybrid_create: final norm kind");
    TL_REQUIRE(c.page_size > 0 && c.num_pages > 0 && c.max_slots > 0 && c.max_pages_per_seq > 0 && c.max_rows > 0, "hybrid_create: pool sizes must be positive");
    TL_REQUIRE(c.embed_dev && c.final_norm_dev && c.head_dev, "hybrid_create: embed, final norm and head are required");
    const bool looped = c.loop_times > 1 || (c.loop_times == 1 && c.loop_stop > c.loop_start);
    if (looped) {
        TL_REQUIRE(c.loop_start >= 0 && c.loop_stop > c.loop_start && c.loop_stop <= c.num_layers, "hybrid_create: loop range outside the layer list");
        TL_REQUIRE(c.loop_step_dev, "hybrid_create: a loop needs its pass offsets");
    }
    auto e = std::make_unique<tl_hybrid>();
    e->cfg = c;
    e->layers.assign(layers, layers + c.num_layers);
    if (stream) e->stream = (hipStream_t)stream;
    else {
        HY_HIP(hipDeviceSynchronize());
        HY_HIP(hipStreamCreateWithFlags(&e->stream, hipStreamNonBlocking));
        e->owns_stream = true;
    }
    int max_in = 0, max_cat = 0, max_q = 0, max_c = 0, max_hv = 0, max_gh = 1, max_da = 1, max_db = 1, vmix_width = 0;
    for (int i = 0; i < c.num_layers; ++i) {
        const tl_hybrid_layer &L = e->layers[i];
        TL_REQUIRE(L.kind == TL_MIX_ATTENTION || L.kind == TL_MIX_DELTA || L.kind == TL_MIX_LINREC || L.kind == TL_MIX_LATENT, "hybrid_create: unknown mixer kind");
        TL_REQUIRE(L.heads > 0 && L.kv_heads > 0 && L.heads % L.kv_heads == 0, "hybrid_create: heads must be a positive multiple of kv_heads");
        TL_REQUIRE(L.dim > 0 && L.dim <= 1024 && L.vdim > 0 && L.vdim <= 512, "hybrid_create: head widths: dim 1..1024, vdim 1..512");
        TL_REQUIRE(L.w_in_dev && L.w_out_dev && L.norm_dev && L.ff >= 0, "hybrid_create: layer matrices and norm are required");
        TL_REQUIRE(L.norm_kind == TL_NORM_RMS || (L.norm_kind == TL_NORM_DYT && L.norm_bias_dev), "hybrid_create: norm kind (Dynamic Tanh needs its bias)");
        if (c.parallel_block == TL_BLOCK_POSTNORM)
            TL_REQUIRE(L.norm_kind == TL_NORM_RMS && !L.ls1_dev && !L.ls2_dev && !looped, "hybrid_create: the block with the norm on the branch's output takes RMS norms, no layer scale and no loop");
        if (c.parallel_block == TL_BLOCK_SANDWICH) {
            TL_REQUIRE(L.norm_kind == TL_NORM_RMS && L.post_norm_dev && (L.ff <= 0 || L.post_norm2_dev), "hybrid_create: the block with norms on both sides takes RMS norms and a weight for every branch's result");
            TL_REQUIRE(L.ff <= 0 || L.ff_kind == TL_FF_PLAIN || L.ff_kind == TL_FF_GATED, "hybrid_create: the block with norms on both sides takes a dense feed-forward");
        }
        TL_REQUIRE((!L.side_gate_dev && !L.side_proj_dev && !L.side_norm_dev) ||
                       (c.parallel_block == TL_BLOCK_SANDWICH && L.side_gate_dev && L.side_proj_dev && L.side_norm_dev && c.side_dim > 0 && L.side_col0 >= 0 &&
                        L.side_col0 + c.side_dim <= c.side_cols),
                   "hybrid_create: a per-layer token input needs its three tensors, the table, and the block with norms on both sides");
        TL_REQUIRE(!L.w_in_bias_dev || c.parallel_block == TL_BLOCK_SANDWICH, "hybrid_create: projection biases are read by the block with norms on both sides only");
        if (c.parallel_block == TL_BLOCK_PARALLEL) {
            TL_REQUIRE(L.ff_kind == TL_FF_PLAIN && !L.ls1_dev && !L.ls2_dev, "hybrid_create: the parallel block takes a plain feed-forward and no layer scale");
        } else if (L.ff > 0) {
            TL_REQUIRE(L.norm2_dev && L.w_in2_dev && L.w_out2_dev && (L.norm_kind != TL_NORM_DYT || L.norm2_bias_dev),
                       "hybrid_create: a sequential block's feed-forward needs its norm and matrices");
            TL_REQUIRE(L.ff_kind == TL_FF_PLAIN || L.ff_kind == TL_FF_GATED || L.ff_kind == TL_FF_MOE, "hybrid_create: unknown feed-forward kind");
            if (L.ff_kind == TL_FF_MOE) {
                const int ET = L.experts + L.identity;
                TL_REQUIRE(L.experts >= 0 && L.identity >= 0 && ET >= 1 && ET <= 256, "hybrid_create: between 1 and 256 experts (identity experts included)");
                TL_REQUIRE(L.groups >= 1 && ET % L.groups == 0 && L.keep >= 1 && L.keep <= L.groups, "hybrid_create: expert groups must divide the experts; 1 <= keep <= groups");
                TL_REQUIRE(L.top >= 1 && L.top <= L.keep * (ET / L.groups), "hybrid_create: top exceeds the experts of the kept groups");
                TL_REQUIRE(L.expert_ff >= 0 && L.shared_ff >= 0 && L.ff == L.shared_ff + L.experts * L.expert_ff,
                           "hybrid_create: mixture of experts: ff = shared_ff + experts * expert_ff");
                TL_REQUIRE(L.correction_dev || L.moe_router == TL_ROUTER_SIGMOID, "hybrid_create: a softmax router needs its correction vector");
                TL_REQUIRE(L.moe_router == TL_ROUTER_SOFTMAX || L.moe_router == TL_ROUTER_SIGMOID, "hybrid_create: unknown router kind");
                TL_REQUIRE(L.moe_gated || (!L.moe_scale_input && !L.moe_shared_sg), "hybrid_create: a weight on the expert's input needs gated experts");
            }
        }
        if (L.kind == TL_MIX_ATTENTION) {
            TL_REQUIRE(L.rot_dims >= 0 && L.rot_dims % 2 == 0 && L.rot_dims <= L.dim, "hybrid_create: rot_dims must be even and at most dim");
            TL_REQUIRE(!L.qk_norm || (L.q_norm_dev && L.k_norm_dev), "hybrid_create: a norm over the whole q / k projection needs its weights");
            TL_REQUIRE(!(L.qk_unit_rms && (L.qk_norm || L.rot_half || L.v_mix != TL_VMIX_NONE)),
                       "hybrid_create: unit-RMS heads after the rotation do not combine with the whole-projection norm, half-split rotation pairs or value mixing");
            TL_REQUIRE(L.chunk >= 0 && L.v_mix >= TL_VMIX_NONE && L.v_mix <= TL_VMIX_BLEND, "hybrid_create: chunk >= 0, v_mix 0..2");
            TL_REQUIRE(L.gated >= 0 && L.gated <= 2 && L.window >= 0, "hybrid_create: gated 0..2, window >= 0");
            if (L.diff_maps || L.qk_head_norm || L.window > 0 || L.gated == 2) {
                TL_REQUIRE(!L.qk_unit_rms && !L.qk_norm && L.v_mix == TL_VMIX_NONE && !L.talk_dev && !L.sink_dev && L.chunk == 0,
                           "hybrid_create: per-head norms, maps, a window and per-head gates do not combine with unit-RMS heads, the whole-projection norm, value mixing, "
                           "mixed scores, learned sinks or a chunked mask");
                TL_REQUIRE(!L.qk_head_norm || (L.q_norm_dev && L.k_norm_dev), "hybrid_create: a norm per head needs its weights");
                TL_REQUIRE(!L.diff_maps || !L.sink, "hybrid_create: differential attention takes no sink");
            }
            if (L.v_mix != TL_VMIX_NONE) {
                if (vmix_width == 0) {
                    TL_REQUIRE(L.v_mix == TL_VMIX_FIRST, "hybrid_create: the first value-mixing layer keeps its values (v_mix 1), later ones blend (v_mix 2)");
                    vmix_width = L.kv_heads * L.vdim;
                } else
                    TL_REQUIRE(L.v_mix == TL_VMIX_BLEND && L.kv_heads * L.vdim == vmix_width, "hybrid_create: value-mixing layers share one values width");
            }
        } else if (L.kind == TL_MIX_LINREC) {
            TL_REQUIRE(L.kv_heads == L.heads && (L.out_norm_dev || L.rec_kind == TL_REC_FIXED), "hybrid_create: a linear recurrence has one key head per head and an output norm weight");
            if (L.rec_kind == TL_REC_FIXED)
                TL_REQUIRE(L.decay_dev && L.rot_dims >= 0 && L.rot_dims % 2 == 0 && L.rot_dims <= L.dim, "hybrid_create: a constant decay needs its values; rot_dims even and at most dim");
            else if (L.rec_kind == TL_REC_CHANNEL)
                TL_REQUIRE(L.a_rank >= 1 && L.a2_dev && L.a2_bias_dev && L.tau > 0.f, "hybrid_create: channel decay needs its projection pair, bias and tau > 0");
            else
                TL_REQUIRE(L.rec_kind == TL_REC_EXPGATE && L.i_bias_dev && L.f_bias_dev && L.gate_cap > 0.f, "hybrid_create: exponential gates need biases and a cap > 0");
        } else if (L.kind == TL_MIX_LATENT) {
            TL_REQUIRE(L.q_rank >= 1 && L.kv_rank >= 1 && L.rot_dim >= 0 && L.dq_norm_dev && L.uq_dev && L.uk_t_dev && L.uv_dev,
                       "hybrid_create: latent attention needs its ranks and per-head projections");
            TL_REQUIRE(L.rot_dims >= 0 && L.rot_dims % 2 == 0 && L.rot_dims <= L.rot_dim, "hybrid_create: rot_dims must be even and at most rot_dim");
            TL_REQUIRE(L.kv_rank + L.rot_dim <= 1024 && L.kv_rank <= 512, "hybrid_create: latent widths: kv_rank + rot_dim <= 1024, kv_rank <= 512");
            if (L.kv_from >= 0) {
                TL_REQUIRE(L.kv_from < i, "hybrid_create: kv_from must name an earlier layer");
                const tl_hybrid_layer &J = e->layers[L.kv_from];
                TL_REQUIRE(J.kind == TL_MIX_LATENT && J.kv_from < 0 && J.kv_rank == L.kv_rank && J.rot_dim == L.rot_dim,
                           "hybrid_create: kv_from must name a latent-attention layer with its own latent of the same widths");
            } else {
                TL_REQUIRE(L.dkv_norm_dev, "hybrid_create: a latent of its own needs its norm weight");
            }
        } else {
            TL_REQUIRE(L.conv_taps >= 1 && L.conv_taps <= 64 && L.conv_dev && L.a_log_dev && L.dt_bias_dev && L.out_norm_dev,
                       "hybrid_create: a delta layer needs conv taps and weights, a_log, dt_bias and its output norm");
        }
        const bool par = c.parallel_block == TL_BLOCK_PARALLEL;
        max_in = std::max(max_in, par ? mixer_cols(L) + L.ff : std::max(mixer_cols(L), ff_in_cols(L)));
        max_cat = std::max(max_cat, par ? L.heads * L.vdim + L.ff : std::max(L.heads * L.vdim, L.ff));
        max_hv = std::max(max_hv, attn_maps(L) * L.heads * (L.vdim + 1));
        max_gh = std::max(max_gh, L.heads);
        if (L.side_gate_dev) max_in = std::max(max_in, c.side_dim), max_cat = std::max(max_cat, c.side_dim);
        if (L.kind == TL_MIX_ATTENTION) max_q = std::max(max_q, attn_maps(L) * L.heads * L.dim);
        else if (L.kind == TL_MIX_LATENT) {
            max_q = std::max(max_q, L.heads * (L.kv_rank + L.rot_dim));
            max_c = std::max(max_c, L.heads * (L.dim + L.rot_dim));
            max_da = std::max(max_da, std::max(L.q_rank, L.heads * L.kv_rank));
            max_db = std::max(max_db, L.heads * L.dim);
        } else if (L.kind == TL_MIX_LINREC) {
            max_c = std::max(max_c, L.heads * L.dim);
            max_da = std::max(max_da, L.a_rank);
        } else max_c = std::max(max_c, conv_channels(L));
    }
    // layer runs
    for (int i = 0; i < c.num_layers;) {
        if (looped && i == c.loop_start) {
            for (int t = 0; t < c.loop_times; ++t)
                for (int j = c.loop_start; j < c.loop_stop; ++j) {
                    Run r;
                    r.layer = j;
                    r.pass = t;
                    r.enters_pass = j == c.loop_start;
                    e->runs.push_back(r);
                }
            i = c.loop_stop;
        } else {
            Run r;
            r.layer = i++;
            e->runs.push_back(r);
        }
    }
    tl_hybrid *p = e.get();
    const size_t es = esize(c.dtype);
    e->inv_freq.assign(c.num_layers, nullptr);
    e->rot_mult.assign(c.num_layers, 1.f);
    for (int i = 0; i < c.num_layers; ++i) {
        const tl_hybrid_layer &L = e->layers[i];
        if (L.kind != TL_MIX_ATTENTION && L.kind != TL_MIX_LATENT && !(L.kind == TL_MIX_LINREC && L.rec_kind == TL_REC_FIXED)) continue;
        const int half = std::max(1, L.rot_dims / 2);
        std::vector<float> f(half, 0.f);
        for (int k = 0; k < L.rot_dims / 2; ++k) f[k] = (float)std::pow((double)L.rot_base, -2.0 * k / (double)L.rot_dims);
        if (L.rot_factor > 0.f && L.rot_dims > 0 && L.rot_scaling_kind == 1) {
            // rescaled by wavelength l = 2 pi / f: kept below original / fast, slowed by `factor` above original / slow, blended in original / l between
            const double two_pi = 6.283185307179586476925287, dims = L.rot_dims, orig = L.rot_original, hi = L.rot_fast, lo = L.rot_slow, fac = L.rot_factor;
            for (int k = 0; k < L.rot_dims / 2; ++k) {
                const double fk = std::pow((double)L.rot_base, -2.0 * k / dims), l = two_pi / fk;
                double v = fk;
                if (l > orig / lo) v = fk / fac;
                else if (!(l < orig / hi)) {
                    const double sm = (orig / l - lo) / (hi - lo);
                    v = (1.0 - sm) * fk / fac + sm * fk;
                }
                f[k] = (float)v;
            }
        } else if (L.rot_factor > 0.f && L.rot_dims > 0) {
            // rescaled frequencies: where(t) = the dimension that turns t times over `original` positions; dimensions below where(fast) keep
            // their frequency, those above where(slow) are slowed by `factor`, a linear ramp between; cos and sin grow by 0.1 ln(factor) + 1
            const double two_pi = 6.283185307179586476925287, dims = L.rot_dims, lb = std::log((double)L.rot_base);
            auto where = [&](double turns) { return dims * std::log((double)L.rot_original / (two_pi * turns)) / (2.0 * lb); };
            const double lo = std::max(std::floor(where(L.rot_fast)), 0.0), hi = std::min(std::ceil(where(L.rot_slow)), dims - 1.0);
            for (int k = 0; k < L.rot_dims / 2; ++k) {
                const double fk = std::pow((double)L.rot_base, -2.0 * k / dims);
                const double ramp = std::min(1.0, std::max(0.0, (k - lo) / std::max(hi - lo, 0.001)));
                f[k] = (float)(fk / (double)L.rot_factor * ramp + fk * (1.0 - ramp));
            }
            e->rot_mult[i] = (float)(0.1 * std::log((double)L.rot_factor) + 1.0);
        }
        HY_TRY(dev_alloc(p, &e->inv_freq[i], half));
        HY_HIP(hipMemcpy(e->inv_freq[i], f.data(), half * 4, hipMemcpyHostToDevice));
    }
    for (size_t ri = 0; ri < e->runs.size(); ++ri) {
        Run &r = e->runs[ri];
        const tl_hybrid_layer &L = e->layers[r.layer];
        if (L.kind == TL_MIX_LATENT) {
            if (L.kv_from >= 0) {  // the pages of the latest earlier run of that layer (the same loop pass, or the last pass before)
                for (size_t rj = ri; rj-- > 0;)
                    if (e->runs[rj].layer == L.kv_from) {
                        r.kpool = e->runs[rj].kpool;
                        break;
                    }
                TL_REQUIRE(r.kpool, "hybrid_create: kv_from names a layer that has not run before this one");
            } else {
                const size_t kb = (size_t)c.num_pages * c.page_size * (L.kv_rank + L.rot_dim) * es;
                HY_TRY(dev_alloc(p, (char **)&r.kpool, kb, true));
                e->stats.kv_bytes += kb;
            }
        } else if (L.kind == TL_MIX_LINREC) {
            const size_t sb = (size_t)c.max_slots * L.heads * L.dim * (L.vdim + (L.rec_kind == TL_REC_EXPGATE ? 1 : 0)), mb = (size_t)c.max_slots * L.heads;
            HY_TRY(dev_alloc(p, &r.state, sb, true));
            HY_TRY(dev_alloc(p, &r.conv_state, mb, true));
            e->stats.state_bytes += (sb + mb) * 4;
        } else if (L.kind == TL_MIX_ATTENTION) {
            const size_t kb = (size_t)c.num_pages * attn_maps(L) * L.kv_heads * c.page_size * L.dim * es, vb = (size_t)c.num_pages * L.kv_heads * c.page_size * L.vdim * es;
            HY_TRY(dev_alloc(p, (char **)&r.kpool, kb, true));
            HY_TRY(dev_alloc(p, (char **)&r.vpool, vb, true));
            e->stats.kv_bytes += kb + vb;
        } else {
            const size_t sb = (size_t)c.max_slots * L.heads * L.dim * L.vdim, cb = (size_t)c.max_slots * std::max(1, L.conv_taps - 1) * conv_channels(L);
            HY_TRY(dev_alloc(p, &r.state, sb, true));
            HY_TRY(dev_alloc(p, &r.conv_state, cb, true));
            e->stats.state_bytes += (sb + cb) * 4;
        }
    }
    e->pool = std::make_unique<PagePool>(c.num_pages, c.page_size, c.max_slots, c.max_pages_per_seq);
    const int R = c.max_rows, W = c.width;
    e->ld_proj = (max_in + 7) / 8 * 8;
    e->ld_cat = (max_cat + 7) / 8 * 8;
    HY_TRY(dev_alloc(p, &e->x, (size_t)R * W));
    HY_TRY(dev_alloc(p, &e->x0, (size_t)R * W));
    if (c.parallel_block == TL_BLOCK_POSTNORM) {
        HY_TRY(dev_alloc(p, &e->y, (size_t)R * W));
        HY_TRY(dev_alloc(p, &e->moe_mask, 1, true));
    } else if (c.parallel_block == TL_BLOCK_SANDWICH)
        HY_TRY(dev_alloc(p, &e->y, (size_t)R * W));
    if (vmix_width > 0) HY_TRY(dev_alloc(p, &e->vref, (size_t)R * vmix_width));
    HY_TRY(dev_alloc(p, &e->proj, (size_t)R * e->ld_proj));
    HY_TRY(dev_alloc(p, &e->qbuf, (size_t)R * std::max(1, max_q)));
    HY_TRY(dev_alloc(p, &e->f32a, (size_t)R * std::max(1, max_c)));
    HY_TRY(dev_alloc(p, &e->gates, (size_t)R * max_gh * 3));
    HY_TRY(dev_alloc(p, &e->idw, (size_t)R));
    HY_TRY(dev_alloc(p, (char **)&e->da, (size_t)R * max_da * es));
    HY_TRY(dev_alloc(p, (char **)&e->db, (size_t)R * max_db * es));
    HY_TRY(dev_alloc(p, &e->obuf, (size_t)R * std::max(1, max_hv)));
    HY_TRY(dev_alloc(p, &e->logits, (size_t)R * c.vocab));
    int max_h = 1, max_v = 1;
    for (const tl_hybrid_layer &L : e->layers)
        if (L.kind == TL_MIX_ATTENTION) max_h = std::max(max_h, attn_maps(L) * L.heads), max_v = std::max(max_v, L.vdim);
        else if (L.kind == TL_MIX_LATENT) max_h = std::max(max_h, L.heads), max_v = std::max(max_v, L.kv_rank);
    HY_TRY(dev_alloc(p, &e->part_acc, (size_t)c.max_slots * max_h * 64 * max_v));
    HY_TRY(dev_alloc(p, &e->part_ml, (size_t)c.max_slots * max_h * 64 * 2));
    if (const char *v = getenv("TL_HYBRID_ATTN_ROWS")) e->attn_rows_only = v[0] != '\0' && v[0] != '0';
    HY_TRY(dev_alloc(p, (char **)&e->h, (size_t)R * W * es));
    HY_TRY(dev_alloc(p, (char **)&e->hsel, (size_t)R * W * es));
    HY_TRY(dev_alloc(p, (char **)&e->cat, (size_t)R * e->ld_cat * es, true));
    HY_TRY(dev_alloc(p, (char **)&e->cat2, (size_t)R * 2 * W * es));
    e->stats.workspace_bytes = (size_t)R * (2 * W + e->ld_proj + max_q + max_c + max_hv + c.vocab) * 4 + (size_t)R * (4 * W + e->ld_cat) * es;
    const size_t mi = meta_ints(R, c.max_slots);
    HY_TRY(dev_alloc(p, &e->meta_dev, mi));
    HY_TRY(dev_alloc(p, &e->dmeta_dev, mi, true));
    HY_HIP(hipHostMalloc((void **)&e->meta_host, mi * 4, hipHostMallocDefault));
    e->meta = carve(e->meta_dev, R, c.max_slots);
    e->dmeta = carve(e->dmeta_dev, R, c.max_slots);
    HY_TRY(dev_alloc(p, &e->table_dev, (size_t)c.max_slots * c.max_pages_per_seq));
    HY_TRY(dev_alloc(p, &e->ctx_dev, (size_t)c.max_slots, true));
    HY_TRY(dev_alloc(p, &e->pending_dev, (size_t)c.max_slots, true));
    HY_TRY(dev_alloc(p, &e->argmax_dev, (size_t)R, true));
    e->stats.layer_runs = (int)e->runs.size();
    HY_HIP(hipDeviceSynchronize());
    *out = e.release();
    return TL_OK;
}

extern "C" void tl_hybrid_destroy(tl_hybrid *e) {
    if (!e) return;
    (void)hipStreamSynchronize(e->stream);
    for (auto &g : e->graphs) (void)hipGraphExecDestroy(g.second);
    for (void *p : e->allocs) (void)hipFree(p);
    if (e->meta_host) (void)hipHostFree(e->meta_host);
    if (e->trace_buf) (void)hipFree(e->trace_buf);
    if (e->owns_stream) (void)hipStreamDestroy(e->stream);
    delete e;
}

extern "C" int tl_hybrid_synchronize(tl_hybrid *e) {
    TL_REQUIRE(e, "hybrid: null engine");
    HY_HIP(hipStreamSynchronize(e->stream));
    return TL_OK;
}

extern "C" int tl_hybrid_begin(tl_hybrid *e, int slot) {
    TL_REQUIRE(e, "hybrid: null engine");
    TL_REQUIRE(slot >= 0 && slot < e->cfg.max_slots, "hybrid_begin: slot out of range");
    TL_REQUIRE(!e->pool->live(slot), "hybrid_begin: slot is live");
    e->pool->begin(slot);
    for (Run &r : e->runs) {  // the slot's recurrent state starts at zero (fill kernels: a caller may have a capture open on this stream)
        const tl_hybrid_layer &L = e->layers[r.layer];
        if (L.kind != TL_MIX_DELTA && L.kind != TL_MIX_LINREC) continue;
        const size_t sn = state_floats(L), cn = aux_floats(L);
        hipLaunchKernelGGL(fill_kernel, dim3((unsigned)std::min<size_t>(1024, (sn + 255) / 256)), dim3(256), 0, e->stream, r.state + slot * sn, sn, 0.f);
        hipLaunchKernelGGL(fill_kernel, dim3((unsigned)std::min<size_t>(1024, (cn + 255) / 256)), dim3(256), 0, e->stream, r.conv_state + slot * cn, cn, 0.f);
        TL_CHECK_LAUNCH("hybrid_begin: state fill");
    }
    return TL_OK;
}

extern "C" int tl_hybrid_release(tl_hybrid *e, int slot) {
    TL_REQUIRE(e, "hybrid: null engine");
    TL_REQUIRE(slot >= 0 && slot < e->cfg.max_slots, "hybrid_release: slot out of range");
    TL_REQUIRE(e->pool->live(slot), "hybrid_release: slot holds no sequence");
    e->pool->release(slot);
    e->table_dirty = true;
    return TL_OK;
}

extern "C" int tl_hybrid_move(tl_hybrid *e, int src, int dst) {
    TL_REQUIRE(e, "hybrid: null engine");
    TL_REQUIRE(src >= 0 && src < e->cfg.max_slots && dst >= 0 && dst < e->cfg.max_slots && src != dst, "hybrid_move: slot out of range");
    TL_REQUIRE(e->pool->live(src) && !e->pool->live(dst), "hybrid_move: src must hold a sequence and dst must be free");
    for (Run &r : e->runs) {  // recurrent state and convolution inputs travel with the sequence; K/V pages stay where they are
        const tl_hybrid_layer &L = e->layers[r.layer];
        if (L.kind != TL_MIX_DELTA && L.kind != TL_MIX_LINREC) continue;
        const size_t sn = state_floats(L), cn = aux_floats(L);
        HY_HIP(hipMemcpyAsync(r.state + dst * sn, r.state + src * sn, sn * 4, hipMemcpyDeviceToDevice, e->stream));
        HY_HIP(hipMemcpyAsync(r.conv_state + dst * cn, r.conv_state + src * cn, cn * 4, hipMemcpyDeviceToDevice, e->stream));
    }
    int32_t tok = 0;
    HY_HIP(hipMemcpyAsync(&tok, e->pending_dev + src, 4, hipMemcpyDeviceToHost, e->stream));
    HY_HIP(hipStreamSynchronize(e->stream));
    HY_HIP(hipMemcpyAsync(e->pending_dev + dst, &tok, 4, hipMemcpyHostToDevice, e->stream));
    HY_HIP(hipStreamSynchronize(e->stream));
    e->pool->move(src, dst);
    e->table_dirty = true;
    return TL_OK;
}

extern "C" int tl_hybrid_context_len(const tl_hybrid *e, int slot) {
    if (!e || slot < 0 || slot >= e->cfg.max_slots || !e->pool->live(slot)) return -1;
    return e->pool->context(slot);
}

extern "C" int tl_hybrid_step(tl_hybrid *e, int n_seqs, const int *slots, const int32_t *tokens, const int *lens, int n_want, const int *want_rows) {
    TL_REQUIRE(e && slots && tokens && lens, "hybrid_step: null argument");
    HY_TRY(check_slots(e, n_seqs, slots));
    const tl_hybrid_config &c = e->cfg;
    long rows = 0;
    for (int i = 0; i < n_seqs; ++i) {
        TL_REQUIRE(lens[i] >= 1, "hybrid_step: every chunk holds at least one token");
        rows += lens[i];
    }
    TL_REQUIRE(rows <= c.max_rows, "hybrid_step: more rows than max_rows");
    TL_REQUIRE(n_want >= 0 && n_want <= c.max_rows && (n_want == 0 || want_rows), "hybrid_step: wanted rows out of range");
    for (int j = 0; j < n_want; ++j) TL_REQUIRE(want_rows[j] >= 0 && want_rows[j] < rows, "hybrid_step: wanted row outside the step");
    for (long t = 0; t < rows; ++t) TL_REQUIRE(tokens[t] >= 0 && tokens[t] < c.vocab, "hybrid_step: token id outside the vocabulary");
    HY_TRY(reserve_all(e, n_seqs, slots, lens));
    HY_HIP(hipStreamSynchronize(e->stream));  // the pinned staging below may still be read by the previous step's copy
    const int R = c.max_rows, S = c.max_slots;
    Meta hm = carve(e->meta_host, R, S);
    int r = 0;
    std::vector<int> slot_of_row(rows);
    for (int i = 0; i < n_seqs; ++i) {
        hm.seq_row0[i] = r;
        hm.seq_slot[i] = slots[i];
        const int ctx = e->pool->context(slots[i]);
        for (int k = 0; k < lens[i]; ++k, ++r) {
            hm.tokens[r] = tokens[r];
            hm.row_seq[r] = i;
            hm.row_pos[r] = ctx + k;
            slot_of_row[r] = slots[i];
        }
    }
    hm.seq_row0[n_seqs] = r;
    for (int j = 0; j < n_want; ++j) {
        hm.want_rows[j] = want_rows[j];
        hm.want_slot[j] = slot_of_row[want_rows[j]];
    }
    HY_HIP(hipMemcpyAsync(e->meta_dev, e->meta_host, meta_ints(R, S) * 4, hipMemcpyHostToDevice, e->stream));
    HY_TRY(sync_table(e));
    StepShape sh{(int)rows, n_seqs, 0};
    int ctx_bound = 0;
    for (int i = 0; i < n_seqs; ++i) {
        sh.max_len = std::max(sh.max_len, lens[i]);
        ctx_bound = std::max(ctx_bound, e->pool->context(slots[i]) + lens[i]);
    }
    plan_splits(sh, ctx_bound);
    HY_TRY(forward(e, e->meta, sh));
    HY_TRY(head(e, e->meta, n_want, true));
    for (int i = 0; i < n_seqs; ++i) e->pool->advance(slots[i], lens[i]);
    e->last_rows = n_want;
    e->trace_rows = (int)rows;
    e->stats.steps++;
    e->stats.rows += rows;
    return TL_OK;
}

extern "C" int tl_hybrid_set_token(tl_hybrid *e, int slot, int32_t token) {
    TL_REQUIRE(e, "hybrid: null engine");
    TL_REQUIRE(slot >= 0 && slot < e->cfg.max_slots && e->pool->live(slot), "hybrid_set_token: slot holds no sequence");
    TL_REQUIRE(token >= 0 && token < e->cfg.vocab, "hybrid_set_token: token id outside the vocabulary");
    HY_HIP(hipMemcpyAsync(e->pending_dev + slot, &token, 4, hipMemcpyHostToDevice, e->stream));
    HY_HIP(hipStreamSynchronize(e->stream));
    return TL_OK;
}

extern "C" int tl_hybrid_decode(tl_hybrid *e, int n_seqs, const int *slots, int steps, int use_graph) {
    TL_REQUIRE(e && slots, "hybrid_decode: null argument");
    TL_REQUIRE(steps >= 1, "hybrid_decode: steps must be positive");
    HY_TRY(check_slots(e, n_seqs, slots));
    const tl_hybrid_config &c = e->cfg;
    TL_REQUIRE(n_seqs <= c.max_rows, "hybrid_decode: more sequences than max_rows");
    std::vector<int> extra(n_seqs, steps);
    HY_TRY(reserve_all(e, n_seqs, slots, extra.data()));
    StepShape sh{n_seqs, n_seqs, 1};
    int ctx_bound = 0;
    for (int i = 0; i < n_seqs; ++i) ctx_bound = std::max(ctx_bound, e->pool->context(slots[i]) + steps);
    plan_splits(sh, ctx_bound);
    const std::vector<int> slot_list(slots, slots + n_seqs);
    std::vector<int> key(slot_list);  // a captured step holds its slots and its split of the key range
    key.push_back(sh.n_splits);
    key.push_back(sh.keys_per_split);
    HY_HIP(hipStreamSynchronize(e->stream));
    const int R = c.max_rows, S = c.max_slots;
    if (e->dmeta_slots != slot_list) {  // static part of the decode metadata: row i <-> sequence i <-> slots[i]
        Meta hm = carve(e->meta_host, R, S);
        std::memset(e->meta_host, 0, meta_ints(R, S) * 4);
        for (int i = 0; i < n_seqs; ++i) {
            hm.row_seq[i] = i;
            hm.seq_row0[i] = i;
            hm.seq_slot[i] = slots[i];
            hm.want_rows[i] = i;
            hm.want_slot[i] = slots[i];
        }
        hm.seq_row0[n_seqs] = n_seqs;
        HY_HIP(hipMemcpyAsync(e->dmeta_dev, e->meta_host, meta_ints(R, S) * 4, hipMemcpyHostToDevice, e->stream));
        HY_HIP(hipStreamSynchronize(e->stream));
        e->dmeta_slots = slot_list;
    }
    std::vector<int32_t> ctx(S, 0);
    for (int s = 0; s < S; ++s) ctx[s] = e->pool->live(s) ? e->pool->context(s) : 0;
    HY_HIP(hipMemcpyAsync(e->ctx_dev, ctx.data(), S * 4, hipMemcpyHostToDevice, e->stream));
    HY_TRY(sync_table(e));
    HY_HIP(hipStreamSynchronize(e->stream));
    auto one_step = [&]() -> int {
        hipLaunchKernelGGL(decode_meta_kernel, dim3((n_seqs + 63) / 64), dim3(64), 0, e->stream, e->dmeta.seq_slot, n_seqs, e->pending_dev, e->ctx_dev,
                           e->dmeta.tokens, e->dmeta.row_pos, 0);
        TL_CHECK_LAUNCH("hybrid decode meta");
        HY_TRY(forward(e, e->dmeta, sh));
        HY_TRY(head(e, e->dmeta, n_seqs, true));
        hipLaunchKernelGGL(decode_meta_kernel, dim3((n_seqs + 63) / 64), dim3(64), 0, e->stream, e->dmeta.seq_slot, n_seqs, e->pending_dev, e->ctx_dev,
                           e->dmeta.tokens, e->dmeta.row_pos, 1);
        TL_CHECK_LAUNCH("hybrid decode advance");
        return TL_OK;
    };
    const bool graph = use_graph && !e->trace;
    if (graph) {
        auto it = e->graphs.find(key);
        if (it == e->graphs.end()) {
            if (e->graphs.size() >= 32) {
                for (auto &g : e->graphs) (void)hipGraphExecDestroy(g.second);
                e->graphs.clear();
            }
            hipGraph_t g = nullptr;
            HY_HIP(hipStreamBeginCapture(e->stream, hipStreamCaptureModeThreadLocal));
            const int s = one_step();
            const hipError_t ce = hipStreamEndCapture(e->stream, &g);
            if (s != 0) {
                if (g) (void)hipGraphDestroy(g);
                return s;
            }
            HY_HIP(ce);
            hipGraphExec_t ex = nullptr;
            HY_HIP(hipGraphInstantiate(&ex, g, nullptr, nullptr, 0));
            (void)hipGraphDestroy(g);
            it = e->graphs.emplace(key, ex).first;
            e->stats.graph_captures++;
        }
        for (int k = 0; k < steps; ++k) {
            HY_HIP(hipGraphLaunch(it->second, e->stream));
            e->stats.graph_replays++;
        }
    } else {
        for (int k = 0; k < steps; ++k) HY_TRY(one_step());
    }
    for (int i = 0; i < n_seqs; ++i) e->pool->advance(slots[i], steps);
    e->last_rows = n_seqs;
    e->trace_rows = n_seqs;
    e->stats.steps += steps;
    e->stats.rows += (long)steps * n_seqs;
    return TL_OK;
}

extern "C" int tl_hybrid_read_pending(tl_hybrid *e, int n, const int *slots, int32_t *out) {
    TL_REQUIRE(e && slots && out, "hybrid_read_pending: null argument");
    std::vector<int32_t> all(e->cfg.max_slots);
    HY_HIP(hipMemcpyAsync(all.data(), e->pending_dev, all.size() * 4, hipMemcpyDeviceToHost, e->stream));
    HY_HIP(hipStreamSynchronize(e->stream));
    for (int i = 0; i < n; ++i) {
        TL_REQUIRE(slots[i] >= 0 && slots[i] < e->cfg.max_slots, "hybrid_read_pending: slot out of range");
        out[i] = all[slots[i]];
    }
    return TL_OK;
}

extern "C" int tl_hybrid_copy_logits(tl_hybrid *e, void *dst_dev, int rows) {
    TL_REQUIRE(e && dst_dev, "hybrid_copy_logits: null argument");
    TL_REQUIRE(rows >= 0 && rows <= e->last_rows, "hybrid_copy_logits: more rows than the last step produced");
    if (rows) HY_HIP(hipMemcpyAsync(dst_dev, e->logits, (size_t)rows * e->cfg.vocab * 4, hipMemcpyDeviceToDevice, e->stream));
    return TL_OK;
}

extern "C" int tl_hybrid_read_logits(tl_hybrid *e, float *dst_host, int rows) {
    TL_REQUIRE(e && dst_host, "hybrid_read_logits: null argument");
    TL_REQUIRE(rows >= 0 && rows <= e->last_rows, "hybrid_read_logits: more rows than the last step produced");
    if (rows) HY_HIP(hipMemcpyAsync(dst_host, e->logits, (size_t)rows * e->cfg.vocab * 4, hipMemcpyDeviceToHost, e->stream));
    HY_HIP(hipStreamSynchronize(e->stream));
    return TL_OK;
}

extern "C" int tl_hybrid_read_argmax(tl_hybrid *e, int rows, int32_t *out) {
    TL_REQUIRE(e && out, "hybrid_read_argmax: null argument");
    TL_REQUIRE(rows >= 0 && rows <= e->last_rows, "hybrid_read_argmax: more rows than the last step produced");
    if (rows) HY_HIP(hipMemcpyAsync(out, e->argmax_dev, (size_t)rows * 4, hipMemcpyDeviceToHost, e->stream));
    HY_HIP(hipStreamSynchronize(e->stream));
    return TL_OK;
}

extern "C" int tl_hybrid_set_trace(tl_hybrid *e, int on) {
    TL_REQUIRE(e, "hybrid: null engine");
    if (on && !e->trace_buf) HY_HIP(hipMalloc((void **)&e->trace_buf, e->runs.size() * (size_t)e->cfg.max_rows * e->cfg.width * 4));
    e->trace = on != 0;
    return TL_OK;
}

extern "C" int tl_hybrid_read_trace(tl_hybrid *e, int run, float *dst_host, int rows) {
    TL_REQUIRE(e && dst_host && e->trace_buf, "hybrid_read_trace: tracing is off");
    TL_REQUIRE(run >= 0 && run < (int)e->runs.size() && rows >= 0 && rows <= e->trace_rows, "hybrid_read_trace: run or rows out of range");
    HY_HIP(hipStreamSynchronize(e->stream));
    HY_HIP(hipMemcpy(dst_host, e->trace_buf + (size_t)run * e->cfg.max_rows * e->cfg.width, (size_t)rows * e->cfg.width * 4, hipMemcpyDeviceToHost));
    return TL_OK;
}

extern "C" int tl_hybrid_get_stats(const tl_hybrid *e, tl_hybrid_stats *out) {
    TL_REQUIRE(e && out, "hybrid_get_stats: null argument");
    tl_hybrid_stats s = e->stats;
    const PagePoolStats &p = e->pool->stats();
    s.pages_in_use = p.pages_in_use;
    s.pages_free = e->pool->free_pages();
    s.peak_pages_in_use = p.peak_pages_in_use;
    s.page_allocations = p.page_allocations;
    s.reused_page_allocations = p.reused_page_allocations;
    s.slot_begins = p.slot_begins;
    s.reused_slot_begins = p.reused_slot_begins;
    *out = s;
    return TL_OK;
}

extern "C" int tl_hybrid_linear(int dtype, const void *a_dev, int lda, const void *w_dev, float *out_dev, int ldc, int M, int N, int K, int force_kernel,
                                void *stream) {
    TL_REQUIRE(a_dev && w_dev && out_dev, "hybrid_linear: null argument");
    TL_REQUIRE(dtype == TL_HY_BF16 || dtype == TL_HY_F32, "hybrid_linear: dtype must be bfloat16 or float32");
    TL_REQUIRE(M > 0 && N > 0 && K > 0 && lda >= K && ldc >= N, "hybrid_linear: bad shape");
    if (dtype == TL_HY_BF16) return linear_t<BF16>(a_dev, lda, w_dev, out_dev, ldc, M, N, K, 0, 1.f, nullptr, force_kernel, (hipStream_t)stream);
    return linear_t<F32>(a_dev, lda, w_dev, out_dev, ldc, M, N, K, 0, 1.f, nullptr, force_kernel, (hipStream_t)stream);
}
