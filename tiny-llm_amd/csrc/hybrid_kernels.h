// Kernels of the layer-list engine (include/tinyllm_hybrid.h).  D = F32 or BF16 (common.h): the type of matrices, of
// activations entering a matrix product and of K/V pages.  Everything else is float32.
//
// Packed rows: a step's tokens lie back to back, sequence after sequence.  Per row: row_seq (index into the step's
// sequence list) and row_pos (position in its sequence).  Per sequence: seq_row0 (first row; seq_row0[n] = rows),
// seq_slot (state slot = block-table row).
#pragma once
#include "common.h"

namespace tl {
namespace hy {

template <typename D>
__device__ __forceinline__ float ld(const typename D::storage *p, size_t i) { return D::to_float(p[i]); }

// generic block reduction (sum), blockDim.x a multiple of 64 and <= 1024; red = 16 floats of LDS
__device__ __forceinline__ float block_sum(float v, float *red) {
    v = wave_sum(v);
    const int w = threadIdx.x >> 6, nw = blockDim.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; ++i) t += red[i];
    return t;
}

__device__ __forceinline__ float sigmoid_f(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float silu_f(float x) { return x / (1.f + expf(-x)); }
__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }
__device__ __forceinline__ float act_f(float z, int kind) {
    if (kind == 0) return 0.5f * z * (1.f + erff(z * 0.70710678118654752440f));
    if (kind == 1) {  // 0.5 z (1 + tanh u) = z / (1 + exp(-2 u)), u = sqrt(2/pi) (z + 0.044715 z^3): one exponential instead of tanhf
        const float u = 0.79788456080286535588f * (z + 0.044715f * z * z * z);
        return z / (1.f + expf(-2.f * u));
    }
    return silu_f(z);
}

// ---- embedding gather: x0 = x = embed[token] * scale; with nw the row then passes an RMS norm, * (noffset + nw) ------
template <typename D>
__global__ void embed_kernel(const int32_t *tokens, const typename D::storage *embed, float *x0, float *x, int width, int vocab, float scale,
                             const float *nw, float noffset, float eps) {
    __shared__ float red[16];
    const int t = blockIdx.x;
    int tok = tokens[t];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
    float inv = 1.f, keep[16];  // (the row's first 16 elements a thread stay in registers between the two passes)
    if (nw) {
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int c = threadIdx.x + i * blockDim.x;
            keep[i] = c < width ? ld<D>(embed, (size_t)tok * width + c) * scale : 0.f;
            ss += keep[i] * keep[i];
        }
        for (int c = threadIdx.x + 16 * blockDim.x; c < width; c += blockDim.x) {
            const float v = ld<D>(embed, (size_t)tok * width + c) * scale;
            ss += v * v;
        }
        ss = block_sum(ss, red);
        inv = 1.f / sqrtf(ss / (float)width + eps);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int c = threadIdx.x + i * blockDim.x;
            if (c < width) {
                const float v = keep[i] * inv * (noffset + nw[c]);
                x0[(size_t)t * width + c] = v;
                x[(size_t)t * width + c] = v;
            }
        }
    }
    for (int c = threadIdx.x + (nw ? 16 * blockDim.x : 0); c < width; c += blockDim.x) {
        float v = ld<D>(embed, (size_t)tok * width + c) * scale;
        if (nw) v = v * inv * (noffset + nw[c]);
        x0[(size_t)t * width + c] = v;
        x[(size_t)t * width + c] = v;
    }
}

// ---- RMS norm of float32 rows -> D rows: x / sqrt(mean(x^2) + eps) * (offset + w).  rows_idx: optional gather. ----
template <typename D>
__global__ void norm_kernel(const float *x, const float *w, float offset, float eps, typename D::storage *out, int width,
                            const int32_t *rows_idx) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const float *src = x + (size_t)(rows_idx ? rows_idx[r] : r) * width;
    float ss = 0.f;
    for (int c = threadIdx.x; c < width; c += blockDim.x) ss += src[c] * src[c];
    ss = block_sum(ss, red);
    const float inv = 1.f / sqrtf(ss / (float)width + eps);
    for (int c = threadIdx.x; c < width; c += blockDim.x) out[(size_t)r * width + c] = D::from_float(src[c] * inv * (offset + w[c]));
}

// ---- [x ; x0] as D rows of 2*width (input of the loop-entry projection) ------------------------------------------
template <typename D>
__global__ void pack2_kernel(const float *x, const float *x0, typename D::storage *out, int width) {
    const int t = blockIdx.x;
    for (int c = threadIdx.x; c < 2 * width; c += blockDim.x)
        out[(size_t)t * 2 * width + c] = D::from_float(c < width ? x[(size_t)t * width + c] : x0[(size_t)t * width + c - width]);
}

// ---- tile matrix product: out[M, N] (+)= A[M, K] . W[N, K]^T, float32 accumulation on the matrix cores ------------
// 64 x 64 output tile per 256-thread workgroup, 4 waves of 32 x 32 (2 x 2 MFMA 16x16 tiles), K in steps of 32 through LDS.
// bf16: v_mfma_f32_16x16x32_bf16; fp32: v_mfma_f32_16x16x4_f32 (full fp32 products).  Any M, N, K: edges are zero-filled in LDS.
// EPI 0: out = acc   1: out += alpha * acc   2: out = acc + bias[n]   3: out += alpha * bias[n] * acc (a per-column scale on the way into the sum)
//     4: as 3, and the Dynamic Tanh norm of the new sum leaves with it: nout[m, n] = tanh(nalpha * out) * nw[n] + nb[n] (D rows of N; the norm is
//        element-wise, so the product that completes a residual sum can hand the next product its input)
// blockIdx.y = a batch of independent products of one shape (the heads of a per-head projection): operands advance by sa / sw / sc elements.
template <typename D, int EPI>
__global__ __launch_bounds__(256) void gemm_tile_kernel(const typename D::storage *A, int lda, const typename D::storage *W, float *out,
                                                        int ldc, int M, int N, int K, float alpha, const float *bias, int vec_ok, long sa, long sw,
                                                        long sc, const float *nw, const float *nb, float nalpha, typename D::storage *nout) {
    using S = typename D::storage;
    A += (size_t)blockIdx.y * sa, W += (size_t)blockIdx.y * sw, out += (size_t)blockIdx.y * sc;
    constexpr bool BF = sizeof(S) == 2;
    constexpr int KT = 32, LD = BF ? KT + 8 : KT + 1;
    __shared__ S As[64 * LD];
    __shared__ S Ws[64 * LD];
    // XCD-aware tile order: consecutive workgroup ids go to different XCDs (round robin over 8), so give each XCD a contiguous run of tiles
    const int nt_n = (N + 63) / 64, nt_m = (M + 63) / 64, total = nt_n * nt_m;
    int id = blockIdx.x;
    {
        const int per = (total + 7) / 8, xcd = id & 7, k = id >> 3;
        const int mapped = xcd * per + k;
        id = (total % 8 == 0) ? mapped : id;
    }
    const int tm = id / nt_n, tn = id % nt_n;
    const int m0 = tm * 64, n0 = tn * 64;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    f32x4 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int lr = tid >> 2, lk = (tid & 3) * 8;  // loader: row of the tile, first of 8 consecutive k
    for (int k0 = 0; k0 < K; k0 += KT) {
        __syncthreads();
        {
            const int gm = m0 + lr, gn = n0 + lr, gk = k0 + lk;
            S av[8], wv[8];
            if (vec_ok && gm < M && gk + 8 <= K) {
                if constexpr (BF) *reinterpret_cast<u32x4 *>(av) = *reinterpret_cast<const u32x4 *>(A + (size_t)gm * lda + gk);
                else {
                    *reinterpret_cast<u32x4 *>(av) = *reinterpret_cast<const u32x4 *>(A + (size_t)gm * lda + gk);
                    *reinterpret_cast<u32x4 *>(av + 4) = *reinterpret_cast<const u32x4 *>(A + (size_t)gm * lda + gk + 4);
                }
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) av[i] = (gm < M && gk + i < K) ? A[(size_t)gm * lda + gk + i] : (S)0;
            }
            if (vec_ok && gn < N && gk + 8 <= K) {
                if constexpr (BF) *reinterpret_cast<u32x4 *>(wv) = *reinterpret_cast<const u32x4 *>(W + (size_t)gn * K + gk);
                else {
                    *reinterpret_cast<u32x4 *>(wv) = *reinterpret_cast<const u32x4 *>(W + (size_t)gn * K + gk);
                    *reinterpret_cast<u32x4 *>(wv + 4) = *reinterpret_cast<const u32x4 *>(W + (size_t)gn * K + gk + 4);
                }
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) wv[i] = (gn < N && gk + i < K) ? W[(size_t)gn * K + gk + i] : (S)0;
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                As[lr * LD + lk + i] = av[i];
                Ws[lr * LD + lk + i] = wv[i];
            }
        }
        __syncthreads();
        if constexpr (BF) {
            bf16x8_t af[2], bfr[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const S *pa = As + (wm * 32 + i * 16 + (lane & 15)) * LD + (lane >> 4) * 8;
                const S *pb = Ws + (wn * 32 + i * 16 + (lane & 15)) * LD + (lane >> 4) * 8;
                u32x4 ua = *reinterpret_cast<const u32x4 *>(pa), ub = *reinterpret_cast<const u32x4 *>(pb);
                af[i] = __builtin_bit_cast(bf16x8_t, ua);
                bfr[i] = __builtin_bit_cast(bf16x8_t, ub);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
        } else {
#pragma unroll
            for (int ks = 0; ks < KT; ks += 4) {
                float a[2], b[2];
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    a[i] = As[(wm * 32 + i * 16 + (lane & 15)) * LD + ks + (lane >> 4)];
                    b[i] = Ws[(wn * 32 + i * 16 + (lane & 15)) * LD + ks + (lane >> 4)];
                }
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], b[j], acc[i][j], 0, 0, 0);
            }
        }
    }
    // D layout of the 16x16 MFMA: lane holds column (lane & 15), rows 4 * (lane >> 4) + r
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int gm = m0 + wm * 32 + i * 16 + (lane >> 4) * 4 + r, gn = n0 + wn * 32 + j * 16 + (lane & 15);
                if (gm < M && gn < N) {
                    float *o = out + (size_t)gm * ldc + gn;
                    const float v = acc[i][j][r];
                    if constexpr (EPI == 0) *o = v;
                    else if constexpr (EPI == 1) *o += alpha * v;
                    else if constexpr (EPI == 2) *o = v + bias[gn];
                    else if constexpr (EPI == 3) *o += alpha * bias[gn] * v;
                    else {
                        const float xn = *o + alpha * bias[gn] * v;
                        *o = xn;
                        nout[(size_t)gm * N + gn] = D::from_float(tanhf(nalpha * xn) * nw[gn] + nb[gn]);
                    }
                }
            }
}

// Segments of a matrix that a step does not need (the experts no row of a small step takes): bit e of *mask says whether segment e is needed.
// on_k 0: OUTPUT columns n < limit belong to segment (n % period - lead) / len when n % period >= lead; columns of unneeded segments are not computed
// (their consumers do not read them).  on_k 1: the K range [lead + e len, lead + (e + 1) len) belongs to segment e; the activations there are zero, so
// the weights are not read (lead and len are multiples of 8: a 16-byte piece lies in one segment).  At most 64 segments.
struct SegSkip {
    const unsigned long long *mask = nullptr;
    int lead = 0, len = 1, period = 1, limit = 0, on_k = 0;
};

// ---- row matrix product for a few rows (decode): each wave owns one output column and streams its weight row once ----
// M <= 8.  Lanes stride over K, 8 elements at a time where the layout allows 16-byte loads.
template <typename D, int EPI>
__global__ __launch_bounds__(256) void gemm_rows_kernel(const typename D::storage *A, int lda, const typename D::storage *W, float *out,
                                                        int ldc, int M, int N, int K, float alpha, const float *bias, int vec_ok, long sa, long sw,
                                                        long sc, const float *nw, const float *nb, float nalpha, typename D::storage *nout,
                                                        SegSkip skip) {
    using S = typename D::storage;
    A += (size_t)blockIdx.y * sa, W += (size_t)blockIdx.y * sw, out += (size_t)blockIdx.y * sc;
    const int lane = threadIdx.x & 63;
    const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (n >= N) return;
    const unsigned long long need = skip.mask ? *skip.mask : ~0ull;
    if (skip.mask && !skip.on_k && n < skip.limit) {
        const int c = n % skip.period;
        if (c >= skip.lead && !((need >> ((c - skip.lead) / skip.len)) & 1ull)) return;
    }
    const bool k_skip = skip.mask && skip.on_k;
    float acc[8];
#pragma unroll
    for (int m = 0; m < 8; ++m) acc[m] = 0.f;
    const S *wrow = W + (size_t)n * K;
    if (vec_ok) {
        for (int k = lane * 8; k + 8 <= K; k += 64 * 8) {
            if (k_skip && k >= skip.lead && !((need >> ((k - skip.lead) / skip.len)) & 1ull)) continue;
            float wf[8];
            if constexpr (sizeof(S) == 2) {
                u32x4 u = *reinterpret_cast<const u32x4 *>(wrow + k);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    wf[2 * i] = __uint_as_float(u[i] << 16);
                    wf[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u);
                }
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) wf[i] = D::to_float(wrow[k + i]);
            }
#pragma unroll
            for (int m = 0; m < 8; ++m) {
                if (m < M) {
                    const S *arow = A + (size_t)m * lda + k;
#pragma unroll
                    for (int i = 0; i < 8; ++i) acc[m] += wf[i] * D::to_float(arow[i]);
                }
            }
        }
        for (int k = (K / 8) * 8 + lane; k < K; k += 64) {
            const float wf = D::to_float(wrow[k]);
#pragma unroll
            for (int m = 0; m < 8; ++m)
                if (m < M) acc[m] += wf * D::to_float(A[(size_t)m * lda + k]);
        }
    } else {
        for (int k = lane; k < K; k += 64) {
            const float wf = D::to_float(wrow[k]);
#pragma unroll
            for (int m = 0; m < 8; ++m)
                if (m < M) acc[m] += wf * D::to_float(A[(size_t)m * lda + k]);
        }
    }
#pragma unroll
    for (int m = 0; m < 8; ++m) {
        if (m < M) {  // M is uniform over the grid
            const float v = wave_sum(acc[m]);
            if (lane == 0) {
                float *o = out + (size_t)m * ldc + n;
                if constexpr (EPI == 0) *o = v;
                else if constexpr (EPI == 1) *o += alpha * v;
                else if constexpr (EPI == 2) *o = v + bias[n];
                else if constexpr (EPI == 3) *o += alpha * bias[n] * v;
                else {
                    const float xn = *o + alpha * bias[n] * v;
                    *o = xn;
                    nout[(size_t)m * N + n] = D::from_float(tanhf(nalpha * xn) * nw[n] + nb[n]);
                }
            }
        }
    }
}

// ---- attention, step 1: rotary positions + unit-RMS on q and k; k and v rows appended to their pages -----------------
// proj: [rows, ldp] float32 with q | k | v at columns 0 | H*dim | (H+G)*dim.  One wave per (row, head of q|k|v).
// Rotation of the pair (2i, 2i+1) by pos * inv_freq[i] for i < rot_dims/2.
template <typename D>
__global__ __launch_bounds__(64) void attn_prep_kernel(const float *proj, int ldp, const int32_t *row_seq, const int32_t *row_pos,
                                                       const int32_t *seq_slot, const int32_t *block_table, int max_pages, int page_size,
                                                       const float *inv_freq, int rot_dims, int unit_rms, float eps, int H, int G, int dim,
                                                       int vdim, float *qbuf, typename D::storage *kpool, typename D::storage *vpool) {
    const int t = blockIdx.x, hh = blockIdx.y, lane = threadIdx.x;
    const int pos = row_pos[t], slot = seq_slot[row_seq[t]];
    const int page = block_table[(size_t)slot * max_pages + pos / page_size], in_page = pos % page_size;
    if (hh >= H + G) {  // a value head: copy
        const int g = hh - H - G;
        const float *src = proj + (size_t)t * ldp + (size_t)(H + G) * dim + (size_t)g * vdim;
        typename D::storage *dst = vpool + (((size_t)page * G + g) * page_size + in_page) * vdim;
        for (int c = lane; c < vdim; c += 64) dst[c] = D::from_float(src[c]);
        return;
    }
    const float *src = proj + (size_t)t * ldp + (size_t)hh * dim;
    // pairs are rotated by the lane that owns the even element; elements beyond rot_dims pass
    float ss = 0.f;
    const int npairs = (dim + 1) / 2;
    const bool is_q = hh < H;
    float *qdst = qbuf + ((size_t)t * H + hh) * dim;
    typename D::storage *kdst = is_q ? nullptr : kpool + (((size_t)page * G + (hh - H)) * page_size + in_page) * dim;
    // pass 1: rotate into registers (at most 8 pairs per lane: dim <= 1024), accumulate the sum of squares
    float ra[8], rb[8];
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const int p = lane + it * 64;
        ra[it] = rb[it] = 0.f;
        if (p < npairs) {
            const int c = 2 * p;
            float u = src[c], v = (c + 1 < dim) ? src[c + 1] : 0.f;
            if (c + 1 < rot_dims) {
                const float a = (float)pos * inv_freq[p];
                float sn, cs;
                sincosf(a, &sn, &cs);
                const float nu = u * cs - v * sn, nv = v * cs + u * sn;
                u = nu;
                v = nv;
            }
            ra[it] = u;
            rb[it] = v;
            ss += u * u + v * v;
        }
    }
    ss = wave_sum(ss);
    const float inv = unit_rms ? 1.f / sqrtf(ss / (float)dim + eps) : 1.f;
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const int p = lane + it * 64;
        if (p < npairs) {
            const int c = 2 * p;
            if (is_q) {
                qdst[c] = ra[it] * inv;
                if (c + 1 < dim) qdst[c + 1] = rb[it] * inv;
            } else {
                kdst[c] = D::from_float(ra[it] * inv);
                if (c + 1 < dim) kdst[c + 1] = D::from_float(rb[it] * inv);
            }
        }
    }
}

// ---- attention, step 2 (row form): one wave per (row, query head) walks the keys 0 .. pos of its sequence ---------------
// float32 scores and weights, running maximum; the sink is the start value of the running pair (max 0, sum 1).
// out: cat[t, h*vdim + c] = (sum_j p_j v_j[c]) * sigmoid(gate[t, h*vdim + c])   (D rows of ldo)
template <typename D>
__global__ __launch_bounds__(64) void attn_rows_kernel(const float *qbuf, const typename D::storage *kpool, const typename D::storage *vpool,
                                                       const int32_t *row_seq, const int32_t *row_pos, const int32_t *seq_slot,
                                                       const int32_t *block_table, int max_pages, int page_size, int H, int G, int dim, int vdim,
                                                       float scale, int sink, const float *gate, int ldg, typename D::storage *out, int ldo, int v_row,
                                                       int window, int vshare, int gate_per_head, float *out32) {
    extern __shared__ float smem[];
    float *qs = smem;        // [dim]
    float *ps = smem + dim;  // [64]
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int pos = row_pos[t], slot = seq_slot[row_seq[t]], g = h / (H / G);
    // window > 0: the keys start window - 1 positions before the query.  vshare K/V heads in a row read one value head.
    const int Gv = G / vshare, gv = g / vshare, k_lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int32_t *bt = block_table + (size_t)slot * max_pages;
    for (int c = lane; c < dim; c += 64) qs[c] = qbuf[((size_t)t * H + h) * dim + c];
    __syncthreads();
    float m = sink ? 0.f : -INFINITY, l = sink ? 1.f : 0.f;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};  // vdim <= 512
    for (int kb = k_lo; kb <= pos; kb += 64) {
        const int j = kb + lane;
        float s = -INFINITY;
        if (j <= pos) {
            const typename D::storage *kr = kpool + (((size_t)bt[j / page_size] * G + g) * page_size + j % page_size) * dim;
            float d = 0.f;
            for (int c = 0; c < dim; ++c) d += qs[c] * D::to_float(kr[c]);
            s = d * scale;
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float p = (j <= pos) ? expf(s - m_new) : 0.f;
        const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
        l = l * corr + wave_sum(p);
        m = m_new;
        __syncthreads();
        ps[lane] = p;
        __syncthreads();
        const int cnt = min(64, pos - kb + 1);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] *= corr;
        for (int jj = 0; jj < cnt; ++jj) {
            const int jg = kb + jj;
            const typename D::storage *vr = vpool + (((size_t)bt[jg / page_size] * Gv + gv) * page_size + jg % page_size) * v_row;
            const float pj = ps[jj];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int c = lane + i * 64;
                if (c < vdim) acc[i] += pj * D::to_float(vr[c]);
            }
        }
    }
    const float invl = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int c = lane + i * 64;
        if (c < vdim) {
            float o = acc[i] * invl;
            if (gate) o *= sigmoid_f(gate[(size_t)t * ldg + (gate_per_head ? (size_t)h : (size_t)h * vdim + c)]);
            if (out32) out32[((size_t)t * H + h) * vdim + c] = o;
            else out[(size_t)t * ldo + (size_t)h * vdim + c] = D::from_float(o);
        }
    }
}

// ---- attention, step 2 (tile form): float32 MFMA flash attention over the paged K/V, grouped heads sharing the staged tiles -----------
// A workgroup (4 waves) owns 64 "query rows" of one sequence and one K/V head: row rho = (token rho / HGB, head-in-group rho % HGB), HGB = the
// group's query heads rounded up to a power of two (<= 16; larger groups take several workgroups), so K and V tiles are staged once for
// every query head that reads them.  Keys come in tiles of 64, converted to float32 in LDS; both products run on v_mfma_f32_16x16x4_f32
// (full float32 products), transposed so that no value crosses lanes between them:
//   S^T[key, row]  = K . Q^T      A = K tile (LDS), B = this wave's 16 query rows (registers, scale folded in)
//   O^T[vcol, row] = V^T . P^T    A = V tile (LDS), B = the weights exactly where the first product left them: the k-slot of lane group g in
//                                 step r is key 4 g + r of the 16-key sub-tile (a sum does not care in which order its terms are paired)
// Per query row (= per lane column) a running maximum and sum; the sink is their start value (0, 1).  The key range may be split over
// gridDim.z (decode steps over long contexts): then unnormalised partial sums + (max, sum) go to part_* and attn_merge_kernel finishes.
template <typename D, int DK4, int VT, bool WSPLIT, bool EXT>
__global__ __launch_bounds__(256) void attn_tile_kernel(const float *qbuf, const typename D::storage *kpool, const typename D::storage *vpool,
                                                        const int32_t *seq_row0, const int32_t *seq_slot, const int32_t *row_pos,
                                                        const int32_t *block_table, int max_pages, int page_size, int H, int G, int dim, int vdim,
                                                        float scale, int sink, int HGB, int n_hblk, int keys_per_split, int n_splits, const float *gate,
                                                        int ldg, typename D::storage *out, int ldo, float *part_acc, float *part_ml, int page_shift,
                                                        int vec_ok, int v_row, int window_, int vshare_, int gate_per_head_, float *out32_) {
    using S = typename D::storage;
    extern __shared__ float smem[];
    // EXT false: plain causal attention into D rows, the four options folded away at compile time
    const int window = EXT ? window_ : 0, vshare = EXT ? vshare_ : 1, gate_per_head = EXT ? gate_per_head_ : 0;
    float *const out32 = EXT ? out32_ : nullptr;
    // window > 0: a query sees key j <= its position only if position - j < window; the walk starts at the first key the tile's first row sees,
    // and a split key range (decode steps) is counted from there.  vshare: that many K/V heads in a row read one value head (maps over shared
    // values).  out32: the read-out as float32 rows [row, head, vdim] instead of D rows of `out` (no gate).
    // LDS rows as wide as the template: zeros behind dim / vdim, no guards in the product loops.  bfloat16 pages: the K tile stays bfloat16
    // in LDS ([64][4 DK4 + 8] 16-bit elements) and S^T runs on v_mfma_f32_16x16x32_bf16 (q rounded to bfloat16 like every other input of a
    // bfloat16 product, float32 sums, the scale applied to the float32 result); the weights and P V are float32 in either case.
    constexpr bool KB16 = sizeof(S) == 2;
    constexpr int DKP = KB16 ? (4 * DK4 + 8) / 2 : 4 * DK4 + 4, VP = 16 * VT + 4;  // (DKP in floats)
    float *Ks = smem;             // [64][DKP]
    float *Vs = smem + 64 * DKP;  // [64][VP]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g4 = lane >> 4, col = lane & 15;
    const int seq = blockIdx.z / n_splits, split = blockIdx.z % n_splits;
    const int kvh = blockIdx.y / n_hblk, hblk = blockIdx.y % n_hblk, HG = H / G, TQ = 64 / HGB;
    const int r0 = seq_row0[seq], len = seq_row0[seq + 1] - r0, t0 = blockIdx.x * TQ;
    if (t0 >= len) return;
    const int pos0 = row_pos[r0], slot = seq_slot[seq];
    const int32_t *bt = block_table + (size_t)slot * max_pages;
    const int k_end_tile = pos0 + min(t0 + TQ, len);  // keys the tile's last query row sees
    const int k_lo = window > 0 ? max(0, pos0 + t0 - window + 1) : 0;
    const int k_begin = k_lo + split * keys_per_split, k_end = min(k_end_tile, k_lo + (split + 1) * keys_per_split);
    const int Gv = G / vshare, kvh_v = kvh / vshare;
    // this lane's query row (column of the transposed products)
    // WSPLIT (a tile with at most 16 query rows, i.e. decode steps): every wave holds the SAME 16 rows and takes the 16 keys `wave` of each
    // 64-key tile -- a quarter of the products per wave -- and the four partial (max, sum, O) sets are merged through LDS at the end
    const int rho = (WSPLIT ? 0 : wave * 16) + col, tl = rho / HGB, hb = hblk * HGB + rho % HGB;
    constexpr int NN = WSPLIT ? 1 : 4;  // 16-key sub-tiles a wave takes per tile
    const int nb = WSPLIT ? wave : 0;
    const bool row_ok = t0 + tl < len && hb < HG;
    const int trow = r0 + t0 + tl, head = kvh * HG + hb, qpos = pos0 + t0 + tl;
    const bool owns_sink = sink && split == 0 && (!WSPLIT || wave == 0);
    float m_run = owns_sink ? 0.f : -INFINITY, l_run = owns_sink ? 1.f : 0.f;
    f32x4 o[VT];
#pragma unroll
    for (int v = 0; v < VT; ++v) o[v] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (k_begin < k_end) {
        float qf[KB16 ? 1 : DK4];       // float32 pages: B operand of the 16x16x4 product, scale folded in
        u32x4 qb[KB16 ? DK4 / 8 : 1];   // bfloat16 pages: B operand of the 16x16x32 product, 8 consecutive k per lane
        if constexpr (KB16) {
#pragma unroll
            for (int ks8 = 0; ks8 < DK4 / 8; ++ks8) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int d = 32 * ks8 + 8 * g4 + 2 * e;
                    const float *qrow = qbuf + ((size_t)trow * H + head) * dim;
                    qb[ks8][e] = BF16::pack2((row_ok && d < dim) ? qrow[d] : 0.f, (row_ok && d + 1 < dim) ? qrow[d + 1] : 0.f);
                }
            }
        } else {
#pragma unroll
            for (int kk = 0; kk < DK4; ++kk) {
                const int d = 4 * kk + g4;
                qf[kk] = (row_ok && d < dim) ? qbuf[((size_t)trow * H + head) * dim + d] * scale : 0.f;
            }
        }
        // Staging: a tile is 64 (ck + cv) chunks of 8 elements; thread t owns chunks t, t + 256, ... -- the same (key, column) places in every
        // tile, worked out once.  The next tile's chunks are loaded into registers before the current tile's products start, and go to LDS
        // (as float32) after them: the loads' latency hides behind the matrix pipe.
        constexpr int NIT = (DK4 / 2 + 2 * VT) / 4;
        constexpr int ck = DK4 / 2, cv = 2 * VT, n_chunks = 64 * (ck + cv);
        int place[NIT];  // key in tile | first column / 8 << 8 | is V << 24; -1: no chunk
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            const int q = tid + 256 * it;
            if (q >= n_chunks) place[it] = -1;
            else if (q < 64 * ck) place[it] = (q / ck) | ((q % ck) << 8);
            else place[it] = ((q - 64 * ck) / cv) | (((q - 64 * ck) % cv) << 8) | (1 << 24);
        }
        S raw[NIT][8];
        auto load_tile = [&](int kb) __attribute__((always_inline)) {
#pragma unroll
            for (int it = 0; it < NIT; ++it) {
                const int pl = place[it], j = kb + (pl & 255), c8 = 8 * ((pl >> 8) & 0xffff);
                const bool is_v = (pl >> 24) & 1;
#pragma unroll
                for (int e = 0; e < 8; ++e) raw[it][e] = (S)0;
                if (pl >= 0 && j < k_end && c8 < (is_v ? vdim : dim)) {
                    const int pg = page_shift >= 0 ? (j >> page_shift) : (j / page_size), in_pg = j - pg * page_size;
                    const int wd = is_v ? vdim : dim;  // v_row: the width of a row of vpool (vdim, or the key row's when the values are its leading columns)
                    const S *src = (is_v ? vpool + (((size_t)bt[pg] * Gv + kvh_v) * page_size + in_pg) * v_row
                                         : kpool + (((size_t)bt[pg] * G + kvh) * page_size + in_pg) * dim) + c8;
                    if (vec_ok) {  // (widths are multiples of 8: a chunk is whole or absent)
                        if constexpr (sizeof(S) == 2) *reinterpret_cast<u32x4 *>(raw[it]) = *reinterpret_cast<const u32x4 *>(src);
                        else {
                            *reinterpret_cast<u32x4 *>(raw[it]) = *reinterpret_cast<const u32x4 *>(src);
                            *reinterpret_cast<u32x4 *>(raw[it] + 4) = *reinterpret_cast<const u32x4 *>(src + 4);
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            if (c8 + e < wd) raw[it][e] = src[e];
                    }
                }
            }
        };
        auto store_tile = [&]() __attribute__((always_inline)) {
#pragma unroll
            for (int it = 0; it < NIT; ++it) {
                const int pl = place[it];
                if (pl < 0) continue;
                if constexpr (KB16) {
                    if (!((pl >> 24) & 1)) {  // a K chunk: 8 bfloat16 as they are
                        *reinterpret_cast<u32x4 *>(reinterpret_cast<uint16_t *>(Ks) + (pl & 255) * (2 * DKP) + 8 * ((pl >> 8) & 0xffff)) =
                            *reinterpret_cast<const u32x4 *>(raw[it]);
                        continue;
                    }
                }
                float *dst = ((pl >> 24) & 1) ? Vs + (pl & 255) * VP + 8 * ((pl >> 8) & 0xffff) : Ks + (pl & 255) * DKP + 8 * ((pl >> 8) & 0xffff);
                f32x4 lo, hi;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    lo[e] = D::to_float(raw[it][e]);
                    hi[e] = D::to_float(raw[it][4 + e]);
                }
                *reinterpret_cast<f32x4 *>(dst) = lo;
                *reinterpret_cast<f32x4 *>(dst + 4) = hi;
            }
        };
        load_tile(k_begin);
        for (int kb = k_begin; kb < k_end; kb += 64) {
            __syncthreads();  // every wave is done with the previous tile
            store_tile();
            __syncthreads();
            if (kb + 64 < k_end) load_tile(kb + 64);
            f32x4 sc[NN];
            float m_tile = -INFINITY;
#pragma unroll
            for (int nn = 0; nn < NN; ++nn) {
                const int n = nb + nn;
                f32x4 a4{0.f, 0.f, 0.f, 0.f};
                if constexpr (KB16) {
                    const uint16_t *kr = reinterpret_cast<const uint16_t *>(Ks) + (16 * n + col) * (2 * DKP) + 8 * g4;
#pragma unroll
                    for (int ks8 = 0; ks8 < DK4 / 8; ++ks8) {
                        const u32x4 ka = *reinterpret_cast<const u32x4 *>(kr + 32 * ks8);
                        a4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ka), __builtin_bit_cast(bf16x8_t, qb[ks8]), a4, 0, 0, 0);
                    }
#pragma unroll
                    for (int r = 0; r < 4; ++r) a4[r] *= scale;
                } else {
                    const float *kr = Ks + (16 * n + col) * DKP + g4;
#pragma unroll
                    for (int kk = 0; kk < DK4; ++kk) a4 = __builtin_amdgcn_mfma_f32_16x16x4f32(kr[4 * kk], qf[kk], a4, 0, 0, 0);
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int j = kb + 16 * n + 4 * g4 + r;
                    a4[r] = (row_ok && j <= qpos && j < k_end && (window <= 0 || qpos - j < window)) ? a4[r] : -INFINITY;
                    m_tile = fmaxf(m_tile, a4[r]);
                }
                sc[nn] = a4;
            }
            m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 16, 64));
            m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32, 64));
            const float m_new = fmaxf(m_run, m_tile);
            const float corr = (m_run == -INFINITY) ? 0.f : expf(m_run - m_new);
            float psum = 0.f;
#pragma unroll
            for (int nn = 0; nn < NN; ++nn)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float p = (sc[nn][r] == -INFINITY) ? 0.f : expf(sc[nn][r] - m_new);
                    sc[nn][r] = p;
                    psum += p;
                }
            psum += __shfl_xor(psum, 16, 64);
            psum += __shfl_xor(psum, 32, 64);
            l_run = l_run * corr + psum;
            m_run = m_new;
#pragma unroll
            for (int v = 0; v < VT; ++v)
#pragma unroll
                for (int r = 0; r < 4; ++r) o[v][r] *= corr;
#pragma unroll
            for (int nn = 0; nn < NN; ++nn)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float *vr = Vs + (16 * (nb + nn) + 4 * g4 + r) * VP + col;
#pragma unroll
                    for (int v = 0; v < VT; ++v)
                        o[v] = __builtin_amdgcn_mfma_f32_16x16x4f32(vr[16 * v], sc[nn][r], o[v], 0, 0, 0);
                }
        }
    }
    if constexpr (WSPLIT) {
        // four waves, four partial sets of the same 16 rows: through LDS (the tiles are no longer needed) to wave 0
        float *xm = smem, *xl = smem + 64, *xo = smem + 128;  // [4][16], [4][16], [4][64][4 VT]
        __syncthreads();
        if (g4 == 0) {
            xm[wave * 16 + col] = m_run;
            xl[wave * 16 + col] = l_run;
        }
#pragma unroll
        for (int v = 0; v < VT; ++v) *reinterpret_cast<f32x4 *>(xo + ((size_t)(wave * 64 + lane) * VT + v) * 4) = o[v];
        __syncthreads();
        if (wave != 0) return;
        float M = -INFINITY;
#pragma unroll
        for (int w = 0; w < 4; ++w) M = fmaxf(M, xm[w * 16 + col]);
        float L = 0.f;
#pragma unroll
        for (int v = 0; v < VT; ++v) o[v] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float mw = xm[w * 16 + col];
            const float f = (mw == -INFINITY) ? 0.f : expf(mw - M);
            L += xl[w * 16 + col] * f;
#pragma unroll
            for (int v = 0; v < VT; ++v) {
                const f32x4 ow = *reinterpret_cast<const f32x4 *>(xo + ((size_t)(w * 64 + lane) * VT + v) * 4);
#pragma unroll
                for (int r = 0; r < 4; ++r) o[v][r] += ow[r] * f;
            }
        }
        m_run = M;
        l_run = L;
    }
    if (!row_ok) return;
    if (n_splits == 1) {
        const float invl = l_run > 0.f ? 1.f / l_run : 0.f;
#pragma unroll
        for (int v = 0; v < VT; ++v)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int c = 16 * v + 4 * g4 + r;
                if (c < vdim) {
                    float val = o[v][r] * invl;
                    if (gate) val *= sigmoid_f(gate[(size_t)trow * ldg + (gate_per_head ? (size_t)head : (size_t)head * vdim + c)]);
                    if (out32) out32[((size_t)trow * H + head) * vdim + c] = val;
                    else out[(size_t)trow * ldo + (size_t)head * vdim + c] = D::from_float(val);
                }
            }
    } else {
        const size_t pi = ((size_t)trow * H + head) * n_splits + split;
#pragma unroll
        for (int v = 0; v < VT; ++v)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int c = 16 * v + 4 * g4 + r;
                if (c < vdim) part_acc[pi * vdim + c] = o[v][r];
            }
        if (g4 == 0) {
            part_ml[2 * pi] = m_run;
            part_ml[2 * pi + 1] = l_run;
        }
    }
}

// the splits of a row's key range put together: one wave per (row, query head), n_splits <= 64.  Lane s owns split s for the maximum, the
// sum and the weights exp(m_s - M); then the lanes turn to the value columns and walk the splits with those weights.
template <typename D>
__global__ __launch_bounds__(64) void attn_merge_kernel(const float *part_acc, const float *part_ml, int n_splits, int H, int vdim, const float *gate,
                                                        int ldg, typename D::storage *out, int ldo, int gate_per_head, float *out32) {
    __shared__ float ws[64];
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const size_t p0 = ((size_t)t * H + h) * n_splits;
    const float m = lane < n_splits ? part_ml[2 * (p0 + lane)] : -INFINITY;
    const float l = lane < n_splits ? part_ml[2 * (p0 + lane) + 1] : 0.f;
    const float M = wave_max(m);
    const float w = (m == -INFINITY) ? 0.f : expf(m - M);
    const float L = wave_sum(l * w);
    ws[lane] = w;
    __syncthreads();
    const float invl = L > 0.f ? 1.f / L : 0.f;
    for (int c = lane; c < vdim; c += 64) {
        float acc = 0.f;
#pragma unroll 8
        for (int s = 0; s < n_splits; ++s) acc += part_acc[(p0 + s) * vdim + c] * ws[s];
        float val = acc * invl;
        if (gate) val *= sigmoid_f(gate[(size_t)t * ldg + (gate_per_head ? (size_t)h : (size_t)h * vdim + c)]);
        if (out32) out32[((size_t)t * H + h) * vdim + c] = val;
        else out[(size_t)t * ldo + (size_t)h * vdim + c] = D::from_float(val);
    }
}

// ---- attention, step 1 (head form with a norm ahead of the rotation): one wave per (row, head and map of q | k, value head) ------------------
// proj: q | k | v at columns 0 | H*M*dim | (H+G)*M*dim; M maps per head lie side by side ([map 1 | map 2] with M = 2).  Every (head, map) of q and
// k: x / sqrt(mean x^2 + eps) * w over dim (qw / kw [dim], shared by all heads and maps; head_norm 0: none), then the rotation of the first
// rot_dims dimensions by pos * inv_freq[i]: pairs (i, i + rot_dims/2) with rot_half, (2i, 2i+1) without.
// q goes to qbuf as H*M heads ordered [K/V head][map][head in group], k to kpool as G*M K/V heads [K/V head][map]: query head e of that order reads
// K/V head e / (H/G), and K/V head g reads value head g / M.
template <typename D>
__global__ __launch_bounds__(64) void attn_prep_head_kernel(const float *proj, int ldp, const int32_t *row_seq, const int32_t *row_pos, const int32_t *seq_slot,
                                                            const int32_t *block_table, int max_pages, int page_size, const float *inv_freq, int rot_dims,
                                                            int rot_half, int head_norm, const float *qw, const float *kw, float eps, int H, int G, int M, int dim,
                                                            int vdim, float *qbuf, typename D::storage *kpool, typename D::storage *vpool, const float *bias) {
    const int t = blockIdx.x, hh = blockIdx.y, lane = threadIdx.x;
    const int pos = row_pos[t], slot = seq_slot[row_seq[t]];
    const int page = block_table[(size_t)slot * max_pages + pos / page_size], in_page = pos % page_size;
    const int HM = H * M, GM = G * M;
    if (hh >= HM + GM) {  // a value head: copy
        const int g = hh - HM - GM;
        const size_t col = (size_t)(HM + GM) * dim + (size_t)g * vdim;
        const float *src = proj + (size_t)t * ldp + col;
        typename D::storage *dst = vpool + (((size_t)page * G + g) * page_size + in_page) * vdim;
        for (int c = lane; c < vdim; c += 64) dst[c] = D::from_float(src[c] + (bias ? bias[col + c] : 0.f));
        return;
    }
    const bool is_q = hh < HM;
    const float *src = proj + (size_t)t * ldp + (size_t)hh * dim;
    const float *bs = bias ? bias + (size_t)hh * dim : nullptr;  // bias (NULL: none): the projection's, over the columns of proj, added here
    const float *w = head_norm ? (is_q ? qw : kw) : nullptr;
    float inv = 1.f;
    if (head_norm) {
        float ss = 0.f;
        for (int c = lane; c < dim; c += 64) {
            const float v = src[c] + (bs ? bs[c] : 0.f);
            ss += v * v;
        }
        ss = wave_sum(ss);
        inv = 1.f / sqrtf(ss / (float)dim + eps);
    }
    float *qdst = nullptr;
    typename D::storage *kdst = nullptr;
    if (is_q) {
        const int h = hh / M, mp = hh % M, HG = H / G;
        qdst = qbuf + ((size_t)t * HM + ((size_t)(h / HG) * M + mp) * HG + h % HG) * dim;
    } else
        kdst = kpool + (((size_t)page * GM + (hh - HM)) * page_size + in_page) * dim;
    const int half = rot_dims / 2, units = dim - half;  // `half` rotation pairs, then the dimensions that pass
    for (int u = lane; u < units; u += 64) {
        int c0, c1 = -1;
        if (u < half) c0 = rot_half ? u : 2 * u, c1 = rot_half ? u + half : 2 * u + 1;
        else c0 = u + half;
        float a = (src[c0] + (bs ? bs[c0] : 0.f)) * inv * (w ? w[c0] : 1.f), b2 = 0.f;
        if (c1 >= 0) {
            b2 = (src[c1] + (bs ? bs[c1] : 0.f)) * inv * (w ? w[c1] : 1.f);
            float sn, cs;
            sincosf((float)pos * inv_freq[u], &sn, &cs);
            const float na = a * cs - b2 * sn, nb = b2 * cs + a * sn;
            a = na, b2 = nb;
        }
        if (is_q) {
            qdst[c0] = a;
            if (c1 >= 0) qdst[c1] = b2;
        } else {
            kdst[c0] = D::from_float(a);
            if (c1 >= 0) kdst[c1] = D::from_float(b2);
        }
    }
}

// ---- differential attention, last step: one wave per (row, head).  a [rows, H*2, vdim] float32 in the order attn_prep_head_kernel gives the
// maps ([K/V head][map][head in group]); o = a1 - lambda a2;  o / sqrt(mean o^2 + eps) * (1 - init) * sigmoid(gate) -> D rows.
// gate (may be NULL): one number per head (gate_per_head) or per output channel.
template <typename D>
__global__ __launch_bounds__(64) void diff_combine_kernel(const float *a, float lambda, float init, float eps, const float *gate, int ldg, int gate_per_head,
                                                          int H, int G, int vdim, typename D::storage *out, int ldo) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x, HG = H / G;
    const float *a1 = a + ((size_t)t * 2 * H + ((size_t)(h / HG) * 2) * HG + h % HG) * vdim, *a2 = a1 + (size_t)HG * vdim;
    float o[8], ss = 0.f;  // vdim <= 512
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int c = lane + 64 * i;
        o[i] = c < vdim ? a1[c] - lambda * a2[c] : 0.f;
        ss += o[i] * o[i];
    }
    ss = wave_sum(ss);
    const float mul = (1.f - init) / sqrtf(ss / (float)vdim + eps);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int c = lane + 64 * i;
        if (c < vdim) {
            float v = o[i] * mul;
            if (gate) v *= sigmoid_f(gate[(size_t)t * ldg + (gate_per_head ? (size_t)h : (size_t)h * vdim + c)]);
            out[(size_t)t * ldo + (size_t)h * vdim + c] = D::from_float(v);
        }
    }
}

// ---- attention, step 1 (row form): one workgroup per row prepares q, k and v with the options the head-wise kernel above does not have ----
// qk_norm: q (all heads) and k (all K/V heads) are each divided by the RMS of their WHOLE projection and multiplied by qw / kw, before the rotation.
// Rotation of the first rot_dims dimensions of each head by pos * inv_freq[i]: pairs (i, i + rot_dims/2) with rot_half, (2i, 2i+1) without.
// v_mix 1: the row's values are kept in vref [rows, G*vdim]; 2: v <- (1 - lambda) v + lambda vref before they go to their page.
template <typename D>
__global__ __launch_bounds__(1024) void attn_prep_row_kernel(const float *proj, int ldp, const int32_t *row_seq, const int32_t *row_pos, const int32_t *seq_slot,
                                                            const int32_t *block_table, int max_pages, int page_size, const float *inv_freq, int rot_dims,
                                                            int rot_half, int qk_norm, const float *qw, const float *kw, float eps, int H, int G, int dim, int vdim,
                                                            int v_mix, float lambda, float *vref, float *qbuf, typename D::storage *kpool,
                                                            typename D::storage *vpool) {
    __shared__ float red[16];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int pos = row_pos[t], slot = seq_slot[row_seq[t]];
    const int page = block_table[(size_t)slot * max_pages + pos / page_size], in_page = pos % page_size;
    const float *row = proj + (size_t)t * ldp;
    const int nq = H * dim, nk = G * dim, nv = G * vdim;
    float inv_q = 1.f, inv_k = 1.f;
    if (qk_norm) {
        float sq = 0.f, sk = 0.f;
        for (int c = tid; c < nq; c += blockDim.x) sq += row[c] * row[c];
        for (int c = tid; c < nk; c += blockDim.x) sk += row[nq + c] * row[nq + c];
        sq = block_sum(sq, red);
        sk = block_sum(sk, red);
        inv_q = 1.f / sqrtf(sq / (float)nq + eps);
        inv_k = 1.f / sqrtf(sk / (float)nk + eps);
    }
    const int half = rot_dims / 2, units = dim - half;  // per head: `half` rotation pairs, then the dimensions that pass
    for (int e = tid; e < (H + G) * units; e += blockDim.x) {
        const int hh = e / units, u = e % units;
        const bool is_q = hh < H;
        const float *src = row + (size_t)hh * dim;  // (k heads follow the q heads in the row)
        const float *w = qk_norm ? (is_q ? qw + (size_t)hh * dim : kw + (size_t)(hh - H) * dim) : nullptr;
        const float inv = is_q ? inv_q : inv_k;
        int c0, c1 = -1;
        if (u < half) c0 = rot_half ? u : 2 * u, c1 = rot_half ? u + half : 2 * u + 1;
        else c0 = u + half;
        float a = src[c0] * inv * (w ? w[c0] : 1.f), b2 = 0.f;
        if (c1 >= 0) {
            b2 = src[c1] * inv * (w ? w[c1] : 1.f);
            float sn, cs;
            sincosf((float)pos * inv_freq[u], &sn, &cs);
            const float na = a * cs - b2 * sn, nb = b2 * cs + a * sn;
            a = na, b2 = nb;
        }
        if (is_q) {
            float *dst = qbuf + (size_t)t * nq + (size_t)hh * dim;
            dst[c0] = a;
            if (c1 >= 0) dst[c1] = b2;
        } else {
            typename D::storage *dst = kpool + (((size_t)page * G + (hh - H)) * page_size + in_page) * dim;
            dst[c0] = D::from_float(a);
            if (c1 >= 0) dst[c1] = D::from_float(b2);
        }
    }
    for (int e = tid; e < nv; e += blockDim.x) {
        float v = row[nq + nk + e];
        if (v_mix == 1) vref[(size_t)t * nv + e] = v;
        else if (v_mix == 2) v = (1.f - lambda) * v + lambda * vref[(size_t)t * nv + e];
        vpool[(((size_t)page * G + e / vdim) * page_size + in_page) * vdim + e % vdim] = D::from_float(v);
    }
}

// ---- attention, step 2 with scores mixed across heads (row form): one workgroup per row, a wave per mixed head ----------------------------
// For every tile of 64 keys the waves first form the raw scores of ALL query heads (lane = key; head h reads K/V head h / (H/G)) in LDS; then wave
// w mixes them for its head, s'_h = sum_g talk[h, g] s_g (talk NULL: s_h), and keeps a running maximum / sum / weighted value sum in float32.
// chunk > 0: the keys start at the first position of the query's chunk.  sink: the running pair starts at (sinks[h] or 0, 1).
// More heads than waves: the waves take the heads in passes and the raw scores are formed again per pass.
template <typename D>
__global__ __launch_bounds__(1024) void attn_talk_rows_kernel(const float *qbuf, const typename D::storage *kpool, const typename D::storage *vpool,
                                                              const int32_t *row_seq, const int32_t *row_pos, const int32_t *seq_slot,
                                                              const int32_t *block_table, int max_pages, int page_size, int H, int G, int dim, int vdim,
                                                              float scale, const float *talk, int sink, const float *sinks, int chunk, const float *gate,
                                                              int ldg, typename D::storage *out, int ldo) {
    extern __shared__ float smem[];
    const int nw = blockDim.x >> 6, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    float *qs = smem;                 // [H][dim]
    float *sc = qs + (size_t)H * dim; // [H][64] raw scores of the tile
    float *ps = sc + (size_t)H * 64;  // [nw][64] weights of the tile, per wave
    const int t = blockIdx.x;
    const int pos = row_pos[t], slot = seq_slot[row_seq[t]], HG = H / G;
    const int32_t *bt = block_table + (size_t)slot * max_pages;
    const int lo = chunk > 0 ? (pos / chunk) * chunk : 0;
    for (int c = threadIdx.x; c < H * dim; c += blockDim.x) qs[c] = qbuf[(size_t)t * H * dim + c];
    __syncthreads();
    for (int h0 = 0; h0 < H; h0 += nw) {
        const int hm = h0 + wave;
        const bool live = hm < H;
        const int gm = live ? hm / HG : 0;
        float m = sink ? (sinks && live ? sinks[hm] : 0.f) : -INFINITY, l = sink ? 1.f : 0.f;
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};  // vdim <= 512
        for (int kb = lo; kb <= pos; kb += 64) {
            const int j = kb + lane;
            for (int h = wave; h < H; h += nw) {
                float d = 0.f;
                if (j <= pos) {
                    const typename D::storage *kr = kpool + (((size_t)bt[j / page_size] * G + h / HG) * page_size + j % page_size) * dim;
                    const float *q = qs + (size_t)h * dim;
                    for (int c = 0; c < dim; ++c) d += q[c] * D::to_float(kr[c]);
                }
                sc[h * 64 + lane] = d * scale;
            }
            __syncthreads();
            if (live) {
                float s;
                if (talk) {
                    s = 0.f;
                    for (int g = 0; g < H; ++g) s += talk[hm * H + g] * sc[g * 64 + lane];
                } else s = sc[hm * 64 + lane];
                if (j > pos) s = -INFINITY;
                const float m_new = fmaxf(m, wave_max(s));
                const float p = (j <= pos) ? expf(s - m_new) : 0.f;
                const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
                l = l * corr + wave_sum(p);
                m = m_new;
                ps[wave * 64 + lane] = p;  // (read by this wave only: its lanes run in lockstep)
                __builtin_amdgcn_wave_barrier();
                const int cnt = min(64, pos - kb + 1);
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[i] *= corr;
                for (int jj = 0; jj < cnt; ++jj) {
                    const int jg = kb + jj;
                    const typename D::storage *vr = vpool + (((size_t)bt[jg / page_size] * G + gm) * page_size + jg % page_size) * vdim;
                    const float pj = ps[wave * 64 + jj];
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        const int c = lane + i * 64;
                        if (c < vdim) acc[i] += pj * D::to_float(vr[c]);
                    }
                }
            }
            __syncthreads();
        }
        if (live) {
            const float invl = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int c = lane + i * 64;
                if (c < vdim) {
                    float o = acc[i] * invl;
                    if (gate) o *= sigmoid_f(gate[(size_t)t * ldg + (size_t)hm * vdim + c]);
                    out[(size_t)t * ldo + (size_t)hm * vdim + c] = D::from_float(o);
                }
            }
        }
    }
}

// ---- attention, step 2 with scores mixed across heads (tile form): MFMA flash attention in which a workgroup sees EVERY query head of its tokens ----
// Mixing needs the scores of all heads of a (query, key) pair at once, so a workgroup owns TQB = 16 / HGB tokens with all their heads: G row blocks of 16
// rows, block g = the query heads of K/V head g (row = token * HGB + head in group, HGB = the group's heads rounded up to a power of two).  It forms the raw
// scores of all G blocks, but weights and values only of the NP blocks blockIdx.y * NP ..: prompts take up to four blocks per workgroup, single-token steps
// one (the chain of a step is short, the raw scores are cheap to repeat).  The four waves split the KEYS: of every 64-key tile wave w takes keys 16 w ..
// 16 w + 15 and keeps its own running (max, sum, O) per row; the four partial sets are merged through LDS at the end.  Nothing in the key loop is shared
// between waves but read-only LDS (queries, mixing matrix), so it runs without workgroup barriers.  Per tile and wave:
//   S^T_g[key, row] = K_g . Q_g^T  for g < G      A = the wave's 16 key rows of K/V head g straight from their pages (a lane's 8 consecutive bfloat16, or
//                                                 DK4 consecutive float32: a dot product does not care in which order its terms are paired; the next tile's
//                                                 rows are loaded ahead of the value products), B = the block's query rows from LDS (bfloat16 pages:
//                                                 v_mfma_f32_16x16x32_bf16 with float32 sums; float32 pages: v_mfma_f32_16x16x4_f32)
//   mix: the raw scores go to the wave's LDS region as [key][token][head]; every lane reads the heads of its (key, token) back and forms
//        s'_h = sum_g talk[h, g] s_g for its head in each of its blocks (the matrix lies in LDS over the padded heads; no mixing = identity)
//   mask (causal; chunked: keys from the first position of the query's chunk), running maximum and sum per row -- the sink is their start value (sink_h, 1)
//   O^T_g[vcol, row] += V_g^T . P_g^T           A = the wave's 16 rows of V_g, loaded at the tile's start and staged in its LDS region as float32,
//                                                 B = the weights where the mix left them (v_mfma_f32_16x16x4_f32)
// The key range may be split over gridDim.z (decode steps over long contexts): partial sums + (max, sum) go to part_* and attn_merge_kernel finishes.
template <typename D, int DK4, int VT, int NP>
__global__ __launch_bounds__(256) void attn_talk_tile_kernel(const float *qbuf, const typename D::storage *kpool, const typename D::storage *vpool,
                                                             const int32_t *seq_row0, const int32_t *seq_slot, const int32_t *row_pos,
                                                             const int32_t *block_table, int max_pages, int page_size, int H, int G, int dim, int vdim,
                                                             float scale, const float *talk, int sink, const float *sinks, int chunk, int HGB,
                                                             int keys_per_split, int n_splits, const float *gate, int ldg, typename D::storage *out, int ldo,
                                                             float *part_acc, float *part_ml, int page_shift, int vec_ok) {
    using S = typename D::storage;
    extern __shared__ float smem[];
    constexpr bool KB16 = sizeof(S) == 2;
    constexpr int VP = 16 * VT + 4, NITV = VT / 2;
    constexpr int QP = KB16 ? (4 * DK4 + 8) / 2 : 4 * DK4 + 4;  // floats per query row in LDS (bfloat16 rows: 4 DK4 + 8 16-bit elements)
    constexpr int NKA = KB16 ? DK4 / 8 : DK4 / 4;               // 16-byte pieces of a key row a lane holds
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g4 = lane >> 4, col = lane & 15;
    // the exponential of a weight: with bfloat16 pages the hardware's (the values it multiplies carry 8 bits); float32 pages keep the exact one
    auto exp_t = [](float x) __attribute__((always_inline)) { return KB16 ? __expf(x) : expf(x); };
    const int seq = blockIdx.z / n_splits, split = blockIdx.z % n_splits;
    const int HG = H / G, TQB = 16 / HGB, HP = G * HGB, XW = 16 * G + 4, g_own0 = blockIdx.y * NP;
    const int r0 = seq_row0[seq], len = seq_row0[seq + 1] - r0, t0 = blockIdx.x * TQB;
    if (t0 >= len) return;
    float *Tl = smem;                                                       // [HP][HP] mixing matrix over padded heads
    float *Qs = smem + HP * HP;                                             // [G][16][QP] query rows of every block
    float *Vw = Qs + (size_t)G * 16 * QP + wave * (16 * VP + 16 * XW);      // [16][VP] this wave's value rows of one K/V head
    float *Sx = Vw + 16 * VP;                                               // [16][XW] this wave's raw scores: [key][token * HP + block * HGB + head in group]
    const int pos0 = row_pos[r0], slot = seq_slot[seq];
    for (int i = tid; i < HP * HP; i += 256) {
        const int tp = i / HP, sp = i % HP, gt = tp / HGB, ht = tp % HGB, gs = sp / HGB, hs = sp % HGB;
        const bool ok = ht < HG && hs < HG;
        Tl[i] = ok ? (talk ? talk[(size_t)(gt * HG + ht) * H + gs * HG + hs] : (tp == sp ? 1.f : 0.f)) : 0.f;
    }
    for (int i = tid; i < G * 16 * (2 * DK4); i += 256) {  // pairs of dimensions; rows beyond the chunk's tokens and heads beyond the group are zero
        const int d = 2 * (i % (2 * DK4)), rw = (i / (2 * DK4)) % 16, g = i / (2 * DK4 * 16);
        const int t = rw / HGB, h = rw % HGB;
        const bool ok = t0 + t < len && h < HG;
        const float *qrow = qbuf + ((size_t)(r0 + t0 + t) * H + (size_t)g * HG + h) * dim;
        const float a = (ok && d < dim) ? qrow[d] : 0.f, b2 = (ok && d + 1 < dim) ? qrow[d + 1] : 0.f;
        if constexpr (KB16) reinterpret_cast<uint32_t *>(Qs)[((size_t)g * 16 + rw) * QP + d / 2] = BF16::pack2(a, b2);
        else {
            Qs[((size_t)g * 16 + rw) * QP + d] = a * scale;
            Qs[((size_t)g * 16 + rw) * QP + d + 1] = b2 * scale;
        }
    }
    __syncthreads();
    const int32_t *bt = block_table + (size_t)slot * max_pages;
    const int tl = col / HGB, hb = col % HGB;
    const bool row_ok = t0 + tl < len && hb < HG;
    const int trow = r0 + t0 + tl, qpos = pos0 + t0 + tl;
    const int qlo = chunk > 0 ? (qpos / chunk) * chunk : 0;
    const int q_first = pos0 + t0, q_last = pos0 + min(t0 + TQB, len) - 1;
    const int k_lo = chunk > 0 ? (q_first / chunk) * chunk : 0;
    const int k_begin = max(k_lo, split * keys_per_split), k_end = min(q_last + 1, (split + 1) * keys_per_split);
    const bool owns_sink = sink && split == 0 && wave == 0;
    float m_run[NP], l_run[NP];
    f32x4 o[NP][VT];
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        const int head = min(g_own0 + i, G - 1) * HG + min(hb, HG - 1);
        m_run[i] = owns_sink ? (sinks ? sinks[head] : 0.f) : -INFINITY;
        l_run[i] = owns_sink ? 1.f : 0.f;
#pragma unroll
        for (int v = 0; v < VT; ++v) o[i][v] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    if (k_begin < k_end) {
        // a lane's pieces of the key rows of four K/V heads (key kb + 16 wave + col): bfloat16 pages: dimensions 32 ks8 + 8 g4 .. + 7; float32 pages:
        // dimensions g4 * DK4 + 4 c .. + 3
        u32x4 ka[4][NKA];
        auto load_k = [&](int gc, int kb) __attribute__((always_inline)) {
            const int jk = kb + 16 * wave + col;
            const bool key_ok = jk < k_end;
            const int pgk = key_ok ? (page_shift >= 0 ? (jk >> page_shift) : (jk / page_size)) : 0, in_pgk = jk - pgk * page_size;
            const size_t krow0 = key_ok ? ((size_t)bt[pgk] * G * page_size + in_pgk) : 0;
#pragma unroll
            for (int gi = 0; gi < 4; ++gi) {
                const int g = gc + gi;
                const S *kr = kpool + (krow0 + (size_t)min(g, G - 1) * page_size) * dim;
                const bool ok = key_ok && g < G;
#pragma unroll
                for (int c = 0; c < NKA; ++c) {
                    const int d = KB16 ? 32 * c + 8 * g4 : g4 * DK4 + 4 * c;
                    constexpr int NE = KB16 ? 8 : 4;
                    ka[gi][c] = u32x4{0u, 0u, 0u, 0u};
                    if (ok && d < dim) {
                        if (vec_ok) ka[gi][c] = *reinterpret_cast<const u32x4 *>(kr + d);
                        else {
                            S tmp[NE];
#pragma unroll
                            for (int e = 0; e < NE; ++e) tmp[e] = d + e < dim ? kr[d + e] : (S)0;
                            ka[gi][c] = *reinterpret_cast<const u32x4 *>(tmp);
                        }
                    }
                }
            }
        };
        // this lane's value chunks of its blocks: 16 keys x 2 VT chunks of 8 columns, lane + 64 it
        S vraw[NP][NITV][8];
        auto load_v = [&](int i, int kb) __attribute__((always_inline)) {
#pragma unroll
            for (int it = 0; it < NITV; ++it) {
                const int g = g_own0 + i, q = lane + 64 * it, j = kb + 16 * wave + q / (2 * VT), c8 = 8 * (q % (2 * VT));
#pragma unroll
                for (int e = 0; e < 8; ++e) vraw[i][it][e] = (S)0;
                if (g < G && j < k_end && c8 < vdim) {
                    const int pg = page_shift >= 0 ? (j >> page_shift) : (j / page_size), in_pg = j - pg * page_size;
                    const S *src = vpool + (((size_t)bt[pg] * G + g) * page_size + in_pg) * vdim + c8;
                    if (vec_ok) {
                        if constexpr (KB16) *reinterpret_cast<u32x4 *>(vraw[i][it]) = *reinterpret_cast<const u32x4 *>(src);
                        else {
                            *reinterpret_cast<u32x4 *>(vraw[i][it]) = *reinterpret_cast<const u32x4 *>(src);
                            *reinterpret_cast<u32x4 *>(vraw[i][it] + 4) = *reinterpret_cast<const u32x4 *>(src + 4);
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            if (c8 + e < vdim) vraw[i][it][e] = src[e];
                    }
                }
            }
        };
        load_k(0, k_begin);
#pragma unroll
        for (int i = 0; i < NP; ++i) load_v(i, k_begin);
        for (int kb = k_begin; kb < k_end; kb += 64) {
            // ---- raw scores of every block for this wave's 16 keys, four K/V heads at a time ----
            for (int gc = 0; gc < G; gc += 4) {
                if (gc > 0) load_k(gc, kb);
#pragma unroll
                for (int gi = 0; gi < 4; ++gi) {
                    const int g = gc + gi;
                    if (g < G) {
                        f32x4 a4{0.f, 0.f, 0.f, 0.f};
                        if constexpr (KB16) {
                            const uint16_t *qr = reinterpret_cast<const uint16_t *>(Qs) + ((size_t)g * 16 + col) * (2 * QP) + 8 * g4;
#pragma unroll
                            for (int ks8 = 0; ks8 < DK4 / 8; ++ks8) {
                                const u32x4 qv = *reinterpret_cast<const u32x4 *>(qr + 32 * ks8);
                                a4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ka[gi][ks8]), __builtin_bit_cast(bf16x8_t, qv), a4, 0, 0, 0);
                            }
#pragma unroll
                            for (int r = 0; r < 4; ++r) a4[r] *= scale;
                        } else {
                            const float *qr = Qs + ((size_t)g * 16 + col) * QP + g4 * DK4;
#pragma unroll
                            for (int c = 0; c < DK4 / 4; ++c) {
                                const f32x4 qv = *reinterpret_cast<const f32x4 *>(qr + 4 * c);
#pragma unroll
                                for (int e = 0; e < 4; ++e) a4 = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(ka[gi][c][e]), qv[e], a4, 0, 0, 0);
                            }
                        }
#pragma unroll
                        for (int r = 0; r < 4; ++r) Sx[(4 * g4 + r) * XW + tl * HP + g * HGB + hb] = a4[r];
                    }
                }
            }
            if (kb + 64 < k_end) load_k(0, kb + 64);  // lands while the values are multiplied
            __builtin_amdgcn_wave_barrier();
            // ---- mix across heads for the blocks of this workgroup ----
            f32x4 sc[NP];
#pragma unroll
            for (int i = 0; i < NP; ++i) sc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
            if ((HP & 3) == 0) {
                for (int sp = 0; sp < HP; sp += 4) {
                    f32x4 x[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) x[r] = *reinterpret_cast<const f32x4 *>(Sx + (4 * g4 + r) * XW + tl * HP + sp);
#pragma unroll
                    for (int i = 0; i < NP; ++i) {
                        const f32x4 c = *reinterpret_cast<const f32x4 *>(Tl + (size_t)(min(g_own0 + i, G - 1) * HGB + hb) * HP + sp);
#pragma unroll
                        for (int r = 0; r < 4; ++r) sc[i][r] += c[0] * x[r][0] + c[1] * x[r][1] + c[2] * x[r][2] + c[3] * x[r][3];
                    }
                }
            } else {
                for (int sp = 0; sp < HP; ++sp) {
#pragma unroll
                    for (int i = 0; i < NP; ++i) {
                        const float c = Tl[(size_t)(min(g_own0 + i, G - 1) * HGB + hb) * HP + sp];
#pragma unroll
                        for (int r = 0; r < 4; ++r) sc[i][r] += c * Sx[(4 * g4 + r) * XW + tl * HP + sp];
                    }
                }
            }
            __builtin_amdgcn_wave_barrier();
            // ---- mask, running maximum and sum per row and block (all blocks first: their lane exchanges overlap) ----
            float corr[NP];
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                const bool blk_ok = row_ok && g_own0 + i < G;
                float m_tile = -INFINITY;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int j = kb + 16 * wave + 4 * g4 + r;
                    sc[i][r] = (blk_ok && j <= qpos && j >= qlo && j < k_end) ? sc[i][r] : -INFINITY;
                    m_tile = fmaxf(m_tile, sc[i][r]);
                }
                m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 16, 64));
                m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32, 64));
                const float m_new = fmaxf(m_run[i], m_tile);
                corr[i] = (m_run[i] == -INFINITY) ? 0.f : (m_new == m_run[i] ? 1.f : exp_t(m_run[i] - m_new));
                float psum = 0.f;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float p = (sc[i][r] == -INFINITY) ? 0.f : exp_t(sc[i][r] - m_new);
                    sc[i][r] = p;
                    psum += p;
                }
                psum += __shfl_xor(psum, 16, 64);
                psum += __shfl_xor(psum, 32, 64);
                l_run[i] = l_run[i] * corr[i] + psum;
                m_run[i] = m_new;
            }
            // ---- the values of each block; the block's rows of the next tile are loaded as soon as this tile's are in LDS ----
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                if (__any(corr[i] != 1.f && l_run[i] != 0.f)) {  // (most tiles move no row's maximum: the sums keep their scale)
#pragma unroll
                    for (int v = 0; v < VT; ++v)
#pragma unroll
                        for (int r = 0; r < 4; ++r) o[i][v][r] *= corr[i];
                }
#pragma unroll
                for (int it = 0; it < NITV; ++it) {
                    const int q = lane + 64 * it;
                    float *dst = Vw + (q / (2 * VT)) * VP + 8 * (q % (2 * VT));
                    f32x4 lo, hi;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        lo[e] = D::to_float(vraw[i][it][e]);
                        hi[e] = D::to_float(vraw[i][it][4 + e]);
                    }
                    *reinterpret_cast<f32x4 *>(dst) = lo;
                    *reinterpret_cast<f32x4 *>(dst + 4) = hi;
                }
                __builtin_amdgcn_wave_barrier();
                if (kb + 64 < k_end) load_v(i, kb + 64);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float *vr = Vw + (4 * g4 + r) * VP + col;
#pragma unroll
                    for (int v = 0; v < VT; ++v) o[i][v] = __builtin_amdgcn_mfma_f32_16x16x4f32(vr[16 * v], sc[i][r], o[i][v], 0, 0, 0);
                }
                __builtin_amdgcn_wave_barrier();
            }
        }
    }
    // four waves, four partial sets of the same rows: block by block through LDS (the key loop's regions are no longer needed); wave i & 3 finishes block i
    float *xm = smem, *xl = smem + 64, *xo = smem + 128;  // [4][16], [4][16], [4][64][4 VT]
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        __syncthreads();
        if (g4 == 0) {
            xm[wave * 16 + col] = m_run[i];
            xl[wave * 16 + col] = l_run[i];
        }
#pragma unroll
        for (int v = 0; v < VT; ++v) *reinterpret_cast<f32x4 *>(xo + ((size_t)(wave * 64 + lane) * VT + v) * 4) = o[i][v];
        __syncthreads();
        const int g = g_own0 + i;
        if (wave != (i & 3) || g >= G) continue;
        float M = -INFINITY;
#pragma unroll
        for (int w = 0; w < 4; ++w) M = fmaxf(M, xm[w * 16 + col]);
        float L = 0.f;
        f32x4 of[VT];
#pragma unroll
        for (int v = 0; v < VT; ++v) of[v] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float mw = xm[w * 16 + col];
            const float f = (mw == -INFINITY) ? 0.f : expf(mw - M);
            L += xl[w * 16 + col] * f;
#pragma unroll
            for (int v = 0; v < VT; ++v) {
                const f32x4 ow = *reinterpret_cast<const f32x4 *>(xo + ((size_t)(w * 64 + lane) * VT + v) * 4);
#pragma unroll
                for (int r = 0; r < 4; ++r) of[v][r] += ow[r] * f;
            }
        }
        if (n_splits == 1) {
            // the block's 16 rows x vdim through the wave's LDS region, so that a lane writes 8 consecutive columns of one row (and reads its gate as such)
            float *xt = smem + 128 + 4 * 64 * 4 * VT + (i & 3) * 16 * VP;  // [16][VP], behind the partial sets
            const float invl = L > 0.f ? 1.f / L : 0.f;
#pragma unroll
            for (int v = 0; v < VT; ++v) {
                f32x4 t4;
#pragma unroll
                for (int r = 0; r < 4; ++r) t4[r] = of[v][r] * invl;
                *reinterpret_cast<f32x4 *>(xt + col * VP + 16 * v + 4 * g4) = t4;
            }
            __builtin_amdgcn_wave_barrier();
            const int orow = lane >> 2, otl = orow / HGB, ohb = orow % HGB;
            if (t0 + otl < len && ohb < HG) {
                const size_t orow_g = (size_t)(r0 + t0 + otl), ohead = (size_t)g * HG + ohb;
#pragma unroll
                for (int k = 0; k < VT / 2; ++k) {
                    const int c8 = 8 * ((lane & 3) + 4 * k);
                    if (c8 >= vdim) continue;
                    const f32x4 lo = *reinterpret_cast<const f32x4 *>(xt + orow * VP + c8), hi = *reinterpret_cast<const f32x4 *>(xt + orow * VP + c8 + 4);
                    float val[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    const float *gp = gate ? gate + orow_g * ldg + ohead * vdim + c8 : nullptr;
                    S *op = out + orow_g * ldo + ohead * vdim + c8;
                    if (vec_ok && (ldg & 3) == 0 && (ldo & 7) == 0 && ((uintptr_t)gate & 15) == 0 && ((uintptr_t)out & 15) == 0) {
                        if (gp) {
                            const f32x4 ga = *reinterpret_cast<const f32x4 *>(gp), gb = *reinterpret_cast<const f32x4 *>(gp + 4);
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                val[e] *= sigmoid_f(ga[e]);
                                val[4 + e] *= sigmoid_f(gb[e]);
                            }
                        }
                        S pk[8];
#pragma unroll
                        for (int e = 0; e < 8; ++e) pk[e] = D::from_float(val[e]);
                        if constexpr (KB16) *reinterpret_cast<u32x4 *>(op) = *reinterpret_cast<const u32x4 *>(pk);
                        else {
                            *reinterpret_cast<u32x4 *>(op) = *reinterpret_cast<const u32x4 *>(pk);
                            *reinterpret_cast<u32x4 *>(op + 4) = *reinterpret_cast<const u32x4 *>(pk + 4);
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            if (c8 + e < vdim) op[e] = D::from_float(gp ? val[e] * sigmoid_f(gp[e]) : val[e]);
                    }
                }
            }
            continue;
        }
        if (!row_ok) continue;
        const int head = g * HG + hb;
        {
            const size_t pi = ((size_t)trow * H + head) * n_splits + split;
#pragma unroll
            for (int v = 0; v < VT; ++v)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int c = 16 * v + 4 * g4 + r;
                    if (c < vdim) part_acc[pi * vdim + c] = of[v][r];
                }
            if (g4 == 0) {
                part_ml[2 * pi] = M;
                part_ml[2 * pi + 1] = L;
            }
        }
    }
}

// ---- the block whose norm sits on the branch's output: x += mult * y / sqrt(mean y^2 + eps) * (offset + w); h = x as D rows (the next sublayer's input) ----
template <typename D>
__global__ void postnorm_add_kernel(float *x, const float *y, const float *w, float offset, float eps, float mult, typename D::storage *h, int width) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const float *src = y + (size_t)r * width;
    float ss = 0.f;
    for (int c = threadIdx.x; c < width; c += blockDim.x) ss += src[c] * src[c];
    ss = block_sum(ss, red);
    const float inv = 1.f / sqrtf(ss / (float)width + eps);
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        const float v = x[(size_t)r * width + c] + mult * (src[c] * inv * (offset + w[c]));
        x[(size_t)r * width + c] = v;
        h[(size_t)r * width + c] = D::from_float(v);
    }
}
// ---- the block with norms on both sides: x += mult * ls * (y / sqrt(mean y^2 + eps) * (offset + w))  (ls NULL: 1), and what reads the new
// stream next leaves with it: next 1: h = x as D rows;  next 2: h = x / sqrt(mean x^2 + eps) * (noffset + nw) as D rows;  0: nothing ----
template <typename D>
__global__ void sandwich_add_kernel(float *x, const float *y, const float *w, float offset, float eps, float mult, const float *ls, int next,
                                    const float *nw, float noffset, typename D::storage *h, int width) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const float *src = y + (size_t)r * width;
    float *xr = x + (size_t)r * width;
    float ss = 0.f;
    for (int c = threadIdx.x; c < width; c += blockDim.x) ss += src[c] * src[c];
    ss = block_sum(ss, red);
    const float inv = 1.f / sqrtf(ss / (float)width + eps);
    float s2 = 0.f;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        const float v = xr[c] + mult * (ls ? ls[c] : 1.f) * (src[c] * inv * (offset + w[c]));
        xr[c] = v;
        s2 += v * v;
        if (next == 1) h[(size_t)r * width + c] = D::from_float(v);
    }
    if (next != 2) return;
    s2 = block_sum(s2, red);
    const float inv2 = 1.f / sqrtf(s2 / (float)width + eps);
    for (int c = threadIdx.x; c < width; c += blockDim.x) h[(size_t)r * width + c] = D::from_float(xr[c] * inv2 * (noffset + nw[c]));  // (this thread's own writes)
}
// per-layer token input, middle step: cat[t, c] = gelu_tanh(proj[t, c]) * table[token[t], col0 + c], c < n
template <typename D>
__global__ void side_act_kernel(const float *proj, int ldp, const int32_t *tokens, const typename D::storage *table, int table_cols, int col0, int n, int vocab,
                                typename D::storage *out, int ldo, int rows) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)rows * n) return;
    const int t = (int)(i / n), c = (int)(i % n);
    int tok = tokens[t];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
    out[(size_t)t * ldo + c] = D::from_float(act_f(proj[(size_t)t * ldp + c], 1) * ld<D>(table, (size_t)tok * table_cols + col0 + c));
}
// float32 rows -> D rows (the input of a sublayer that reads the stream itself)
template <typename D>
__global__ void cast_rows_kernel(const float *x, typename D::storage *out, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = D::from_float(x[i]);
}
__global__ void scale_kernel(float *x, float a, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] *= a;
}

// ---- feed-forward activation: cat[t, col0 + c] = act(proj[t, up0 + c]) ---------------------------------------------------
template <typename D>
__global__ void ff_act_kernel(const float *proj, int ldp, int up0, int ff, int kind, typename D::storage *out, int ldo, int col0, int rows) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)rows * ff) return;
    const int t = (int)(i / ff), c = (int)(i % ff);
    out[(size_t)t * ldo + col0 + c] = D::from_float(act_f(proj[(size_t)t * ldp + up0 + c], kind));
}

// ---- short causal depthwise convolution + SiLU over the first C columns of proj -------------------------------------------
// state: [slots, taps-1, C] float32 = the last taps-1 inputs of the sequence, oldest first (zeros at its start).
__global__ void conv_kernel(const float *proj, int ldp, const float *w, int taps, int C, const int32_t *row_seq, const int32_t *seq_row0,
                            const int32_t *seq_slot, const float *state, float *out, int rows) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)rows * C) return;
    const int t = (int)(i / C), c = (int)(i % C);
    const int s = row_seq[t], r0 = seq_row0[s], li = t - r0;
    const float *st = state + (size_t)seq_slot[s] * (taps - 1) * C;
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
        const int idx = li - (taps - 1) + j;
        const float v = idx >= 0 ? proj[(size_t)(r0 + idx) * ldp + c] : st[(size_t)(taps - 1 + idx) * C + c];
        acc += w[(size_t)c * taps + j] * v;
    }
    out[(size_t)t * C + c] = silu_f(acc);
}
// the convolution's inputs move on: the last taps-1 inputs after this chunk.  One thread per (sequence, channel).
__global__ void conv_state_kernel(const float *proj, int ldp, int taps, int C, const int32_t *seq_row0, const int32_t *seq_slot, float *state,
                                  int n_seqs) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)n_seqs * C) return;
    const int s = (int)(i / C), c = (int)(i % C);
    const int r0 = seq_row0[s], n = seq_row0[s + 1] - r0;
    float *st = state + (size_t)seq_slot[s] * (taps - 1) * C;
    for (int j = 0; j < taps - 1; ++j) {  // ascending: st[j + n] is read before it is written
        const int src = n - (taps - 1) + j;
        st[(size_t)j * C + c] = src >= 0 ? proj[(size_t)(r0 + src) * ldp + c] : st[(size_t)(j + n) * C + c];
    }
}

// ---- gated delta rule, token by token ------------------------------------------------------------------------------------
// grid (heads, sequences, blocks of 256 / LPC state columns), 256 threads: LPC lanes (16 = one DPP row, 32, or 64 = a wave) share a column of the
// state, each holding RPT of its key_dim rows in registers (key_dim <= LPC RPT), so the two dot products of a token are RPT multiply-adds and
// one DPP / wave sum each.  The token loop is a dependency chain: a wave per column (LPC 64) keeps the per-wave work smallest and puts two waves
// on a SIMD at common sizes; LPC 16 serves narrow keys.
// Per token:  S *= g;  u = beta (v - S^T k);  S += k u^T;  o = S^T q.   State in memory: [slot, head, value_dim, key_dim] (a column's rows
// are contiguous: the 16 lanes of a column read and write one run).
// qkv: [rows, C] float32 after convolution + SiLU, q | k | v at 0 | G*dim | 2*G*dim.  q and k become unit vectors here
// (x / sqrt(sum x^2 + unit_eps); q also * dim^-1/2).  proj columns a0 + h (decay input) and b0 + h (beta input).
// sum over the LPC adjacent lanes that share a state column (every lane of the wave takes part)
template <int LPC>
__device__ __forceinline__ float column_sum(float v, int lane) {
    if constexpr (LPC == 64) return wave_sum(v);
    v = group16_sum(v);
    if constexpr (LPC == 32) v += lane_xor16(v, lane);
    return v;
}
template <int RPT, int LPC>
__global__ __launch_bounds__(256) void delta_kernel(const float *qkv, int C, const float *proj, int ldp, int a0, int b0, const float *a_log,
                                                    const float *dt_bias, float unit_eps, const int32_t *seq_row0, const int32_t *seq_slot, float *state,
                                                    float *obuf, int H, int G, int dim, int vdim) {
    constexpr int DP = LPC * RPT;                    // padded key width: zeros behind dim
    constexpr int CPB = 256 / LPC;                   // state columns of a workgroup
    constexpr int TB = 4096 / DP < 32 ? 4096 / DP : 32;  // tokens per LDS tile (q and k tiles of 16 KB each at most)
    constexpr int NIT = TB * DP / 256;               // q / k elements a thread stages per tile
    __shared__ float qs[TB * DP], ks[TB * DP], vs[TB * CPB], gs[TB], bs[TB], iqs[TB], iks[TB], os[TB * CPB];
    const int h = blockIdx.x, s = blockIdx.y, j0 = blockIdx.z * CPB;
    const int kh = h / (H / G);
    const int r0 = seq_row0[s], n = seq_row0[s + 1] - r0, slot = seq_slot[s];
    const int tid = threadIdx.x;
    const int jl = tid / LPC, r = tid % LPC, j = j0 + jl;
    const bool active = j < vdim;
    float S[RPT];
    float *sp = state + (((size_t)slot * H + h) * vdim + (active ? j : 0)) * dim + r * RPT;
#pragma unroll
    for (int i = 0; i < RPT; ++i) S[i] = (active && r * RPT + i < dim) ? sp[i] : 0.f;
    const float decay_rate = -expf(a_log[h]), bias = dt_bias[h], qscale = 1.f / sqrtf((float)dim);
    // The next tile's inputs travel through registers: loaded before the current tile's recurrence starts, written to LDS after it, so the
    // loads' latency hides behind the token loop.
    float rq[NIT], rk[NIT], rv[(TB * CPB + 255) / 256], ra = 0.f, rb = 0.f;
    auto fetch = [&](int t0) __attribute__((always_inline)) {
        const int nt = min(TB, n - t0);
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            const int i = tid + 256 * it, tt = i / DP, d = i % DP;
            const bool ok = tt < nt && d < dim;
            const float *row = qkv + (size_t)(r0 + t0 + (ok ? tt : 0)) * C;
            rq[it] = ok ? row[(size_t)kh * dim + d] : 0.f;
            rk[it] = ok ? row[(size_t)(G + kh) * dim + d] : 0.f;
        }
#pragma unroll
        for (int it = 0; it < (TB * CPB + 255) / 256; ++it) {
            const int i = tid + 256 * it, tt = i / CPB, c = i % CPB;
            rv[it] = (tt < nt && j0 + c < vdim) ? qkv[(size_t)(r0 + t0 + tt) * C + (size_t)2 * G * dim + (size_t)h * vdim + j0 + c] : 0.f;
        }
        if (tid < nt) {
            const float *prow = proj + (size_t)(r0 + t0 + tid) * ldp;
            ra = prow[a0 + h];
            rb = prow[b0 + h];
        }
    };
    if (n > 0) fetch(0);
    for (int t0 = 0; t0 < n; t0 += TB) {
        const int nt = min(TB, n - t0);
        __syncthreads();  // the previous tile's recurrence is done with the LDS
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            qs[tid + 256 * it] = rq[it];
            ks[tid + 256 * it] = rk[it];
        }
#pragma unroll
        for (int it = 0; it < (TB * CPB + 255) / 256; ++it)
            if (tid + 256 * it < TB * CPB) vs[tid + 256 * it] = rv[it];
        if (tid < nt) {
            gs[tid] = expf(decay_rate * softplus_f(ra + bias));
            bs[tid] = sigmoid_f(rb);
        }
        __syncthreads();
        {   // unit vectors: 256 / TB lanes per token form |q|^2 and |k|^2; the scales wait in LDS, outside the token loop's dependency chain
            constexpr int LPT = 256 / TB;
            const int tt = tid / LPT, sub = tid % LPT;
            float sq = 0.f, sk = 0.f;
            for (int d = sub; d < DP; d += LPT) {
                sq += qs[tt * DP + d] * qs[tt * DP + d];
                sk += ks[tt * DP + d] * ks[tt * DP + d];
            }
#pragma unroll
            for (int o = 1; o < LPT; o <<= 1) {
                sq += __shfl_xor(sq, o, 64);
                sk += __shfl_xor(sk, o, 64);
            }
            if (sub == 0) {
                iqs[tt] = qscale / sqrtf(sq + unit_eps);
                iks[tt] = 1.f / sqrtf(sk + unit_eps);
            }
        }
        __syncthreads();
        if (t0 + TB < n) fetch(t0 + TB);
        // every lane runs the recurrence (the DPP sums want whole rows; idle columns store nothing); the next token's operands are read from
        // LDS while the current token's chain runs
        float g, b, vj, ik, iq, kv[RPT], qv[RPT];
        auto read_token = [&](int tt, float &g_, float &b_, float &v_, float &ik_, float &iq_, float (&k_)[RPT], float (&q_)[RPT]) __attribute__((always_inline)) {
            g_ = gs[tt], b_ = bs[tt], v_ = vs[tt * CPB + jl], ik_ = iks[tt], iq_ = iqs[tt];
            const float *kt = ks + tt * DP + r * RPT, *qt = qs + tt * DP + r * RPT;
            if constexpr (RPT % 4 == 0) {
#pragma unroll
                for (int i = 0; i < RPT; i += 4) {
                    const f32x4 k4 = *reinterpret_cast<const f32x4 *>(kt + i), q4 = *reinterpret_cast<const f32x4 *>(qt + i);
#pragma unroll
                    for (int e = 0; e < 4; ++e) k_[i + e] = k4[e], q_[i + e] = q4[e];
                }
            } else if constexpr (RPT == 2) {
                const f32x2 k2 = *reinterpret_cast<const f32x2 *>(kt), q2 = *reinterpret_cast<const f32x2 *>(qt);
                k_[0] = k2[0], k_[1] = k2[1], q_[0] = q2[0], q_[1] = q2[1];
            } else {
#pragma unroll
                for (int i = 0; i < RPT; ++i) k_[i] = kt[i], q_[i] = qt[i];
            }
        };
        read_token(0, g, b, vj, ik, iq, kv, qv);
        for (int tt = 0; tt < nt; ++tt) {
            float ng, nb, nv, nik, niq, nk[RPT], nq[RPT];
            read_token(tt + 1 < nt ? tt + 1 : tt, ng, nb, nv, nik, niq, nk, nq);
            float dot0 = 0.f, dot1 = 0.f;
#pragma unroll
            for (int i = 0; i < RPT; ++i) {
                S[i] *= g;
                if (i & 1) dot1 += S[i] * kv[i];
                else dot0 += S[i] * kv[i];
            }
            const float dot = column_sum<LPC>(dot0 + dot1, tid);
            const float uk = b * (vj - dot * ik) * ik;  // u = beta (v - S^T k^), k^ = k / |k|;  S += k^ u^T = k (u / |k|)
            float od0 = 0.f, od1 = 0.f;
#pragma unroll
            for (int i = 0; i < RPT; ++i) {
                S[i] += kv[i] * uk;
                if (i & 1) od1 += S[i] * qv[i];
                else od0 += S[i] * qv[i];
            }
            const float od = column_sum<LPC>(od0 + od1, tid) * iq;
            if (r == 0) os[tt * CPB + jl] = od;  // (read-outs leave the token loop through LDS: no global store inside the chain)
            g = ng, b = nb, vj = nv, ik = nik, iq = niq;
#pragma unroll
            for (int i = 0; i < RPT; ++i) kv[i] = nk[i], qv[i] = nq[i];
        }
        __syncthreads();
        for (int i = tid; i < nt * CPB; i += 256) {
            const int tt = i / CPB, c = i % CPB;
            if (j0 + c < vdim) obuf[(size_t)(r0 + t0 + tt) * ((size_t)H * vdim) + (size_t)h * vdim + j0 + c] = os[i];
        }
    }
    if (active) {
#pragma unroll
        for (int i = 0; i < RPT; ++i)
            if (r * RPT + i < dim) sp[i] = S[i];
    }
}

// ---- read-out of the delta rule: per (row, head) o / rms(o) * w * silu(gate) -> cat columns h*vdim .. ----------------------
template <typename D>
__global__ __launch_bounds__(64) void delta_out_kernel(const float *obuf, const float *w, float eps, const float *gate, int ldg, int H, int vdim,
                                                       typename D::storage *out, int ldo) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float *o = obuf + ((size_t)t * H + h) * vdim;
    float ss = 0.f;
    for (int c = lane; c < vdim; c += 64) ss += o[c] * o[c];
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / (float)vdim + eps);
    for (int c = lane; c < vdim; c += 64)
        out[(size_t)t * ldo + (size_t)h * vdim + c] = D::from_float(o[c] * inv * w[c] * silu_f(gate[(size_t)t * ldg + (size_t)h * vdim + c]));
}

// ---- Dynamic Tanh norm of float32 rows -> D rows: tanh(alpha x) * w + b (no statistics of the row).  rows_idx: optional gather. ----
template <typename D>
__global__ void dyt_kernel(const float *x, const float *w, const float *b, float alpha, typename D::storage *out, int width, const int32_t *rows_idx) {
    const int r = blockIdx.x;
    const float *src = x + (size_t)(rows_idx ? rows_idx[r] : r) * width;
    for (int c = threadIdx.x; c < width; c += blockDim.x) out[(size_t)r * width + c] = D::from_float(tanhf(alpha * src[c]) * w[c] + b[c]);
}

// ---- RMS norm of n columns of float32 rows (a latent) -> D rows: x / sqrt(mean x^2 + eps) * w.  One workgroup per row. -------------
template <typename D>
__global__ void rms_cols_kernel(const float *in, int ldi, int n, const float *w, float eps, typename D::storage *out, int ldo) {
    __shared__ float red[16];
    const int t = blockIdx.x;
    const float *src = in + (size_t)t * ldi;
    float ss = 0.f;
    for (int c = threadIdx.x; c < n; c += blockDim.x) ss += src[c] * src[c];
    ss = block_sum(ss, red);
    const float inv = 1.f / sqrtf(ss / (float)n + eps);
    for (int c = threadIdx.x; c < n; c += blockDim.x) out[(size_t)t * ldo + c] = D::from_float(src[c] * inv * w[c]);
}

// ---- latent attention, step 1.  Queries q [rows, H, dim + rot] (float32): the plain part -> qn (D, the input of the per-head key
// absorption), the rotated part -> qbuf[t, h, rank ..] after its rotation.  With own_kv (the layer has its own latent projection, columns
// kv0 .. of proj: rank latent columns, then rot columns of one rotated key part shared by all heads): the latent is RMS-normed with
// its weight and appended to the sequence's page row [c (rank) | rotated key part (rot)] -- the whole K/V cache of the layer.
// Rotation: pair (2i, 2i+1) by pos * freq[i], cos and sin times mult.  grid (rows, H + 1), one wave each.
template <typename D>
__global__ __launch_bounds__(64) void latent_prep_kernel(const float *q, int H, int dim, int rot, int rank, const float *proj, int ldp, int kv0,
                                                         const float *c_norm, float eps, int own_kv, const int32_t *row_seq, const int32_t *row_pos,
                                                         const int32_t *seq_slot, const int32_t *block_table, int max_pages, int page_size,
                                                         const float *freq, int rot_dims, float mult, typename D::storage *qn, float *qbuf,
                                                         typename D::storage *pool) {
    const int t = blockIdx.x, hh = blockIdx.y, lane = threadIdx.x;
    const int pos = row_pos[t];
    auto turn = [&](const float *src, int p, float &u, float &v) {
        const int c = 2 * p;
        u = src[c], v = (c + 1 < rot) ? src[c + 1] : 0.f;
        if (c + 1 < rot_dims) {
            float sn, cs;
            sincosf((float)pos * freq[p], &sn, &cs);
            sn *= mult, cs *= mult;
            const float nu = u * cs - v * sn, nv = v * cs + u * sn;
            u = nu, v = nv;
        }
    };
    if (hh < H) {
        const float *src = q + ((size_t)t * H + hh) * (dim + rot);
        for (int c = lane; c < dim; c += 64) qn[((size_t)t * H + hh) * dim + c] = D::from_float(src[c]);
        float *dst = qbuf + ((size_t)t * H + hh) * (rank + rot) + rank;
        for (int p = lane; 2 * p < rot; p += 64) {
            float u, v;
            turn(src + dim, p, u, v);
            dst[2 * p] = u;
            if (2 * p + 1 < rot) dst[2 * p + 1] = v;
        }
        return;
    }
    if (!own_kv) return;
    const int slot = seq_slot[row_seq[t]];
    const int page = block_table[(size_t)slot * max_pages + pos / page_size], in_page = pos % page_size;
    typename D::storage *dst = pool + ((size_t)page * page_size + in_page) * (rank + rot);
    const float *src = proj + (size_t)t * ldp + kv0;
    float ss = 0.f;
    for (int c = lane; c < rank; c += 64) ss += src[c] * src[c];
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / (float)rank + eps);
    for (int c = lane; c < rank; c += 64) dst[c] = D::from_float(src[c] * inv * c_norm[c]);
    for (int p = lane; 2 * p < rot; p += 64) {
        float u, v;
        turn(src + rank, p, u, v);
        dst[rank + 2 * p] = D::from_float(u);
        if (2 * p + 1 < rot) dst[rank + 2 * p + 1] = D::from_float(v);
    }
}

// ---- out[t, c] = in[t, c] * gate(g[t, c]) as D rows.  kind 0: sigmoid, 1: SiLU, 2: no gate (g is not read) ----------------------------
template <typename D>
__global__ void gate_mul_kernel(const float *in, int ldi, const float *g, int ldg, int n, int kind, typename D::storage *out, int ldo, int rows) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)rows * n) return;
    const int t = (int)(i / n), c = (int)(i % n);
    const float z = kind == 2 ? 0.f : g[(size_t)t * ldg + c];
    out[(size_t)t * ldo + c] = D::from_float(in[(size_t)t * ldi + c] * (kind == 2 ? 1.f : (kind == 0 ? sigmoid_f(z) : silu_f(z))));
}

// ---- gated feed-forward activation: cat[t, col0 + c] = act(proj[t, g0 + c]) * proj[t, u0 + c] ------------------------------------
template <typename D>
__global__ void ff_gated_act_kernel(const float *proj, int ldp, int g0, int u0, int ff, int kind, typename D::storage *out, int ldo, int col0, int rows) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)rows * ff) return;
    const int t = (int)(i / ff), c = (int)(i % ff);
    out[(size_t)t * ldo + col0 + c] = D::from_float(act_f(proj[(size_t)t * ldp + g0 + c], kind) * proj[(size_t)t * ldp + u0 + c]);
}

// ---- linear recurrences with a decaying matrix state --------------------------------------------------------------------------------
// log-sigmoid without overflow
__device__ __forceinline__ float logsigmoid_f(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// Exponential gates with a running maximum (mLSTM).  Per (sequence, head), token by token:
//   li = cap tanh((x_i + b_i) / cap),  lf = logsigmoid(cap tanh((x_f + b_f) / cap)),  m' = max(lf + m, li)
//   decay a = exp(lf + m - m'),  input scale b = exp(li - m'),  floor e = exp(-m')       (m starts at 0 with the sequence)
// m -> max(m + A, B) composes associatively ((A1, B1) then (A2, B2) = (A1 + A2, max(B1 + A2, B2))), so a wave scans 64 tokens at a time.
// proj columns i0 + h / f0 + h hold x_i / x_f.  gates: [rows, H, 3] = (a, b, e).  m_state: [slots, H].
__global__ __launch_bounds__(64) void expgate_scan_kernel(const float *proj, int ldp, int i0, int f0, const float *i_bias, const float *f_bias, float cap,
                                                          const int32_t *seq_row0, const int32_t *seq_slot, float *m_state, float *gates, int H) {
    const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int r0 = seq_row0[s], n = seq_row0[s + 1] - r0, slot = seq_slot[s];
    float m = m_state[(size_t)slot * H + h];
    for (int t0 = 0; t0 < n; t0 += 64) {
        const int t = t0 + lane;
        const bool ok = t < n;
        float li = 0.f, lf = 0.f;
        if (ok) {
            const float *row = proj + (size_t)(r0 + t) * ldp;
            li = cap * tanhf((row[i0 + h] + i_bias[h]) / cap);
            lf = logsigmoid_f(cap * tanhf((row[f0 + h] + f_bias[h]) / cap));
        }
        float A = ok ? lf : 0.f, B = ok ? li : -INFINITY;  // lanes past the end: the identity
        for (int off = 1; off < 64; off <<= 1) {
            const float pa = __shfl_up(A, off, 64), pb = __shfl_up(B, off, 64);
            if (lane >= off) {
                B = fmaxf(pb + A, B);
                A = pa + A;
            }
        }
        const float m_t = fmaxf(m + A, B);
        float m_prev = __shfl_up(m_t, 1, 64);
        if (lane == 0) m_prev = m;
        if (ok) {
            float *g = gates + ((size_t)(r0 + t) * H + h) * 3;
            g[0] = expf(lf + m_prev - m_t);
            g[1] = expf(li - m_t);
            g[2] = expf(-m_t);
        }
        m = __shfl(m_t, min(63, n - 1 - t0), 64);
    }
    if (lane == 0) m_state[(size_t)slot * H + h] = m;
}

// decay per key channel (gated linear attention): z[t, c] <- sigmoid(z + bias[c])^(1/tau) = exp(logsigmoid(z + bias) / tau), in place
__global__ void channel_decay_kernel(float *z, const float *bias, int n, float inv_tau, int rows) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)rows * n) return;
    z[i] = expf(logsigmoid_f(z[i] + bias[i % n]) * inv_tau);
}
// float32 columns of proj -> D rows (the input of a second, low-rank projection)
template <typename D>
__global__ void cast_cols_kernel(const float *in, int ldi, int c0, int n, typename D::storage *out, int ldo, int rows) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)rows * n) return;
    const int t = (int)(i / n), c = (int)(i % n);
    out[(size_t)t * ldo + c] = D::from_float(in[(size_t)t * ldi + c0 + c]);
}

// The recurrence itself, token by token:   S <- diag(a_t) S + b_t k_t v_t^T;   o_t = S^T q_t      (S: [key_dim, columns] per head, float32)
//   CHAN false: a_t one number per head (gates[.., 0]), b_t = gates[.., 1]     CHAN true: a_t per key channel (decay[t, h, d]), b_t = 1
// ones != 0 appends one column whose value is 1 for every token: it carries the normaliser n_t = a n + b k, read out as n_t . q_t.
// grid (heads, sequences, blocks of 256 / LPC columns), 256 threads; LPC lanes share a column, RPT key rows each in registers (as delta_kernel).
// q | k | v at columns q0 | k0 | v0 of proj (head-major).  State [slot, head, column, key_dim].  obuf [rows, H, VE], VE = vdim + ones.
template <int RPT, int LPC, bool CHAN>
__global__ __launch_bounds__(256) void linrec_kernel(const float *proj, int ldp, int q0, int k0, int v0, const float *gates, const float *decay,
                                                     const int32_t *seq_row0, const int32_t *seq_slot, float *state, float *obuf, int H, int dim,
                                                     int vdim, int ones) {
    constexpr int DP = LPC * RPT, CPB = 256 / LPC;
    constexpr int TB = 4096 / DP < 32 ? 4096 / DP : 32;
    __shared__ __attribute__((aligned(16))) float qs[TB * DP], ks[TB * DP], as[CHAN ? TB * DP : TB];
    __shared__ float vs[TB * CPB], bs[TB], os[TB * CPB];
    const int h = blockIdx.x, s = blockIdx.y, j0 = blockIdx.z * CPB, VE = vdim + ones;
    const int r0 = seq_row0[s], n = seq_row0[s + 1] - r0, slot = seq_slot[s];
    const int tid = threadIdx.x, jl = tid / LPC, r = tid % LPC, j = j0 + jl;
    const bool active = j < VE;
    float S[RPT];
    float *sp = state + (((size_t)slot * H + h) * VE + (active ? j : 0)) * dim + r * RPT;
#pragma unroll
    for (int i = 0; i < RPT; ++i) S[i] = (active && r * RPT + i < dim) ? sp[i] : 0.f;
    // The next tile's inputs travel through registers: loaded before the current tile's recurrence starts, written to LDS after it, so the
    // loads' latency hides behind the token loop (as in delta_kernel).
    constexpr int NIT = TB * DP / 256, NV = (TB * CPB + 255) / 256;
    float rq[NIT], rk[NIT], ra[CHAN ? NIT : 1], rv[NV], rg = 1.f, rb = 0.f;
    auto fetch = [&](int t0) __attribute__((always_inline)) {
        const int nt = min(TB, n - t0);
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            const int i = tid + 256 * it, tt = i / DP, d = i % DP;
            const bool ok = tt < nt && d < dim;
            const float *row = proj + (size_t)(r0 + t0 + (ok ? tt : 0)) * ldp + (size_t)h * dim + (ok ? d : 0);
            rq[it] = ok ? row[q0] : 0.f;
            rk[it] = ok ? row[k0] : 0.f;
            if constexpr (CHAN) ra[it] = ok ? decay[((size_t)(r0 + t0 + tt) * H + h) * dim + d] : 1.f;
        }
#pragma unroll
        for (int it = 0; it < NV; ++it) {
            const int i = tid + 256 * it, tt = i / CPB, c = j0 + i % CPB;
            rv[it] = (tt < nt && c < VE) ? (c < vdim ? proj[(size_t)(r0 + t0 + tt) * ldp + v0 + (size_t)h * vdim + c] : 1.f) : 0.f;
        }
        if (tid < nt) {
            if constexpr (!CHAN) rg = gates[((size_t)(r0 + t0 + tid) * H + h) * 3];
            rb = CHAN ? 1.f : gates[((size_t)(r0 + t0 + tid) * H + h) * 3 + 1];
        }
    };
    if (n > 0) fetch(0);
    for (int t0 = 0; t0 < n; t0 += TB) {
        const int nt = min(TB, n - t0);
        __syncthreads();  // the previous tile's recurrence is done with the LDS
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            qs[tid + 256 * it] = rq[it];
            ks[tid + 256 * it] = rk[it];
            if constexpr (CHAN) as[tid + 256 * it] = ra[it];
        }
#pragma unroll
        for (int it = 0; it < NV; ++it)
            if (tid + 256 * it < TB * CPB) vs[tid + 256 * it] = rv[it];
        if (tid < TB) {
            if constexpr (!CHAN) as[tid] = rg;
            bs[tid] = rb;
        }
        __syncthreads();
        if (t0 + TB < n) fetch(t0 + TB);
        // the state's chain is one multiply-add per token and element; the next token's operands are read from LDS while the current one runs
        float bv, kv[RPT], qv[RPT], av[CHAN ? RPT : 1];
        auto read_token = [&](int tt, float &bv_, float (&k_)[RPT], float (&q_)[RPT], float (&a_)[CHAN ? RPT : 1]) __attribute__((always_inline)) {
            bv_ = bs[tt] * vs[tt * CPB + jl];
            const float *kt = ks + tt * DP + r * RPT, *qt = qs + tt * DP + r * RPT, *at = as + (CHAN ? tt * DP + r * RPT : tt);
            if constexpr (RPT % 4 == 0) {
#pragma unroll
                for (int i = 0; i < RPT; i += 4) {
                    const f32x4 k4 = *reinterpret_cast<const f32x4 *>(kt + i), q4 = *reinterpret_cast<const f32x4 *>(qt + i);
#pragma unroll
                    for (int e = 0; e < 4; ++e) k_[i + e] = k4[e], q_[i + e] = q4[e];
                    if constexpr (CHAN) {
                        const f32x4 a4 = *reinterpret_cast<const f32x4 *>(at + i);
#pragma unroll
                        for (int e = 0; e < 4; ++e) a_[i + e] = a4[e];
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < RPT; ++i) {
                    k_[i] = kt[i], q_[i] = qt[i];
                    if constexpr (CHAN) a_[i] = at[i];
                }
            }
            if constexpr (!CHAN) a_[0] = at[0];
        };
        read_token(0, bv, kv, qv, av);
        for (int tt = 0; tt < nt; ++tt) {
            float nbv, nk[RPT], nq[RPT], na[CHAN ? RPT : 1];
            read_token(tt + 1 < nt ? tt + 1 : tt, nbv, nk, nq, na);
            float od0 = 0.f, od1 = 0.f;
#pragma unroll
            for (int i = 0; i < RPT; ++i) {
                S[i] = S[i] * av[CHAN ? i : 0] + kv[i] * bv;
                if (i & 1) od1 += S[i] * qv[i];
                else od0 += S[i] * qv[i];
            }
            const float od = column_sum<LPC>(od0 + od1, tid);
            if (r == 0) os[tt * CPB + jl] = od;
            bv = nbv;
#pragma unroll
            for (int i = 0; i < RPT; ++i) kv[i] = nk[i], qv[i] = nq[i];
#pragma unroll
            for (int i = 0; i < (CHAN ? RPT : 1); ++i) av[i] = na[i];
        }
        __syncthreads();
        for (int i = tid; i < nt * CPB; i += 256) {
            const int tt = i / CPB, c = i % CPB;
            if (j0 + c < VE) obuf[((size_t)(r0 + t0 + tt) * H + h) * VE + j0 + c] = os[i];
        }
    }
    if (active) {
#pragma unroll
        for (int i = 0; i < RPT; ++i)
            if (r * RPT + i < dim) sp[i] = S[i];
    }
}

// Constant decay per head (retention), ahead of the recurrence: q and k of every (row, head) turn in place (float32 columns q0 / k0 of proj) on their
// first rot_dims dimensions by pos * inv_freq[i] -- pairs (i, i + rot_dims/2) with rot_half, (2i, 2i+1) without -- then k is multiplied by k_scale;
// gates[t, h] = (decay[h], 1, -).  One wave per (row, head).
__global__ __launch_bounds__(64) void fixed_decay_prep_kernel(float *proj, int ldp, int q0, int k0, const int32_t *row_pos, const float *inv_freq, int rot_dims,
                                                              int rot_half, float k_scale, const float *decay, float *gates, int H, int dim) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int pos = row_pos[t], half = rot_dims / 2;
    float *q = proj + (size_t)t * ldp + q0 + (size_t)h * dim, *k = proj + (size_t)t * ldp + k0 + (size_t)h * dim;
    for (int u = lane; u < dim - half; u += 64) {
        if (u < half) {
            const int c0 = rot_half ? u : 2 * u, c1 = rot_half ? u + half : 2 * u + 1;
            float sn, cs;
            sincosf((float)pos * inv_freq[u], &sn, &cs);
            const float qa = q[c0], qb = q[c1], ka = k[c0], kb = k[c1];
            q[c0] = qa * cs - qb * sn, q[c1] = qb * cs + qa * sn;
            k[c0] = (ka * cs - kb * sn) * k_scale, k[c1] = (kb * cs + ka * sn) * k_scale;
        } else
            k[u + half] *= k_scale;
    }
    if (lane == 0) {
        float *g = gates + ((size_t)t * H + h) * 3;
        g[0] = decay[h], g[1] = 1.f, g[2] = 0.f;
    }
}

// read-out of a linear recurrence, one wave per (row, head):  o = obuf[t, h, :vdim] * qscale;  with ones: o /= max(|n.q|, e) + 1e-6 where n.q is
// the appended column (times qscale) and e the gate floor;  then o / rms(o) * w[h * w_stride + c] * gate(g)   (gate_kind 0 sigmoid, 1 SiLU)
template <typename D>
__global__ __launch_bounds__(64) void linrec_out_kernel(const float *obuf, int VE, int ones, const float *gates, float qscale, const float *w,
                                                        int w_stride, float eps, const float *gate, int ldg, int gate_kind, int H, int vdim,
                                                        typename D::storage *out, int ldo) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float *o = obuf + ((size_t)t * H + h) * VE;
    float mul = qscale;
    if (ones) mul = qscale / (fmaxf(fabsf(o[vdim] * qscale), gates[((size_t)t * H + h) * 3 + 2]) + 1e-6f);
    float ss = 0.f;
    for (int c = lane; c < vdim; c += 64) {
        const float v = o[c] * mul;
        ss += v * v;
    }
    ss = wave_sum(ss);
    const float inv = mul / sqrtf(ss / (float)vdim + eps);
    for (int c = lane; c < vdim; c += 64) {
        const float z = gate[(size_t)t * ldg + (size_t)h * vdim + c];
        out[(size_t)t * ldo + (size_t)h * vdim + c] = D::from_float(o[c] * inv * (w ? w[(size_t)h * w_stride + c] : 1.f) * (gate_kind == 0 ? sigmoid_f(z) : silu_f(z)));
    }
}

// ---- mixture of experts: routing and activation, one workgroup per row -----------------------------------------------------------------
// proj columns of the row: shared up [ffs] at su0, directly behind it expert e's up [ffe] at eu0 + e * ffe (eu0 = su0 + ffs); router logits
// z [ET] at r0 (ET = experts + identity experts); shared gate (1) at sg0.  s = softmax(z); choice = s + correction; the experts form `groups` equal runs of neighbours, a
// group scores its largest choice, only the `keep` best groups can be taken; the `top` largest choices among them are taken (ties: the lower
// index); weights are their s, not renormalised.  The last `identity` experts return their input: their weights are summed into idw[t].
// cat row: [ sigmoid(sg) * relu(up)^2  (ffs) | w_e * relu(up_e)^2 (ffe each; 0 for experts not taken) ].
// the router of one row, by every thread of a 256-thread workgroup: scores s = softmax(z) or sigmoid(z) (router 0 / 1); choice = s + correction
// (NULL: 0); groups, kept groups, the `top` largest choices (ties: the lower index).  Leaves sw[e] = s_e for the experts taken, 0 for the others.
__device__ __forceinline__ void moe_route_row(const float *row, int r0, int ET, int top, int groups, int keep, const float *correction, int router, float *sw,
                                              float *sc, float *gm) {
    const int tid = threadIdx.x;
    if (tid < 64) {  // one wave scores (ET <= 256: four experts a lane at most)
        float z[4], mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = tid + 64 * i;
            z[i] = e < ET ? row[r0 + e] : -INFINITY;
            mx = fmaxf(mx, z[i]);
        }
        float sum = 1.f;
        if (router == 0) {
            mx = wave_max(mx);
            sum = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                z[i] = (tid + 64 * i) < ET ? expf(z[i] - mx) : 0.f;
                sum += z[i];
            }
            sum = wave_sum(sum);
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) z[i] = (tid + 64 * i) < ET ? sigmoid_f(z[i]) : 0.f;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = tid + 64 * i;
            if (e < ET) {
                const float s = router == 0 ? z[i] / sum : z[i];
                sw[e] = s;
                sc[e] = s + (correction ? correction[e] : 0.f);
            }
        }
    }
    __syncthreads();
    if (tid == 0 && groups > 1) {  // groups, then the top choices: a few dozen comparisons
        const int per = ET / groups;
        for (int g = 0; g < groups; ++g) {
            float m = -INFINITY;
            for (int e = g * per; e < (g + 1) * per; ++e) m = fmaxf(m, sc[e]);
            gm[g] = m;
        }
        for (int g = 0; g < groups; ++g) {  // rank of the group: how many beat it (ties: the lower index first)
            int rank = 0;
            for (int o = 0; o < groups; ++o) rank += (gm[o] > gm[g]) || (gm[o] == gm[g] && o < g);
            if (rank >= keep)
                for (int e = g * per; e < (g + 1) * per; ++e) sc[e] = -INFINITY;
        }
    }
    __syncthreads();
    float wgt = 0.f;
    if (tid < ET) {
        const float c = sc[tid];
        int rank = 0;
        for (int o = 0; o < ET; ++o) rank += (sc[o] > c) || (sc[o] == c && o < tid);
        wgt = (rank < top && !(c == -INFINITY)) ? sw[tid] : 0.f;
    }
    __syncthreads();
    if (tid < ET) sw[tid] = wgt;
    __syncthreads();
}

template <typename D>
__global__ __launch_bounds__(256) void moe_route_act_kernel(const float *proj, int ldp, int r0, int sg0, int su0, int eu0, int experts, int identity, int top,
                                                            int groups, int keep, int ffe, int ffs, const float *correction,
                                                            typename D::storage *out, int ldo, int col0, float *idw, int router) {
    __shared__ float sw[256], sc[256];
    __shared__ float gm[256];
    // blockIdx.y: a share of the row's columns (every share routes the row again: a few dozen comparisons against thousands of columns)
    const int t = blockIdx.x, tid = threadIdx.x, ET = experts + identity;
    const float *row = proj + (size_t)t * ldp;
    moe_route_row(row, r0, ET, top, groups, keep, correction, router, sw, sc, gm);
    if (tid == 0 && blockIdx.y == 0) {
        float a = 0.f;
        for (int e = experts; e < ET; ++e) a += sw[e];
        idw[t] = a;
    }
    const float sgate = ffs > 0 ? sigmoid_f(row[sg0]) : 0.f;
    typename D::storage *o = out + (size_t)t * ldo + col0;
    const int n = ffs + experts * ffe, per = (n + gridDim.y - 1) / gridDim.y, c_end = min(n, (int)(blockIdx.y + 1) * per);
    for (int c = blockIdx.y * per + tid; c < c_end; c += 256) {  // shared columns first, then the experts' (su0 + ffs == eu0)
        const float w = c < ffs ? sgate : sw[(c - ffs) / ffe], u = fmaxf(row[su0 + c], 0.f);
        o[c] = D::from_float(w * u * u);
    }
}
// which experts the rows of a small step take: bit e of *mask is set when some row's router takes expert e (the products around the activation then leave the
// others out, see SegSkip).  One workgroup; experts <= 64.
__global__ __launch_bounds__(256) void moe_taken_mask_kernel(const float *proj, int ldp, int r0, int rows, int experts, int identity, int top, int groups, int keep,
                                                             const float *correction, int router, unsigned long long *mask) {
    __shared__ float sw[256], sc[256];
    __shared__ float gm[256];
    __shared__ unsigned long long taken;
    if (threadIdx.x == 0) taken = 0ull;
    __syncthreads();
    for (int t = 0; t < rows; ++t) {
        moe_route_row(proj + (size_t)t * ldp, r0, experts + identity, top, groups, keep, correction, router, sw, sc, gm);
        if ((int)threadIdx.x < experts && sw[threadIdx.x] != 0.f) atomicOr(&taken, 1ull << threadIdx.x);
        __syncthreads();
    }
    if (threadIdx.x == 0) *mask = taken;
}
// the same with gated experts, W_down (act(W_gate h) * W_up h): proj columns g0 .. = shared gate [ffs] | expert gates [ffe each], u0 .. = shared up | expert ups,
// router logits at r0, the shared expert's scalar gate at sg0 (sg0 < 0: the shared expert is not scaled).  The router's weight w_e multiplies the
// expert's OUTPUT (scale_input 0: w act(g) u) or its INPUT (1: the expert of w h, i.e. act(w g) (w u), both projections being linear).
// cat row: [ shared (ffs) | expert columns (ffe each; 0 for experts not taken) ].
template <typename D>
__global__ __launch_bounds__(256) void moe_gated_act_kernel(const float *proj, int ldp, int r0, int sg0, int g0, int u0, int experts, int identity, int top,
                                                            int groups, int keep, int ffe, int ffs, const float *correction, typename D::storage *out,
                                                            int ldo, int col0, float *idw, int router, int scale_input, int act) {
    __shared__ float sw[256], sc[256];
    __shared__ float gm[256];
    const int t = blockIdx.x, tid = threadIdx.x, ET = experts + identity;
    const float *row = proj + (size_t)t * ldp;
    moe_route_row(row, r0, ET, top, groups, keep, correction, router, sw, sc, gm);
    if (tid == 0 && blockIdx.y == 0) {
        float a = 0.f;
        for (int e = experts; e < ET; ++e) a += sw[e];
        idw[t] = a;
    }
    const float sgate = sg0 >= 0 ? sigmoid_f(row[sg0]) : 1.f;
    typename D::storage *o = out + (size_t)t * ldo + col0;
    const int n = ffs + experts * ffe, per = (n + gridDim.y - 1) / gridDim.y, c_end = min(n, (int)(blockIdx.y + 1) * per);
    for (int c = blockIdx.y * per + tid; c < c_end; c += 256) {
        const float g = row[g0 + c], u = row[u0 + c];
        float v;
        if (c < ffs) v = sgate * act_f(g, act) * u;
        else {
            const float w = sw[(c - ffs) / ffe];
            v = w == 0.f ? 0.f : (scale_input ? act_f(w * g, act) * (w * u) : w * act_f(g, act) * u);
        }
        o[c] = D::from_float(v);
    }
}
// identity experts: x[t, c] += ls[c] * idw[t] * h[t, c]  (ls may be null: 1)
template <typename D>
__global__ void identity_axpy_kernel(float *x, const typename D::storage *h, const float *idw, const float *ls, float mult, int width, int rows) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)rows * width) return;
    const int t = (int)(i / width), c = (int)(i % width);
    x[i] += mult * (ls ? ls[c] : 1.f) * idw[t] * D::to_float(h[i]);
}

// ---- small helpers -----------------------------------------------------------------------------------------------------------
__global__ void add_rowvec_kernel(float *x, const float *v, int width, int rows) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < (size_t)rows * width) x[i] += v[i % width];
}
__global__ void fill_kernel(float *p, size_t n, float v) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v;
}
// argmax of each logits row (first index wins on ties); also the next input token of the row's slot when slot_of_row is given
__global__ __launch_bounds__(1024) void argmax_kernel(const float *logits, int vocab, int32_t *out, const int32_t *slot_of_row, int32_t *pending) {
    __shared__ float bv[16];
    __shared__ int bi[16];
    const int r = blockIdx.x, tid = threadIdx.x, lane = tid & 63;
    const float *row = logits + (size_t)r * vocab;
    float best = -INFINITY;
    int idx = 0x7fffffff;
    auto take = [&](float v, int c) {
        if (v > best || (v == best && c < idx)) best = v, idx = c;
    };
    if (vocab % 4 == 0) {
        for (int c = 4 * tid; c < vocab; c += 4096) {
            const f32x4 v = *reinterpret_cast<const f32x4 *>(row + c);
#pragma unroll
            for (int e = 0; e < 4; ++e) take(v[e], c + e);
        }
    } else {
        for (int c = tid; c < vocab; c += 1024) take(row[c], c);
    }
    for (int o = 32; o > 0; o >>= 1) take(__shfl_xor(best, o, 64), __shfl_xor(idx, o, 64));
    if (lane == 0) {
        bv[tid >> 6] = best;
        bi[tid >> 6] = idx;
    }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < 16; ++w) take(bv[w], bi[w]);
        if (idx == 0x7fffffff) idx = 0;
        out[r] = idx;
        if (slot_of_row) pending[slot_of_row[r]] = idx;
    }
}
// decode bookkeeping on the device: the step's rows are one token per listed slot; tokens come from `pending`, positions from `ctx`
__global__ void decode_meta_kernel(const int32_t *slots, int n, const int32_t *pending, int32_t *ctx, int32_t *tokens, int32_t *row_pos,
                                   int advance) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int s = slots[i];
    if (advance) ctx[s] += 1;
    else {
        tokens[i] = pending[s];
        row_pos[i] = ctx[s];
    }
}

}  // namespace hy
}  // namespace tl
