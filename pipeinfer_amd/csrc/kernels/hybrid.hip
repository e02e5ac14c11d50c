// Operators of hybrid decoder blocks (recurrent and low-rank-attention mixers, routed feed-forwards).  Everything here is fp32: norms, scores, soft-max, recurrent
// state, router.  Matrices are bfloat16 pi_weights (widened exactly); `exact` = 0 rounds the activations that enter an expert's matrices to bfloat16 as pi_op_dense does.
//
//   k_rms_scale          y = x / sqrt(mean(x^2) + eps) * (w + w_offset) [* gate];  out = [residual +] mult * y;  rows may be written into the cache cells of the pass
//   k_linear_attention   per head S <- lambda * S + k v^T, o = S^T q over a run of tokens of one sequence; S lives in HBM per (slot, head) between calls
//   k_latent_attention   attention over a shared low-rank latent c: the key up-projection is folded into the query (q~ = W_uk^T q), the value up-projection applied to the
//                        probability-weighted sum of latents — the cache is read once for all heads of a tile and K / V are never materialised; soft-max with a sink term
//   k_moe_route          router logits, soft-max over all router outputs, bias-corrected top-k choice, weights = uncorrected scores
//   k_moe_up / _down     the chosen experts of every token (gathered mat-vecs), identity experts pass their input through
#include "ops_common.h"
#include "kernel_timing.h"

#include <algorithm>
#include <cmath>

static __device__ __forceinline__ float hy_widen(uint16_t b) { return __uint_as_float((uint32_t) b << 16); }
static __device__ __forceinline__ float hy_round(float f) { const uint32_t u = __float_as_uint(f); return __uint_as_float(((u + 0x7fffu + ((u >> 16) & 1u)) >> 16) << 16); }

// sum over the 256 threads of a block (every thread gets the total); red: 4 floats of LDS, reusable after the call
static __device__ __forceinline__ float hy_block_sum(float v, float * red) {
    v = pi_lanes_sum<64>(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = 0.0f;
    for (int i = 0; i < (int) (blockDim.x >> 6); i++) s += red[i];
    return s;
}
static __device__ __forceinline__ float hy_block_max(float v, float * red) {
    v = pi_wave_max(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = red[0];
    for (int i = 1; i < (int) (blockDim.x >> 6); i++) s = fmaxf(s, red[i]);
    return s;
}

// ---- RMS norm with its usual companions ---------------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) k_rms_scale(const float * __restrict__ x, int64_t xs, const float * __restrict__ w, float w_off, float eps, int n,
                                                   const float * __restrict__ gate, int64_t gs, const float * __restrict__ res, int64_t rs, float mult,
                                                   float * __restrict__ out, int64_t os, const int32_t * __restrict__ dyn, int to_cells, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    __shared__ float red[4];
    const int t = blockIdx.x;
    const float * xr = x + (int64_t) t * xs;
    float ss = 0.0f;
    for (int i = threadIdx.x; i < n; i += 256) ss = fmaf(xr[i], xr[i], ss);
    ss = hy_block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float) n + eps);
    const int64_t orow = to_cells ? pi_cell_of(dyn, 0, t) : t;
    for (int i = threadIdx.x; i < n; i += 256) {
        float y = xr[i] * inv * (w[i] + w_off);
        if (gate) y *= gate[(int64_t) t * gs + i];
        y *= mult;
        if (res) y = res[(int64_t) t * rs + i] + y;
        out[orow * os + i] = y;
    }
}

extern "C" int pi_op_rms_scale(const float * x, int64_t x_stride, const float * w, float w_offset, float eps, int n, int n_tok, const float * gate, int64_t gate_stride,
                               const float * residual, int64_t residual_stride, float mult, float * out, int64_t out_stride, const int32_t * dyn_dev, int to_cells, void * stream) {
    if (n_tok <= 0 || n <= 0) return 0;
    if (to_cells && !dyn_dev) { pi_set_error("pi_op_rms_scale: rows go to cache cells but no cell table was given"); return -1; }
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 12.0 * n * n_tok, k_rms_scale, dim3((unsigned) n_tok), dim3(256), 0, (hipStream_t) stream, x, x_stride, w, w_offset, eps, n, gate, gate_stride,
                 residual, residual_stride, mult, out, out_stride, dyn_dev, to_cells, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}

// ---- linear attention with a per-head decay -------------------------------------------------------------------------------------------------------
// rec[t] = state slot of token t (| 1 << 30 on the first token of a sequence whose state starts from zero), tokens of one slot are consecutive.  Workgroup (head, column block,
// segment ordinal): thread (column j, part sp of R) keeps S[i][j] for its DPT rows i in registers, walks the segment's tokens in order and leaves S in HBM.
#define LA_TB 16                                  // tokens whose q and k are staged in LDS at a time
#define LA_FRESH (1 << 30)
template <int DPT>
__global__ void __launch_bounds__(256) k_linear_attention(const float * __restrict__ q, const float * __restrict__ k, const float * __restrict__ v, int64_t stride, int heads, int dim, int vdim, int R,
                                                          const float * __restrict__ decay, float * __restrict__ state, const int32_t * __restrict__ rec, int n_tok,
                                                          float * __restrict__ out, int64_t os, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    extern __shared__ float lds[];                // q tile [LA_TB][dim] | k tile [LA_TB][dim] | the slot words of the pass [n_tok]
    __shared__ int seg[3];                        // first token, length, slot word
    const int h = blockIdx.x, tid = threadIdx.x;
    int * recs = (int *) (lds + 2 * LA_TB * dim);
    for (int t = tid; t < n_tok; t += blockDim.x) recs[t] = rec[t];
    __syncthreads();
    if (tid == 0) {
        int ord = -1, first = 0, len = 0, word = -1, prev = -1;
        for (int t = 0; t < n_tok; t++) {
            const int s = recs[t] & ~LA_FRESH;
            if (t == 0 || s != prev) { if (ord == (int) blockIdx.z) break; ord++; first = t; len = 0; word = recs[t]; }
            prev = s; len++;
        }
        if (ord != (int) blockIdx.z) len = 0;
        seg[0] = first; seg[1] = len; seg[2] = word;
    }
    __syncthreads();
    const int first = seg[0], len = seg[1], word = seg[2];
    if (len == 0 || word < 0) return;
    const int slot = word & ~LA_FRESH;
    const int cols = blockDim.x / R;
    const int j = blockIdx.y * cols + tid / R, sp = tid % R;
    const bool col_ok = j < vdim;
    const float lam = decay[h];
    float * S_hbm = state + ((int64_t) slot * heads + h) * dim * vdim;
    float S[DPT];
#pragma unroll
    for (int ii = 0; ii < DPT; ii++) {
        const int i = sp * DPT + ii;
        S[ii] = (col_ok && i < dim && !(word & LA_FRESH)) ? S_hbm[(int64_t) i * vdim + j] : 0.0f;
    }
    float * qt = lds, * kt = lds + LA_TB * dim;
    for (int t0 = 0; t0 < len; t0 += LA_TB) {
        const int nt = min(LA_TB, len - t0);
        __syncthreads();
        for (int idx = tid; idx < nt * dim; idx += blockDim.x) {
            const int tt = idx / dim, i = idx % dim;
            const int64_t off = (int64_t) (first + t0 + tt) * stride + (int64_t) h * dim + i;
            qt[idx] = q[off]; kt[idx] = k[off];
        }
        __syncthreads();
        for (int tt = 0; tt < nt; tt++) {
            const int t = first + t0 + tt;
            const float vj = col_ok ? v[(int64_t) t * stride + (int64_t) h * vdim + j] : 0.0f;
            float o = 0.0f;
#pragma unroll
            for (int ii = 0; ii < DPT; ii++) {
                const int i = sp * DPT + ii;
                if (i < dim) {
                    S[ii] = fmaf(kt[tt * dim + i], vj, lam * S[ii]);
                    o = fmaf(S[ii], qt[tt * dim + i], o);
                }
            }
            for (int d = R >> 1; d > 0; d >>= 1) o += __shfl_xor(o, d, PI_WAVE);
            if (col_ok && sp == 0) out[(int64_t) t * os + (int64_t) h * vdim + j] = o;
        }
    }
    if (col_ok)
#pragma unroll
        for (int ii = 0; ii < DPT; ii++) { const int i = sp * DPT + ii; if (i < dim) S_hbm[(int64_t) i * vdim + j] = S[ii]; }
}

extern "C" int pi_op_linear_attention(const float * q, const float * k, const float * v, int64_t stride, int heads, int dim, int vdim, const float * decay_dev, float * state_dev,
                                      const int32_t * rec_dev, int n_tok, int max_segments, float * out, int64_t out_stride, void * stream) {
    if (n_tok <= 0) return 0;
    if (dim <= 0 || vdim <= 0 || heads <= 0 || dim > 1024) { pi_set_error("pi_op_linear_attention: head sizes %d x %d outside the kernel's range (key width <= 1024)", dim, vdim); return -1; }
    const int dpt = dim <= 16 ? 16 : dim <= 32 ? 32 : 64;
    int R = 1; while (R * dpt < dim) R *= 2;
    int threads = std::min(256, (vdim * R + 63) / 64 * 64);
    const int cols = threads / R;
    const dim3 grid((unsigned) heads, (unsigned) ((vdim + cols - 1) / cols), (unsigned) std::max(1, std::min(n_tok, max_segments)));
    const size_t lds = ((size_t) 2 * LA_TB * dim + (size_t) n_tok) * sizeof(float);
    const double bytes = 4.0 * n_tok * heads * (2.0 * dim + 2.0 * vdim) + 8.0 * heads * dim * vdim;
    hipStream_t s = (hipStream_t) stream;
#define LA_GO(D) PI_KT_LAUNCH(PI_KT_ATT, 0, std::min(n_tok, PI_KT_MAXNT - 1), bytes, k_linear_attention<D>, grid, dim3(threads), lds, s, q, k, v, stride, heads, dim, vdim, R, decay_dev, state_dev, rec_dev, n_tok, out, out_stride, pi_abort_word())
    if (dpt == 16) LA_GO(16); else if (dpt == 32) LA_GO(32); else LA_GO(64);
#undef LA_GO
    PI_CHECK_LAUNCH(); return 0;
}

// copies the state of one slot to another, all heads of one layer (sequence copy)
__global__ void k_copy_f32(const float * __restrict__ src, float * __restrict__ dst, int64_t n) {
    for (int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t) gridDim.x * 256) dst[i] = src[i];
}
extern "C" int pi_op_copy_f32(const float * src, float * dst, int64_t n, void * stream) {
    if (n <= 0) return 0;
    hipLaunchKernelGGL(k_copy_f32, dim3((unsigned) std::max<int64_t>(1, std::min<int64_t>(1024, (n + 255) / 256))), dim3(256), 0, (hipStream_t) stream, src, dst, n);
    PI_CHECK_LAUNCH(); return 0;
}

// ---- attention over a shared latent -----------------------------------------------------------------------------------------------------------------
// grid (token, head tile of HT); LDS: qa [HT][rank] (absorbed, pre-scaled queries) | ol [4 waves][HT][rank] | sc [HT][cap] scores then probabilities
template <int HT>
__global__ void __launch_bounds__(256) k_latent_attention(const float * __restrict__ q, int64_t qs, const float * __restrict__ cache, const uint32_t * __restrict__ mask,
                                                          const uint16_t * __restrict__ wuk, const uint16_t * __restrict__ wuv, const float * __restrict__ sink, float scale,
                                                          int heads, int dim, int vdim, int rank, int n_kv_arg, int cap, float * __restrict__ out, int64_t os,
                                                          const int32_t * __restrict__ dyn, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w, 5)) return;
    extern __shared__ float lds[];
    __shared__ float red[4], hm[HT], hden[HT];
    const int t = blockIdx.x, h0 = blockIdx.y * HT, nh = min(HT, heads - h0), tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n_kv = min(dyn ? dyn[1] : n_kv_arg, cap);
    const int words = (n_kv_arg + 31) / 32;
    float * qa = lds, * ol = qa + HT * rank, * sc = ol + 4 * HT * rank;
    for (int idx = tid; idx < nh * rank; idx += 256) {
        const int hh = idx / rank, r = idx % rank;
        const float * qh = q + (int64_t) t * qs + (int64_t) (h0 + hh) * dim;
        const uint16_t * wk = wuk + (int64_t) (h0 + hh) * dim * rank + r;
        float a = 0.0f;
        for (int d = 0; d < dim; d++) a = fmaf(qh[d], hy_widen(wk[(int64_t) d * rank]), a);
        qa[idx] = a * scale;
    }
    __syncthreads();
    const uint32_t * mrow = mask + (int64_t) t * words;
    float lmax[HT];
#pragma unroll
    for (int hh = 0; hh < HT; hh++) lmax[hh] = -INFINITY;
    for (int j = tid; j < n_kv; j += 256) {
        const bool vis = (mrow[j >> 5] >> (j & 31)) & 1u;
        float a[HT];
#pragma unroll
        for (int hh = 0; hh < HT; hh++) a[hh] = 0.0f;
        if (vis) {
            const float * c = cache + (int64_t) j * rank;
            if ((rank & 3) == 0) {
                for (int r = 0; r < rank; r += 4) {
                    const float4 cv = *(const float4 *) (c + r);
#pragma unroll
                    for (int hh = 0; hh < HT; hh++) {
                        const float * qq = qa + hh * rank + r;
                        a[hh] = fmaf(qq[0], cv.x, a[hh]); a[hh] = fmaf(qq[1], cv.y, a[hh]); a[hh] = fmaf(qq[2], cv.z, a[hh]); a[hh] = fmaf(qq[3], cv.w, a[hh]);
                    }
                }
            } else {
                for (int r = 0; r < rank; r++) {
                    const float cv = c[r];
#pragma unroll
                    for (int hh = 0; hh < HT; hh++) a[hh] = fmaf(qa[hh * rank + r], cv, a[hh]);
                }
            }
        }
#pragma unroll
        for (int hh = 0; hh < HT; hh++) {
            const float s = vis ? a[hh] : -INFINITY;
            if (hh < nh) sc[hh * cap + j] = s;
            lmax[hh] = fmaxf(lmax[hh], s);
        }
    }
#pragma unroll
    for (int hh = 0; hh < HT; hh++) {
        const float m = hy_block_max(lmax[hh], red);
        if (tid == 0 && hh < nh) hm[hh] = fmaxf(m, sink[h0 + hh]);
    }
    __syncthreads();
#pragma unroll
    for (int hh = 0; hh < HT; hh++) {
        float l = 0.0f;
        if (hh < nh) {
            const float m = hm[hh];
            for (int j = tid; j < n_kv; j += 256) { const float p = expf(sc[hh * cap + j] - m); sc[hh * cap + j] = p; l += p; }
        }
        l = hy_block_sum(l, red);
        if (tid == 0 && hh < nh) hden[hh] = l + expf(sink[h0 + hh] - hm[hh]);
    }
    __syncthreads();
    // probability-weighted sum of latents: wave w takes cells w, w + 4, ...; lanes walk the (head, r) pairs
    for (int base = 0; base < nh * rank; base += 64) {
        const int idx = base + lane;
        const bool ok = idx < nh * rank;
        const int hh = ok ? idx / rank : 0, r = ok ? idx % rank : 0;
        float a = 0.0f;
        for (int j = wave; j < n_kv; j += 4) {
            const float p = sc[hh * cap + j];
            if (p != 0.0f) a = fmaf(p, cache[(int64_t) j * rank + r], a);
        }
        if (ok) ol[wave * HT * rank + idx] = a;
    }
    __syncthreads();
    for (int idx = tid; idx < nh * rank; idx += 256)
        ol[idx] = (ol[idx] + ol[HT * rank + idx] + ol[2 * HT * rank + idx] + ol[3 * HT * rank + idx]) / hden[idx / rank];
    __syncthreads();
    // value up-projection: one wave per output value
    for (int o = wave; o < nh * vdim; o += 4) {
        const int hh = o / vdim, vv = o % vdim;
        const uint16_t * wv = wuv + ((int64_t) (h0 + hh) * vdim + vv) * rank;
        float a = 0.0f;
        for (int r = lane; r < rank; r += 64) a = fmaf(hy_widen(wv[r]), ol[hh * rank + r], a);
        a = pi_lanes_sum<64>(a);
        if (lane == 0) out[(int64_t) t * os + (int64_t) (h0 + hh) * vdim + vv] = a;
    }
}

#define LAT_LDS_BUDGET (144 * 1024)
static int latent_tile(int heads, int rank, int cap, int n_tok) {
    int ht = n_tok >= 8 ? 8 : 1;                                     // single tokens: one head per workgroup (more workgroups); prompts: the cache row is read once for 8 heads
    while (ht > 1 && (ht / 2 >= heads || ((size_t) 5 * ht * rank + (size_t) ht * cap) * 4 > LAT_LDS_BUDGET)) ht /= 2;
    return ht;
}
extern "C" int pi_op_latent_attention_max_cells(int rank) { return (int) std::min<int64_t>(LAT_LDS_BUDGET / 4 - 5 * (int64_t) rank, 1 << 20); }
extern "C" int pi_op_latent_attention_reserve(void) {
    PI_CHECK_HIP(hipFuncSetAttribute((const void *) k_latent_attention<1>, hipFuncAttributeMaxDynamicSharedMemorySize, LAT_LDS_BUDGET));
    PI_CHECK_HIP(hipFuncSetAttribute((const void *) k_latent_attention<2>, hipFuncAttributeMaxDynamicSharedMemorySize, LAT_LDS_BUDGET));
    PI_CHECK_HIP(hipFuncSetAttribute((const void *) k_latent_attention<4>, hipFuncAttributeMaxDynamicSharedMemorySize, LAT_LDS_BUDGET));
    PI_CHECK_HIP(hipFuncSetAttribute((const void *) k_latent_attention<8>, hipFuncAttributeMaxDynamicSharedMemorySize, LAT_LDS_BUDGET));
    return 0;
}
extern "C" int pi_op_latent_attention(const float * q, int64_t q_stride, const float * cache, const uint32_t * mask, const pi_weight * wuk, const pi_weight * wuv, const float * sink_dev,
                                      float scale, int heads, int dim, int vdim, int rank, int n_tok, int n_kv, float * out, int64_t out_stride, const int32_t * dyn_dev, void * stream) {
    if (n_tok <= 0) return 0;
    if (!wuk || !wuv || wuk->type != PI_BF16 || wuv->type != PI_BF16 || wuk->ne0 != rank || wuv->ne0 != rank || wuk->ne1 != (int64_t) heads * dim || wuv->ne1 != (int64_t) heads * vdim) {
        pi_set_error("pi_op_latent_attention: the up-projections must be bfloat16 [heads * dim][rank] and [heads * vdim][rank]"); return -1;
    }
    if (((size_t) 5 * rank + (size_t) n_kv) * 4 > LAT_LDS_BUDGET) { pi_set_error("pi_op_latent_attention: %d cells of rank %d do not fit a workgroup's score row", n_kv, rank); return -1; }
    const int ht = latent_tile(heads, rank, n_kv, n_tok);
    const size_t lds = ((size_t) 5 * ht * rank + (size_t) ht * n_kv) * 4;
    const dim3 grid((unsigned) n_tok, (unsigned) ((heads + ht - 1) / ht));
    const int acct = pi_account_n_kv() > 0 ? pi_account_n_kv() : n_kv;
    const double bytes = 4.0 * acct * rank + 2.0 * rank * heads * (dim + vdim) + 4.0 * n_tok * heads * (dim + vdim);
    hipStream_t s = (hipStream_t) stream;
#define LAT_GO(H) PI_KT_LAUNCH(PI_KT_ATT, PI_BF16, std::min(n_tok, PI_KT_MAXNT - 1), bytes, k_latent_attention<H>, grid, dim3(256), lds, s, q, q_stride, cache, mask, (const uint16_t *) wuk->p0, (const uint16_t *) wuv->p0, \
                                sink_dev, scale, heads, dim, vdim, rank, n_kv, n_kv, out, out_stride, dyn_dev, pi_abort_word())
    if (ht == 8) LAT_GO(8); else if (ht == 4) LAT_GO(4); else if (ht == 2) LAT_GO(2); else LAT_GO(1);
#undef LAT_GO
    PI_CHECK_LAUNCH(); return 0;
}

// ---- routed feed-forward ------------------------------------------------------------------------------------------------------------------------------
// one workgroup per token: logits of all router outputs (a wave per output), soft-max, choice = score + correction, `top` rounds of arg-max (lowest index wins a tie)
__global__ void __launch_bounds__(256) k_moe_route(const uint16_t * __restrict__ router, int64_t width, int n_out, const float * __restrict__ corr, const float * __restrict__ x, int64_t xs,
                                                   int top, int exact, int32_t * __restrict__ sel, float * __restrict__ selw, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    extern __shared__ float z[];                  // [n_out] logits -> scores | [n_out] choice
    float * ch = z + n_out;
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float * xr = x + (int64_t) t * xs;
    for (int e = wave; e < n_out; e += 4) {
        const uint16_t * w = router + (int64_t) e * width;
        float a = 0.0f;
        for (int64_t i = lane; i < width; i += 64) a = fmaf(hy_widen(w[i]), exact ? xr[i] : hy_round(xr[i]), a);
        a = pi_lanes_sum<64>(a);
        if (lane == 0) z[e] = a;
    }
    __syncthreads();
    if (wave != 0) return;
    float m = -INFINITY;
    for (int e = lane; e < n_out; e += 64) m = fmaxf(m, z[e]);
    m = pi_wave_max(m);
    float l = 0.0f;
    for (int e = lane; e < n_out; e += 64) { const float p = expf(z[e] - m); z[e] = p; l += p; }
    l = pi_lanes_sum<64>(l);
    for (int e = lane; e < n_out; e += 64) { z[e] = z[e] / l; ch[e] = z[e] + corr[e]; }
    for (int kk = 0; kk < top; kk++) {
        float bv = -INFINITY; int bi = 0x7fffffff;
        for (int e = lane; e < n_out; e += 64) { const float c = ch[e]; if (c > bv || (c == bv && e < bi)) { bv = c; bi = e; } }
        for (int d = 32; d > 0; d >>= 1) {
            const float ov = __shfl_xor(bv, d, PI_WAVE); const int oi = __shfl_xor(bi, d, PI_WAVE);
            if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
        }
        if (bi == 0x7fffffff) bi = 0;             // (fewer finite choices than `top`: cannot happen with finite logits)
        if (lane == 0) { sel[(int64_t) t * top + kk] = bi; selw[(int64_t) t * top + kk] = z[bi]; ch[bi] = -INFINITY; }
    }
}

// up[t][kk][f] = relu(W_up[e] x_t)^2 for the kk-th chosen expert e of token t (nothing for identity experts); a wave per row f
__global__ void __launch_bounds__(256) k_moe_up(const uint16_t * __restrict__ wup, int64_t width, int ff, int n_exp, const float * __restrict__ x, int64_t xs, const int32_t * __restrict__ sel,
                                                int top, int exact, float * __restrict__ up, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w, 0)) return;
    const int lane = threadIdx.x & 63, f = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int slot = blockIdx.y, e = sel[slot];
    if (f >= ff || e >= n_exp) return;
    const int t = slot / top;
    const float * xr = x + (int64_t) t * xs;
    const uint16_t * w = wup + ((int64_t) e * ff + f) * width;
    float a = 0.0f;
    for (int64_t i = lane; i < width; i += 64) a = fmaf(hy_widen(w[i]), exact ? xr[i] : hy_round(xr[i]), a);
    a = pi_lanes_sum<64>(a);
    if (lane == 0) { const float r = fmaxf(a, 0.0f); up[(int64_t) slot * ff + f] = r * r; }
}
// out[t][n] = sum_kk w_kk * (identity ? x[t][n] : W_down[e_kk][n] . up[t][kk]); a wave per output n
__global__ void __launch_bounds__(256) k_moe_down(const uint16_t * __restrict__ wdown, int64_t width, int ff, int n_exp, int top, const float * __restrict__ x, int64_t xs,
                                                  const int32_t * __restrict__ sel, const float * __restrict__ selw, const float * __restrict__ up, int exact, float * __restrict__ out, int64_t os,
                                                  const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w, 0)) return;
    const int lane = threadIdx.x & 63;
    const int64_t n = (int64_t) blockIdx.x * 4 + (threadIdx.x >> 6);
    const int t = blockIdx.y;
    if (n >= width) return;
    float acc = 0.0f;
    for (int kk = 0; kk < top; kk++) {
        const int e = sel[(int64_t) t * top + kk];
        const float wgt = selw[(int64_t) t * top + kk];
        if (e >= n_exp) { acc = fmaf(wgt, x[(int64_t) t * xs + n], acc); continue; }
        const uint16_t * w = wdown + ((int64_t) e * width + n) * ff;
        const float * u = up + ((int64_t) t * top + kk) * ff;
        float a = 0.0f;
        for (int i = lane; i < ff; i += 64) a = fmaf(hy_widen(w[i]), exact ? u[i] : hy_round(u[i]), a);
        a = pi_lanes_sum<64>(a);
        acc = fmaf(wgt, a, acc);
    }
    if (lane == 0) out[(int64_t) t * os + n] = acc;
}

extern "C" int pi_op_moe_route(const pi_weight * router, const float * correction_dev, const float * x, int64_t x_stride, int n_tok, int top, int exact, int32_t * sel_dev, float * selw_dev, void * stream) {
    if (n_tok <= 0) return 0;
    if (!router || router->type != PI_BF16 || top < 1 || top > router->ne1 || router->ne1 > 8192) { pi_set_error("pi_op_moe_route: a bfloat16 router of at most 8192 outputs and 1 <= top <= outputs are required"); return -1; }
    PI_KT_LAUNCH(PI_KT_OTHER, PI_BF16, 1, 2.0 * router->ne0 * router->ne1 + 4.0 * n_tok * router->ne0, k_moe_route, dim3((unsigned) n_tok), dim3(256), (size_t) 8 * router->ne1, (hipStream_t) stream,
                 (const uint16_t *) router->p0, router->ne0, (int) router->ne1, correction_dev, x, x_stride, top, exact, sel_dev, selw_dev, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}
// wup: [n_exp * ff][width], wdown: [n_exp * width][ff] (the experts' matrices one after the other); up_dev: scratch [n_tok][top][ff]
extern "C" int pi_op_moe_experts(const pi_weight * wup, const pi_weight * wdown, int n_exp, int ff, const float * x, int64_t x_stride, const int32_t * sel_dev, const float * selw_dev, int n_tok, int top,
                                 int exact, float * up_dev, float * out, int64_t out_stride, void * stream) {
    if (n_tok <= 0) return 0;
    hipStream_t s = (hipStream_t) stream;
    int64_t width = 0;
    if (n_exp > 0) {
        if (!wup || !wdown || wup->type != PI_BF16 || wdown->type != PI_BF16 || wup->ne1 != (int64_t) n_exp * ff || wdown->ne0 != ff || wdown->ne1 != (int64_t) n_exp * wup->ne0) {
            pi_set_error("pi_op_moe_experts: expert matrices must be bfloat16 [experts * ff][width] and [experts * width][ff]"); return -1;
        }
        width = wup->ne0;
        const double b_up = std::min<double>(n_tok * top, n_exp) * 2.0 * ff * width + 4.0 * n_tok * (width + (double) top * ff);
        PI_KT_LAUNCH(PI_KT_MATVEC, PI_BF16, std::min(n_tok, PI_KT_MAXNT - 1), b_up, k_moe_up, dim3((unsigned) ((ff + 3) / 4), (unsigned) (n_tok * top)), dim3(256), 0, s,
                     (const uint16_t *) wup->p0, width, ff, n_exp, x, x_stride, sel_dev, top, exact, up_dev, pi_abort_word());
        PI_CHECK_LAUNCH();
    } else width = out_stride;
    const double b_dn = std::min<double>(n_tok * top, std::max(n_exp, 1)) * 2.0 * ff * width + 4.0 * n_tok * (width + (double) top * ff);
    PI_KT_LAUNCH(PI_KT_MATVEC, PI_BF16, std::min(n_tok, PI_KT_MAXNT - 1), b_dn, k_moe_down, dim3((unsigned) ((width + 3) / 4), (unsigned) n_tok), dim3(256), 0, s,
                 n_exp > 0 ? (const uint16_t *) wdown->p0 : nullptr, width, ff, n_exp, top, x, x_stride, sel_dev, selw_dev, up_dev, exact, out, out_stride, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}

// ---- the same for a prompt's worth of tokens: grouped by expert, on the matrix cores ---------------------------------------------------------------------
// k_moe_group sorts the (token, choice) slots of a pass by expert (a counting sort in one workgroup) and cuts every expert's run into tiles of 64 slots; k_moe_up_mfma /
// k_moe_down_mfma compute 64 slots x 64 rows per workgroup with v_mfma_f32_16x16x32_bf16 (operand layout as k_dense_mfma: A = 16 weight rows, B = 16 slots, 8 consecutive k per
// lane) — an expert's matrices are read once per 64 of its tokens instead of once per token; k_moe_combine sums a token's weighted choices (identity experts: the input itself).
// idx layout (int32): [0] number of tiles | tile expert [max_tiles] | tile start [max_tiles] | tile length [max_tiles] | order [n_slots]
typedef __bf16 hy_bf16x8 __attribute__((ext_vector_type(8)));
typedef float hy_f32x4 __attribute__((ext_vector_type(4)));
typedef uint16_t hy_u16x8 __attribute__((ext_vector_type(8)));
#define MOE_GROUP_MAX_EXPERTS 1024
static inline int moe_max_tiles(int n_slots, int n_exp) { return (n_slots + 63) / 64 + std::min(n_exp, n_slots); }

__global__ void __launch_bounds__(256) k_moe_group(const int32_t * __restrict__ sel, int n_slots, int n_exp, int max_tiles, int32_t * __restrict__ idx, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    __shared__ int cnt[MOE_GROUP_MAX_EXPERTS], cur[MOE_GROUP_MAX_EXPERTS];
    int32_t * tile_e = idx + 1, * tile_s = tile_e + max_tiles, * tile_n = tile_s + max_tiles, * order = tile_n + max_tiles;
    for (int e = threadIdx.x; e < n_exp; e += 256) cnt[e] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < n_slots; i += 256) { const int e = sel[i]; if (e >= 0 && e < n_exp) atomicAdd(&cnt[e], 1); }
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0, nt = 0;
        for (int e = 0; e < n_exp; e++) {
            cur[e] = at;
            for (int k = 0; k < cnt[e]; k += 64) { tile_e[nt] = e; tile_s[nt] = at + k; tile_n[nt] = min(64, cnt[e] - k); nt++; }
            at += cnt[e];
        }
        idx[0] = nt;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n_slots; i += 256) { const int e = sel[i]; if (e >= 0 && e < n_exp) order[atomicAdd(&cur[e], 1)] = i; }
}

// acc[j] += W[rows j*16 + (l % 16)][k] * B[slot (l % 16)][k] over K (K % 8 == 0); brow: this lane's B row (nullptr: zeros), wrow[j]: this lane's A rows (nullptr: zeros)
static __device__ __forceinline__ void hy_mfma_rows(const uint16_t * const wrow[4], const float * brow, int64_t K, int kb, hy_f32x4 acc[4]) {
    for (int64_t k0 = 0; k0 < K; k0 += 32) {
        const int64_t k = k0 + kb * 8;
        const bool k_ok = k < K;
        hy_u16x8 b = hy_u16x8{0, 0, 0, 0, 0, 0, 0, 0};
        if (k_ok && brow) {
            const float4 v0 = *(const float4 *) (brow + k), v1 = *(const float4 *) (brow + k + 4);
            const float f[8] = { v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w };
#pragma unroll
            for (int i = 0; i < 8; i++) { const uint32_t u = __float_as_uint(f[i]); b[i] = (uint16_t) ((u + 0x7fffu + ((u >> 16) & 1u)) >> 16); }
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            hy_u16x8 a = hy_u16x8{0, 0, 0, 0, 0, 0, 0, 0};
            if (k_ok && wrow[j]) a = *(const hy_u16x8 *) (wrow[j] + k);
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(hy_bf16x8, a), __builtin_bit_cast(hy_bf16x8, b), acc[j], 0, 0, 0);
        }
    }
}

// UP: B rows are the tokens' inputs x[slot / top], A rows W_up[e], out up[slot][f] = relu(.)^2;  !UP: B rows up[slot] (K = ff), A rows W_down[e], out dn[slot][n]
template <bool UP>
__global__ void __launch_bounds__(256) k_moe_mfma(const uint16_t * __restrict__ W, int64_t K, int rows, const float * __restrict__ B, int64_t bs, int top, const int32_t * __restrict__ idx,
                                                  int max_tiles, float * __restrict__ out, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w, 1)) return;
    const int tile = blockIdx.y;
    if (tile >= idx[0]) return;
    const int32_t * tile_e = idx + 1, * tile_s = tile_e + max_tiles, * tile_n = tile_s + max_tiles, * order = tile_n + max_tiles;
    const int e = tile_e[tile], start = tile_s[tile], len = tile_n[tile];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, li = lane & 15, kb = lane >> 4;
    if (wave * 16 >= len) return;                                  // (whole waves: no barrier follows)
    const int si = wave * 16 + li;
    const int slot = si < len ? order[start + si] : -1;
    const float * brow = slot < 0 ? nullptr : B + (int64_t) (UP ? slot / top : slot) * bs;
    const int n0 = blockIdx.x * 64;
    const uint16_t * wrow[4];
#pragma unroll
    for (int j = 0; j < 4; j++) { const int r = n0 + j * 16 + li; wrow[j] = r < rows ? W + ((int64_t) e * rows + r) * K : nullptr; }
    hy_f32x4 acc[4];
#pragma unroll
    for (int j = 0; j < 4; j++) acc[j] = hy_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    hy_mfma_rows(wrow, brow, K, kb, acc);
    if (slot < 0) return;
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int row = n0 + j * 16 + kb * 4 + r;
            if (row < rows) { float v = acc[j][r]; if (UP) { v = fmaxf(v, 0.0f); v *= v; } out[(int64_t) slot * rows + row] = v; }
        }
}

__global__ void __launch_bounds__(256) k_moe_combine(const float * __restrict__ dn, int64_t width, int n_exp, int top, const float * __restrict__ x, int64_t xs, const int32_t * __restrict__ sel,
                                                     const float * __restrict__ selw, float * __restrict__ out, int64_t os, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    const int t = blockIdx.y;
    const int64_t n = (int64_t) blockIdx.x * 256 + threadIdx.x;
    if (n >= width) return;
    float acc = 0.0f;
    for (int kk = 0; kk < top; kk++) {
        const int e = sel[(int64_t) t * top + kk];
        acc = fmaf(selw[(int64_t) t * top + kk], e >= n_exp ? x[(int64_t) t * xs + n] : dn[((int64_t) t * top + kk) * width + n], acc);
    }
    out[(int64_t) t * os + n] = acc;
}

// ints of index scratch the grouped path needs for a pass of n_tok tokens
extern "C" size_t pi_op_moe_grouped_index_ints(int n_tok, int top, int n_exp) { const int ns = n_tok * top; return (size_t) 1 + 3 * (size_t) moe_max_tiles(ns, n_exp) + (size_t) ns; }
// whether a pass of this shape takes the grouped matrix-core path (otherwise pi_op_moe_experts: gathered mat-vecs)
extern "C" int pi_op_moe_grouped_ok(const pi_weight * wup, const pi_weight * wdown, int n_exp, int ff, int n_tok, int top, int exact) {
    static const int min_slots = getenv("PI_MOE_GROUPED_MIN") ? atoi(getenv("PI_MOE_GROUPED_MIN")) : 32;
    return !exact && n_exp > 0 && n_exp <= MOE_GROUP_MAX_EXPERTS && wup && wdown && n_tok * top >= min_slots && wup->ne0 % 8 == 0 && ff % 8 == 0 &&
           ((uintptr_t) wup->p0 % 16) == 0 && ((uintptr_t) wdown->p0 % 16) == 0;
}
// up_dev: [n_tok * top][ff], dn_dev: [n_tok * top][width], idx_dev: pi_op_moe_grouped_index_ints ints
extern "C" int pi_op_moe_experts_grouped(const pi_weight * wup, const pi_weight * wdown, int n_exp, int ff, const float * x, int64_t x_stride, const int32_t * sel_dev, const float * selw_dev, int n_tok, int top,
                                         float * up_dev, float * dn_dev, int32_t * idx_dev, float * out, int64_t out_stride, void * stream) {
    if (!pi_op_moe_grouped_ok(wup, wdown, n_exp, ff, n_tok, top, 0)) { pi_set_error("pi_op_moe_experts_grouped: this shape takes pi_op_moe_experts"); return -1; }
    if (wup->type != PI_BF16 || wdown->type != PI_BF16 || wup->ne1 != (int64_t) n_exp * ff || wdown->ne0 != ff || wdown->ne1 != (int64_t) n_exp * wup->ne0 || x_stride % 4 || ((uintptr_t) x % 16)) {
        pi_set_error("pi_op_moe_experts_grouped: expert matrices must be bfloat16 [experts * ff][width] and [experts * width][ff], inputs 16-byte aligned rows"); return -1;
    }
    hipStream_t s = (hipStream_t) stream;
    const int64_t width = wup->ne0;
    const int ns = n_tok * top, mt = moe_max_tiles(ns, n_exp), nta = std::min(n_tok, PI_KT_MAXNT - 1);
    const double wbytes = std::min<double>(ns, n_exp) * 2.0 * ff * width;
    PI_KT_LAUNCH(PI_KT_OTHER, PI_BF16, 1, 8.0 * ns, k_moe_group, dim3(1), dim3(256), 0, s, sel_dev, ns, n_exp, mt, idx_dev, pi_abort_word());
    PI_CHECK_LAUNCH();
    PI_KT_LAUNCH(PI_KT_MMQ, PI_BF16, nta, wbytes + 4.0 * ns * (width + ff), k_moe_mfma<true>, dim3((unsigned) ((ff + 63) / 64), (unsigned) mt), dim3(256), 0, s,
                 (const uint16_t *) wup->p0, width, ff, x, x_stride, top, idx_dev, mt, up_dev, pi_abort_word());
    PI_CHECK_LAUNCH();
    PI_KT_LAUNCH(PI_KT_MMQ, PI_BF16, nta, wbytes + 4.0 * ns * (width + ff), k_moe_mfma<false>, dim3((unsigned) ((width + 63) / 64), (unsigned) mt), dim3(256), 0, s,
                 (const uint16_t *) wdown->p0, (int64_t) ff, (int) width, up_dev, (int64_t) ff, top, idx_dev, mt, dn_dev, pi_abort_word());
    PI_CHECK_LAUNCH();
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 4.0 * n_tok * width * (top + 2), k_moe_combine, dim3((unsigned) ((width + 255) / 256), (unsigned) n_tok), dim3(256), 0, s,
                 dn_dev, width, n_exp, top, x, x_stride, sel_dev, selw_dev, out, out_stride, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}
