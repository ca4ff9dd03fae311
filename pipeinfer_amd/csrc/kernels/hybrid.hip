// Operators of hybrid decoder blocks (recurrent and low-rank-attention mixers, routed feed-forwards).  Everything here is fp32: norms, scores, soft-max, recurrent
// state, router.  Matrices are bfloat16 pi_weights (widened exactly); `exact` = 0 rounds the activations that enter an expert's matrices to bfloat16 as pi_op_dense does.
//
//   k_rms_scale          y = x / sqrt(mean(x^2) + eps) * (w + w_offset) [* gate];  out = [residual +] mult * y;  rows may be written into the cache cells of the pass
//   k_linear_attention   per head S <- lambda * S + k v^T, o = S^T q over a run of tokens of one sequence; S lives in HBM per (slot, head) between calls
//   k_latent_attention   attention over a shared low-rank latent c: the key up-projection is folded into the query (q~ = W_uk^T q), the value up-projection applied to the
//                        probability-weighted sum of latents — the cache is read once for all heads of a tile and K / V are never materialised; soft-max with a sink term
//   k_norm_chain(_reg)   y = ((ca * a + cb * b) - mean) / sqrt(variance + eps) * w + bias;  out = [residual +] y   (layer norm of one input or of the weighted sum of two), and
//                        the three row operations at the end of a block in one launch: post-norm + residual, the depth average, the next sublayer's pre-norm
//   k_depth_mix          out = sum_j coef[j] * X_j over the stream's earlier states (a learned average over depth)
//   k_moe_route          router logits, soft-max over all router outputs, bias-corrected top-k choice, weights = uncorrected scores
//   k_moe_up / _down     the chosen experts of every token (gathered mat-vecs), identity experts pass their input through
#include "ops_common.h"
#include "kernel_timing.h"

#include <algorithm>
#include <cmath>

static __device__ __forceinline__ float hy_widen(uint16_t b) { return __uint_as_float((uint32_t) b << 16); }
static __device__ __forceinline__ float hy_round(float f) { const uint32_t u = __float_as_uint(f); return __uint_as_float(((u + 0x7fffu + ((u >> 16) & 1u)) >> 16) << 16); }

typedef uint16_t hy_u16x8v __attribute__((ext_vector_type(8)));
// this lane's share of w . x over n values (bfloat16 row w, fp32 row x); vec: n % 8 == 0 and both rows 16-byte aligned — 16-byte weight loads, several in flight
static __device__ __forceinline__ float hy_dot_lane(const uint16_t * __restrict__ w, const float * __restrict__ x, int64_t n, int lane, bool exact, bool vec) {
    float a = 0.0f;
    if (vec) {
#pragma unroll 4
        for (int64_t i = (int64_t) lane * 8; i < n; i += 512) {
            const hy_u16x8v wv = *(const hy_u16x8v *) (w + i);
            const float4 x0 = *(const float4 *) (x + i), x1 = *(const float4 *) (x + i + 4);
            const float xf[8] = { x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w };
#pragma unroll
            for (int k = 0; k < 8; k++) a = fmaf(hy_widen(wv[k]), exact ? xf[k] : hy_round(xf[k]), a);
        }
    } else {
        for (int64_t i = lane; i < n; i += 64) a = fmaf(hy_widen(w[i]), exact ? x[i] : hy_round(x[i]), a);
    }
    return a;
}

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
                                                   float * __restrict__ out, int64_t os, const int32_t * __restrict__ dyn, int to_cells, int vec, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    __shared__ float red[4];
    const int t = blockIdx.x;
    const float * xr = x + (int64_t) t * xs;
    float ss = 0.0f;
    if (vec) { for (int i = threadIdx.x * 4; i < n; i += 1024) { const float4 v = *(const float4 *) (xr + i); ss = fmaf(v.x, v.x, ss); ss = fmaf(v.y, v.y, ss); ss = fmaf(v.z, v.z, ss); ss = fmaf(v.w, v.w, ss); } }
    else for (int i = threadIdx.x; i < n; i += 256) ss = fmaf(xr[i], xr[i], ss);
    ss = hy_block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float) n + eps);
    const int64_t orow = to_cells ? pi_cell_of(dyn, 0, t) : t;
    if (vec) {
        for (int i = threadIdx.x * 4; i < n; i += 1024) {
            const float4 xv = *(const float4 *) (xr + i), wv = *(const float4 *) (w + i);
            float y[4] = { xv.x * inv * (wv.x + w_off), xv.y * inv * (wv.y + w_off), xv.z * inv * (wv.z + w_off), xv.w * inv * (wv.w + w_off) };
            if (gate) { const float4 g = *(const float4 *) (gate + (int64_t) t * gs + i); y[0] *= g.x; y[1] *= g.y; y[2] *= g.z; y[3] *= g.w; }
#pragma unroll
            for (int k = 0; k < 4; k++) y[k] *= mult;
            if (res) { const float4 r = *(const float4 *) (res + (int64_t) t * rs + i); y[0] = r.x + y[0]; y[1] = r.y + y[1]; y[2] = r.z + y[2]; y[3] = r.w + y[3]; }
            *(float4 *) (out + orow * os + i) = make_float4(y[0], y[1], y[2], y[3]);
        }
        return;
    }
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
    auto al = [](const void * p, int64_t stride) { return !p || (((uintptr_t) p % 16) == 0 && stride % 4 == 0); };
    const int vec = n % 4 == 0 && al(x, x_stride) && al(w, 0) && al(gate, gate_stride) && al(residual, residual_stride) && al(out, out_stride);
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 12.0 * n * n_tok, k_rms_scale, dim3((unsigned) n_tok), dim3(256), 0, (hipStream_t) stream, x, x_stride, w, w_offset, eps, n, gate, gate_stride,
                 residual, residual_stride, mult, out, out_stride, dyn_dev, to_cells, vec, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}

// ---- layer norm (weight and bias) over one or the weighted sum of two inputs, optional residual; the row operations at the end of a block -----------------------------
// The end of a block as one launch, per token row:  v = [residual +] LN_A(ca * a + cb * b)  -> out_a;   (n_hist > 0)  v = sum_(j < n_hist - 1) coef[j] * hist[j] + coef[n_hist - 1] * v
// -> out_mix  (out_a is hist[n_hist - 1]: the block's result joins the history it is averaged with);   (w_c)  LN_C(v) -> out_c  (the next sublayer's input).
// A thread re-reads only what it wrote itself, so no barrier is needed between the stages beyond those of the sums.
__global__ void __launch_bounds__(256) k_norm_chain(const float * __restrict__ a, int64_t as, float ca, const float * __restrict__ b, int64_t bs, float cb, const float * __restrict__ w,
                                                    const float * __restrict__ bias, float eps, int n, const float * __restrict__ res, int64_t rs, float * __restrict__ out_a, int64_t oas,
                                                    const float * __restrict__ hist, int64_t hist_stride, int n_hist, const float * __restrict__ coef, float * __restrict__ out_mix, int64_t oms,
                                                    const float * __restrict__ w_c, const float * __restrict__ bias_c, float * __restrict__ out_c, int64_t ocs, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    __shared__ float red[4];
    const int t = blockIdx.x;
    const float * ar = a + (int64_t) t * as, * br = b ? b + (int64_t) t * bs : nullptr;
    auto val = [&](int i) { const float v = ca * ar[i]; return br ? fmaf(cb, br[i], v) : v; };
    float sum = 0.0f;
    for (int i = threadIdx.x; i < n; i += 256) sum += val(i);
    const float mean = hy_block_sum(sum, red) / (float) n;
    float ss = 0.0f;
    for (int i = threadIdx.x; i < n; i += 256) { const float d = val(i) - mean; ss = fmaf(d, d, ss); }
    const float inv = 1.0f / sqrtf(hy_block_sum(ss, red) / (float) n + eps);
    float * oa = out_a + (int64_t) t * oas;
    float * last = oa;                                                 // the row the next stage reads (this thread's own elements)
    float sum_c = 0.0f;
    for (int i = threadIdx.x; i < n; i += 256) {
        float y = (val(i) - mean) * inv * w[i] + (bias ? bias[i] : 0.0f);
        if (res) y = res[(int64_t) t * rs + i] + y;
        oa[i] = y;
        if (n_hist > 0) {
            float m = 0.0f;
            for (int j = 0; j < n_hist - 1; j++) m = fmaf(coef[j], hist[(int64_t) j * hist_stride + (int64_t) t * n + i], m);
            y = fmaf(coef[n_hist - 1], y, m);
            out_mix[(int64_t) t * oms + i] = y;
        }
        sum_c += y;
    }
    if (!w_c) return;
    if (n_hist > 0) last = out_mix + (int64_t) t * oms;
    const float mean_c = hy_block_sum(sum_c, red) / (float) n;
    float ss_c = 0.0f;
    for (int i = threadIdx.x; i < n; i += 256) { const float d = last[i] - mean_c; ss_c = fmaf(d, d, ss_c); }
    const float inv_c = 1.0f / sqrtf(hy_block_sum(ss_c, red) / (float) n + eps);
    for (int i = threadIdx.x; i < n; i += 256) out_c[(int64_t) t * ocs + i] = (last[i] - mean_c) * inv_c * w_c[i] + (bias_c ? bias_c[i] : 0.0f);
}
// The same with the row in registers (n <= 256 * NPT): every input is loaded once, all loads are issued before the first sum, and the stages only exchange their sums
template <int NPT>
__global__ void __launch_bounds__(256) k_norm_chain_reg(const float * __restrict__ a, int64_t as, float ca, const float * __restrict__ b, int64_t bs, float cb, const float * __restrict__ w,
                                                        const float * __restrict__ bias, float eps, int n, const float * __restrict__ res, int64_t rs, float * __restrict__ out_a, int64_t oas,
                                                        const float * __restrict__ hist, int64_t hist_stride, int n_hist, const float * __restrict__ coef, float * __restrict__ out_mix, int64_t oms,
                                                        const float * __restrict__ w_c, const float * __restrict__ bias_c, float * __restrict__ out_c, int64_t ocs, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    __shared__ float red[4];
    const int t = blockIdx.x;
    const float * ar = a + (int64_t) t * as, * br = b ? b + (int64_t) t * bs : nullptr;
    float v[NPT], wv[NPT], bv[NPT], rv[NPT], mv[NPT];
    float sum = 0.0f;
#pragma unroll
    for (int k = 0; k < NPT; k++) {
        const int i = threadIdx.x + k * 256;
        const bool ok = i < n;
        float x = ok ? ca * ar[i] : 0.0f;
        if (ok && br) x = fmaf(cb, br[i], x);
        v[k] = x; sum += x;
        wv[k] = ok ? w[i] : 0.0f; bv[k] = ok && bias ? bias[i] : 0.0f; rv[k] = ok && res ? res[(int64_t) t * rs + i] : 0.0f;
        float m = 0.0f;
        if (ok) for (int j = 0; j < n_hist - 1; j++) m = fmaf(coef[j], hist[(int64_t) j * hist_stride + (int64_t) t * n + i], m);
        mv[k] = m;
    }
    const float mean = hy_block_sum(sum, red) / (float) n;
    float ss = 0.0f;
#pragma unroll
    for (int k = 0; k < NPT; k++) if (threadIdx.x + k * 256 < n) { const float d = v[k] - mean; ss = fmaf(d, d, ss); }
    const float inv = 1.0f / sqrtf(hy_block_sum(ss, red) / (float) n + eps);
    const float c_last = n_hist > 0 ? coef[n_hist - 1] : 0.0f;
    float sum_c = 0.0f;
#pragma unroll
    for (int k = 0; k < NPT; k++) {
        const int i = threadIdx.x + k * 256;
        if (i < n) {
            float y = (v[k] - mean) * inv * wv[k] + bv[k];
            if (res) y = rv[k] + y;
            out_a[(int64_t) t * oas + i] = y;
            if (n_hist > 0) { y = fmaf(c_last, y, mv[k]); out_mix[(int64_t) t * oms + i] = y; }
            v[k] = y; sum_c += y;
        }
    }
    if (!w_c) return;
#pragma unroll
    for (int k = 0; k < NPT; k++) { const int i = threadIdx.x + k * 256; wv[k] = i < n ? w_c[i] : 0.0f; bv[k] = i < n && bias_c ? bias_c[i] : 0.0f; }
    const float mean_c = hy_block_sum(sum_c, red) / (float) n;
    float ss_c = 0.0f;
#pragma unroll
    for (int k = 0; k < NPT; k++) if (threadIdx.x + k * 256 < n) { const float d = v[k] - mean_c; ss_c = fmaf(d, d, ss_c); }
    const float inv_c = 1.0f / sqrtf(hy_block_sum(ss_c, red) / (float) n + eps);
#pragma unroll
    for (int k = 0; k < NPT; k++) { const int i = threadIdx.x + k * 256; if (i < n) out_c[(int64_t) t * ocs + i] = (v[k] - mean_c) * inv_c * wv[k] + bv[k]; }
}
// ... and with 16-byte accesses: a thread owns NG groups of four neighbouring values (n % 4 == 0, rows 16-byte aligned, n <= 1024 * NG); one barrier per sum (each has its own LDS words)
static __device__ __forceinline__ float hy_block_sum_once(float v, float * red) {
    v = pi_lanes_sum<64>(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return red[0] + red[1] + red[2] + red[3];
}
template <int NG>
__global__ void __launch_bounds__(256) k_norm_chain_vec(const float * __restrict__ a, int64_t as, float ca, const float * __restrict__ b, int64_t bs, float cb, const float * __restrict__ w,
                                                        const float * __restrict__ bias, float eps, int n, const float * __restrict__ res, int64_t rs, float * __restrict__ out_a, int64_t oas,
                                                        const float * __restrict__ hist, int64_t hist_stride, int n_hist, const float * __restrict__ coef, float * __restrict__ out_mix, int64_t oms,
                                                        const float * __restrict__ w_c, const float * __restrict__ bias_c, float * __restrict__ out_c, int64_t ocs, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    __shared__ float red[4][4];
    const int t = blockIdx.x;
    const float * ar = a + (int64_t) t * as, * br = b ? b + (int64_t) t * bs : nullptr;
    const float4 zero = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    float4 v[NG], wv[NG], bv[NG], rv[NG], mv[NG];
    float sum = 0.0f;
#pragma unroll
    for (int g = 0; g < NG; g++) {
        const int i = (threadIdx.x + g * 256) * 4;
        const bool ok = i < n;
        float4 x = ok ? *(const float4 *) (ar + i) : zero;
        x.x *= ca; x.y *= ca; x.z *= ca; x.w *= ca;
        if (ok && br) { const float4 y = *(const float4 *) (br + i); x.x = fmaf(cb, y.x, x.x); x.y = fmaf(cb, y.y, x.y); x.z = fmaf(cb, y.z, x.z); x.w = fmaf(cb, y.w, x.w); }
        v[g] = x; sum += (x.x + x.y) + (x.z + x.w);
        wv[g] = ok ? *(const float4 *) (w + i) : zero;
        bv[g] = ok && bias ? *(const float4 *) (bias + i) : zero;
        rv[g] = ok && res ? *(const float4 *) (res + (int64_t) t * rs + i) : zero;
        float4 m = zero;
        if (ok) for (int j = 0; j < n_hist - 1; j++) {
            const float c = coef[j]; const float4 h = *(const float4 *) (hist + (int64_t) j * hist_stride + (int64_t) t * n + i);
            m.x = fmaf(c, h.x, m.x); m.y = fmaf(c, h.y, m.y); m.z = fmaf(c, h.z, m.z); m.w = fmaf(c, h.w, m.w);
        }
        mv[g] = m;
    }
    const float mean = hy_block_sum_once(sum, red[0]) / (float) n;
    float ss = 0.0f;
#pragma unroll
    for (int g = 0; g < NG; g++) if ((threadIdx.x + g * 256) * 4 < n) {
        const float d0 = v[g].x - mean, d1 = v[g].y - mean, d2 = v[g].z - mean, d3 = v[g].w - mean;
        ss = fmaf(d0, d0, ss); ss = fmaf(d1, d1, ss); ss = fmaf(d2, d2, ss); ss = fmaf(d3, d3, ss);
    }
    const float inv = 1.0f / sqrtf(hy_block_sum_once(ss, red[1]) / (float) n + eps);
    const float c_last = n_hist > 0 ? coef[n_hist - 1] : 0.0f;
    float sum_c = 0.0f;
#pragma unroll
    for (int g = 0; g < NG; g++) {
        const int i = (threadIdx.x + g * 256) * 4;
        if (i < n) {
            float4 y = make_float4((v[g].x - mean) * inv * wv[g].x + bv[g].x, (v[g].y - mean) * inv * wv[g].y + bv[g].y, (v[g].z - mean) * inv * wv[g].z + bv[g].z, (v[g].w - mean) * inv * wv[g].w + bv[g].w);
            if (res) { y.x = rv[g].x + y.x; y.y = rv[g].y + y.y; y.z = rv[g].z + y.z; y.w = rv[g].w + y.w; }
            *(float4 *) (out_a + (int64_t) t * oas + i) = y;
            if (n_hist > 0) {
                y.x = fmaf(c_last, y.x, mv[g].x); y.y = fmaf(c_last, y.y, mv[g].y); y.z = fmaf(c_last, y.z, mv[g].z); y.w = fmaf(c_last, y.w, mv[g].w);
                *(float4 *) (out_mix + (int64_t) t * oms + i) = y;
            }
            v[g] = y; sum_c += (y.x + y.y) + (y.z + y.w);
        }
    }
    if (!w_c) return;
#pragma unroll
    for (int g = 0; g < NG; g++) { const int i = (threadIdx.x + g * 256) * 4; wv[g] = i < n ? *(const float4 *) (w_c + i) : zero; bv[g] = i < n && bias_c ? *(const float4 *) (bias_c + i) : zero; }
    const float mean_c = hy_block_sum_once(sum_c, red[2]) / (float) n;
    float ss_c = 0.0f;
#pragma unroll
    for (int g = 0; g < NG; g++) if ((threadIdx.x + g * 256) * 4 < n) {
        const float d0 = v[g].x - mean_c, d1 = v[g].y - mean_c, d2 = v[g].z - mean_c, d3 = v[g].w - mean_c;
        ss_c = fmaf(d0, d0, ss_c); ss_c = fmaf(d1, d1, ss_c); ss_c = fmaf(d2, d2, ss_c); ss_c = fmaf(d3, d3, ss_c);
    }
    const float inv_c = 1.0f / sqrtf(hy_block_sum_once(ss_c, red[3]) / (float) n + eps);
#pragma unroll
    for (int g = 0; g < NG; g++) {
        const int i = (threadIdx.x + g * 256) * 4;
        if (i < n) *(float4 *) (out_c + (int64_t) t * ocs + i) = make_float4((v[g].x - mean_c) * inv_c * wv[g].x + bv[g].x, (v[g].y - mean_c) * inv_c * wv[g].y + bv[g].y,
                                                                              (v[g].z - mean_c) * inv_c * wv[g].z + bv[g].z, (v[g].w - mean_c) * inv_c * wv[g].w + bv[g].w);
    }
}
extern "C" int pi_op_layer_norm_mix(const float * a, int64_t a_stride, float ca, const float * b, int64_t b_stride, float cb, const float * w_dev, const float * bias_dev, float eps, int n, int n_tok,
                                    const float * residual, int64_t residual_stride, float * out, int64_t out_stride, void * stream) {
    return pi_op_norm_chain(a, a_stride, ca, b, b_stride, cb, w_dev, bias_dev, eps, n, n_tok, residual, residual_stride, out, out_stride, nullptr, 0, 0, nullptr, nullptr, 0, nullptr, nullptr, nullptr, 0, stream);
}
extern "C" int pi_op_norm_chain(const float * a, int64_t a_stride, float ca, const float * b, int64_t b_stride, float cb, const float * w_dev, const float * bias_dev, float eps, int n, int n_tok,
                                const float * residual, int64_t residual_stride, float * out_a, int64_t out_a_stride, const float * hist, int64_t hist_stride, int n_hist, const float * coef_dev,
                                float * out_mix, int64_t out_mix_stride, const float * w_next, const float * bias_next, float * out_next, int64_t out_next_stride, void * stream) {
    if (n_tok <= 0 || n <= 0) return 0;
    if (n_hist > 0 && (!hist || !coef_dev || !out_mix || out_a != hist + (int64_t) (n_hist - 1) * hist_stride || out_a_stride != n)) {
        pi_set_error("pi_op_norm_chain: the block's result must be written into the last entry of the history it is averaged with"); return -1;
    }
    if (w_next && (!out_next || out_next == out_a || out_next == out_mix)) { pi_set_error("pi_op_norm_chain: the next norm needs an output of its own"); return -1; }
    const double bytes = 4.0 * n * n_tok * (3.0 + (b ? 1 : 0) + (residual ? 1 : 0) + n_hist + (w_next ? 2 : 0));
#define NC_GO(K) PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, bytes, K, dim3((unsigned) n_tok), dim3(256), 0, (hipStream_t) stream, a, a_stride, ca, b, b_stride, cb, w_dev, bias_dev, eps, n, residual, residual_stride, \
                              out_a, out_a_stride, hist, hist_stride, n_hist, coef_dev, out_mix, out_mix_stride, w_next, bias_next, out_next, out_next_stride, pi_abort_word())
    auto al = [](const void * p, int64_t stride) { return !p || (((uintptr_t) p % 16) == 0 && stride % 4 == 0); };
    const bool vec = n % 4 == 0 && n <= 8192 && al(a, a_stride) && al(b, b_stride) && al(w_dev, 0) && al(bias_dev, 0) && al(residual, residual_stride) && al(out_a, out_a_stride) && al(hist, hist_stride) &&
                     al(out_mix, out_mix_stride) && al(w_next, 0) && al(bias_next, 0) && al(out_next, out_next_stride);
    if (vec) { if (n <= 1024) NC_GO(k_norm_chain_vec<1>); else if (n <= 2048) NC_GO(k_norm_chain_vec<2>); else if (n <= 4096) NC_GO(k_norm_chain_vec<4>); else NC_GO(k_norm_chain_vec<8>); }
    else if (n <= 1024) NC_GO(k_norm_chain_reg<4>); else if (n <= 2048) NC_GO(k_norm_chain_reg<8>); else if (n <= 4096) NC_GO(k_norm_chain_reg<16>); else if (n <= 8192) NC_GO(k_norm_chain_reg<32>); else NC_GO(k_norm_chain);
#undef NC_GO
    PI_CHECK_LAUNCH(); return 0;
}

// out[t][i] = sum_j coef[j] * hist[j][t][i], j ascending; hist: n_hist arrays [n_tok rows][n], `hist_stride` floats apart
__global__ void __launch_bounds__(256) k_depth_mix(const float * __restrict__ hist, int64_t hist_stride, int n_hist, const float * __restrict__ coef, int n, float * __restrict__ out, int64_t os,
                                                   const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    const int t = blockIdx.y, i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float a = 0.0f;
    for (int j = 0; j < n_hist; j++) a = fmaf(coef[j], hist[(int64_t) j * hist_stride + (int64_t) t * n + i], a);
    out[(int64_t) t * os + i] = a;
}
extern "C" int pi_op_depth_mix(const float * hist, int64_t hist_stride, int n_hist, const float * coef_dev, int n, int n_tok, float * out, int64_t out_stride, void * stream) {
    if (n_tok <= 0 || n <= 0 || n_hist <= 0) return 0;
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 4.0 * n * n_tok * (n_hist + 1.0), k_depth_mix, dim3((unsigned) ((n + 255) / 256), (unsigned) n_tok), dim3(256), 0, (hipStream_t) stream, hist, hist_stride, n_hist, coef_dev, n,
                 out, out_stride, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}

// x <- cap * tanh(x / cap) in place
__global__ void k_softcap(float * __restrict__ x, int64_t n, float cap, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    for (int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t) gridDim.x * 256) x[i] = cap * tanhf(x[i] / cap);
}
extern "C" int pi_op_softcap(float * x, int64_t n, float cap, void * stream) {
    if (n <= 0) return 0;
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 8.0 * n, k_softcap, dim3((unsigned) std::max<int64_t>(1, std::min<int64_t>(4096, (n + 255) / 256))), dim3(256), 0, (hipStream_t) stream, x, n, cap, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}

// out[t][f] = in[t][f] * in[t][ff + f]  (a gated feed-forward whose gate and up rows are one matrix; the gate's activation ran in the projection's epilogue)
__global__ void k_glu_mul(const float * __restrict__ in, int64_t is, int ff, float * __restrict__ out, int64_t os, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    const int t = blockIdx.y, f = blockIdx.x * 256 + threadIdx.x;
    if (f < ff) out[(int64_t) t * os + f] = in[(int64_t) t * is + f] * in[(int64_t) t * is + ff + f];
}
extern "C" int pi_op_glu_mul(const float * in, int64_t in_stride, int ff, int n_tok, float * out, int64_t out_stride, void * stream) {
    if (n_tok <= 0 || ff <= 0) return 0;
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 12.0 * ff * n_tok, k_glu_mul, dim3((unsigned) ((ff + 255) / 256), (unsigned) n_tok), dim3(256), 0, (hipStream_t) stream, in, in_stride, ff, out, out_stride, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}

// a gated hidden layer from its raw halves: PI_GLU_SILU silu(g) * u; PI_GLU_CLIPPED g' sigmoid(1.702 g') (u' + 1) with g' = min(g, limit), u' = clip(u, -limit, limit) (limit <= 0: no bounds)
static __device__ __forceinline__ float hy_glu(float g, float u, int glu, float limit) {
    if (glu == PI_GLU_CLIPPED) {
        if (limit > 0.0f) { g = fminf(g, limit); u = fminf(fmaxf(u, -limit), limit); }
        return g / (1.0f + expf(-1.702f * g)) * (u + 1.0f);
    }
    return glu == PI_GLU_SILU ? g / (1.0f + expf(-g)) * u : g * u;
}
__global__ void k_glu_mul_ex(const float * __restrict__ in, int64_t is, int ff, int glu, float limit, int64_t gate_col, float * __restrict__ out, int64_t os, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    const int t = blockIdx.y, f = blockIdx.x * 256 + threadIdx.x;
    if (f >= ff) return;
    const float * r = in + (int64_t) t * is;
    float y = hy_glu(r[f], r[ff + f], glu, limit);
    if (gate_col >= 0) y *= 1.0f / (1.0f + expf(-r[gate_col]));
    out[(int64_t) t * os + f] = y;
}
extern "C" int pi_op_glu_mul_ex(const float * in, int64_t in_stride, int ff, int glu, float limit, int64_t gate_col, int n_tok, float * out, int64_t out_stride, void * stream) {
    if (n_tok <= 0 || ff <= 0) return 0;
    if (glu < PI_GLU_OFF || glu > PI_GLU_CLIPPED || gate_col >= in_stride) { pi_set_error("pi_op_glu_mul_ex: hidden layer of kind %d, gate column %lld of rows %lld floats apart", glu, (long long) gate_col, (long long) in_stride); return -1; }
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 12.0 * ff * n_tok, k_glu_mul_ex, dim3((unsigned) ((ff + 255) / 256), (unsigned) n_tok), dim3(256), 0, (hipStream_t) stream, in, in_stride, ff, glu, limit, gate_col, out, out_stride, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}

// ---- rows of the stream: copies, and a layer's end with the next tanh norm --------------------------------------------------------------------------------------
__global__ void k_copy_rows(const float * __restrict__ src, int64_t ss, float * __restrict__ dst, int64_t ds, int n, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    const int t = blockIdx.y, i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[(int64_t) t * ds + i] = src[(int64_t) t * ss + i];
}
extern "C" int pi_op_copy_rows(const float * src, int64_t src_stride, float * dst, int64_t dst_stride, int n, int n_tok, void * stream) {
    if (n_tok <= 0 || n <= 0) return 0;
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 8.0 * n * n_tok, k_copy_rows, dim3((unsigned) ((n + 255) / 256), (unsigned) n_tok), dim3(256), 0, (hipStream_t) stream, src, src_stride, dst, dst_stride, n, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}
// x_out = x + a + b + c (summed in this order); h = tanh(alpha * x_out) * w + bias: no statistics, so a thread needs nobody else's values
__global__ void k_sum_tanh_norm(const float * __restrict__ x, int64_t xs, const float * __restrict__ a, int64_t as, const float * __restrict__ b, int64_t bs, const float * __restrict__ c, int64_t cs, int n,
                                float * __restrict__ xo, int64_t xos, const float * __restrict__ alpha, const float * __restrict__ w, const float * __restrict__ bias, float * __restrict__ ho, int64_t hos,
                                const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    const int t = blockIdx.y, i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float v = x[(int64_t) t * xs + i];
    if (a) v += a[(int64_t) t * as + i];
    if (b) v += b[(int64_t) t * bs + i];
    if (c) v += c[(int64_t) t * cs + i];
    if (xo) xo[(int64_t) t * xos + i] = v;
    if (w) ho[(int64_t) t * hos + i] = fmaf(tanhf(alpha[0] * v), w[i], bias ? bias[i] : 0.0f);
}
extern "C" int pi_op_sum_tanh_norm(const float * x, int64_t x_stride, const float * a, int64_t a_stride, const float * b, int64_t b_stride, const float * c, int64_t c_stride, int n, int n_tok,
                                   float * x_out, int64_t x_out_stride, const float * alpha_dev, const float * w_dev, const float * bias_dev, float * h_out, int64_t h_out_stride, void * stream) {
    if (n_tok <= 0 || n <= 0) return 0;
    if (w_dev && (!alpha_dev || !h_out)) { pi_set_error("pi_op_sum_tanh_norm: the norm needs its scalar and an output"); return -1; }
    if (!w_dev && !x_out) return 0;
    const int rows = 1 + (a != nullptr) + (b != nullptr) + (c != nullptr) + (x_out != nullptr) + (w_dev != nullptr);
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 4.0 * n * n_tok * rows, k_sum_tanh_norm, dim3((unsigned) ((n + 255) / 256), (unsigned) n_tok), dim3(256), 0, (hipStream_t) stream, x, x_stride, a, a_stride, b, b_stride, c, c_stride, n,
                 x_out, x_out_stride, alpha_dev, w_dev, bias_dev, h_out, h_out_stride, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}

// the same with the token shift of the norm's output behind it, m = h + (h_prev - h) * mu (h_prev: the sequence's previous token; pi_op_token_shift's state and slot words), for passes of at most
// 32 tokens in ONE launch: the thread of a run's first token walks the run for its column with h_prev in a register and leaves the state, so nothing it writes is read by another thread
#define STN_FRESH (1 << 30)
#define STN_WALK_MAX_TOKENS 32
__global__ void __launch_bounds__(256) k_sum_tanh_norm_walk(const float * __restrict__ x, int64_t xs, const float * __restrict__ a, int64_t as, const float * __restrict__ b, int64_t bs, const float * __restrict__ c, int64_t cs,
                                                            int n, int n_tok, float * __restrict__ xo, int64_t xos, const float * __restrict__ alpha, const float * __restrict__ w, const float * __restrict__ bias,
                                                            float * __restrict__ ho, int64_t hos, const float * __restrict__ mu, float * __restrict__ state, const int32_t * __restrict__ rec, float * __restrict__ mo,
                                                            int64_t mos, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    const int t = blockIdx.x, i = blockIdx.y * 256 + threadIdx.x;
    const int word = rec[t], slot = word & ~STN_FRESH;
    if (i >= n || (t > 0 && (rec[t - 1] & ~STN_FRESH) == slot)) return;
    const float al = alpha[0], wi = w[i], bi = bias ? bias[i] : 0.0f, mi = mu[i];
    float prev = (word & STN_FRESH) ? 0.0f : state[(int64_t) slot * n + i];
    for (int tt = t; tt < n_tok && (rec[tt] & ~STN_FRESH) == slot; tt++) {
        float v = x[(int64_t) tt * xs + i];
        if (a) v += a[(int64_t) tt * as + i];
        if (b) v += b[(int64_t) tt * bs + i];
        if (c) v += c[(int64_t) tt * cs + i];
        if (xo) xo[(int64_t) tt * xos + i] = v;
        const float h = fmaf(tanhf(al * v), wi, bi);
        ho[(int64_t) tt * hos + i] = h;
        mo[(int64_t) tt * mos + i] = fmaf(prev - h, mi, h);
        prev = h;
    }
    state[(int64_t) slot * n + i] = prev;
}
extern "C" int pi_op_sum_tanh_norm_shift(const float * x, int64_t x_stride, const float * a, int64_t a_stride, const float * b, int64_t b_stride, const float * c, int64_t c_stride, int n, int n_tok,
                                         float * x_out, int64_t x_out_stride, const float * alpha_dev, const float * w_dev, const float * bias_dev, float * h_out, int64_t h_out_stride,
                                         const float * mu_dev, float * state_dev, const int32_t * rec_dev, float * m_out, int64_t m_out_stride, void * stream) {
    if (n_tok <= 0 || n <= 0) return 0;
    if (!w_dev || !alpha_dev || !h_out || !mu_dev || !state_dev || !rec_dev || !m_out || m_out == h_out) { pi_set_error("pi_op_sum_tanh_norm_shift: the norm, the shift factors, the sequences' state and slot words and two outputs are required"); return -1; }
    if (n_tok > STN_WALK_MAX_TOKENS) {
        if (pi_op_sum_tanh_norm(x, x_stride, a, a_stride, b, b_stride, c, c_stride, n, n_tok, x_out, x_out_stride, alpha_dev, w_dev, bias_dev, h_out, h_out_stride, stream) != 0) return -1;
        return pi_op_token_shift(h_out, h_out_stride, n, mu_dev, 1, state_dev, rec_dev, n_tok, m_out, m_out_stride, stream);
    }
    const int rows = 3 + (a != nullptr) + (b != nullptr) + (c != nullptr) + (x_out != nullptr);
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 4.0 * n * n_tok * rows + 8.0 * n, k_sum_tanh_norm_walk, dim3((unsigned) n_tok, (unsigned) ((n + 255) / 256)), dim3(256), 0, (hipStream_t) stream, x, x_stride, a, a_stride, b, b_stride,
                 c, c_stride, n, n_tok, x_out, x_out_stride, alpha_dev, w_dev, bias_dev, h_out, h_out_stride, mu_dev, state_dev, rec_dev, m_out, m_out_stride, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}

// ---- linear attention with a per-head decay -------------------------------------------------------------------------------------------------------
// rec[t] = state slot of token t (| 1 << 30 on the first token of a sequence whose state starts from zero), tokens of one slot are consecutive.  Workgroup (head, column block,
// piece): thread (column j, part sp of R) keeps S[i][j] for its DPT rows i in registers and walks the piece's tokens in order.
// A pass of up to LA_TB tokens is one launch: a piece is a sequence's whole run, S comes from and goes back to HBM.  Longer passes cut every sequence's run into pieces of LA_TB
// tokens and take three launches, so that the serial depth is two pieces instead of the whole prompt (the recurrence is linear in S):
//   mode 1  every piece but a run's last: the state it would build from ZERO, L_p = sum_j lambda^(len-1-j) k_j v_j^T, into scratch
//   k_linear_state_scan  per run, piece by piece: S_in(p + 1) = lambda^len_p * S_in(p) + L_p, S_in(0) = the slot's state (or zero); scratch[p] <- S_in(p)
//   mode 2  every piece from its true S_in(p): outputs; a run's last piece leaves the slot's new state
#define LA_TB 32                                  // tokens of a piece; q, k and v of a piece are staged in LDS
#define LA_FRESH (1 << 30)
#define LA_MAXRUNS 256                            // sequences a pass may carry (the host checks)
// the first tokens of the pass's runs, in order (every thread of the block calls; bnd / nb in LDS): a thread looks at its own tokens only, one thread sorts the few it found
static __device__ __forceinline__ int la_runs(const int * recs, int n_tok, int * bnd, int * nb) {
    if (threadIdx.x == 0) *nb = 0;
    __syncthreads();
    for (int t = threadIdx.x; t < n_tok; t += blockDim.x)
        if (t == 0 || (recs[t] & ~LA_FRESH) != (recs[t - 1] & ~LA_FRESH)) { const int k = atomicAdd(nb, 1); if (k < LA_MAXRUNS) bnd[k] = t; }
    __syncthreads();
    const int n = min(*nb, LA_MAXRUNS);
    if (threadIdx.x == 0)
        for (int i = 1; i < n; i++) { const int v = bnd[i]; int j = i - 1; while (j >= 0 && bnd[j] > v) { bnd[j + 1] = bnd[j]; j--; } bnd[j + 1] = v; }
    __syncthreads();
    return n;
}
// piece number `want` of the pass (lseg = 0: pieces are whole runs): first token, length, slot word, whether it is its run's last piece
static __device__ __forceinline__ bool la_find_piece(const int * recs, int n_tok, const int * bnd, int n_runs, int lseg, int want, int & first, int & len, int & word, int & last) {
    int ord = 0;
    for (int r = 0; r < n_runs; r++) {
        const int t = bnd[r], e = r + 1 < n_runs ? bnd[r + 1] : n_tok;
        const int nsub = lseg > 0 ? (e - t + lseg - 1) / lseg : 1;
        if (want < ord + nsub) {
            const int p = want - ord;
            first = lseg > 0 ? t + p * lseg : t; len = lseg > 0 ? min(lseg, e - first) : e - t; word = recs[t]; last = p == nsub - 1;
            return true;
        }
        ord += nsub;
    }
    return false;
}
template <int DPT>
__global__ void __launch_bounds__(256) k_linear_attention(const float * __restrict__ q, const float * __restrict__ k, const float * __restrict__ v, int64_t stride, int heads, int hpg, int dim, int vdim, int R,
                                                          const float * __restrict__ decay, const float * __restrict__ tdecay, const float * __restrict__ tscale, int64_t tds, const float * __restrict__ skip,
                                                          float * __restrict__ state, const int32_t * __restrict__ rec, int n_tok, int mode, float * __restrict__ scratch,
                                                          float * __restrict__ out, int64_t os, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    extern __shared__ float lds[];                // q tile [LA_TB][dim] | k tile [LA_TB][dim] | v tile [LA_TB][cols] | the slot words of the pass [n_tok]
    __shared__ int seg[4], bnd[LA_MAXRUNS], nbnd; // seg: first token, length, slot word, last piece of its run
    __shared__ float lam_t[LA_TB], sc_t[LA_TB];   // per token of the tile: decay and the factor on k v^T
    const int h = blockIdx.x, tid = threadIdx.x;
    int * recs = (int *) (lds + 2 * LA_TB * dim + LA_TB * (blockDim.x / R));
    for (int t = tid; t < n_tok; t += blockDim.x) recs[t] = rec[t];
    __syncthreads();
    const int n_runs = la_runs(recs, n_tok, bnd, &nbnd);
    if (tid == 0) {
        int first = 0, len = 0, word = -1, last = 1;
        if (!la_find_piece(recs, n_tok, bnd, n_runs, mode ? LA_TB : 0, blockIdx.z, first, len, word, last)) len = 0;
        seg[0] = first; seg[1] = len; seg[2] = word; seg[3] = last;
    }
    __syncthreads();
    const int first = seg[0], len = seg[1], word = seg[2], last = seg[3];
    if (len == 0 || word < 0 || (mode == 1 && last)) return;
    const int slot = word & ~LA_FRESH;
    const int cols = blockDim.x / R;
    const int j = blockIdx.y * cols + tid / R, sp = tid % R;
    const bool col_ok = j < vdim;
    const float lam = decay ? decay[h] : 1.0f, skp = skip ? skip[h] : 0.0f;
    const int hq = h / hpg;                                            // the q / k head this head reads (hpg heads share one)
    float * S_hbm = state + ((int64_t) slot * heads + h) * dim * vdim;
    float * S_scr = scratch ? scratch + ((int64_t) blockIdx.z * heads + h) * dim * vdim : nullptr;
    const float * S_from = mode == 2 ? S_scr : mode == 1 || (word & LA_FRESH) ? nullptr : S_hbm;
    float S[DPT];
#pragma unroll
    for (int ii = 0; ii < DPT; ii++) {
        const int i = sp * DPT + ii;
        S[ii] = (col_ok && i < dim && S_from) ? S_from[(int64_t) i * vdim + j] : 0.0f;
    }
    float * qt = lds, * kt = lds + LA_TB * dim, * vt = kt + LA_TB * dim;
    const bool dim4 = (dim & 3) == 0;
    for (int t0 = 0; t0 < len; t0 += LA_TB) {
        const int nt = min(LA_TB, len - t0);
        __syncthreads();
        for (int idx = tid; idx < nt * dim; idx += blockDim.x) {
            const int tt = idx / dim, i = idx % dim;
            const int64_t off = (int64_t) (first + t0 + tt) * stride + (int64_t) hq * dim + i;
            if (mode != 1) qt[idx] = q[off];
            kt[idx] = k[off];
        }
        if (tid < nt) {
            lam_t[tid] = tdecay ? tdecay[(int64_t) (first + t0 + tid) * tds + h] : lam;
            sc_t[tid] = tscale ? tscale[(int64_t) (first + t0 + tid) * tds + h] : 1.0f;
        }
        for (int idx = tid; idx < nt * cols; idx += blockDim.x) {
            const int tt = idx / cols, jj = blockIdx.y * cols + idx % cols;
            vt[idx] = jj < vdim ? v[(int64_t) (first + t0 + tt) * stride + (int64_t) h * vdim + jj] : 0.0f;
        }
        __syncthreads();
        if (mode == 1) {                                              // the state only
            for (int tt = 0; tt < nt; tt++) {
                const float vj = vt[tt * cols + tid / R] * sc_t[tt], lam = lam_t[tt];
                const float * kr = kt + tt * dim + sp * DPT;
#pragma unroll
                for (int ii = 0; ii < DPT; ii++) if (sp * DPT + ii < dim) S[ii] = fmaf(kr[ii], vj, lam * S[ii]);
            }
            continue;
        }
        for (int tt = 0; tt < nt; tt++) {
            const float vraw = vt[tt * cols + tid / R], vj = vraw * sc_t[tt], lam = lam_t[tt];
            const float * kr = kt + tt * dim + sp * DPT, * qr = qt + tt * dim + sp * DPT;
            float o = 0.0f;
            if (dim4) {
#pragma unroll
                for (int ii = 0; ii < DPT; ii += 4) {
                    if (sp * DPT + ii < dim) {
                        const float4 kv = *(const float4 *) (kr + ii), qv = *(const float4 *) (qr + ii);
                        S[ii] = fmaf(kv.x, vj, lam * S[ii]);         o = fmaf(S[ii], qv.x, o);
                        S[ii + 1] = fmaf(kv.y, vj, lam * S[ii + 1]); o = fmaf(S[ii + 1], qv.y, o);
                        S[ii + 2] = fmaf(kv.z, vj, lam * S[ii + 2]); o = fmaf(S[ii + 2], qv.z, o);
                        S[ii + 3] = fmaf(kv.w, vj, lam * S[ii + 3]); o = fmaf(S[ii + 3], qv.w, o);
                    }
                }
            } else {
#pragma unroll
                for (int ii = 0; ii < DPT; ii++)
                    if (sp * DPT + ii < dim) { S[ii] = fmaf(kr[ii], vj, lam * S[ii]); o = fmaf(S[ii], qr[ii], o); }
            }
            if (R == 2) o += pi_partner<1>(o);
            else if (R == 4) { o += pi_partner<2>(o); o += pi_partner<1>(o); }
            else for (int d = R >> 1; d > 0; d >>= 1) o += __shfl_xor(o, d, PI_WAVE);
            if (col_ok && sp == 0) out[(int64_t) (first + t0 + tt) * os + (int64_t) h * vdim + j] = fmaf(skp, vraw, o);
        }
    }
    float * S_to = mode == 1 ? S_scr : last ? S_hbm : nullptr;
    if (col_ok && S_to)
#pragma unroll
        for (int ii = 0; ii < DPT; ii++) { const int i = sp * DPT + ii; if (i < dim) S_to[(int64_t) i * vdim + j] = S[ii]; }
}

// grid (head, blocks over dim * vdim, run): scratch[piece] holds L_p coming in and S_in(p) going out
__global__ void __launch_bounds__(256) k_linear_state_scan(int heads, int dim, int vdim, const float * __restrict__ decay, const float * __restrict__ tdecay, int64_t tds, const float * __restrict__ state,
                                                           const int32_t * __restrict__ rec, int n_tok, float * __restrict__ scratch, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    __shared__ int seg[4], bnd[LA_MAXRUNS], nbnd; // seg: slot word, first piece ordinal, pieces of the run (0: no such run), the run's first token
    extern __shared__ int recs[];                 // the slot words of the pass
    for (int t = threadIdx.x; t < n_tok; t += 256) recs[t] = rec[t];
    __syncthreads();
    const int n_runs = la_runs(recs, n_tok, bnd, &nbnd);
    if (threadIdx.x == 0) {
        int ord = 0, nsub = 0, word = -1, sub0 = 0, tfirst = 0;
        for (int r = 0; r < n_runs; r++) {
            const int t = bnd[r], e = r + 1 < n_runs ? bnd[r + 1] : n_tok;
            const int ns = (e - t + LA_TB - 1) / LA_TB;
            if (r == (int) blockIdx.z) { nsub = ns; word = recs[t]; sub0 = ord; tfirst = t; break; }
            ord += ns;
        }
        seg[0] = word; seg[1] = sub0; seg[2] = nsub; seg[3] = tfirst;
    }
    __syncthreads();
    const int word = seg[0], sub0 = seg[1], nsub = seg[2], tfirst = seg[3];
    if (nsub == 0 || word < 0) return;
    const int h = blockIdx.x, slot = word & ~LA_FRESH;
    const int64_t per = (int64_t) dim * vdim, idx = (int64_t) blockIdx.y * 256 + threadIdx.x;
    if (idx >= per) return;
    float lp = 1.0f;                                                   // lambda^LA_TB: every piece but a run's last has LA_TB tokens
    if (!tdecay) for (int i = 0; i < LA_TB; i++) lp *= decay[h];
    float run = (word & LA_FRESH) ? 0.0f : state[((int64_t) slot * heads + h) * per + idx];
    for (int p0 = 0; p0 < nsub; p0 += 8) {                             // eight pieces at a time: their loads are in flight together, then the chain runs on registers
        float lpart[8];
#pragma unroll
        for (int i = 0; i < 8; i++) lpart[i] = p0 + i < nsub - 1 ? scratch[((int64_t) (sub0 + p0 + i) * heads + h) * per + idx] : 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++)
            if (p0 + i < nsub) {
                scratch[((int64_t) (sub0 + p0 + i) * heads + h) * per + idx] = run;
                if (tdecay && p0 + i < nsub - 1) {                     // per-token decays: the product over the piece's tokens
                    lp = 1.0f;
                    const float * td = tdecay + (int64_t) (tfirst + (p0 + i) * LA_TB) * tds + h;
                    for (int j = 0; j < LA_TB; j++) lp *= td[(int64_t) j * tds];
                }
                run = fmaf(lp, run, lpart[i]);
            }
    }
}

// once per process, outside graph capture: the tiles of wide keys (q, k of 32 tokens) need more dynamic LDS than a kernel gets by default
#define LA_LDS_MAX (150 * 1024)
extern "C" int pi_op_linear_attention_reserve(void) {
    static bool done = false;
    if (done) return 0;
    PI_CHECK_HIP(hipFuncSetAttribute((const void *) k_linear_attention<8>, hipFuncAttributeMaxDynamicSharedMemorySize, LA_LDS_MAX));
    PI_CHECK_HIP(hipFuncSetAttribute((const void *) k_linear_attention<16>, hipFuncAttributeMaxDynamicSharedMemorySize, LA_LDS_MAX));
    PI_CHECK_HIP(hipFuncSetAttribute((const void *) k_linear_attention<32>, hipFuncAttributeMaxDynamicSharedMemorySize, LA_LDS_MAX));
    done = true;
    return 0;
}
static int la_max_pieces(int n_tok, int max_segments) { return n_tok / LA_TB + std::min(n_tok, std::max(1, max_segments)) + 1; }
extern "C" size_t pi_op_linear_attention_scratch_floats(int heads, int dim, int vdim, int n_tok, int max_segments) {
    return n_tok <= LA_TB ? 0 : (size_t) la_max_pieces(n_tok, max_segments) * heads * dim * vdim;
}
extern "C" int pi_op_linear_attention(const float * q, const float * k, const float * v, int64_t stride, int heads, int dim, int vdim, const float * decay_dev, float * state_dev,
                                      const int32_t * rec_dev, int n_tok, int max_segments, float * scratch_dev, size_t scratch_floats, float * out, int64_t out_stride, void * stream) {
    return pi_op_linear_attention_ex(q, k, v, stride, heads, heads, dim, vdim, decay_dev, nullptr, nullptr, 0, nullptr, state_dev, rec_dev, n_tok, max_segments, scratch_dev, scratch_floats, out, out_stride, stream);
}
extern "C" int pi_op_linear_attention_ex(const float * q, const float * k, const float * v, int64_t stride, int heads, int qk_heads, int dim, int vdim, const float * decay_dev, const float * tdecay_dev,
                                         const float * tscale_dev, int64_t t_stride, const float * skip_dev, float * state_dev, const int32_t * rec_dev, int n_tok, int max_segments, float * scratch_dev,
                                         size_t scratch_floats, float * out, int64_t out_stride, void * stream) {
    if (n_tok <= 0) return 0;
    if (qk_heads < 1 || heads % qk_heads) { pi_set_error("pi_op_linear_attention: %d heads do not divide over %d query / key heads", heads, qk_heads); return -1; }
    if (!decay_dev && !tdecay_dev) { pi_set_error("pi_op_linear_attention: neither per-head nor per-token decays were given"); return -1; }
    const int hpg = heads / qk_heads;
    if (dim <= 0 || vdim <= 0 || heads <= 0 || dim > 1024) { pi_set_error("pi_op_linear_attention: head sizes %d x %d outside the kernel's range (key width <= 1024)", dim, vdim); return -1; }
    if (max_segments > LA_MAXRUNS) { pi_set_error("pi_op_linear_attention: at most %d sequences in a pass", LA_MAXRUNS); return -1; }
    const int dpt = dim <= 8 ? 8 : dim <= 16 ? 16 : 32;                // state values a thread keeps in registers (more would spill in the token loop)
    int R = 1; while (R * dpt < dim) R *= 2;
    int threads = std::min(256, (vdim * R + 63) / 64 * 64);
    const int cols = threads / R;
    const bool pieces = n_tok > LA_TB;
    if (pieces && (!scratch_dev || scratch_floats < pi_op_linear_attention_scratch_floats(heads, dim, vdim, n_tok, max_segments))) { pi_set_error("pi_op_linear_attention: a pass of %d tokens needs %zu floats of scratch", n_tok, pi_op_linear_attention_scratch_floats(heads, dim, vdim, n_tok, max_segments)); return -1; }
    const unsigned gz = pieces ? (unsigned) la_max_pieces(n_tok, max_segments) : (unsigned) std::max(1, std::min(n_tok, max_segments));
    const dim3 grid((unsigned) heads, (unsigned) ((vdim + cols - 1) / cols), gz);
    const size_t lds = ((size_t) 2 * LA_TB * dim + (size_t) LA_TB * cols + (size_t) n_tok) * sizeof(float);
    if (lds > LA_LDS_MAX) { pi_set_error("pi_op_linear_attention: a key width of %d with %d tokens in the pass needs %zu bytes of LDS (at most %d)", dim, n_tok, lds, LA_LDS_MAX); return -1; }
    if (lds > 48 * 1024 && pi_op_linear_attention_reserve() != 0) return -1;
    const double bytes = 4.0 * n_tok * heads * (2.0 * dim + 2.0 * vdim) + 8.0 * heads * dim * vdim;
    hipStream_t s = (hipStream_t) stream;
    const int nta = std::min(n_tok, PI_KT_MAXNT - 1);
#define LA_GO(D, MODE) PI_KT_LAUNCH(PI_KT_ATT, 0, nta, bytes, k_linear_attention<D>, grid, dim3(threads), lds, s, q, k, v, stride, heads, hpg, dim, vdim, R, decay_dev, tdecay_dev, tscale_dev, t_stride, skip_dev, state_dev, rec_dev, n_tok, MODE, scratch_dev, out, out_stride, pi_abort_word())
#define LA_ANY(MODE) do { if (dpt == 8) LA_GO(8, MODE); else if (dpt == 16) LA_GO(16, MODE); else LA_GO(32, MODE); } while (0)
    if (!pieces) { LA_ANY(0); PI_CHECK_LAUNCH(); return 0; }
    LA_ANY(1);
    PI_CHECK_LAUNCH();
    PI_KT_LAUNCH(PI_KT_ATT, 0, nta, 12.0 * gz * heads * dim * vdim, k_linear_state_scan, dim3((unsigned) heads, (unsigned) (((int64_t) dim * vdim + 255) / 256), (unsigned) std::max(1, std::min(n_tok, max_segments))), dim3(256), (size_t) 4 * n_tok, s,
                 heads, dim, vdim, decay_dev, tdecay_dev, t_stride, state_dev, rec_dev, n_tok, scratch_dev, pi_abort_word());
    PI_CHECK_LAUNCH();
    LA_ANY(2);
#undef LA_ANY
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
// Three launches.  (1) k_latent_absorb folds the key up-projection and the score scale into the query: qa[t][h][:] = scale * W_uk[h]^T q[t][h] (rank values per head).
// (2) k_latent_scores, grid (token, head tile of M heads, split of the cell range): a thread owns a cell in the score phase — its latent row streams through registers once and
// feeds M accumulators, the M queries come through wave-uniform (scalar) loads — and a slice of the latent's rank in the value phase, where the probabilities of a cell are
// broadcast from LDS to M x RPT accumulators; every split leaves an un-normalised partial (max, sum, sum of p * c) in scratch.  (3) k_latent_combine merges the splits with
// the sink term, normalises and applies the value up-projection.  K / V are never materialised; single tokens are spread over the chip by the splits (64 cells each),
// prompts take splits only when a score row would not fit LDS.
// scratch (floats): qa [n_tok][heads][rank] | pol [n_tok][heads][S][rank] | pml [n_tok][heads][S][2]
#define LAT_LDS_BUDGET (128 * 1024)
struct lat_plan { int M, RPT, cap, S; size_t lds, scratch; };
static lat_plan latent_plan(int heads, int rank, int n_tok, int n_ctx) {
    lat_plan p;
    const bool single = n_tok <= 8;
    int best = 1;                                                     // heads per workgroup: the largest tile that leaves at most a quarter of its accumulator rows idle
    for (int m : { 2, 4, 8, 16 }) { if (single && m > 4) break; if (3 * ((heads + m - 1) / m * m) <= 4 * heads) best = m; }
    p.M = best;
    p.RPT = rank > 512 ? 4 : rank > 256 ? 2 : 1;
    const int rthreads = (rank + p.RPT - 1) / p.RPT, G = std::max(1, 256 / rthreads);
    const int cap_max = std::max(64, (int) (((LAT_LDS_BUDGET / 4 - (size_t) G * p.M * rank - 256 * p.M) / p.M) / 64 * 64));
    p.cap = single ? 64 : std::min(cap_max, 2048);
    p.cap = std::min(p.cap, (n_ctx + 63) / 64 * 64);
    p.S = (n_ctx + p.cap - 1) / p.cap;
    p.lds = ((size_t) p.cap * p.M + (size_t) G * p.M * rank + 8 * p.M + 8 + 256 * p.M) * 4;
    p.scratch = (size_t) n_tok * heads * rank * (1 + p.S) + (size_t) n_tok * heads * p.S * 2;
    return p;
}

// grid (token tile of 4, head, 64 values of the rank): lane = one rank value, the four waves take a quarter of the head's dim each and meet in LDS
__global__ void __launch_bounds__(256) k_latent_absorb(const float * __restrict__ q, int64_t qs, const uint16_t * __restrict__ wuk, float scale, int heads, int dim, int rank, int n_tok,
                                                       float * __restrict__ qa, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w, 5)) return;
    __shared__ float part[4][4][64];
    extern __shared__ float4 qsh[];                                    // [dim]: the head's query values of the four tokens, side by side
    const int t0 = blockIdx.x * 4, h = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = blockIdx.z * 64 + lane;
    for (int idx = threadIdx.x; idx < 4 * dim; idx += 256) {
        const int tt = idx / dim, d = idx % dim;
        ((float *) qsh)[d * 4 + tt] = q[(int64_t) min(t0 + tt, n_tok - 1) * qs + (int64_t) h * dim + d];
    }
    __syncthreads();
    const int dq = (dim + 3) / 4, d0 = wave * dq, d1 = min(dim, d0 + dq);
    float acc[4] = { 0.0f, 0.0f, 0.0f, 0.0f };
    const uint16_t * w = wuk + (int64_t) h * dim * rank + min(r, rank - 1);
#pragma unroll 8
    for (int d = d0; d < d1; d++) {
        const float wv = hy_widen(w[(int64_t) d * rank]);
        const float4 qv = qsh[d];
        acc[0] = fmaf(qv.x, wv, acc[0]); acc[1] = fmaf(qv.y, wv, acc[1]); acc[2] = fmaf(qv.z, wv, acc[2]); acc[3] = fmaf(qv.w, wv, acc[3]);
    }
#pragma unroll
    for (int tt = 0; tt < 4; tt++) part[wave][tt][lane] = acc[tt];
    __syncthreads();
    const int tt = wave;                                              // wave tt writes token t0 + tt
    if (t0 + tt < n_tok && r < rank) qa[((int64_t) (t0 + tt) * heads + h) * rank + r] = (part[0][tt][lane] + part[1][tt][lane] + part[2][tt][lane] + part[3][tt][lane]) * scale;
}

template <int M, int RPT>
__global__ void __launch_bounds__(256) k_latent_scores(const float * __restrict__ qa, const float * __restrict__ cache, const uint32_t * __restrict__ mask, int heads, int rank, int n_kv_arg,
                                                       int cap, int S, float * __restrict__ pol, float * __restrict__ pml, const int32_t * __restrict__ dyn, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w, 5)) return;
    extern __shared__ float lds[];
    const int t = blockIdx.x, h0 = blockIdx.y * M, split = blockIdx.z, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int rthreads = (rank + RPT - 1) / RPT, G = max(1, 256 / rthreads);
    float * sc = lds, * part = sc + (size_t) cap * M, * red = part + (size_t) G * M * rank, * wsc = red + 8 * M + 8;     // red: [4 waves][M] twice; wsc: [4 waves][64 cells][M]
    __shared__ int hi_s;
    const int n_kv = min(dyn ? dyn[1] : n_kv_arg, n_kv_arg);
    const int words = (n_kv_arg + 31) / 32;
    const uint32_t * mrow = mask + (int64_t) t * words;
    const int c0 = split * cap;
    int c1 = min(n_kv, c0 + cap);
    if (tid == 0) hi_s = 0;
    __syncthreads();
    {   // cells past the last visible one of this token are not walked (a prompt's early tokens see little of the pass's cells)
        int hi = 0;
        for (int w = (c0 >> 5) + tid; w < (c1 + 31) >> 5; w += 256) { const uint32_t bits = mrow[w]; if (bits) hi = max(hi, w * 32 + 32 - __clz(bits)); }
        if (hi) atomicMax(&hi_s, hi);
    }
    __syncthreads();
    c1 = min(c1, hi_s);
    const int nh = min(M, heads - h0);
    const float * qat = qa + ((int64_t) t * heads + h0) * rank;
    float * pol_t = pol + (((int64_t) t * heads + h0) * S + split) * rank, * pml_t = pml + (((int64_t) t * heads + h0) * S + split) * 2;
    if (c1 <= c0) {                                                   // nothing of this token lives in this split: an empty partial
        for (int m = 0; m < nh; m++) {
            for (int r = tid; r < rank; r += 256) pol_t[(int64_t) m * S * rank + r] = 0.0f;
            if (tid == 0) { pml_t[(int64_t) m * S * 2] = -INFINITY; pml_t[(int64_t) m * S * 2 + 1] = 0.0f; }
        }
        return;
    }
    // scores: a thread per cell; a split of 64 cells (single tokens) gives every wave a quarter of the rank instead, so that all four waves stream the 64 latents
    float lmax[M];
#pragma unroll
    for (int m = 0; m < M; m++) lmax[m] = -INFINITY;
    if (cap == 64 && (rank & 15) == 0) {
        const int j = c0 + lane, rq = rank >> 2, rb = wave * rq;
        const bool vis = j < c1 && ((mrow[j >> 5] >> (j & 31)) & 1u);
        float a[M];
#pragma unroll
        for (int m = 0; m < M; m++) a[m] = 0.0f;
        if (vis) {
            const float * c = cache + (int64_t) j * rank + rb;
#pragma unroll 8
            for (int r = 0; r < rq; r += 4) {
                const float4 cv = *(const float4 *) (c + r);
#pragma unroll
                for (int m = 0; m < M; m++) {
                    const float * qq = qat + (m < nh ? m : 0) * rank + rb + r;                    // (wave-uniform address)
                    a[m] = fmaf(qq[0], cv.x, a[m]); a[m] = fmaf(qq[1], cv.y, a[m]); a[m] = fmaf(qq[2], cv.z, a[m]); a[m] = fmaf(qq[3], cv.w, a[m]);
                }
            }
        }
#pragma unroll
        for (int m = 0; m < M; m++) wsc[((size_t) wave * 64 + lane) * M + m] = a[m];
        __syncthreads();
        if (wave == 0 && j < c1) {
#pragma unroll
            for (int m = 0; m < M; m++) {
                const float sv = vis ? wsc[(size_t) lane * M + m] + wsc[((size_t) 64 + lane) * M + m] + wsc[((size_t) 128 + lane) * M + m] + wsc[((size_t) 192 + lane) * M + m] : -INFINITY;
                sc[(size_t) lane * M + m] = sv; lmax[m] = sv;
            }
        }
        __syncthreads();
    } else
    for (int j = c0 + tid; j < c1; j += 256) {
        const bool vis = (mrow[j >> 5] >> (j & 31)) & 1u;
        float a[M];
#pragma unroll
        for (int m = 0; m < M; m++) a[m] = 0.0f;
        if (vis) {
            const float * c = cache + (int64_t) j * rank;
            if ((rank & 3) == 0) {
#pragma unroll 2
                for (int r = 0; r < rank; r += 4) {
                    const float4 cv = *(const float4 *) (c + r);
#pragma unroll
                    for (int m = 0; m < M; m++) {
                        const float * qq = qat + (m < nh ? m : 0) * rank + r;                     // (wave-uniform address)
                        a[m] = fmaf(qq[0], cv.x, a[m]); a[m] = fmaf(qq[1], cv.y, a[m]); a[m] = fmaf(qq[2], cv.z, a[m]); a[m] = fmaf(qq[3], cv.w, a[m]);
                    }
                }
            } else {
                for (int r = 0; r < rank; r++) {
                    const float cv = c[r];
#pragma unroll
                    for (int m = 0; m < M; m++) a[m] = fmaf(qat[(m < nh ? m : 0) * rank + r], cv, a[m]);
                }
            }
        }
#pragma unroll
        for (int m = 0; m < M; m++) { const float sv = vis ? a[m] : -INFINITY; sc[(size_t) (j - c0) * M + m] = sv; lmax[m] = fmaxf(lmax[m], sv); }
    }
    // per head: max over the split, then p = exp(s - max) and its sum (every thread revisits its own cells)
#pragma unroll
    for (int m = 0; m < M; m++) { const float v = pi_wave_max(lmax[m]); if (lane == 0) red[wave * M + m] = v; }
    __syncthreads();
    float mx[M], lsum[M];
#pragma unroll
    for (int m = 0; m < M; m++) { mx[m] = fmaxf(fmaxf(red[m], red[M + m]), fmaxf(red[2 * M + m], red[3 * M + m])); lsum[m] = 0.0f; }
    for (int j = c0 + tid; j < c1; j += 256)
#pragma unroll
        for (int m = 0; m < M; m++) {
            const float sv = sc[(size_t) (j - c0) * M + m];
            const float pv = sv == -INFINITY ? 0.0f : expf(sv - mx[m]);
            sc[(size_t) (j - c0) * M + m] = pv; lsum[m] += pv;
        }
    float * red2 = red + 4 * M;
#pragma unroll
    for (int m = 0; m < M; m++) { const float v = pi_lanes_sum<64>(lsum[m]); if (lane == 0) red2[wave * M + m] = v; }
    __syncthreads();
    if (tid < nh) {
        pml_t[(int64_t) tid * S * 2] = fmaxf(fmaxf(red[tid], red[M + tid]), fmaxf(red[2 * M + tid], red[3 * M + tid]));
        pml_t[(int64_t) tid * S * 2 + 1] = red2[tid] + red2[M + tid] + red2[2 * M + tid] + red2[3 * M + tid];
    }
    // sum of p * c: thread (cell group g, rank slice rt)
    const int g = tid / rthreads, rt = tid % rthreads, r0 = rt * RPT;
    float o[M][RPT];
#pragma unroll
    for (int m = 0; m < M; m++)
#pragma unroll
        for (int i = 0; i < RPT; i++) o[m][i] = 0.0f;
    if (g < G) {
#pragma unroll 8
        for (int j = c0 + g; j < c1; j += G) {                          // (a masked cell has p = 0: its latent — zeros or an earlier owner's finite values — adds nothing)
            float cv[RPT];
#pragma unroll
            for (int i = 0; i < RPT; i++) cv[i] = r0 + i < rank ? cache[(int64_t) j * rank + r0 + i] : 0.0f;
            const float * pj = sc + (size_t) (j - c0) * M;
#pragma unroll
            for (int m = 0; m < M; m++) {
                const float pv = pj[m];
#pragma unroll
                for (int i = 0; i < RPT; i++) o[m][i] = fmaf(pv, cv[i], o[m][i]);
            }
        }
        if (G > 1)
#pragma unroll
            for (int m = 0; m < M; m++)
#pragma unroll
                for (int i = 0; i < RPT; i++) if (r0 + i < rank) part[((size_t) g * M + m) * rank + r0 + i] = o[m][i];
    }
    if (G > 1) {
        __syncthreads();
        for (int idx = tid; idx < nh * rank; idx += 256) {
            const int m = idx / rank, r = idx % rank;
            float v = 0.0f;
            for (int gg = 0; gg < G; gg++) v += part[((size_t) gg * M + m) * rank + r];
            pol_t[(int64_t) m * S * rank + r] = v;
        }
    } else if (g == 0) {
#pragma unroll
        for (int m = 0; m < M; m++)
            if (m < nh)
#pragma unroll
                for (int i = 0; i < RPT; i++) if (r0 + i < rank) pol_t[(int64_t) m * S * rank + r0 + i] = o[m][i];
    }
}

// grid (token tile of 4, head, 16 output values): merges the splits (with the sink), normalises, applies its rows of W_uv[h]
__global__ void __launch_bounds__(256) k_latent_combine(const float * __restrict__ pol, const float * __restrict__ pml, const uint16_t * __restrict__ wuv, const float * __restrict__ sink,
                                                        int heads, int vdim, int rank, int S, int n_tok, float * __restrict__ out, int64_t os, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w, 5)) return;
    extern __shared__ float ol[];                                     // [4][rank]
    __shared__ float wgt[4][64 + 1];                                  // per token: weight of every split (S <= 64 at a time), [64]: 1 / denominator
    const int t0 = blockIdx.x * 4, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nt = min(4, n_tok - t0);
    for (int idx = tid; idx < 4 * rank; idx += 256) ol[idx] = 0.0f;
    // (the wave `tt` owns token t0 + tt's bookkeeping)
    float mstar = -INFINITY, den = 0.0f;
    const float sk = sink[h];
    const float * pml_t = pml + ((int64_t) (t0 + min(wave, nt - 1)) * heads + h) * S * 2;
    {
        float m = sk;
        for (int s = lane; s < S; s += 64) m = fmaxf(m, pml_t[s * 2]);
        mstar = pi_wave_max(m);
        float d = 0.0f;
        for (int s = lane; s < S; s += 64) { const float ms = pml_t[s * 2]; if (ms != -INFINITY) d += pml_t[s * 2 + 1] * expf(ms - mstar); }
        den = pi_lanes_sum<64>(d) + expf(sk - mstar);
    }
    for (int sb = 0; sb < S; sb += 64) {
        __syncthreads();
        if (wave < nt) {
            const int s = sb + lane;
            const float ms = s < S ? pml_t[s * 2] : -INFINITY;
            wgt[wave][lane] = ms == -INFINITY ? 0.0f : expf(ms - mstar) / den;
        }
        __syncthreads();
        for (int idx = tid; idx < nt * rank; idx += 256) {
            const int tt = idx / rank, r = idx % rank;
            const float * p = pol + (((int64_t) (t0 + tt) * heads + h) * S + sb) * rank + r;
            float v = ol[idx];
#pragma unroll 8
            for (int s = 0; s < min(64, S - sb); s++) v = fmaf(wgt[tt][s], p[(int64_t) s * rank], v);                 // (an empty split: weight 0, partial written as zeros)
            ol[idx] = v;
        }
    }
    __syncthreads();
    for (int vv = blockIdx.z * 16 + wave; vv < min(vdim, (int) blockIdx.z * 16 + 16); vv += 4) {
        const uint16_t * wv = wuv + ((int64_t) h * vdim + vv) * rank;
        float a[4] = { 0.0f, 0.0f, 0.0f, 0.0f };
#pragma unroll 4
        for (int r = lane; r < rank; r += 64) {
            const float w = hy_widen(wv[r]);
#pragma unroll
            for (int tt = 0; tt < 4; tt++) a[tt] = fmaf(w, ol[tt * rank + r], a[tt]);
        }
#pragma unroll
        for (int tt = 0; tt < 4; tt++) { const float v = pi_lanes_sum<64>(a[tt]); if (lane == 0 && tt < nt) out[(int64_t) (t0 + tt) * os + (int64_t) h * vdim + vv] = v; }
    }
}

extern "C" int pi_op_latent_attention_max_cells(int rank) { (void) rank; return 1 << 22; }       // (long contexts are cut into splits: no score row has to fit LDS whole)
extern "C" size_t pi_op_latent_attention_scratch_floats(int heads, int rank, int n_tok, int n_ctx) {
    return std::max(latent_plan(heads, rank, n_tok, n_ctx).scratch, latent_plan(heads, rank, std::min(n_tok, 8), n_ctx).scratch);
}
template <int M, int RPT> static int latent_reserve_one() {
    PI_CHECK_HIP(hipFuncSetAttribute((const void *) k_latent_scores<M, RPT>, hipFuncAttributeMaxDynamicSharedMemorySize, LAT_LDS_BUDGET + 4096));
    return 0;
}
extern "C" int pi_op_latent_attention_reserve(void) {
    static bool done = false;
    if (done) return 0;
#define LAT_RES(M) if (latent_reserve_one<M, 1>() || latent_reserve_one<M, 2>() || latent_reserve_one<M, 4>()) return -1;
    LAT_RES(1) LAT_RES(2) LAT_RES(4) LAT_RES(8) LAT_RES(16)
#undef LAT_RES
    done = true;
    return 0;
}
template <int M, int RPT>
static void latent_scores_launch(const lat_plan & p, dim3 grid, hipStream_t s, double bytes, int nta, const float * qa, const float * cache, const uint32_t * mask, int heads, int rank, int n_kv,
                                 float * pol, float * pml, const int32_t * dyn) {
    PI_KT_LAUNCH(PI_KT_ATT, PI_BF16, nta, bytes, (k_latent_scores<M, RPT>), grid, dim3(256), p.lds, s, qa, cache, mask, heads, rank, n_kv, p.cap, p.S, pol, pml, dyn, pi_abort_word());
}
extern "C" int pi_op_latent_attention(const float * q, int64_t q_stride, const float * cache, const uint32_t * mask, const pi_weight * wuk, const pi_weight * wuv, const float * sink_dev,
                                      float scale, int heads, int dim, int vdim, int rank, int n_tok, int n_kv, float * scratch_dev, size_t scratch_floats, float * out, int64_t out_stride,
                                      const int32_t * dyn_dev, void * stream) {
    if (n_tok <= 0) return 0;
    if (!wuk || !wuv || wuk->type != PI_BF16 || wuv->type != PI_BF16 || wuk->ne0 != rank || wuv->ne0 != rank || wuk->ne1 != (int64_t) heads * dim || wuv->ne1 != (int64_t) heads * vdim) {
        pi_set_error("pi_op_latent_attention: the up-projections must be bfloat16 [heads * dim][rank] and [heads * vdim][rank]"); return -1;
    }
    if (rank > 1024) { pi_set_error("pi_op_latent_attention: latent width %d above 1024", rank); return -1; }
    const lat_plan p = latent_plan(heads, rank, n_tok, n_kv);
    if (p.scratch > scratch_floats) { pi_set_error("pi_op_latent_attention: %zu floats of scratch needed, %zu given", p.scratch, scratch_floats); return -1; }
    if (p.lds > LAT_LDS_BUDGET + 4096 || (size_t) 4 * rank * 4 > 64 * 1024) { pi_set_error("pi_op_latent_attention: LDS plan does not fit"); return -1; }
    if (pi_op_latent_attention_reserve() != 0) return -1;
    hipStream_t s = (hipStream_t) stream;
    float * qa = scratch_dev, * pol = qa + (size_t) n_tok * heads * rank, * pml = pol + (size_t) n_tok * heads * p.S * rank;
    const int nta = std::min(n_tok, PI_KT_MAXNT - 1);
    const int acct = pi_account_n_kv() > 0 ? pi_account_n_kv() : n_kv;
    PI_KT_LAUNCH(PI_KT_ATT, PI_BF16, nta, 2.0 * rank * heads * dim + 4.0 * n_tok * heads * (dim + rank), k_latent_absorb, dim3((unsigned) ((n_tok + 3) / 4), (unsigned) heads, (unsigned) ((rank + 63) / 64)), dim3(256), (size_t) 16 * dim, s,
                 q, q_stride, (const uint16_t *) wuk->p0, scale, heads, dim, rank, n_tok, qa, pi_abort_word());
    PI_CHECK_LAUNCH();
    const dim3 grid((unsigned) n_tok, (unsigned) ((heads + p.M - 1) / p.M), (unsigned) p.S);
    const double bytes = 4.0 * acct * rank + 4.0 * n_tok * heads * rank * (1.0 + p.S);
#define LAT_GO(M) do { if (p.RPT == 1) latent_scores_launch<M, 1>(p, grid, s, bytes, nta, qa, cache, mask, heads, rank, n_kv, pol, pml, dyn_dev); \
                       else if (p.RPT == 2) latent_scores_launch<M, 2>(p, grid, s, bytes, nta, qa, cache, mask, heads, rank, n_kv, pol, pml, dyn_dev); \
                       else latent_scores_launch<M, 4>(p, grid, s, bytes, nta, qa, cache, mask, heads, rank, n_kv, pol, pml, dyn_dev); } while (0)
    switch (p.M) { case 16: LAT_GO(16); break; case 8: LAT_GO(8); break; case 4: LAT_GO(4); break; case 2: LAT_GO(2); break; default: LAT_GO(1); }
#undef LAT_GO
    PI_CHECK_LAUNCH();
    PI_KT_LAUNCH(PI_KT_ATT, PI_BF16, nta, 2.0 * rank * heads * vdim + 4.0 * n_tok * heads * (rank * p.S + vdim), k_latent_combine, dim3((unsigned) ((n_tok + 3) / 4), (unsigned) heads, (unsigned) ((vdim + 15) / 16)), dim3(256), (size_t) 16 * rank, s,
                 pol, pml, (const uint16_t *) wuv->p0, sink_dev, heads, vdim, rank, p.S, n_tok, out, out_stride, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}

// ---- routed feed-forward ------------------------------------------------------------------------------------------------------------------------------
// one workgroup per token: logits of all router outputs (a wave per output), soft-max, choice = score + correction, `top` rounds of arg-max (lowest index wins a tie)
// n_groups > 0: the scores are sigmoid(logit), consecutive outputs are bundled into n_groups groups of equal size, a group is ranked by top1 + top2 of its members' scores, and the
// choice is restricted to members of the `keep` highest-ranked groups (then by their own score; lowest index wins a tie, among groups as among outputs)
__global__ void __launch_bounds__(256) k_moe_route(const uint16_t * __restrict__ router, int64_t width, int n_out, const float * __restrict__ corr, const float * __restrict__ x, int64_t xs,
                                                   int top, int exact, int vec, int n_groups, int keep, int32_t * __restrict__ sel, float * __restrict__ selw, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    extern __shared__ float z[];                  // [n_out] logits -> scores | [n_out] choice | [n_groups] group scores
    float * ch = z + n_out, * gsc = ch + n_out;
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float * xr = x + (int64_t) t * xs;
    for (int e = wave; e < n_out; e += 4) {
        const float a = pi_lanes_sum<64>(hy_dot_lane(router + (int64_t) e * width, xr, width, lane, exact != 0, vec != 0));
        if (lane == 0) z[e] = a;
    }
    __syncthreads();
    if (wave != 0) return;
    if (n_groups < 0) {                           // by logit (+ bias); the weights are worked out over the chosen ones below
        for (int e = lane; e < n_out; e += 64) { z[e] += corr ? corr[e] : 0.0f; ch[e] = z[e]; }
    } else if (n_groups > 0) {
        const int per = n_out / n_groups;
        for (int e = lane; e < n_out; e += 64) { z[e] = 1.0f / (1.0f + expf(-z[e])); ch[e] = -INFINITY; }
        for (int g = lane; g < n_groups; g += 64) {
            float b0 = -INFINITY, b1 = -INFINITY;
            for (int e = g * per; e < (g + 1) * per; e++) { const float v = z[e]; if (v > b0) { b1 = b0; b0 = v; } else if (v > b1) b1 = v; }
            gsc[g] = b1 == -INFINITY ? b0 : b0 + b1;
        }
        for (int kk = 0; kk < keep; kk++) {
            float bv = -INFINITY; int bi = 0x7fffffff;
            for (int g = lane; g < n_groups; g += 64) { const float c = gsc[g]; if (c > bv || (c == bv && g < bi)) { bv = c; bi = g; } }
            for (int d = 32; d > 0; d >>= 1) {
                const float ov = __shfl_xor(bv, d, PI_WAVE); const int oi = __shfl_xor(bi, d, PI_WAVE);
                if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
            }
            if (bi == 0x7fffffff) break;
            for (int e = bi * per + lane; e < (bi + 1) * per; e += 64) ch[e] = z[e];
            if (lane == 0) gsc[bi] = -INFINITY;
        }
    } else {
    float m = -INFINITY;
    for (int e = lane; e < n_out; e += 64) m = fmaxf(m, z[e]);
    m = pi_wave_max(m);
    float l = 0.0f;
    for (int e = lane; e < n_out; e += 64) { const float p = expf(z[e] - m); z[e] = p; l += p; }
    l = pi_lanes_sum<64>(l);
    for (int e = lane; e < n_out; e += 64) { z[e] = z[e] / l; ch[e] = z[e] + corr[e]; }
    }
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
    if (n_groups < 0 && lane == 0) {              // soft-max over the chosen logits alone (the first chosen is the largest)
        float * wt = selw + (int64_t) t * top;
        const float m = wt[0];
        float l = 0.0f;
        for (int kk = 0; kk < top; kk++) { wt[kk] = expf(wt[kk] - m); l += wt[kk]; }
        for (int kk = 0; kk < top; kk++) wt[kk] = wt[kk] / l;
    }
}

// up[t][kk][f] = relu(W_up[e] x_t)^2 for the kk-th chosen expert e of token t (nothing for identity experts); a wave per row f.
// glu: an expert's first matrix holds 2 * ff rows [gate | up] and up[t][kk][f] = silu(gate_f . x) * (up_f . x)
__global__ void __launch_bounds__(256) k_moe_up(const uint16_t * __restrict__ wup, int64_t width, int ff, int n_exp, const float * __restrict__ x, int64_t xs, const int32_t * __restrict__ sel,
                                                int top, int exact, int vec, int glu, float limit, float * __restrict__ up, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w, 0)) return;
    const int lane = threadIdx.x & 63, f = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int slot = blockIdx.y, e = sel[slot];
    if (f >= ff || e >= n_exp) return;
    const int t = slot / top;
    const float * xr = x + (int64_t) t * xs;
    if (glu) {
        const float g = pi_lanes_sum<64>(hy_dot_lane(wup + ((int64_t) e * 2 * ff + f) * width, xr, width, lane, exact != 0, vec != 0));
        const float u = pi_lanes_sum<64>(hy_dot_lane(wup + ((int64_t) e * 2 * ff + ff + f) * width, xr, width, lane, exact != 0, vec != 0));
        if (lane == 0) up[(int64_t) slot * ff + f] = hy_glu(g, u, glu, limit);
        return;
    }
    const float a = pi_lanes_sum<64>(hy_dot_lane(wup + ((int64_t) e * ff + f) * width, xr, width, lane, exact != 0, vec != 0));
    if (lane == 0) { const float r = fmaxf(a, 0.0f); up[(int64_t) slot * ff + f] = r * r; }
}
// out[t][n] = sum_kk w_kk * (identity ? x[t][n] : W_down[e_kk][n] . up[t][kk]); a wave per output n
__global__ void __launch_bounds__(256) k_moe_down(const uint16_t * __restrict__ wdown, int64_t width, int ff, int n_exp, int top, const float * __restrict__ x, int64_t xs,
                                                  const int32_t * __restrict__ sel, const float * __restrict__ selw, const float * __restrict__ up, int exact, int vec, float * __restrict__ out, int64_t os,
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
        const float a = pi_lanes_sum<64>(hy_dot_lane(wdown + ((int64_t) e * width + n) * ff, up + ((int64_t) t * top + kk) * ff, ff, lane, exact != 0, vec != 0));
        acc = fmaf(wgt, a, acc);
    }
    if (lane == 0) out[(int64_t) t * os + n] = acc;
}

static int moe_route_launch(const pi_weight * router, const float * correction_dev, const float * x, int64_t x_stride, int n_tok, int top, int exact, int n_groups, int keep, int32_t * sel_dev, float * selw_dev, void * stream) {
    if (n_tok <= 0) return 0;
    if (!router || router->type != PI_BF16 || top < 1 || top > router->ne1 || router->ne1 > 8192) { pi_set_error("pi_op_moe_route: a bfloat16 router of at most 8192 outputs and 1 <= top <= outputs are required"); return -1; }
    PI_KT_LAUNCH(PI_KT_OTHER, PI_BF16, 1, 2.0 * router->ne0 * router->ne1 + 4.0 * n_tok * router->ne0, k_moe_route, dim3((unsigned) n_tok), dim3(256), (size_t) 8 * router->ne1 + (size_t) 4 * std::max(n_groups, 1), (hipStream_t) stream,
                 (const uint16_t *) router->p0, router->ne0, (int) router->ne1, correction_dev, x, x_stride, top, exact,
                 (int) (router->ne0 % 8 == 0 && ((uintptr_t) router->p0 % 16) == 0 && ((uintptr_t) x % 16) == 0 && x_stride % 4 == 0), n_groups, keep, sel_dev, selw_dev, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}
extern "C" int pi_op_moe_route(const pi_weight * router, const float * correction_dev, const float * x, int64_t x_stride, int n_tok, int top, int exact, int32_t * sel_dev, float * selw_dev, void * stream) {
    return moe_route_launch(router, correction_dev, x, x_stride, n_tok, top, exact, 0, 0, sel_dev, selw_dev, stream);
}
extern "C" int pi_op_moe_route_top_logits(const pi_weight * router, const float * bias_dev, const float * x, int64_t x_stride, int n_tok, int top, int exact, int32_t * sel_dev, float * selw_dev, void * stream) {
    return moe_route_launch(router, bias_dev, x, x_stride, n_tok, top, exact, -1, 0, sel_dev, selw_dev, stream);
}
extern "C" int pi_op_moe_route_groups(const pi_weight * router, const float * x, int64_t x_stride, int n_tok, int top, int n_groups, int keep, int exact, int32_t * sel_dev, float * selw_dev, void * stream) {
    if (!router || n_groups < 1 || router->ne1 % n_groups || keep < 1 || keep > n_groups || (int64_t) keep * (router->ne1 / n_groups) < top) {
        pi_set_error("pi_op_moe_route_groups: the router's outputs must divide into the groups, and the kept groups must hold at least `top` outputs"); return -1;
    }
    return moe_route_launch(router, nullptr, x, x_stride, n_tok, top, exact, n_groups, keep, sel_dev, selw_dev, stream);
}
// wup: [n_exp * ff][width], wdown: [n_exp * width][ff] (the experts' matrices one after the other); up_dev: scratch [n_tok][top][ff]
extern "C" int pi_op_moe_experts(const pi_weight * wup, const pi_weight * wdown, int n_exp, int ff, const float * x, int64_t x_stride, const int32_t * sel_dev, const float * selw_dev, int n_tok, int top,
                                 int exact, float * up_dev, float * out, int64_t out_stride, void * stream) {
    return pi_op_moe_experts_act(wup, wdown, n_exp, ff, 0, x, x_stride, sel_dev, selw_dev, n_tok, top, exact, up_dev, out, out_stride, stream);
}
extern "C" int pi_op_moe_experts_act(const pi_weight * wup, const pi_weight * wdown, int n_exp, int ff, int glu, const float * x, int64_t x_stride, const int32_t * sel_dev, const float * selw_dev, int n_tok, int top,
                                     int exact, float * up_dev, float * out, int64_t out_stride, void * stream) {
    return pi_op_moe_experts_glu(wup, wdown, n_exp, ff, glu, 0.0f, x, x_stride, sel_dev, selw_dev, n_tok, top, exact, up_dev, out, out_stride, stream);
}
extern "C" int pi_op_moe_experts_glu(const pi_weight * wup, const pi_weight * wdown, int n_exp, int ff, int glu, float limit, const float * x, int64_t x_stride, const int32_t * sel_dev, const float * selw_dev, int n_tok,
                                     int top, int exact, float * up_dev, float * out, int64_t out_stride, void * stream) {
    if (n_tok <= 0) return 0;
    if (glu < PI_GLU_OFF || glu > PI_GLU_CLIPPED) { pi_set_error("pi_op_moe_experts: hidden layer of kind %d is unknown", glu); return -1; }
    const int upr = glu ? 2 : 1;                                       // rows of an expert's first matrix, in units of ff
    hipStream_t s = (hipStream_t) stream;
    int64_t width = 0;
    if (n_exp > 0) {
        if (!wup || !wdown || wup->type != PI_BF16 || wdown->type != PI_BF16 || wup->ne1 != (int64_t) n_exp * ff * upr || wdown->ne0 != ff || wdown->ne1 != (int64_t) n_exp * wup->ne0) {
            pi_set_error("pi_op_moe_experts: expert matrices must be bfloat16 [experts * ff (twice with a gate)][width] and [experts * width][ff]"); return -1;
        }
        width = wup->ne0;
        const double b_up = std::min<double>(n_tok * top, n_exp) * 2.0 * upr * ff * width + 4.0 * n_tok * (width + (double) top * ff);
        PI_KT_LAUNCH(PI_KT_MATVEC, PI_BF16, std::min(n_tok, PI_KT_MAXNT - 1), b_up, k_moe_up, dim3((unsigned) ((ff + 3) / 4), (unsigned) (n_tok * top)), dim3(256), 0, s,
                     (const uint16_t *) wup->p0, width, ff, n_exp, x, x_stride, sel_dev, top, exact,
                     (int) (width % 8 == 0 && ((uintptr_t) wup->p0 % 16) == 0 && ((uintptr_t) x % 16) == 0 && x_stride % 4 == 0), glu, limit, up_dev, pi_abort_word());
        PI_CHECK_LAUNCH();
    } else width = out_stride;
    const double b_dn = std::min<double>(n_tok * top, std::max(n_exp, 1)) * 2.0 * ff * width + 4.0 * n_tok * (width + (double) top * ff);
    PI_KT_LAUNCH(PI_KT_MATVEC, PI_BF16, std::min(n_tok, PI_KT_MAXNT - 1), b_dn, k_moe_down, dim3((unsigned) ((width + 3) / 4), (unsigned) n_tok), dim3(256), 0, s,
                 n_exp > 0 ? (const uint16_t *) wdown->p0 : nullptr, width, ff, n_exp, top, x, x_stride, sel_dev, selw_dev, up_dev, exact,
                 (int) (n_exp > 0 && ff % 8 == 0 && ((uintptr_t) wdown->p0 % 16) == 0 && ((uintptr_t) up_dev % 16) == 0), out, out_stride, pi_abort_word());
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
// glu_off > 0: the B value at k is silu(brow[k]) * brow[glu_off + k] (a gated hidden layer whose two halves were stored raw)
static __device__ __forceinline__ void hy_mfma_rows(const uint16_t * const wrow[4], const float * brow, int64_t K, int kb, hy_f32x4 acc[4], int64_t glu_off = 0, int glu = PI_GLU_SILU, float limit = 0.0f) {
    for (int64_t k0 = 0; k0 < K; k0 += 32) {
        const int64_t k = k0 + kb * 8;
        const bool k_ok = k < K;
        hy_u16x8 b = hy_u16x8{0, 0, 0, 0, 0, 0, 0, 0};
        if (k_ok && brow) {
            const float4 v0 = *(const float4 *) (brow + k), v1 = *(const float4 *) (brow + k + 4);
            float f[8] = { v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w };
            if (glu_off > 0) {
                const float4 u0 = *(const float4 *) (brow + glu_off + k), u1 = *(const float4 *) (brow + glu_off + k + 4);
                const float uf[8] = { u0.x, u0.y, u0.z, u0.w, u1.x, u1.y, u1.z, u1.w };
#pragma unroll
                for (int i = 0; i < 8; i++) f[i] = hy_glu(f[i], uf[i], glu, limit);
            }
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

// UP: B rows are the tokens' inputs x[slot / top], A rows W_up[e], out up[slot][f] = relu(.)^2;  !UP: B rows up[slot] (K = ff), A rows W_down[e], out dn[slot][n].
// glu: UP leaves the 2 * ff rows [gate | up] of an expert raw, !UP forms silu(gate) * up while it reads them (bs = 2 * ff, K = ff)
template <bool UP>
__global__ void __launch_bounds__(256) k_moe_mfma(const uint16_t * __restrict__ W, int64_t K, int rows, const float * __restrict__ B, int64_t bs, int top, const int32_t * __restrict__ idx,
                                                  int max_tiles, int glu, float limit, float * __restrict__ out, const int32_t * __restrict__ abort_w) {
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
    hy_mfma_rows(wrow, brow, K, kb, acc, !UP && glu ? K : 0, glu, limit);
    if (slot < 0) return;
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int row = n0 + j * 16 + kb * 4 + r;
            if (row < rows) { float v = acc[j][r]; if (UP && !glu) { v = fmaxf(v, 0.0f); v *= v; } out[(int64_t) slot * rows + row] = v; }
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
extern "C" int pi_op_moe_grouped_ok(const pi_weight * wup, const pi_weight * wdown, int n_exp, int ff, int glu, int n_tok, int top, int exact) {
    (void) glu;
    static const int min_slots = getenv("PI_MOE_GROUPED_MIN") ? atoi(getenv("PI_MOE_GROUPED_MIN")) : 32;
    return !exact && n_exp > 0 && n_exp <= MOE_GROUP_MAX_EXPERTS && wup && wdown && n_tok * top >= min_slots && wup->ne0 % 8 == 0 && ff % 8 == 0 &&
           ((uintptr_t) wup->p0 % 16) == 0 && ((uintptr_t) wdown->p0 % 16) == 0;
}
// up_dev: [n_tok * top][ff], dn_dev: [n_tok * top][width], idx_dev: pi_op_moe_grouped_index_ints ints
extern "C" int pi_op_moe_experts_grouped(const pi_weight * wup, const pi_weight * wdown, int n_exp, int ff, const float * x, int64_t x_stride, const int32_t * sel_dev, const float * selw_dev, int n_tok, int top,
                                         float * up_dev, float * dn_dev, int32_t * idx_dev, float * out, int64_t out_stride, void * stream) {
    return pi_op_moe_experts_grouped_act(wup, wdown, n_exp, ff, 0, x, x_stride, sel_dev, selw_dev, n_tok, top, up_dev, dn_dev, idx_dev, out, out_stride, stream);
}
// glu: w_up holds [gate | up] per expert (2 * ff rows) and up_dev is [n_tok * top][2 * ff]
extern "C" int pi_op_moe_experts_grouped_act(const pi_weight * wup, const pi_weight * wdown, int n_exp, int ff, int glu, const float * x, int64_t x_stride, const int32_t * sel_dev, const float * selw_dev, int n_tok, int top,
                                             float * up_dev, float * dn_dev, int32_t * idx_dev, float * out, int64_t out_stride, void * stream) {
    return pi_op_moe_experts_grouped_glu(wup, wdown, n_exp, ff, glu, 0.0f, x, x_stride, sel_dev, selw_dev, n_tok, top, up_dev, dn_dev, idx_dev, out, out_stride, stream);
}
extern "C" int pi_op_moe_experts_grouped_glu(const pi_weight * wup, const pi_weight * wdown, int n_exp, int ff, int glu, float limit, const float * x, int64_t x_stride, const int32_t * sel_dev, const float * selw_dev,
                                             int n_tok, int top, float * up_dev, float * dn_dev, int32_t * idx_dev, float * out, int64_t out_stride, void * stream) {
    if (glu < PI_GLU_OFF || glu > PI_GLU_CLIPPED) { pi_set_error("pi_op_moe_experts_grouped: hidden layer of kind %d is unknown", glu); return -1; }
    if (!pi_op_moe_grouped_ok(wup, wdown, n_exp, ff, glu, n_tok, top, 0)) { pi_set_error("pi_op_moe_experts_grouped: this shape takes pi_op_moe_experts"); return -1; }
    const int upr = glu ? 2 : 1;
    if (wup->type != PI_BF16 || wdown->type != PI_BF16 || wup->ne1 != (int64_t) n_exp * ff * upr || wdown->ne0 != ff || wdown->ne1 != (int64_t) n_exp * wup->ne0 || x_stride % 4 || ((uintptr_t) x % 16)) {
        pi_set_error("pi_op_moe_experts_grouped: expert matrices must be bfloat16 [experts * ff][width] and [experts * width][ff], inputs 16-byte aligned rows"); return -1;
    }
    hipStream_t s = (hipStream_t) stream;
    const int64_t width = wup->ne0;
    const int ns = n_tok * top, mt = moe_max_tiles(ns, n_exp), nta = std::min(n_tok, PI_KT_MAXNT - 1);
    const double wbytes = std::min<double>(ns, n_exp) * 2.0 * ff * width * (glu ? 1.5 : 1.0);
    PI_KT_LAUNCH(PI_KT_OTHER, PI_BF16, 1, 8.0 * ns, k_moe_group, dim3(1), dim3(256), 0, s, sel_dev, ns, n_exp, mt, idx_dev, pi_abort_word());
    PI_CHECK_LAUNCH();
    PI_KT_LAUNCH(PI_KT_MMQ, PI_BF16, nta, wbytes + 4.0 * ns * (width + ff), k_moe_mfma<true>, dim3((unsigned) ((ff * upr + 63) / 64), (unsigned) mt), dim3(256), 0, s,
                 (const uint16_t *) wup->p0, width, ff * upr, x, x_stride, top, idx_dev, mt, glu, limit, up_dev, pi_abort_word());
    PI_CHECK_LAUNCH();
    PI_KT_LAUNCH(PI_KT_MMQ, PI_BF16, nta, wbytes + 4.0 * ns * (width + ff), k_moe_mfma<false>, dim3((unsigned) ((width + 63) / 64), (unsigned) mt), dim3(256), 0, s,
                 (const uint16_t *) wdown->p0, (int64_t) ff, (int) width, up_dev, (int64_t) ff * upr, top, idx_dev, mt, glu, limit, dn_dev, pi_abort_word());
    PI_CHECK_LAUNCH();
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 4.0 * n_tok * width * (top + 2), k_moe_combine, dim3((unsigned) ((width + 255) / 256), (unsigned) n_tok), dim3(256), 0, s,
                 dn_dev, width, n_exp, top, x, x_stride, sel_dev, selw_dev, out, out_stride, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}
