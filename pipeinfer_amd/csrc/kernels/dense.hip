// Dense operators over bfloat16 weight matrices stored [rows][K] as the checkpoint has them (no re-ordering: a row is one contiguous run of K values).
//
//   out[t][r] = act(sum_k W[r][k] * in(x[t][k]))          fp32 accumulation, fp32 in and out
//
// `exact` selects what enters the product: 0 (serving precision) rounds the activations to bfloat16 (nearest even), so a product of two bfloat16 values is exact in fp32 and only the
// order of the fp32 sum differs between the kernels below; 1 keeps the activations in fp32 (weights widen exactly), every multiply-add a true fp32 fma.
//
//   k_dense_rows   one wave per output row, K spread over the lanes with 16 / 8 / 2-byte weight loads, TT tokens held in registers: the mat-vec of decode (weights streamed
//                  once from HBM whatever TT is) and every width of the fp32 mode
//   k_dense_mfma_lds  serving precision, >= 96 tokens: 128 tokens x 128 rows per workgroup, both operands staged through LDS as bfloat16, double-buffered
//   k_dense_mfma   serving precision, 16 .. 95 tokens: 64 tokens x 64 rows per workgroup on v_mfma_f32_16x16x32_bf16; a wave owns 16 tokens and four 16-row tiles, operands go
//                  straight from global memory into the lane layout of the instruction (A: weight row l % 16, k block l / 16; B: token l % 16, k block l / 16)
//   k_embed        rows of the table gathered, widened and scaled
#include "ops_common.h"
#include "kernel_timing.h"

#include <algorithm>

typedef __bf16 dn_bf16x8 __attribute__((ext_vector_type(8)));
typedef float dn_f32x4 __attribute__((ext_vector_type(4)));
typedef uint16_t dn_u16x8 __attribute__((ext_vector_type(8)));

static __device__ __forceinline__ float dn_widen(uint16_t b) { return __uint_as_float((uint32_t) b << 16); }
// nearest-even rounding of an fp32 value to bfloat16 precision, kept in an fp32 register
static __device__ __forceinline__ uint32_t dn_round_bits(float f) { const uint32_t u = __float_as_uint(f); return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16; }
static __device__ __forceinline__ float dn_round(float f) { return __uint_as_float(dn_round_bits(f) << 16); }

static __device__ __forceinline__ float dn_act(float v, int act) {
    switch (act) {
        case PI_ACT_SILU:     return v / (1.0f + expf(-v));
        case PI_ACT_SIGMOID:  return 1.0f / (1.0f + expf(-v));
        case PI_ACT_RELU_SQR: { const float r = fmaxf(v, 0.0f); return r * r; }
        case PI_ACT_TANH:     return tanhf(v);
        case PI_ACT_GELU_TANH: return 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
        case PI_ACT_GELU_ERF: return 0.5f * v * (1.0f + erff(v * 0.7071067811865476f));
        default:              return v;
    }
}

__global__ void k_embed(const uint16_t * __restrict__ table, int64_t width, int64_t n_rows, const int32_t * __restrict__ tokens, float scale, float * __restrict__ out, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    const int t = blockIdx.x;
    const int64_t row = tokens[t];
    if (row < 0 || row >= n_rows) { for (int64_t i = threadIdx.x; i < width; i += blockDim.x) out[(int64_t) t * width + i] = 0.0f; return; }
    for (int64_t i = threadIdx.x; i < width; i += blockDim.x) out[(int64_t) t * width + i] = dn_widen(table[row * width + i]) * scale;
}

// VW weights per lane and step (8: one 16-byte load, 4: 8 bytes, 1: any K and alignment)
template <int TT, int VW, bool EXACT>
__global__ void __launch_bounds__(256) k_dense_rows(const uint16_t * __restrict__ W, int64_t K, int64_t N, const float * __restrict__ X, int64_t xs, int T, float * __restrict__ Y, int64_t ys,
                                                    int act_a, int64_t rows_a, int act_b, int64_t seg_rows, int64_t seg_off, int seg_last, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w, 0)) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t row = (int64_t) blockIdx.x * 4 + wave;
    if (row >= N) return;
    if (seg_rows > 0) X += min(row / seg_rows, (int64_t) seg_last) * seg_off;       // rows in segments of seg_rows (the last one takes the rest), every segment with an input of its own
    const int t0 = blockIdx.y * TT;
    float acc[TT];
#pragma unroll
    for (int i = 0; i < TT; i++) acc[i] = 0.0f;
    const uint16_t * w = W + row * K;
    for (int64_t k = (int64_t) lane * VW; k < K; k += 64 * VW) {
        float wf[VW];
        if constexpr (VW == 8) { const dn_u16x8 v = *(const dn_u16x8 *) (w + k); for (int i = 0; i < 8; i++) wf[i] = dn_widen(v[i]); }
        else if constexpr (VW == 4) { const uint2 v = *(const uint2 *) (w + k); wf[0] = __uint_as_float(v.x << 16); wf[1] = __uint_as_float(v.x & 0xffff0000u); wf[2] = __uint_as_float(v.y << 16); wf[3] = __uint_as_float(v.y & 0xffff0000u); }
        else wf[0] = dn_widen(w[k]);
#pragma unroll
        for (int tt = 0; tt < TT; tt++) {
            if (t0 + tt >= T) break;
            const float * x = X + (int64_t) (t0 + tt) * xs + k;
            float xf[VW];
            if constexpr (VW >= 4) {
#pragma unroll
                for (int i = 0; i < VW; i += 4) { const float4 v = *(const float4 *) (x + i); xf[i] = v.x; xf[i + 1] = v.y; xf[i + 2] = v.z; xf[i + 3] = v.w; }
            } else xf[0] = x[0];
#pragma unroll
            for (int i = 0; i < VW; i++) acc[tt] = fmaf(wf[i], EXACT ? xf[i] : dn_round(xf[i]), acc[tt]);
        }
    }
    const int act = row < rows_a ? act_a : act_b;
#pragma unroll
    for (int tt = 0; tt < TT; tt++) {
        if (t0 + tt >= T) break;
        const float s = pi_lanes_sum<64>(acc[tt]);
        if (lane == 0) Y[(int64_t) (t0 + tt) * ys + row] = dn_act(s, act);
    }
}

// 64 tokens x 64 rows per workgroup; K % 8 == 0, 16-byte aligned rows of W and X
__global__ void __launch_bounds__(256) k_dense_mfma(const uint16_t * __restrict__ W, int64_t K, int64_t N, const float * __restrict__ X, int64_t xs, int T, float * __restrict__ Y, int64_t ys,
                                                    int act_a, int64_t rows_a, int act_b, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w, 1)) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int li = lane & 15, kb = lane >> 4;
    const int64_t n0 = (int64_t) blockIdx.x * 64;
    const int tok = blockIdx.y * 64 + wave * 16 + li;                  // the token this lane feeds as operand B
    const bool tok_ok = tok < T;
    const float * xrow = X + (int64_t) (tok_ok ? tok : 0) * xs;
    const uint16_t * wrow[4]; bool row_ok[4];
#pragma unroll
    for (int j = 0; j < 4; j++) { const int64_t r = n0 + j * 16 + li; row_ok[j] = r < N; wrow[j] = W + (row_ok[j] ? r : 0) * K; }
    dn_f32x4 acc[4];
#pragma unroll
    for (int j = 0; j < 4; j++) acc[j] = dn_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    for (int64_t k0 = 0; k0 < K; k0 += 32) {
        const int64_t k = k0 + kb * 8;
        const bool k_ok = k < K;                                       // (K % 8 == 0: a block of 8 is inside or outside as a whole)
        dn_u16x8 b = dn_u16x8{0, 0, 0, 0, 0, 0, 0, 0};
        if (k_ok && tok_ok) {
            const float4 v0 = *(const float4 *) (xrow + k), v1 = *(const float4 *) (xrow + k + 4);
            b[0] = (uint16_t) dn_round_bits(v0.x); b[1] = (uint16_t) dn_round_bits(v0.y); b[2] = (uint16_t) dn_round_bits(v0.z); b[3] = (uint16_t) dn_round_bits(v0.w);
            b[4] = (uint16_t) dn_round_bits(v1.x); b[5] = (uint16_t) dn_round_bits(v1.y); b[6] = (uint16_t) dn_round_bits(v1.z); b[7] = (uint16_t) dn_round_bits(v1.w);
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            dn_u16x8 a = dn_u16x8{0, 0, 0, 0, 0, 0, 0, 0};
            if (k_ok && row_ok[j]) a = *(const dn_u16x8 *) (wrow[j] + k);
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(dn_bf16x8, a), __builtin_bit_cast(dn_bf16x8, b), acc[j], 0, 0, 0);
        }
    }
    // D: lane holds token l % 16 and rows (l / 16) * 4 .. + 3 of each tile
    if (!tok_ok) return;
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int64_t row = n0 + j * 16 + kb * 4 + r;
            if (row < N) Y[(int64_t) tok * ys + row] = dn_act(acc[j][r], row < rows_a ? act_a : act_b);
        }
}

// 128 tokens x 128 rows per workgroup, operands staged through LDS as bfloat16 (activations are rounded once, while they are staged): a wave owns 64 x 64 = sixteen 16 x 16
// tiles, so one K step of 32 costs it eight 16-byte LDS reads for sixteen MFMAs; the next K step's global loads are in flight while the current one is multiplied.
// K % 8 == 0, 16-byte aligned rows of W and X.
__global__ void __launch_bounds__(256) k_dense_mfma_lds(const uint16_t * __restrict__ W, int64_t K, int64_t N, const float * __restrict__ X, int64_t xs, int T, float * __restrict__ Y, int64_t ys,
                                                        int act_a, int64_t rows_a, int act_b, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w, 1)) return;
    __shared__ __attribute__((aligned(16))) uint16_t sw[2][128 * 32], sx[2][128 * 32];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, kb = lane >> 4;
    const int wr = wave >> 1, wt = wave & 1;                           // the wave's 64 rows / 64 tokens inside the tile
    const int64_t n0 = (int64_t) blockIdx.x * 128;
    const int t0 = blockIdx.y * 128;
    // staging: thread -> (row or token tid / 2, 16 k values of half tid % 2)
    const int sr = tid >> 1, sh = tid & 1;
    const bool w_ok = n0 + sr < N, x_ok = t0 + sr < T;
    const uint16_t * wsrc = W + (w_ok ? n0 + sr : 0) * K + sh * 16;
    const float * xsrc = X + (int64_t) (x_ok ? t0 + sr : 0) * xs + sh * 16;
    uint4 wreg[2]; float4 xreg[4];
    auto fetch = [&](int64_t k0) {
#pragma unroll
        for (int i = 0; i < 2; i++) wreg[i] = (w_ok && k0 + sh * 16 + i * 8 < K) ? *(const uint4 *) (wsrc + k0 + i * 8) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; i++) xreg[i] = (x_ok && k0 + sh * 16 + i * 4 < K) ? *(const float4 *) (xsrc + k0 + i * 4) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    };
    auto stage = [&](int buf) {
        *(uint4 *) (sw[buf] + sr * 32 + sh * 16) = wreg[0]; *(uint4 *) (sw[buf] + sr * 32 + sh * 16 + 8) = wreg[1];
        uint32_t pk[8];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            pk[2 * i]     = dn_round_bits(xreg[i].x) | dn_round_bits(xreg[i].y) << 16;
            pk[2 * i + 1] = dn_round_bits(xreg[i].z) | dn_round_bits(xreg[i].w) << 16;
        }
        *(uint4 *) (sx[buf] + sr * 32 + sh * 16) = make_uint4(pk[0], pk[1], pk[2], pk[3]); *(uint4 *) (sx[buf] + sr * 32 + sh * 16 + 8) = make_uint4(pk[4], pk[5], pk[6], pk[7]);
    };
    dn_f32x4 acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 4; b++) acc[a][b] = dn_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    fetch(0);
    stage(0);
    __syncthreads();
    int buf = 0;
    for (int64_t k0 = 0; k0 < K; k0 += 32) {
        const bool more = k0 + 32 < K;
        if (more) fetch(k0 + 32);
        dn_u16x8 af[4], bf[4];
#pragma unroll
        for (int a = 0; a < 4; a++) af[a] = *(const dn_u16x8 *) (sw[buf] + (wr * 64 + a * 16 + li) * 32 + kb * 8);
#pragma unroll
        for (int b = 0; b < 4; b++) bf[b] = *(const dn_u16x8 *) (sx[buf] + (wt * 64 + b * 16 + li) * 32 + kb * 8);
#pragma unroll
        for (int a = 0; a < 4; a++)
#pragma unroll
            for (int b = 0; b < 4; b++)
                acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(dn_bf16x8, af[a]), __builtin_bit_cast(dn_bf16x8, bf[b]), acc[a][b], 0, 0, 0);
        if (more) stage(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }
#pragma unroll
    for (int b = 0; b < 4; b++) {
        const int tok = t0 + wt * 64 + b * 16 + li;
        if (tok >= T) continue;
#pragma unroll
        for (int a = 0; a < 4; a++) {
            const int64_t row = n0 + wr * 64 + a * 16 + kb * 4;
            float v[4];
#pragma unroll
            for (int r = 0; r < 4; r++) v[r] = dn_act(acc[a][b][r], row + r < rows_a ? act_a : act_b);
            float * dst = Y + (int64_t) tok * ys + row;
            if (row + 3 < N && (ys & 3) == 0 && (((uintptr_t) Y) & 15) == 0) *(float4 *) dst = make_float4(v[0], v[1], v[2], v[3]);
            else for (int r = 0; r < 4; r++) if (row + r < N) dst[r] = v[r];
        }
    }
}

extern "C" int pi_op_embed(const pi_weight * w, const int32_t * tokens, int n_tok, float scale, float * out, void * stream) {
    if (!w || w->type != PI_BF16) { pi_set_error("pi_op_embed: the table must be a bfloat16 weight"); return -1; }
    if (n_tok <= 0) return 0;
    PI_KT_LAUNCH(PI_KT_OTHER, PI_BF16, 1, 6.0 * w->ne0 * n_tok, k_embed, dim3((unsigned) n_tok), dim3(256), 0, (hipStream_t) stream, (const uint16_t *) w->p0, w->ne0, w->ne1, tokens, scale, out, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}

static int dense_mfma_min_tokens() { static const int v = getenv("PI_DENSE_MFMA_MIN") ? atoi(getenv("PI_DENSE_MFMA_MIN")) : 16; return v; }

template <int VW, bool EXACT>
static void launch_rows(const pi_weight * w, const float * x, int64_t xs, int n_tok, float * out, int64_t os, int act_a, int64_t rows_a, int act_b, hipStream_t s, double bytes, int64_t seg_rows = 0, int64_t seg_off = 0, int seg_last = 0) {
    const uint16_t * W = (const uint16_t *) w->p0;
    const unsigned gx = (unsigned) ((w->ne1 + 3) / 4);
    const int nt_acct = std::min(n_tok, PI_KT_MAXNT - 1);
    if (n_tok == 1)      PI_KT_LAUNCH(PI_KT_MATVEC, PI_BF16, nt_acct, bytes, (k_dense_rows<1, VW, EXACT>), dim3(gx, 1), dim3(256), 0, s, W, w->ne0, w->ne1, x, xs, n_tok, out, os, act_a, rows_a, act_b, seg_rows, seg_off, seg_last, pi_abort_word());
    else if (n_tok <= 4) PI_KT_LAUNCH(PI_KT_MATVEC, PI_BF16, nt_acct, bytes, (k_dense_rows<4, VW, EXACT>), dim3(gx, 1), dim3(256), 0, s, W, w->ne0, w->ne1, x, xs, n_tok, out, os, act_a, rows_a, act_b, seg_rows, seg_off, seg_last, pi_abort_word());
    else PI_KT_LAUNCH(PI_KT_MATVEC, PI_BF16, nt_acct, bytes, (k_dense_rows<8, VW, EXACT>), dim3(gx, (unsigned) ((n_tok + 7) / 8)), dim3(256), 0, s, W, w->ne0, w->ne1, x, xs, n_tok, out, os, act_a, rows_a, act_b, seg_rows, seg_off, seg_last, pi_abort_word());
}

extern "C" int pi_op_dense(const pi_weight * w, const float * x, int64_t x_stride, int n_tok, float * out, int64_t out_stride, int act_a, int64_t rows_a, int act_b, int exact, void * stream) {
    if (!w || w->type != PI_BF16) { pi_set_error("pi_op_dense: the weight must be bfloat16"); return -1; }
    if (n_tok <= 0 || w->ne1 <= 0) return 0;
    if (x_stride < w->ne0 || out_stride < w->ne1) { pi_set_error("pi_op_dense: row strides (%lld, %lld) below the matrix's sizes (%lld, %lld)", (long long) x_stride, (long long) out_stride, (long long) w->ne0, (long long) w->ne1); return -1; }
    hipStream_t s = (hipStream_t) stream;
    const int64_t K = w->ne0;
    const double bytes = 2.0 * K * w->ne1 + 4.0 * n_tok * (K + w->ne1);
    const bool al16 = K % 8 == 0 && ((uintptr_t) w->p0 % 16) == 0 && ((uintptr_t) x % 16) == 0 && x_stride % 4 == 0;
    const bool al8  = K % 4 == 0 && ((uintptr_t) w->p0 % 8) == 0 && ((uintptr_t) x % 16) == 0 && x_stride % 4 == 0;
    static const int lds_min = getenv("PI_DENSE_LDS_MIN") ? atoi(getenv("PI_DENSE_LDS_MIN")) : 96;
    if (!exact && al16 && n_tok >= lds_min) {
        PI_KT_LAUNCH(PI_KT_MMQ, PI_BF16, std::min(n_tok, PI_KT_MAXNT - 1), bytes, k_dense_mfma_lds, dim3((unsigned) ((w->ne1 + 127) / 128), (unsigned) ((n_tok + 127) / 128)), dim3(256), 0, s,
                     (const uint16_t *) w->p0, K, w->ne1, x, x_stride, n_tok, out, out_stride, act_a, rows_a, act_b, pi_abort_word());
        PI_CHECK_LAUNCH(); return 0;
    }
    if (!exact && al16 && n_tok >= dense_mfma_min_tokens()) {
        PI_KT_LAUNCH(PI_KT_MMQ, PI_BF16, std::min(n_tok, PI_KT_MAXNT - 1), bytes, k_dense_mfma, dim3((unsigned) ((w->ne1 + 63) / 64), (unsigned) ((n_tok + 63) / 64)), dim3(256), 0, s,
                     (const uint16_t *) w->p0, K, w->ne1, x, x_stride, n_tok, out, out_stride, act_a, rows_a, act_b, pi_abort_word());
        PI_CHECK_LAUNCH(); return 0;
    }
    if (al16 && K >= 512) { if (exact) launch_rows<8, true>(w, x, x_stride, n_tok, out, out_stride, act_a, rows_a, act_b, s, bytes); else launch_rows<8, false>(w, x, x_stride, n_tok, out, out_stride, act_a, rows_a, act_b, s, bytes); }
    else if (al8)         { if (exact) launch_rows<4, true>(w, x, x_stride, n_tok, out, out_stride, act_a, rows_a, act_b, s, bytes); else launch_rows<4, false>(w, x, x_stride, n_tok, out, out_stride, act_a, rows_a, act_b, s, bytes); }
    else                  { if (exact) launch_rows<1, true>(w, x, x_stride, n_tok, out, out_stride, act_a, rows_a, act_b, s, bytes); else launch_rows<1, false>(w, x, x_stride, n_tok, out, out_stride, act_a, rows_a, act_b, s, bytes); }
    PI_CHECK_LAUNCH(); return 0;
}

// one matrix whose rows fall into segments that each read an input of their own: rows [g * seg_rows, (g + 1) * seg_rows) read x + g * seg_off (g < n_seg - 1; the last segment takes the remaining
// rows).  Few tokens (the mat-vec kernel): ONE launch; wider passes take a matrix-core launch per segment
extern "C" int pi_op_dense_segments(const pi_weight * w, const float * x, int64_t x_stride, int64_t seg_rows, int64_t seg_off, int n_seg, int n_tok, float * out, int64_t out_stride, int act_a, int64_t rows_a,
                                    int act_b, int exact, void * stream) {
    if (!w || w->type != PI_BF16) { pi_set_error("pi_op_dense: the weight must be bfloat16"); return -1; }
    if (n_tok <= 0 || w->ne1 <= 0) return 0;
    if (n_seg < 1 || seg_rows < 1 || (int64_t) (n_seg - 1) * seg_rows >= w->ne1) { pi_set_error("pi_op_dense_segments: %d segments of %lld rows do not fit %lld rows", n_seg, (long long) seg_rows, (long long) w->ne1); return -1; }
    const int64_t K = w->ne0;
    if (x_stride < (int64_t) (n_seg - 1) * seg_off + K || out_stride < w->ne1) { pi_set_error("pi_op_dense_segments: row strides below the sizes"); return -1; }
    const bool al16 = K % 8 == 0 && ((uintptr_t) w->p0 % 16) == 0 && ((uintptr_t) x % 16) == 0 && x_stride % 4 == 0 && seg_off % 4 == 0;
    if (exact || !al16 || n_tok < dense_mfma_min_tokens()) {
        const bool al8 = K % 4 == 0 && ((uintptr_t) w->p0 % 8) == 0 && ((uintptr_t) x % 16) == 0 && x_stride % 4 == 0 && seg_off % 4 == 0;
        const double bytes = 2.0 * K * w->ne1 + 4.0 * n_tok * (n_seg * K + w->ne1);
        hipStream_t s = (hipStream_t) stream;
        if (al16 && K >= 512) { if (exact) launch_rows<8, true>(w, x, x_stride, n_tok, out, out_stride, act_a, rows_a, act_b, s, bytes, seg_rows, seg_off, n_seg - 1); else launch_rows<8, false>(w, x, x_stride, n_tok, out, out_stride, act_a, rows_a, act_b, s, bytes, seg_rows, seg_off, n_seg - 1); }
        else if (al8)         { if (exact) launch_rows<4, true>(w, x, x_stride, n_tok, out, out_stride, act_a, rows_a, act_b, s, bytes, seg_rows, seg_off, n_seg - 1); else launch_rows<4, false>(w, x, x_stride, n_tok, out, out_stride, act_a, rows_a, act_b, s, bytes, seg_rows, seg_off, n_seg - 1); }
        else                  { if (exact) launch_rows<1, true>(w, x, x_stride, n_tok, out, out_stride, act_a, rows_a, act_b, s, bytes, seg_rows, seg_off, n_seg - 1); else launch_rows<1, false>(w, x, x_stride, n_tok, out, out_stride, act_a, rows_a, act_b, s, bytes, seg_rows, seg_off, n_seg - 1); }
        PI_CHECK_LAUNCH(); return 0;
    }
    for (int g = 0; g < n_seg; g++) {                                  // a view of the segment's rows
        pi_weight view = *w;
        const int64_t r0 = (int64_t) g * seg_rows;
        view.p0 = w->p0 + (size_t) r0 * K * 2; view.ne1 = g == n_seg - 1 ? w->ne1 - r0 : seg_rows;
        const int64_t ra = std::max<int64_t>(0, std::min<int64_t>(view.ne1, rows_a - r0));
        if (pi_op_dense(&view, x + g * seg_off, x_stride, n_tok, out + r0, out_stride, act_a, ra, act_b, exact, stream) != 0) return -1;
    }
    return 0;
}
