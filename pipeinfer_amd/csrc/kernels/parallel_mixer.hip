// Operators of a mixer made of two branches that read the same input: attention with un-normalised sigmoid weights inside position chunks (grouped key / value heads,
// normed and partly rotated queries and keys, unit-norm values, a per-head output gate), and a selective state-space recurrence with a short causal convolution in front
// (state-space duality: per head S_t = a_t S_(t-1) + dt_t B_t x_t^T, y_t = S_t^T C_t + D x_t).  Everything here is fp32 in both precisions of the engine: norms, angles,
// scores, weights, decays, step sizes, states.  The recurrence itself is pi_op_linear_attention_ex (hybrid.hip) with per-token decays and scales.
//
//   k_qkv_prepare        per token: RMS norm (shared per-head weight) + partial rotation of q and k, unit RMS of v; k and v go to the token's cache cell, the cell learns its position
//   k_chunk_attention    out[t][h] = gate[t][h] * sum over visible cells c of sigmoid(q . K[c] * scale + bias[h]) V[c];  visible = the pass's mask bit AND position(c) >= start of t's chunk
//   k_causal_conv        per channel: act(bias + sum_l w[l] * input(t - taps + 1 + l)), inputs before the pass come from the sequence's conv state (zeros for a fresh one)
//   k_conv_state_update  the sequence's last taps - 1 inputs, for the next pass
//   k_causal_conv_walk   both of the above and k_ssd_steps in one launch for passes of at most 32 tokens
//   k_ssd_steps          dt = softplus(raw + bias), a = exp(-exp(A_log) * dt)
//   k_gate_group_norm    u = y * silu(z); each of `groups` equal parts of u divided by its root mean square; * w * mult
#include "ops_common.h"
#include "kernel_timing.h"

#include <algorithm>
#include <cmath>
#include <vector>

#define PM_FRESH (1 << 30)

static __device__ __forceinline__ float pm_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }
static __device__ __forceinline__ float pm_block_sum(float v, float * red) {          // sum over the block's threads (every thread gets it); red: 4 floats, reusable after the call
    v = pi_lanes_sum<64>(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = 0.0f;
    for (int i = 0; i < (int) (blockDim.x >> 6); i++) s += red[i];
    return s;
}

// one pooled row: the token at position p = pos[t] closes a block of `pool` positions ((p + 1) % pool == 0, the caller checks): the cells of the block's positions are found among the cells the
// token's mask row shows, their key / value rows of head g summed in position order, the means left in row pool_off + the token's own cell.  members: `pool` ints of LDS; all 256 threads call
static __device__ __forceinline__ void pm_pool_block(float * __restrict__ kc, float * __restrict__ vc, const int32_t * __restrict__ cell_pos, const uint32_t * __restrict__ mrow, int p, int pool, int64_t pool_off,
                                                     int G, int g, int D, int V, int n_kv, int own_cell, int * members) {
    const int tid = threadIdx.x, p0 = p - pool + 1;
    for (int i = tid; i < pool; i += 256) members[i] = -1;
    __syncthreads();
    for (int c = tid; c < n_kv; c += 256) {
        if (!((mrow[c >> 5] >> (c & 31)) & 1u)) continue;
        const int cp = cell_pos[c];
        if (cp >= p0 && cp <= p) members[cp - p0] = c;
    }
    __syncthreads();
    const int64_t own = pool_off + own_cell;
    for (int i = tid; i < D + V; i += 256) {
        const bool key = i < D;
        const float * cache = key ? kc : vc;
        const int W = key ? D : V, col = key ? i : i - D;
        float sum = 0.0f;
        for (int j = 0; j < pool; j++) { const int c = members[j]; if (c >= 0) sum += cache[((int64_t) c * G + g) * W + col]; }
        (key ? kc : vc)[(own * G + g) * W + col] = sum / (float) pool;
    }
}

// ---- rotation table: cos / sin of p * base^(-2i / dims), angles formed in double on the host ------------------------------------------------------------
struct pi_rotary_table { float2 * cs; int n_pos, half; };
extern "C" void * pi_rotary_table_create(int n_pos, int dims, float base) { return pi_rotary_table_create_scaled(n_pos, dims, base, 1.0f, 1.0f, 1.0f, 0); }
// original > 0: long wavelengths are stretched — an angle step whose wavelength 2 pi / f exceeds original / low is divided by `factor`, one below original / high stays, between the two they blend
extern "C" void * pi_rotary_table_create_scaled(int n_pos, int dims, float base, float factor, float low, float high, int original) {
    if (n_pos < 1 || dims < 0 || (dims & 1)) { pi_set_error("pi_rotary_table_create: %d positions, %d rotated dimensions (an even number)", n_pos, dims); return nullptr; }
    if (original > 0 && (!(factor > 0.0f) || !(low > 0.0f) || !(high > 0.0f))) { pi_set_error("pi_rotary_table_create: stretching needs positive factor, low and high"); return nullptr; }
    pi_rotary_table * t = new pi_rotary_table{ nullptr, n_pos, dims / 2 };
    if (t->half == 0) return t;
    std::vector<float2> h((size_t) n_pos * t->half);
    for (int i = 0; i < t->half; i++) {
        double f = std::pow((double) base, -2.0 * i / dims);
        if (original > 0) {
            const double wl = 2.0 * M_PI / f, lo_wl = (double) original / high, hi_wl = (double) original / low;
            if (wl > hi_wl) f /= factor;
            else if (wl >= lo_wl && high != low) { const double sm = ((double) original / wl - low) / ((double) high - low); f = (1.0 - sm) * f / factor + sm * f; }
        }
        for (int p = 0; p < n_pos; p++) { const double a = (double) p * f; h[(size_t) p * t->half + i] = make_float2((float) std::cos(a), (float) std::sin(a)); }
    }
    t->cs = (float2 *) pi_malloc(h.size() * sizeof(float2));
    if (!t->cs || pi_memcpy_h2d(t->cs, h.data(), h.size() * sizeof(float2), nullptr) != 0 || pi_stream_sync(nullptr) != 0) { pi_free(t->cs); delete t; return nullptr; }
    return t;
}
extern "C" int pi_rotary_table_positions(const void * table) { return table ? ((const pi_rotary_table *) table)->n_pos : 0; }
extern "C" void pi_rotary_table_free(void * table) { pi_rotary_table * t = (pi_rotary_table *) table; if (t) { pi_free(t->cs); delete t; } }

// ---- q / k / v of a pass ------------------------------------------------------------------------------------------------------------------------------
// grid (token, head slot): slots [0, H) are query heads, [H, H + G) key heads, [H + G, H + 2G) value heads; one wave per slot
__global__ void __launch_bounds__(64) k_qkv_prepare(const float * __restrict__ q, const float * __restrict__ k, const float * __restrict__ v, int64_t stride, const float * __restrict__ qw,
                                                    const float * __restrict__ kw, float eps, int H, int G, int D, int V, const float2 * __restrict__ rot, int half, int n_pos,
                                                    const int32_t * __restrict__ pos, float * __restrict__ q_out, int64_t qos, float * __restrict__ kc, float * __restrict__ vc,
                                                    int32_t * __restrict__ cell_pos, const int32_t * __restrict__ dyn, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    const int t = blockIdx.x, slot = blockIdx.y, lane = threadIdx.x;
    const int cell = pi_cell_of(dyn, 0, t);
    const int p = pos[t];
    if (slot == 0 && lane == 0) cell_pos[cell] = p;
    if (slot >= H + G) {                                              // a value head: divided by its root mean square, no weight
        const int g = slot - H - G;
        const float * src = v + (int64_t) t * stride + (int64_t) g * V;
        float ss = 0.0f;
        for (int i = lane; i < V; i += 64) ss = fmaf(src[i], src[i], ss);
        const float inv = 1.0f / sqrtf(pi_lanes_sum<64>(ss) / (float) V + eps);
        float * dst = vc + ((int64_t) cell * G + g) * V;
        for (int i = lane; i < V; i += 64) dst[i] = src[i] * inv;
        return;
    }
    const bool is_q = slot < H;
    const int h = is_q ? slot : slot - H;
    const float * src = (is_q ? q : k) + (int64_t) t * stride + (int64_t) h * D;
    const float * w = is_q ? qw : kw;
    float * dst = is_q ? q_out + (int64_t) t * qos + (int64_t) h * D : kc + ((int64_t) cell * G + h) * D;
    float ss = 0.0f;
    for (int i = lane; i < D; i += 64) ss = fmaf(src[i], src[i], ss);
    const float inv = 1.0f / sqrtf(pi_lanes_sum<64>(ss) / (float) D + eps);
    const float2 * cs = rot + (int64_t) min(p, n_pos - 1) * half;
    for (int i = lane; i < D; i += 64) {
        float y = src[i] * inv * w[i];
        if (i < 2 * half) {                                           // dimension i pairs with i + half (i < half) or i - half
            const int j = i < half ? i + half : i - half, f = i < half ? i : i - half;
            const float o = src[j] * inv * w[j];
            const float2 c = cs[f];
            y = i < half ? y * c.x - o * c.y : y * c.x + o * c.y;
        }
        dst[i] = y;
    }
}

extern "C" int pi_op_qkv_prepare(const float * q, const float * k, const float * v, int64_t stride, const float * q_norm_w, const float * k_norm_w, float eps, int heads, int kv_heads, int dim, int vdim,
                                 const void * rotary_table, const int32_t * pos_dev, int n_tok, float * q_out, int64_t q_out_stride, float * k_cache, float * v_cache, int32_t * cell_pos_dev,
                                 const int32_t * dyn_dev, void * stream) {
    if (n_tok <= 0) return 0;
    const pi_rotary_table * rt = (const pi_rotary_table *) rotary_table;
    if (!rt || 2 * rt->half > dim) { pi_set_error("pi_op_qkv_prepare: a rotation table over at most %d dimensions is required", dim); return -1; }
    if (heads < 1 || kv_heads < 1 || heads % kv_heads) { pi_set_error("pi_op_qkv_prepare: %d query heads do not divide over %d key / value heads", heads, kv_heads); return -1; }
    if (!dyn_dev || !cell_pos_dev) { pi_set_error("pi_op_qkv_prepare: the pass's cell table and the cells' position array are required"); return -1; }
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 8.0 * n_tok * ((double) heads * dim + (double) kv_heads * (dim + vdim)), k_qkv_prepare, dim3((unsigned) n_tok, (unsigned) (heads + 2 * kv_heads)), dim3(64), 0, (hipStream_t) stream,
                 q, k, v, stride, q_norm_w, k_norm_w, eps, heads, kv_heads, dim, vdim, rt->cs, rt->half, rt->n_pos, pos_dev, q_out, q_out_stride, k_cache, v_cache, cell_pos_dev, dyn_dev, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}

// the same with the order and the pairing as parameters.  norm_first: R(.) * w, then the rotation (as above), else the rotation first and R(.) * w over the rotated head; w may be absent (1);
// pairing PI_PAIR_HALVES: dimension i with i + dims / 2, PI_PAIR_NEIGHBOURS: 2i with 2i + 1 (angle number i either way); v_norm = 0: value heads go to their cell as they are
__global__ void __launch_bounds__(64) k_qkv_prepare_any(const float * __restrict__ q, const float * __restrict__ k, const float * __restrict__ v, int64_t stride, const float * __restrict__ qw,
                                                        const float * __restrict__ kw, float eps, int H, int G, int D, int V, const float2 * __restrict__ rot, int half, int n_pos, int norm_first, int pairing, int v_norm,
                                                        const int32_t * __restrict__ pos, float * __restrict__ q_out, int64_t qos, float * __restrict__ kc, float * __restrict__ vc,
                                                        int32_t * __restrict__ cell_pos, const int32_t * __restrict__ dyn, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    const int t = blockIdx.x, slot = blockIdx.y, lane = threadIdx.x;
    const int cell = pi_cell_of(dyn, 0, t);
    const int p = pos[t];
    if (slot == 0 && lane == 0) cell_pos[cell] = p;
    if (slot >= H + G) {
        const int g = slot - H - G;
        const float * src = v + (int64_t) t * stride + (int64_t) g * V;
        float inv = 1.0f;
        if (v_norm) {
            float ss = 0.0f;
            for (int i = lane; i < V; i += 64) ss = fmaf(src[i], src[i], ss);
            inv = 1.0f / sqrtf(pi_lanes_sum<64>(ss) / (float) V + eps);
        }
        float * dst = vc + ((int64_t) cell * G + g) * V;
        for (int i = lane; i < V; i += 64) dst[i] = v_norm ? src[i] * inv : src[i];
        return;
    }
    const bool is_q = slot < H;
    const int h = is_q ? slot : slot - H;
    const float * src = (is_q ? q : k) + (int64_t) t * stride + (int64_t) h * D;
    const float * w = is_q ? qw : kw;
    float * dst = is_q ? q_out + (int64_t) t * qos + (int64_t) h * D : kc + ((int64_t) cell * G + h) * D;
    const bool none = norm_first == PI_QK_NORM_NONE;
    norm_first = norm_first == PI_QK_NORM_FIRST;
    float inv1 = 1.0f;
    if (norm_first) {
        float ss = 0.0f;
        for (int i = lane; i < D; i += 64) ss = fmaf(src[i], src[i], ss);
        inv1 = 1.0f / sqrtf(pi_lanes_sum<64>(ss) / (float) D + eps);
    }
    const float2 * cs = rot + (int64_t) min(p, n_pos - 1) * half;
    auto before = [&](int i) { return norm_first ? src[i] * inv1 * (w ? w[i] : 1.0f) : src[i]; };
    auto turned = [&](int i) {
        float y = before(i);
        if (i < 2 * half) {
            const bool lead = pairing == PI_PAIR_NEIGHBOURS ? !(i & 1) : i < half;                       // the pair's first member: u cos - v sin; its second: v cos + u sin
            const int j = pairing == PI_PAIR_NEIGHBOURS ? (i ^ 1) : (i < half ? i + half : i - half), f = pairing == PI_PAIR_NEIGHBOURS ? (i >> 1) : (i < half ? i : i - half);
            const float o = before(j);
            const float2 c = cs[f];
            y = lead ? y * c.x - o * c.y : y * c.x + o * c.y;
        }
        return y;
    };
    if (norm_first || none) { for (int i = lane; i < D; i += 64) dst[i] = turned(i); return; }
    float ss = 0.0f;
    for (int i = lane; i < D; i += 64) { const float y = turned(i); ss = fmaf(y, y, ss); }
    const float inv = 1.0f / sqrtf(pi_lanes_sum<64>(ss) / (float) D + eps);
    for (int i = lane; i < D; i += 64) dst[i] = turned(i) * inv * (w ? w[i] : 1.0f);
}
extern "C" int pi_op_qkv_prepare_ex(const float * q, const float * k, const float * v, int64_t stride, const float * q_norm_w, const float * k_norm_w, float eps, int heads, int kv_heads, int dim, int vdim,
                                    const void * rotary_table, int norm_first, int pairing, int v_norm, const int32_t * pos_dev, int n_tok, float * q_out, int64_t q_out_stride, float * k_cache, float * v_cache,
                                    int32_t * cell_pos_dev, const int32_t * dyn_dev, void * stream) {
    if (n_tok <= 0) return 0;
    const pi_rotary_table * rt = (const pi_rotary_table *) rotary_table;
    if (!rt || 2 * rt->half > dim) { pi_set_error("pi_op_qkv_prepare: a rotation table over at most %d dimensions is required", dim); return -1; }
    if (heads < 1 || kv_heads < 1 || heads % kv_heads) { pi_set_error("pi_op_qkv_prepare: %d query heads do not divide over %d key / value heads", heads, kv_heads); return -1; }
    if (!dyn_dev || !cell_pos_dev) { pi_set_error("pi_op_qkv_prepare: the pass's cell table and the cells' position array are required"); return -1; }
    if (pairing != PI_PAIR_HALVES && pairing != PI_PAIR_NEIGHBOURS) { pi_set_error("pi_op_qkv_prepare: pairing %d is unknown", pairing); return -1; }
    if (norm_first < 0 || norm_first > PI_QK_NORM_NONE) { pi_set_error("pi_op_qkv_prepare: norm order %d is unknown", norm_first); return -1; }
    if (norm_first == PI_QK_NORM_FIRST && (!q_norm_w || !k_norm_w)) { pi_set_error("pi_op_qkv_prepare: norm weights are required"); return -1; }
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 8.0 * n_tok * ((double) heads * dim + (double) kv_heads * (dim + vdim)), k_qkv_prepare_any, dim3((unsigned) n_tok, (unsigned) (heads + 2 * kv_heads)), dim3(64), 0, (hipStream_t) stream,
                 q, k, v, stride, q_norm_w, k_norm_w, eps, heads, kv_heads, dim, vdim, rt->cs, rt->half, rt->n_pos, norm_first, pairing, v_norm, pos_dev, q_out, q_out_stride, k_cache, v_cache, cell_pos_dev, dyn_dev, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}

// ---- attention with sigmoid weights inside chunks ---------------------------------------------------------------------------------------------------------
// grid (token, key / value head, split of its query heads): the workgroup serves the query heads of its key head (all of them in one workgroup unless they are very many or very wide).  The cells are walked 256 at a time; the visible ones of a round are compacted
// in cell order (so that the sum has one order whatever the launch), their key rows staged in LDS 64 at a time.  Scores: thread (cell, query head); output: thread (query
// head, value column), value rows read from the cache along the columns.
// rows `cells[0 .. nl)` of a cache [cells][G][W] (head g) into LDS rows `pitch` floats apart.  Eight loads per thread are issued before the first LDS store: the compiler cannot
// tell the cell list (LDS) from the tile (LDS) and would otherwise wait for every row's trip to memory before it reads the next cell number
// RPW: rows a wave has in flight per round
template <int RPW>
static __device__ __forceinline__ void ca_stage(const float * __restrict__ cache, const int * cells, int nl, int G, int g, int W, int pitch, float * tile, int tid) {
    const int lane = tid & 63, wave = tid >> 6;
    if (W <= 128) {                                                   // a wave per row, two columns per lane, RPW rows per round: no index arithmetic beyond adds
        for (int r0 = wave; r0 < nl; r0 += 4 * RPW) {
            float tmp[2 * RPW];
#pragma unroll
            for (int u = 0; u < RPW; u++) {
                const int cc = r0 + u * 4;
                const float * row = cache + ((int64_t) cells[min(cc, nl - 1)] * G + g) * W;
                tmp[2 * u] = cc < nl && lane < W ? row[lane] : 0.0f;
                tmp[2 * u + 1] = cc < nl && lane + 64 < W ? row[lane + 64] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < RPW; u++) {
                const int cc = r0 + u * 4;
                if (cc < nl && lane < W) tile[cc * pitch + lane] = tmp[2 * u];
                if (cc < nl && lane + 64 < W) tile[cc * pitch + lane + 64] = tmp[2 * u + 1];
            }
        }
        return;
    }
    const int total = nl * W;
    for (int base = 0; base < total; base += 256 * 8) {
        float tmp[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int i = base + u * 256 + tid;
            tmp[u] = i < total ? cache[((int64_t) cells[i / W] * G + g) * W + i % W] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int i = base + u * 256 + tid;
            if (i < total) tile[(i / W) * pitch + i % W] = tmp[u];
        }
    }
}
#define CA_TILE 64                                // key rows staged at a time (fewer when a row is long: ca_tile)
#define CA_SB 1                                   // blocks of 256 cells whose visibility is worked out in one round
#define CA_MAXOUT 16                              // outputs (query head, value column) a thread accumulates: hpg * vdim <= 256 * CA_MAXOUT
template <int RPW>
__global__ void __launch_bounds__(256) k_chunk_attention(const float * __restrict__ q, int64_t qs, const float * kc, const float * vc, const int32_t * __restrict__ cell_pos,
                                                         const uint32_t * __restrict__ mask, const int32_t * __restrict__ pos, const float * __restrict__ hbias, const float * __restrict__ gate, int64_t gs, int gate_act,
                                                         float scale, float out_mult, int weights, float softcap, int chunk, int H, int G, int D, int V, int n_kv_arg, int tile, int hps, float * __restrict__ out, int64_t os, const int32_t * __restrict__ dyn,
                                                         const float * __restrict__ sink, int mask_kind, int pool, int pool_off, int pool_z, int n_hz, int n_cs, int split_cells, float * __restrict__ part, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w, 5)) return;
    extern __shared__ float lds[];                // q [hpg][D] | key tile [tile][D + 1], then the value tile [tile][V] in the same place | weights [tile][hpg]
    if (pool_z > 0 && (int) blockIdx.z == pool_z) {                   // the extra slice of workgroups: the pooled rows of the blocks this pass's tokens close (no token of the pass reads them: the host checked n_tok <= window)
        const int p = pos[blockIdx.x];
        if ((p + 1) % pool != 0) return;
        pm_pool_block((float *) kc, (float *) vc, cell_pos, mask + (int64_t) blockIdx.x * ((n_kv_arg + 31) / 32), p, pool, pool_off, G, blockIdx.y, D, V, min(dyn ? dyn[1] : n_kv_arg, n_kv_arg), pi_cell_of(dyn, 0, blockIdx.x), (int *) lds);
        return;
    }
    __shared__ int list[256 * CA_SB], wcnt[4 * CA_SB];
    const int t = blockIdx.x, g = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // blockIdx.z = head split + n_hz * cell split.  split_cells > 0 (soft-max kinds, few tokens): this workgroup looks at the cells [cs * split_cells, (cs + 1) * split_cells) only and leaves its running
    // maximum, denominator and un-normalised sums in `part` for k_attention_combine: a single token's tiles then run side by side instead of one after the other
    const int hz = (int) blockIdx.z % n_hz, cs = (int) blockIdx.z / n_hz;
    const int hs = hz * hps, hpg = min(hps, H / G - hs), h0 = g * (H / G) + hs, DP = D + 1;        // this workgroup's query heads: hpg of them from h0 on (all of the key head's unless they are split over blockIdx.z)
    float * qsh = lds, * ksh = qsh + hpg * D, * wsh = ksh + tile * max(DP, V);
    float * m_run = wsh + tile * hps, * l_run = m_run + hps, * f_run = l_run + hps;        // soft-max weights: per query head the running maximum, denominator, and the factor the sums so far take this tile
    const bool soft = weights != PI_WEIGHTS_SIGMOID;
    // (a sink: one more key without a value, of score 0 or of a learned score per head that the scale does not touch)
    if (soft) for (int m = tid; m < hpg; m += 256) {
        const bool has_sink = split_cells == 0 && (sink || weights == PI_WEIGHTS_SOFTMAX_SINK);           // (with cell splits the sink joins in the combine)
        m_run[m] = has_sink ? (sink ? sink[h0 + m] : 0.0f) : -INFINITY; l_run[m] = has_sink ? 1.0f : 0.0f;
    }
    const int n_kv = min(dyn ? dyn[1] : n_kv_arg, n_kv_arg);
    const int words = (n_kv_arg + 31) / 32;
    const uint32_t * mrow = mask + (int64_t) t * words;
    const int p = pos[t];
    // the first position the token sees as itself: the start of its block of `chunk` positions, or of the window of `chunk` positions that ends with the token
    const int first_pos = chunk <= 0 ? 0 : mask_kind == PI_MASK_WINDOW ? p - chunk + 1 : p / chunk * chunk;
    for (int i = tid; i < hpg * D; i += 256) qsh[i] = q[(int64_t) t * qs + (int64_t) h0 * D + i];
    float acc[CA_MAXOUT];
#pragma unroll
    for (int i = 0; i < CA_MAXOUT; i++) acc[i] = 0.0f;
    const int n_out = hpg * V;
    const int c_first = split_cells > 0 ? cs * split_cells : 0, c_end = split_cells > 0 ? min(n_kv, c_first + split_cells) : n_kv;
    for (int c0 = c_first; c0 < c_end; c0 += 256 * CA_SB) {          // CA_SB blocks of 256 cells at a time: their mask words and positions are loaded together
        bool vis[CA_SB], far[CA_SB]; unsigned long long bal[CA_SB];
#pragma unroll
        for (int u = 0; u < CA_SB; u++) {
            const int c = c0 + u * 256 + tid;
            const bool in = c < c_end;
            const uint32_t word = in ? mrow[c >> 5] : 0u;
            const int cp = in ? cell_pos[c] : -1;
            // behind the window a cell counts where it closes a block of `pool` positions, through the block's pooled row (row pool_off + cell of both caches)
            far[u] = pool > 0 && cp < first_pos && cp >= 0 && (cp + 1) % pool == 0;
            vis[u] = in && ((word >> (c & 31)) & 1u) && (cp >= first_pos || far[u]);
        }
#pragma unroll
        for (int u = 0; u < CA_SB; u++) bal[u] = __ballot(vis[u]);
        __syncthreads();                          // (the previous round's list and tiles are no longer read)
        if (lane == 0)
#pragma unroll
            for (int u = 0; u < CA_SB; u++) wcnt[u * 4 + wave] = __popcll(bal[u]);
        __syncthreads();
        int total = 0, mine[CA_SB];               // cell order: block, then wave, then lane
#pragma unroll
        for (int u = 0; u < CA_SB; u++)
#pragma unroll
            for (int w = 0; w < 4; w++) { if (w == wave) mine[u] = total; total += wcnt[u * 4 + w]; }
        if (total == 0) continue;
#pragma unroll
        for (int u = 0; u < CA_SB; u++) if (vis[u]) list[mine[u] + __popcll(bal[u] & ((1ull << lane) - 1ull))] = c0 + u * 256 + tid + (far[u] ? pool_off : 0);
        __syncthreads();
        for (int l0 = 0; l0 < total; l0 += tile) {
            const int nl = min(tile, total - l0);
            if (l0) __syncthreads();                 // (the previous tile's values are no longer read)
            ca_stage<RPW>(kc, list + l0, nl, G, g, D, DP, ksh, tid);
            __syncthreads();
            for (int i = tid; i < nl * hpg; i += 256) {
                const int cc = i % nl, m = i / nl;
                const float * kr = ksh + cc * DP, * qr = qsh + m * D;
                float s = 0.0f;
                for (int d = 0; d < D; d++) s = fmaf(qr[d], kr[d], s);
                s = s * scale + (hbias ? hbias[h0 + m] : 0.0f);
                if (soft && softcap > 0.0f) s = softcap * tanhf(s / softcap);
                wsh[cc * hpg + m] = soft ? s : pm_sigmoid(s);
            }
            __syncthreads();
            if (soft)                             // a wave per query head, a lane per cell of the tile (tile <= 64): new maximum, exponentials in the scores' place, denominator
                for (int m = wave; m < hpg; m += 4) {
                    const float sc = lane < nl ? wsh[lane * hpg + m] : -INFINITY;
                    const float m_old = m_run[m], m_new = fmaxf(m_old, pi_wave_max(sc));
                    const float e = lane < nl ? expf(sc - m_new) : 0.0f;
                    const float sum = pi_lanes_sum<64>(e);
                    if (lane < nl) wsh[lane * hpg + m] = e;
                    if (lane == 0) { const float f = m_old == -INFINITY ? 0.0f : expf(m_old - m_new); m_run[m] = m_new; l_run[m] = fmaf(l_run[m], f, sum); f_run[m] = f; }
                }
            // the value rows take the key tile's place: all their loads are in flight together (read one by one in the sum below, every row would cost a trip to memory)
            ca_stage<RPW>(vc, list + l0, nl, G, g, V, V, ksh, tid);
            __syncthreads();
#pragma unroll
            for (int oi = 0; oi < CA_MAXOUT; oi++) {
                const int o = oi * 256 + tid;
                if (o < n_out) {
                    const int m = o / V, vv = o % V;
                    float a = soft ? acc[oi] * f_run[m] : acc[oi];
                    for (int cc = 0; cc < nl; cc++) a = fmaf(wsh[cc * hpg + m], ksh[cc * V + vv], a);
                    acc[oi] = a;
                }
            }
        }
    }
    if (split_cells > 0) {                                            // this split's share: [V sums | maximum | denominator] per (token, head, split)
        __syncthreads();
#pragma unroll
        for (int oi = 0; oi < CA_MAXOUT; oi++) {
            const int o = oi * 256 + tid;
            if (o < n_out) { const int m = o / V; part[(((int64_t) t * H + h0 + m) * n_cs + cs) * (V + 2) + o % V] = acc[oi]; }
        }
        for (int m = tid; m < hpg; m += 256) { float * pr = part + (((int64_t) t * H + h0 + m) * n_cs + cs) * (V + 2) + V; pr[0] = m_run[m]; pr[1] = l_run[m]; }
        return;
    }
#pragma unroll
    for (int oi = 0; oi < CA_MAXOUT; oi++) {
        const int o = oi * 256 + tid;
        if (o < n_out) {
            const int m = o / V;
            float gt = gate ? gate[(int64_t) t * gs + h0 + m] : 1.0f;
            if (gate && gate_act == PI_ACT_SIGMOID) gt = pm_sigmoid(gt);
            const float den = soft ? l_run[m] : 1.0f;
            out[(int64_t) t * os + (int64_t) h0 * V + o] = (soft ? (den > 0.0f ? acc[oi] / den : 0.0f) : acc[oi]) * gt * out_mult;
        }
    }
}

// the cell splits of a token's head merged: M = max(maxima, sink), out = sum_s e^(m_s - M) sums_s / (e^(sink - M) + sum_s e^(m_s - M) l_s), in split order; grid (token, head)
__global__ void __launch_bounds__(128) k_attention_combine(const float * __restrict__ part, int n_cs, int H, int V, const float * __restrict__ sink, int weights, const float * __restrict__ gate, int64_t gs, int gate_act,
                                                           float out_mult, float * __restrict__ out, int64_t os, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    const int t = blockIdx.x, h = blockIdx.y;
    const float * pr = part + ((int64_t) t * H + h) * n_cs * (V + 2);
    const bool has_sink = sink || weights == PI_WEIGHTS_SOFTMAX_SINK;
    const float sk = sink ? sink[h] : 0.0f;
    float M = has_sink ? sk : -INFINITY;
    for (int s = 0; s < n_cs; s++) M = fmaxf(M, pr[(int64_t) s * (V + 2) + V]);
    float den = has_sink ? expf(sk - M) : 0.0f;
    for (int s = 0; s < n_cs; s++) { const float ms = pr[(int64_t) s * (V + 2) + V]; if (ms != -INFINITY) den = fmaf(pr[(int64_t) s * (V + 2) + V + 1], expf(ms - M), den); }
    float gt = gate ? gate[(int64_t) t * gs + h] : 1.0f;
    if (gate && gate_act == PI_ACT_SIGMOID) gt = pm_sigmoid(gt);
    for (int v = threadIdx.x; v < V; v += 128) {
        float a = 0.0f;
        for (int s = 0; s < n_cs; s++) { const float ms = pr[(int64_t) s * (V + 2) + V]; if (ms != -INFINITY) a = fmaf(pr[(int64_t) s * (V + 2) + v], expf(ms - M), a); }
        out[(int64_t) t * os + (int64_t) h * V + v] = (den > 0.0f ? a / den : 0.0f) * gt * out_mult;
    }
}
// cell splits of a pass of n_tok tokens over n_kv cells: how many, and the floats of scratch they need (0 splits: the pass is wide enough to fill the device by itself)
#define CA_SPLIT_MAX 32
static int ca_cell_splits(int n_tok, int kv_heads, int n_hz, int n_kv, int * split_cells) {
    if ((int64_t) n_tok * kv_heads * n_hz > 64 || n_kv <= 64) return 0;
    const int n_cs = std::min(CA_SPLIT_MAX, (n_kv + 63) / 64);
    *split_cells = ((n_kv + n_cs - 1) / n_cs + 63) / 64 * 64;
    return (n_kv + *split_cells - 1) / *split_cells;
}
extern "C" size_t pi_op_window_attention_scratch_floats(int heads, int vdim, int n_tok) { return (size_t) std::min(n_tok, 64) * heads * CA_SPLIT_MAX * (vdim + 2); }

extern "C" int pi_op_chunk_attention(const float * q, int64_t q_stride, const float * k_cache, const float * v_cache, const int32_t * cell_pos_dev, const uint32_t * mask_dev, const int32_t * pos_dev,
                                     const float * head_bias_dev, const float * gate_dev, int64_t gate_stride, int gate_act, float scale, float out_mult, int chunk, int heads, int kv_heads, int dim, int vdim, int n_tok, int n_kv,
                                     float * out, int64_t out_stride, const int32_t * dyn_dev, void * stream) {
    return pi_op_chunk_attention_ex(q, q_stride, k_cache, v_cache, cell_pos_dev, mask_dev, pos_dev, head_bias_dev, gate_dev, gate_stride, gate_act, scale, out_mult, PI_WEIGHTS_SIGMOID, 0.0f, chunk, heads, kv_heads, dim, vdim,
                                    n_tok, n_kv, out, out_stride, dyn_dev, stream);
}
extern "C" int pi_op_chunk_attention_ex(const float * q, int64_t q_stride, const float * k_cache, const float * v_cache, const int32_t * cell_pos_dev, const uint32_t * mask_dev, const int32_t * pos_dev,
                                        const float * head_bias_dev, const float * gate_dev, int64_t gate_stride, int gate_act, float scale, float out_mult, int weights, float softcap, int chunk, int heads, int kv_heads,
                                        int dim, int vdim, int n_tok, int n_kv, float * out, int64_t out_stride, const int32_t * dyn_dev, void * stream) {
    return pi_op_window_attention(q, q_stride, (float *) k_cache, (float *) v_cache, cell_pos_dev, mask_dev, pos_dev, head_bias_dev, nullptr, gate_dev, gate_stride, gate_act, scale, out_mult, weights, softcap, PI_MASK_CHUNK, chunk, 0, 0, 0,
                                  heads, kv_heads, dim, vdim, n_tok, n_kv, nullptr, 0, out, out_stride, dyn_dev, stream);
}
// the same kernel with the mask kind, pooled far blocks and a learned sink as parameters (`chunk` is the block's or the window's size)
extern "C" int pi_op_window_attention(const float * q, int64_t q_stride, float * k_cache, float * v_cache, const int32_t * cell_pos_dev, const uint32_t * mask_dev, const int32_t * pos_dev,
                                      const float * head_bias_dev, const float * sink_dev, const float * gate_dev, int64_t gate_stride, int gate_act, float scale, float out_mult, int weights, float softcap, int mask_kind, int chunk,
                                      int pool, int64_t pooled_row_offset, int pool_here, int heads, int kv_heads, int dim, int vdim, int n_tok, int n_kv, float * scratch, size_t scratch_floats, float * out, int64_t out_stride,
                                      const int32_t * dyn_dev, void * stream) {
    if (n_tok <= 0) return 0;
    if (mask_kind != PI_MASK_CHUNK && mask_kind != PI_MASK_WINDOW) { pi_set_error("pi_op_window_attention: mask kind %d is unknown", mask_kind); return -1; }
    if (pool < 0 || (pool > 0 && (mask_kind != PI_MASK_WINDOW || chunk < 1 || pooled_row_offset < n_kv || pooled_row_offset > 0x3fffffff))) { pi_set_error("pi_op_window_attention: pooled blocks need a window and their rows behind the %d cells", n_kv); return -1; }
    if (sink_dev && weights == PI_WEIGHTS_SIGMOID) { pi_set_error("pi_op_window_attention: a sink belongs to a soft-max"); return -1; }
    if (pool_here && (pool < 1 || n_tok > chunk || !dyn_dev)) { pi_set_error("pi_op_window_attention: pooled rows can be written in the same launch only where no token of the pass reads them (%d tokens, window %d)", n_tok, chunk); return -1; }
    if (weights != PI_WEIGHTS_SIGMOID && weights != PI_WEIGHTS_SOFTMAX && weights != PI_WEIGHTS_SOFTMAX_SINK) { pi_set_error("pi_op_chunk_attention: weights of kind %d are unknown", weights); return -1; }
    if (heads < 1 || kv_heads < 1 || heads % kv_heads || dim < 1 || vdim < 1 || chunk < 0) { pi_set_error("pi_op_chunk_attention: %d query heads over %d key / value heads, sizes %d / %d, chunk %d", heads, kv_heads, dim, vdim, chunk); return -1; }
    int hpg = heads / kv_heads, splits = 1;                            // query heads of a key head that one workgroup serves: all of them, unless their outputs or the LDS plan say otherwise
    while (hpg > 1 && (hpg * vdim > 256 * CA_MAXOUT || (size_t) hpg * dim * sizeof(float) > 24 * 1024)) { splits *= 2; hpg = (heads / kv_heads + splits - 1) / splits; }
    int tile = CA_TILE;
    auto lds_of = [&](int tl) { return ((size_t) hpg * dim + (size_t) tl * std::max(dim + 1, vdim) + (size_t) tl * hpg + (size_t) 3 * hpg) * sizeof(float); };
    while (tile > 4 && lds_of(tile) > 60 * 1024) tile >>= 1;
    const size_t lds = std::max(lds_of(tile), pool_here ? (size_t) pool * sizeof(int) : (size_t) 0);
    const int n_z = (heads / kv_heads + hpg - 1) / hpg;
    // few tokens and a soft-max: the cell range is cut into splits that run side by side, merged by a second small launch (needs scratch for every split's share)
    int split_cells = 0, n_cs = weights != PI_WEIGHTS_SIGMOID && scratch ? ca_cell_splits(n_tok, kv_heads, n_z, n_kv, &split_cells) : 0;
    if (n_cs < 2 || (size_t) n_tok * heads * n_cs * (vdim + 2) > scratch_floats) { n_cs = 1; split_cells = 0; }
    if (hpg * vdim > 256 * CA_MAXOUT || lds > 60 * 1024) { pi_set_error("pi_op_chunk_attention: %d query heads per key head of sizes %d / %d are beyond the kernel (LDS %zu bytes)", hpg, dim, vdim, lds); return -1; }
    const int acct = pi_account_n_kv() > 0 ? pi_account_n_kv() : n_kv;
    const double visible = chunk > 0 ? std::min(acct, chunk) + (pool > 0 ? std::max(acct - chunk, 0) / pool : 0) : acct;
#define CA_GO(R)     PI_KT_LAUNCH(PI_KT_ATT, 0, std::min(n_tok, PI_KT_MAXNT - 1), 4.0 * visible * kv_heads * (dim + vdim) + 4.0 * n_tok * heads * (dim + vdim), k_chunk_attention<R>, dim3((unsigned) n_tok, (unsigned) kv_heads, (unsigned) (n_z * n_cs + (pool_here ? 1 : 0))), dim3(256), lds, \
                 (hipStream_t) stream, q, q_stride, k_cache, v_cache, cell_pos_dev, mask_dev, pos_dev, head_bias_dev, gate_dev, gate_stride, gate_act, scale, out_mult, weights, softcap, chunk, heads, kv_heads, dim, vdim, n_kv, tile, hpg, out, out_stride, \
                 dyn_dev, sink_dev, mask_kind, pool, (int) pooled_row_offset, pool_here ? n_z * n_cs : 0, n_z, n_cs, split_cells, scratch, pi_abort_word());
    CA_GO(4);                                                          // (deeper rounds were measured for single tokens: no gain, the registers they take cost as much as the trips they save)
#undef CA_GO
    PI_CHECK_LAUNCH();
    if (split_cells > 0) {
        PI_KT_LAUNCH(PI_KT_ATT, 0, std::min(n_tok, PI_KT_MAXNT - 1), 4.0 * n_tok * heads * ((double) n_cs * (vdim + 2) + vdim), k_attention_combine, dim3((unsigned) n_tok, (unsigned) heads), dim3(128), 0, (hipStream_t) stream,
                     scratch, n_cs, heads, vdim, sink_dev, weights, gate_dev, gate_stride, gate_act, out_mult, out, out_stride, pi_abort_word());
        PI_CHECK_LAUNCH();
    }
    return 0;
}

// ---- pooled far blocks: one key / value per block of `pool` positions ------------------------------------------------------------------------------------------
// grid (token, key / value head).  Only a token that closes a block works: it finds the cells of the block's positions among the cells its mask row shows (its own and the pass's earlier ones
// included: call this behind the launch that stores the pass's keys and values), sums their rows in position order and leaves the means in row pool_off + its own cell of both caches.
__global__ void __launch_bounds__(256) k_pool_blocks(float * __restrict__ kc, float * __restrict__ vc, const int32_t * __restrict__ cell_pos, const uint32_t * __restrict__ mask, const int32_t * __restrict__ pos,
                                                     int pool, int64_t pool_off, int G, int D, int V, int n_kv_arg, const int32_t * __restrict__ dyn, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    extern __shared__ int members[];              // [pool] the cell of every position of the block (-1: none)
    const int t = blockIdx.x, g = blockIdx.y;
    const int p = pos[t];
    if ((p + 1) % pool != 0) return;
    const int n_kv = min(dyn ? dyn[1] : n_kv_arg, n_kv_arg), words = (n_kv_arg + 31) / 32;
    pm_pool_block(kc, vc, cell_pos, mask + (int64_t) t * words, p, pool, pool_off, G, g, D, V, n_kv, pi_cell_of(dyn, 0, t), members);
}
extern "C" int pi_op_pool_blocks(float * k_cache, float * v_cache, const int32_t * cell_pos_dev, const uint32_t * mask_dev, const int32_t * pos_dev, int pool, int64_t pooled_row_offset, int kv_heads, int dim, int vdim,
                                 int n_tok, int n_kv, const int32_t * dyn_dev, void * stream) {
    if (n_tok <= 0) return 0;
    if (pool < 1 || pool > 8192 || pooled_row_offset < n_kv || kv_heads < 1 || dim < 1 || vdim < 1 || !dyn_dev) { pi_set_error("pi_op_pool_blocks: blocks of %d positions (1..8192), pooled rows from row %lld on behind %d cells", pool, (long long) pooled_row_offset, n_kv); return -1; }
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 4.0 * ((double) n_tok / pool + 1.0) * kv_heads * (dim + vdim) * (pool + 1), k_pool_blocks, dim3((unsigned) n_tok, (unsigned) kv_heads), dim3(256), (size_t) pool * sizeof(int), (hipStream_t) stream,
                 k_cache, v_cache, cell_pos_dev, mask_dev, pos_dev, pool, pooled_row_offset, kv_heads, dim, vdim, n_kv, dyn_dev, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}

// ---- short causal convolution over the tokens of each sequence ----------------------------------------------------------------------------------------------
// rec[t]: state slot of token t's sequence (| 1 << 30 on the first token of a sequence that starts from nothing); a sequence's tokens are consecutive.
// state: [slots][taps - 1][channels], the sequence's last inputs, oldest first.  grid (token, blocks of 256 channels)
__global__ void __launch_bounds__(256) k_causal_conv(const float * __restrict__ x, int64_t xs, int channels, int taps, const float * __restrict__ w, const float * __restrict__ bias,
                                                     const float * __restrict__ state, const int32_t * __restrict__ rec, int act, float * __restrict__ out, int64_t os, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= channels) return;
    const int slot = rec[t] & ~PM_FRESH;
    int d = 0, fresh = 0;                                             // d: tokens of this sequence in the pass before t (counted up to taps - 1)
    while (d < taps - 1 && t - d - 1 >= 0 && (rec[t - d - 1] & ~PM_FRESH) == slot) d++;
    if (d < taps - 1) fresh = (rec[t - d] & PM_FRESH) != 0;           // (t - d is then the sequence's first token of the pass)
    float a = bias ? bias[c] : 0.0f;
    for (int l = 0; l < taps; l++) {                                  // tap l weighs the input `taps - 1 - l` tokens back
        const int back = taps - 1 - l;
        float v;
        if (back <= d) v = x[(int64_t) (t - back) * xs + c];
        else v = fresh ? 0.0f : state[((int64_t) slot * (taps - 1) + (taps - 1 - (back - d))) * channels + c];
        a = fmaf(w[(int64_t) c * taps + l], v, a);
    }
    if (act == PI_ACT_SILU) a = a / (1.0f + expf(-a));
    out[(int64_t) t * os + c] = a;
}
// grid (token, blocks of 256 channels): only a sequence's last token of the pass works, it rewrites its slot's rows oldest first (a row only ever takes a later row's value)
__global__ void __launch_bounds__(256) k_conv_state_update(const float * __restrict__ x, int64_t xs, int channels, int taps, float * __restrict__ state, const int32_t * __restrict__ rec, int n_tok,
                                                           const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    const int slot = rec[t] & ~PM_FRESH;
    if (t + 1 < n_tok && (rec[t + 1] & ~PM_FRESH) == slot) return;
    if (c >= channels) return;
    int len = 1, fresh = 0;                                           // tokens of the sequence in this pass, counted up to taps - 1
    while (len < taps - 1 && t - len >= 0 && (rec[t - len] & ~PM_FRESH) == slot) len++;
    if (len < taps - 1) fresh = (rec[t - len + 1] & PM_FRESH) != 0;
    float * st = state + (int64_t) slot * (taps - 1) * channels + c;
    for (int i = 0; i < taps - 1; i++) {
        const int from = i + len;                                     // row of (old state, then the pass's tokens) that becomes row i
        float v;
        if (from < taps - 1) v = fresh ? 0.0f : st[(int64_t) from * channels];
        else v = x[(int64_t) (t - len + 1 + from - (taps - 1)) * xs + c];
        st[(int64_t) i * channels] = v;
    }
}

static bool pi_causal_conv_walk_ok(int n_tok, int taps);
static int pi_causal_conv_walk(const float * x, int64_t x_stride, int channels, int taps, const float * w_dev, const float * bias_dev, float * state_dev, const int32_t * rec_dev, int n_tok, int act, float * out,
                               int64_t out_stride, hipStream_t s);
extern "C" int pi_op_causal_conv(const float * x, int64_t x_stride, int channels, int taps, const float * w_dev, const float * bias_dev, float * state_dev, const int32_t * rec_dev, int n_tok, int act,
                                 float * out, int64_t out_stride, void * stream) {
    if (n_tok <= 0 || channels <= 0) return 0;
    if (taps < 1 || taps > 64) { pi_set_error("pi_op_causal_conv: %d taps (1..64)", taps); return -1; }
    if (out == x) { pi_set_error("pi_op_causal_conv: the output may not overwrite the input (later tokens and the state read it)"); return -1; }
    hipStream_t s = (hipStream_t) stream;
    if (pi_causal_conv_walk_ok(n_tok, taps)) return pi_causal_conv_walk(x, x_stride, channels, taps, w_dev, bias_dev, state_dev, rec_dev, n_tok, act, out, out_stride, s);      // short passes: one launch, the state included
    const dim3 grid((unsigned) n_tok, (unsigned) ((channels + 255) / 256));
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 8.0 * n_tok * channels + 4.0 * channels * taps, k_causal_conv, grid, dim3(256), 0, s, x, x_stride, channels, taps, w_dev, bias_dev, state_dev, rec_dev, act, out, out_stride, pi_abort_word());
    PI_CHECK_LAUNCH();
    if (taps > 1) {
        PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 8.0 * (taps - 1) * channels, k_conv_state_update, grid, dim3(256), 0, s, x, x_stride, channels, taps, state_dev, rec_dev, n_tok, pi_abort_word());
        PI_CHECK_LAUNCH();
    }
    return 0;
}

// Short passes (decoding, small portions) in ONE launch: the thread of a sequence's FIRST token of the pass walks that sequence's tokens for its channel with the window in
// registers and leaves the new state, so no other thread reads what it writes; one extra row of blocks computes the recurrence's step sizes and decays meanwhile.
#define CV_MAXTAPS 8
__global__ void __launch_bounds__(256) k_causal_conv_walk(const float * __restrict__ x, int64_t xs, int channels, int taps, const float * __restrict__ w, const float * __restrict__ bias,
                                                          float * __restrict__ state, const int32_t * __restrict__ rec, int n_tok, int act, float * __restrict__ out, int64_t os, int cblocks,
                                                          const float * __restrict__ raw, int64_t raws, const float * __restrict__ dt_bias, const float * __restrict__ a_log, int heads,
                                                          float * __restrict__ dt, float * __restrict__ decay, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    const int t = blockIdx.x;
    if ((int) blockIdx.y == cblocks) {                                // step sizes and decays of token t
        for (int h = threadIdx.x; h < heads; h += 256) {
            const float z = raw[(int64_t) t * raws + h] + dt_bias[h];
            const float sp = z > 20.0f ? z : log1pf(expf(z));
            dt[(int64_t) t * heads + h] = sp;
            decay[(int64_t) t * heads + h] = expf(-expf(a_log[h]) * sp);
        }
        return;
    }
    const int c = blockIdx.y * 256 + threadIdx.x;
    const int word = rec[t], slot = word & ~PM_FRESH;
    if (c >= channels || (t > 0 && (rec[t - 1] & ~PM_FRESH) == slot)) return;
    float win[CV_MAXTAPS - 1], wt[CV_MAXTAPS];                         // right-aligned (the last entries are the most recent input / the current token's tap): every register index is static
    const int off = CV_MAXTAPS - taps;
    float * st = state + (int64_t) slot * (taps - 1) * channels + c;
#pragma unroll
    for (int l = 0; l < CV_MAXTAPS - 1; l++) win[l] = l >= off && !(word & PM_FRESH) ? st[(int64_t) (l - off) * channels] : 0.0f;
#pragma unroll
    for (int l = 0; l < CV_MAXTAPS; l++) wt[l] = l >= off ? w[(int64_t) c * taps + (l - off)] : 0.0f;
    const float b0 = bias ? bias[c] : 0.0f;
    for (int tt = t; tt < n_tok && (rec[tt] & ~PM_FRESH) == slot; tt++) {
        const float v = x[(int64_t) tt * xs + c];
        float a = b0;
#pragma unroll
        for (int l = 0; l < CV_MAXTAPS - 1; l++) a = fmaf(wt[l], win[l], a);       // (entries left of the window carry zero weights)
        a = fmaf(wt[CV_MAXTAPS - 1], v, a);
#pragma unroll
        for (int l = 0; l < CV_MAXTAPS - 2; l++) win[l] = win[l + 1];
        win[CV_MAXTAPS - 2] = v;
        if (act == PI_ACT_SILU) a = a / (1.0f + expf(-a));
        out[(int64_t) tt * os + c] = a;
    }
#pragma unroll
    for (int l = 0; l < CV_MAXTAPS - 1; l++) if (l >= off) st[(int64_t) (l - off) * channels] = win[l];
}
#define CV_WALK_MAX_TOKENS 32
static bool pi_causal_conv_walk_ok(int n_tok, int taps) { return n_tok <= CV_WALK_MAX_TOKENS && taps <= CV_MAXTAPS; }
// the walking kernel without the row of blocks that forms step sizes
static int pi_causal_conv_walk(const float * x, int64_t x_stride, int channels, int taps, const float * w_dev, const float * bias_dev, float * state_dev, const int32_t * rec_dev, int n_tok, int act, float * out,
                               int64_t out_stride, hipStream_t s) {
    const int cblocks = (channels + 255) / 256;
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 8.0 * n_tok * channels + 4.0 * channels * (2 * taps - 1), k_causal_conv_walk, dim3((unsigned) n_tok, (unsigned) cblocks), dim3(256), 0, s,
                 x, x_stride, channels, taps, w_dev, bias_dev, state_dev, rec_dev, n_tok, act, out, out_stride, cblocks, (const float *) nullptr, (int64_t) 0, (const float *) nullptr, (const float *) nullptr, 0,
                 (float *) nullptr, (float *) nullptr, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}
// the convolution and, in the same launch where the pass is short, the step sizes / decays of the recurrence it feeds (raw_dev .. decay_out as for pi_op_ssd_steps)
extern "C" int pi_op_causal_conv_steps(const float * x, int64_t x_stride, int channels, int taps, const float * w_dev, const float * bias_dev, float * state_dev, const int32_t * rec_dev, int n_tok, int act,
                                       float * out, int64_t out_stride, const float * raw, int64_t raw_stride, const float * dt_bias_dev, const float * a_log_dev, int heads, float * dt_out, float * decay_out,
                                       void * stream) {
    if (n_tok <= 0 || channels <= 0) return 0;
    if (taps < 1 || taps > 64) { pi_set_error("pi_op_causal_conv: %d taps (1..64)", taps); return -1; }
    if (n_tok > CV_WALK_MAX_TOKENS || taps > CV_MAXTAPS) {
        if (pi_op_causal_conv(x, x_stride, channels, taps, w_dev, bias_dev, state_dev, rec_dev, n_tok, act, out, out_stride, stream) != 0) return -1;
        return pi_op_ssd_steps(raw, raw_stride, dt_bias_dev, a_log_dev, heads, n_tok, dt_out, decay_out, stream);
    }
    if (out == x) { pi_set_error("pi_op_causal_conv: the output may not overwrite the input"); return -1; }
    const int cblocks = (channels + 255) / 256;
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 8.0 * n_tok * channels + 4.0 * channels * (2 * taps - 1) + 12.0 * n_tok * heads, k_causal_conv_walk, dim3((unsigned) n_tok, (unsigned) (cblocks + 1)), dim3(256), 0, (hipStream_t) stream,
                 x, x_stride, channels, taps, w_dev, bias_dev, state_dev, rec_dev, n_tok, act, out, out_stride, cblocks, raw, raw_stride, dt_bias_dev, a_log_dev, heads, dt_out, decay_out, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}

// ---- step sizes and decays of a selective recurrence ---------------------------------------------------------------------------------------------------------
__global__ void k_ssd_steps(const float * __restrict__ raw, int64_t rs, const float * __restrict__ dt_bias, const float * __restrict__ a_log, int heads, int n_tok, float * __restrict__ dt,
                            float * __restrict__ decay, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n_tok * heads) return;
    const int t = i / heads, h = i % heads;
    const float z = raw[(int64_t) t * rs + h] + dt_bias[h];
    const float sp = z > 20.0f ? z : log1pf(expf(z));                 // (beyond 20 the two agree to the last bit of fp32)
    dt[i] = sp;
    decay[i] = expf(-expf(a_log[h]) * sp);
}
extern "C" int pi_op_ssd_steps(const float * raw, int64_t raw_stride, const float * dt_bias_dev, const float * a_log_dev, int heads, int n_tok, float * dt_out, float * decay_out, void * stream) {
    if (n_tok <= 0) return 0;
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 12.0 * n_tok * heads, k_ssd_steps, dim3((unsigned) ((n_tok * heads + 255) / 256)), dim3(256), 0, (hipStream_t) stream, raw, raw_stride, dt_bias_dev, a_log_dev, heads, n_tok,
                 dt_out, decay_out, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}

// ---- gate, then RMS norm in equal parts -------------------------------------------------------------------------------------------------------------------
// grid (token, part)
__global__ void __launch_bounds__(256) k_gate_group_norm(const float * __restrict__ y, int64_t ys, const float * __restrict__ z, int64_t zs, const float * __restrict__ w, float eps, float mult, int n, int groups,
                                                         float * __restrict__ out, int64_t os, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    __shared__ float red[4];
    const int t = blockIdx.x, part = n / groups, i0 = blockIdx.y * part;
    const float * yr = y + (int64_t) t * ys + i0, * zr = z + (int64_t) t * zs + i0;
    float ss = 0.0f;
    for (int i = threadIdx.x; i < part; i += 256) { const float g = zr[i], u = yr[i] * (g / (1.0f + expf(-g))); ss = fmaf(u, u, ss); }
    ss = pm_block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float) part + eps);
    for (int i = threadIdx.x; i < part; i += 256) { const float g = zr[i], u = yr[i] * (g / (1.0f + expf(-g))); out[(int64_t) t * os + i0 + i] = u * inv * w[i0 + i] * mult; }
}
extern "C" int pi_op_gate_group_norm(const float * y, int64_t y_stride, const float * z, int64_t z_stride, const float * w_dev, float eps, float mult, int n, int groups, int n_tok, float * out, int64_t out_stride, void * stream) {
    if (n_tok <= 0 || n <= 0) return 0;
    if (groups < 1 || n % groups) { pi_set_error("pi_op_gate_group_norm: %d values do not divide into %d equal parts", n, groups); return -1; }
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 16.0 * n * n_tok, k_gate_group_norm, dim3((unsigned) n_tok, (unsigned) groups), dim3(256), 0, (hipStream_t) stream, y, y_stride, z, z_stride, w_dev, eps, mult, n, groups, out, out_stride,
                 pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}
