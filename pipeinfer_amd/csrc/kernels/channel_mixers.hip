// Operators of blocks whose norm comes AFTER the sum (x <- R(alpha x + ls * sublayer(x)) * w) and of recurrent mixers whose state decays per key channel:
//
//   k_embed_pair         token row * scale + a row of a second table (a hashed pair embedding: the host names the row of every token)
//   k_rms_post           the end of a sublayer in one launch: [the mean of two RMS-normed branch outputs ->] layer scale -> + alpha x -> RMS norm [-> a second RMS norm for what reads x next]
//   k_token_shift(_walk) m_s = h + (h_prev - h) * mu_s for several s at once; h_prev of a sequence's first token of the pass comes from (and its last token goes to) the sequence's state
//   k_channel_recurrence per head a [dim][vdim] state, per token and key channel a decay.  Two rules:
//                          delta   S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q        (the read-out sees the token's own write)
//                          bonus   o = (S + diag(b) k v^T)^T q;  S <- diag(g) S + k v^T                         (the read-out sees the token through the bonus only)
//                        decays arrive raw and are formed here (exp(-exp(raw + bias)) or exp(-exp(A_h) softplus(raw + bias))), q / k can be made unit vectors here, beta is sigmoid(raw)
//   k_head_norm_gate     every head's output divided by its root mean square, * weight (shared by the heads or one per head), * gate (as is, sigmoid or silu of it)
//
// Everything is fp32 in both precisions of the engine.
#include "ops_common.h"
#include "kernel_timing.h"

#include <algorithm>
#include <cmath>

#define CM_FRESH (1 << 30)

static __device__ __forceinline__ float cm_widen(uint16_t b) { return __uint_as_float((uint32_t) b << 16); }
static __device__ __forceinline__ float cm_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }
static __device__ __forceinline__ float cm_softplus(float z) { return z > 20.0f ? z : log1pf(expf(z)); }        // (beyond 20 the two agree to the last bit of fp32)
static __device__ __forceinline__ float cm_block_sum(float v, float * red) {          // sum over the block's threads (every thread gets it); red: 4 floats, reusable after the call
    v = pi_lanes_sum<64>(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = 0.0f;
    for (int i = 0; i < (int) (blockDim.x >> 6); i++) s += red[i];
    return s;
}

// ---- embedding: token row * scale + a row of a second table ---------------------------------------------------------------------------------------------
__global__ void k_embed_pair(const uint16_t * __restrict__ table, int64_t width, int64_t n_rows, const int32_t * __restrict__ tokens, float scale, const uint16_t * __restrict__ table2, int64_t n_rows2,
                             const int32_t * __restrict__ rows2, float * __restrict__ out, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    const int t = blockIdx.x;
    const int64_t row = tokens[t], row2 = rows2[t];
    const bool ok = row >= 0 && row < n_rows, ok2 = row2 >= 0 && row2 < n_rows2;
    for (int64_t i = threadIdx.x; i < width; i += blockDim.x)
        out[(int64_t) t * width + i] = (ok ? cm_widen(table[row * width + i]) * scale : 0.0f) + (ok2 ? cm_widen(table2[row2 * width + i]) : 0.0f);
}
extern "C" int pi_op_embed_pair(const pi_weight * w, const int32_t * tokens, int n_tok, float scale, const pi_weight * w2, const int32_t * rows2, float * out, void * stream) {
    if (!w || w->type != PI_BF16 || !w2 || w2->type != PI_BF16 || w->ne0 != w2->ne0) { pi_set_error("pi_op_embed_pair: two bfloat16 tables of the same width are required"); return -1; }
    if (n_tok <= 0) return 0;
    PI_KT_LAUNCH(PI_KT_OTHER, PI_BF16, 1, 8.0 * w->ne0 * n_tok, k_embed_pair, dim3((unsigned) n_tok), dim3(256), 0, (hipStream_t) stream, (const uint16_t *) w->p0, w->ne0, w->ne1, tokens, scale,
                 (const uint16_t *) w2->p0, w2->ne1, rows2, out, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}

// ---- the end of a sublayer whose norm comes after the sum ------------------------------------------------------------------------------------------------
// per token row:  m = b ? mb * (R(a) * wa + R(b) * wb) : a;   v = alpha * x + ls * m;   out = R(v) * w;   (w_next)  out_next = R(out) * w_next.   R(y) = y / sqrt(mean(y^2) + eps).
// A thread keeps its NPT values of every row in registers; out may be x.  PRE: every input (rows and weight vectors) is loaded before the first block sum, so that the launch makes ONE
// trip to memory instead of one per stage (rows up to 4096 wide; wider rows would not fit the registers and load stage by stage).
template <int NPT, bool PRE>
__global__ void __launch_bounds__(256) k_rms_post(const float * __restrict__ a, int64_t as, const float * __restrict__ wa, const float * __restrict__ b, int64_t bs, const float * __restrict__ wb, float mb,
                                                  const float * __restrict__ ls, const float * __restrict__ x, int64_t xs, float alpha, const float * __restrict__ w, float eps, int n,
                                                  float * __restrict__ out, int64_t os, const float * __restrict__ w_next, float * __restrict__ out_next, int64_t ons, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    __shared__ float red[4];
    const int t = blockIdx.x, tid = threadIdx.x;
    float m[NPT], v[NPT];
    float pwa[PRE ? NPT : 1], pwb[PRE ? NPT : 1], pls[PRE ? NPT : 1], px[PRE ? NPT : 1], pw[PRE ? NPT : 1], pwn[PRE ? NPT : 1];
#pragma unroll
    for (int j = 0; j < NPT; j++) {
        const int i = j * 256 + tid;
        m[j] = i < n ? a[(int64_t) t * as + i] : 0.0f;
        v[j] = b && i < n ? b[(int64_t) t * bs + i] : 0.0f;
        if (PRE) {
            pwa[j] = b && i < n ? wa[i] : 0.0f; pwb[j] = b && i < n ? wb[i] : 0.0f;
            pls[j] = ls && i < n ? ls[i] : 1.0f; px[j] = i < n ? x[(int64_t) t * xs + i] : 0.0f; pw[j] = i < n ? w[i] : 0.0f; pwn[j] = w_next && i < n ? w_next[i] : 0.0f;
        }
    }
    if (b) {
        float sa = 0.0f, sb = 0.0f;
#pragma unroll
        for (int j = 0; j < NPT; j++) { sa = fmaf(m[j], m[j], sa); sb = fmaf(v[j], v[j], sb); }
        sa = cm_block_sum(sa, red); sb = cm_block_sum(sb, red);
        const float ia = 1.0f / sqrtf(sa / (float) n + eps), ib = 1.0f / sqrtf(sb / (float) n + eps);
#pragma unroll
        for (int j = 0; j < NPT; j++) { const int i = j * 256 + tid; if (i < n) m[j] = mb * (m[j] * ia * (PRE ? pwa[j] : wa[i]) + v[j] * ib * (PRE ? pwb[j] : wb[i])); }
    }
    float ss = 0.0f;
#pragma unroll
    for (int j = 0; j < NPT; j++) {
        const int i = j * 256 + tid;
        v[j] = i < n ? fmaf(alpha, PRE ? px[j] : x[(int64_t) t * xs + i], (PRE ? pls[j] : ls ? ls[i] : 1.0f) * m[j]) : 0.0f;
        ss = fmaf(v[j], v[j], ss);
    }
    ss = cm_block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float) n + eps);
    float s2 = 0.0f;
#pragma unroll
    for (int j = 0; j < NPT; j++) { const int i = j * 256 + tid; if (i < n) { v[j] = v[j] * inv * (PRE ? pw[j] : w[i]); out[(int64_t) t * os + i] = v[j]; s2 = fmaf(v[j], v[j], s2); } }
    if (!w_next) return;
    s2 = cm_block_sum(s2, red);
    const float inv2 = 1.0f / sqrtf(s2 / (float) n + eps);
#pragma unroll
    for (int j = 0; j < NPT; j++) { const int i = j * 256 + tid; if (i < n) out_next[(int64_t) t * ons + i] = v[j] * inv2 * (PRE ? pwn[j] : w_next[i]); }
}
extern "C" int pi_op_rms_post(const float * a, int64_t a_stride, const float * wa, const float * b, int64_t b_stride, const float * wb, float mean_mult, const float * layer_scale, const float * x, int64_t x_stride,
                              float alpha, const float * w, float eps, int n, int n_tok, float * out, int64_t out_stride, const float * w_next, float * out_next, int64_t out_next_stride, void * stream) {
    if (n_tok <= 0 || n <= 0) return 0;
    if (n > 256 * 32) { pi_set_error("pi_op_rms_post: rows of %d values (at most %d)", n, 256 * 32); return -1; }
    if (b && (!wa || !wb)) { pi_set_error("pi_op_rms_post: two inputs need the weights of their norms"); return -1; }
    if (w_next && !out_next) { pi_set_error("pi_op_rms_post: a second norm needs a place for its result"); return -1; }
    const double bytes = 4.0 * n * n_tok * (3.0 + (b ? 1 : 0) + (w_next ? 1 : 0));
#define RP_GO(N, P) PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, bytes, (k_rms_post<N, P>), dim3((unsigned) n_tok), dim3(256), 0, (hipStream_t) stream, a, a_stride, wa, b, b_stride, wb, mean_mult, layer_scale, x, x_stride, alpha, w, eps, n, \
                              out, out_stride, w_next, out_next, out_next_stride, pi_abort_word())
    if (n <= 256 * 2) RP_GO(2, true); else if (n <= 256 * 4) RP_GO(4, true); else if (n <= 256 * 8) RP_GO(8, true); else if (n <= 256 * 16) RP_GO(16, true); else RP_GO(32, false);
#undef RP_GO
    PI_CHECK_LAUNCH(); return 0;
}

// ---- token shift: every mix of a token with the token before it ------------------------------------------------------------------------------------------------
// out[t][s][i] = h[t][i] + (prev[i] - h[t][i]) * mu[s][i], s < n_mix; prev = h[t - 1] inside a sequence's run, the sequence's state (zeros on a fresh slot) at the run's first token.
// rec as for the recurrences; state: [slots][n].  grid (token, blocks of 256 values)
__global__ void __launch_bounds__(256) k_token_shift(const float * __restrict__ h, int64_t hs, int n, const float * __restrict__ mu, int n_mix, const float * __restrict__ state, const int32_t * __restrict__ rec,
                                                     float * __restrict__ out, int64_t os, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    const int t = blockIdx.x, i = blockIdx.y * 256 + threadIdx.x;
    if (i >= n) return;
    const int word = rec[t], slot = word & ~CM_FRESH;
    const bool inside = t > 0 && (rec[t - 1] & ~CM_FRESH) == slot;
    const float cur = h[(int64_t) t * hs + i];
    const float prev = inside ? h[(int64_t) (t - 1) * hs + i] : (word & CM_FRESH) ? 0.0f : state[(int64_t) slot * n + i];
    const float d = prev - cur;
    for (int s = 0; s < n_mix; s++) out[(int64_t) t * os + (int64_t) s * n + i] = fmaf(d, mu[(int64_t) s * n + i], cur);
}
// a run's last token becomes the sequence's state (its own launch: the run's first token reads the state in the launch above)
__global__ void __launch_bounds__(256) k_token_shift_state(const float * __restrict__ h, int64_t hs, int n, float * __restrict__ state, const int32_t * __restrict__ rec, int n_tok, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    const int t = blockIdx.x, i = blockIdx.y * 256 + threadIdx.x;
    const int slot = rec[t] & ~CM_FRESH;
    if (i >= n || (t + 1 < n_tok && (rec[t + 1] & ~CM_FRESH) == slot)) return;
    state[(int64_t) slot * n + i] = h[(int64_t) t * hs + i];
}
// short passes in ONE launch: the thread of a run's first token walks the run for its value and leaves the state, so nothing it writes is read by another thread
__global__ void __launch_bounds__(256) k_token_shift_walk(const float * __restrict__ h, int64_t hs, int n, const float * __restrict__ mu, int n_mix, float * __restrict__ state, const int32_t * __restrict__ rec, int n_tok,
                                                          float * __restrict__ out, int64_t os, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    const int t = blockIdx.x, i = blockIdx.y * 256 + threadIdx.x;
    const int word = rec[t], slot = word & ~CM_FRESH;
    if (i >= n || (t > 0 && (rec[t - 1] & ~CM_FRESH) == slot)) return;
    float prev = (word & CM_FRESH) ? 0.0f : state[(int64_t) slot * n + i];
    for (int tt = t; tt < n_tok && (rec[tt] & ~CM_FRESH) == slot; tt++) {
        const float cur = h[(int64_t) tt * hs + i], d = prev - cur;
        for (int s = 0; s < n_mix; s++) out[(int64_t) tt * os + (int64_t) s * n + i] = fmaf(d, mu[(int64_t) s * n + i], cur);
        prev = cur;
    }
    state[(int64_t) slot * n + i] = prev;
}
#define TS_WALK_MAX_TOKENS 32
extern "C" int pi_op_token_shift(const float * h, int64_t h_stride, int n, const float * mu_dev, int n_mix, float * state_dev, const int32_t * rec_dev, int n_tok, float * out, int64_t out_stride, void * stream) {
    if (n_tok <= 0 || n <= 0) return 0;
    if (n_mix < 1 || out_stride < (int64_t) n_mix * n) { pi_set_error("pi_op_token_shift: %d mixes of %d values do not fit rows %lld floats apart", n_mix, n, (long long) out_stride); return -1; }
    if (out == h) { pi_set_error("pi_op_token_shift: the output may not overwrite the input (the next token reads it)"); return -1; }
    hipStream_t s = (hipStream_t) stream;
    const dim3 grid((unsigned) n_tok, (unsigned) ((n + 255) / 256));
    const double bytes = 4.0 * n * n_tok * (1.0 + n_mix) + 4.0 * n * n_mix;
    if (n_tok <= TS_WALK_MAX_TOKENS) {
        PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, bytes, k_token_shift_walk, grid, dim3(256), 0, s, h, h_stride, n, mu_dev, n_mix, state_dev, rec_dev, n_tok, out, out_stride, pi_abort_word());
        PI_CHECK_LAUNCH(); return 0;
    }
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, bytes, k_token_shift, grid, dim3(256), 0, s, h, h_stride, n, mu_dev, n_mix, state_dev, rec_dev, out, out_stride, pi_abort_word());
    PI_CHECK_LAUNCH();
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 8.0 * n, k_token_shift_state, grid, dim3(256), 0, s, h, h_stride, n, state_dev, rec_dev, n_tok, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}

// ---- recurrences with a decay per key channel ------------------------------------------------------------------------------------------------------------------
// Workgroup (head, block of value columns, piece of the pass): thread (column j, part sp of R) keeps S[i][j] for its DPT rows i in registers and walks the piece's tokens in order; q, k,
// the decays and v of CR_TB tokens at a time are staged (and finished: decays formed, unit vectors, sigmoid) in LDS.  A value column never meets another: o_j, u_j and S[:, j]
// depend on column j alone, so the only exchange is the sum over the R parts of a column (neighbouring lanes).
//   delta:  S <- g S;  a = S^T k, c = S^T q (one pass over the registers);  u = beta (v - a);  o = c + u (k . q);  S <- S + k u
//   bonus:  c = S^T q;  o = c + v (sum_i q_i b_i k_i);  S <- g S + k v
// A pass of up to CR_TB tokens (or keys too wide for the scan's tile) is ONE launch, mode 0: a piece is a sequence's whole run, S comes from and goes back to HBM.  Longer passes cut
// every run into pieces of CR_PIECE tokens that run side by side, because a column's step is affine in the column, s <- A_t s + b_t v_j with A_t the same for every column:
//   mode 1  every piece but a run's last, with extra columns: L_p = the state the piece builds from ZERO, and T_p = A_n .. A_1.  Delta rule: dim extra columns, column c of T_p is what the
//           piece makes of the unit vector e_c with v = 0 — the same walk over a column that starts as e_c.  Bonus rule: A_t is diagonal, ONE extra column that starts as all ones ends as
//           the diagonal of T_p.  Both into scratch [piece][head][dim][vdim + extra]
//   k_channel_state_scan / _diag  per run, piece by piece: S_in(p + 1) = T_p S_in(p) + L_p, S_in(0) = the slot's state (or zero); scratch[p][..][0 .. vdim) <- S_in(p)
//   mode 2  every piece from its true S_in(p): outputs; a run's last piece leaves the slot's new state
#define CR_TB 32                                  // tokens staged in LDS at a time
#define CR_PIECE 64                               // most tokens of a piece of a long pass (the launcher picks 32 or 64: longer pieces leave the scan fewer to chain, shorter ones put more side by side)
#define CR_MAXRUNS 256
#define CR_SCAN_MAXDIM 128                        // widest key whose transition matrix the scan keeps in LDS
// the pass's runs in order (a run: the consecutive tokens of one slot): every thread looks at its own tokens for a run's first one, the few found are ranked by position.  first[r] in `sorted`
static __device__ __forceinline__ int cr_runs(const int32_t * __restrict__ rec, int n_tok, int * bnd, int * sorted, int * nb) {
    if (threadIdx.x == 0) *nb = 0;
    __syncthreads();
    for (int t = threadIdx.x; t < n_tok; t += blockDim.x)
        if (t == 0 || (rec[t] & ~CM_FRESH) != (rec[t - 1] & ~CM_FRESH)) { const int at = atomicAdd(nb, 1); if (at < CR_MAXRUNS) bnd[at] = t; }
    __syncthreads();
    const int n = min(*nb, CR_MAXRUNS);
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        int rank = 0;
        for (int o = 0; o < n; o++) rank += bnd[o] < bnd[i];
        sorted[rank] = bnd[i];
    }
    __syncthreads();
    return n;
}
// (amdgpu_waves_per_eu(1, 2): at most two workgroups fit a compute unit's LDS anyway, so the registers of the other waves a SIMD could hold are free for a token's reads)
template <int DPT, int RULE>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 2))) k_channel_recurrence(const float * __restrict__ q, int64_t qs, const float * __restrict__ k, int64_t ks, const float * __restrict__ v, int64_t vs,
                                                            const float * __restrict__ draw, int64_t ds, int decay_mode, const float * __restrict__ dbias, const float * __restrict__ a_log,
                                                            const float * __restrict__ braw, int64_t bs, const float * __restrict__ bonus, int qk_unit, float q_mult,
                                                            int heads, int hpg, int dim, int vdim, int R, float * __restrict__ state, const int32_t * __restrict__ rec, int n_tok, int mode, int tb, int piece,
                                                            float * __restrict__ scratch, float * __restrict__ out, int64_t os, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    extern __shared__ float lds[];                // q [CR_TB][dp] | k [CR_TB][dp] | g [CR_TB][dp] | v [CR_TB][cols];  a row is R parts of DPT values, DPT + 4 floats apart (the parts of one wave-wide read then fall into different banks), dp = R * (DPT + 4); rows end in zeros so that the token loop needs no bounds
    __shared__ int seg[4], bnd[CR_MAXRUNS], sorted[CR_MAXRUNS], nbnd;      // seg: first token, length, slot word of this workgroup's piece, whether it is its run's last
    __shared__ float beta_t[CR_TB], dot_t[CR_TB];
    const int h = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nw = blockDim.x >> 6;
    const int n_runs = n_tok == 1 ? 1 : cr_runs(rec, n_tok, bnd, sorted, &nbnd);      // (a single token is its own run: no search, no barrier)
    if (n_tok == 1) { if (tid == 0) { seg[0] = 0; seg[1] = blockIdx.z == 0 ? 1 : 0; seg[2] = rec[0]; seg[3] = 1; } }
    else if (tid == 0) {                          // piece number blockIdx.z of the pass (mode 0: pieces are whole runs)
        const int lseg = mode ? piece : 0, want = blockIdx.z;
        int ord = 0;
        seg[1] = 0; seg[2] = -1;
        for (int r = 0; r < n_runs; r++) {
            const int t = sorted[r], e = r + 1 < n_runs ? sorted[r + 1] : n_tok;
            const int nsub = lseg > 0 ? (e - t + lseg - 1) / lseg : 1;
            if (want < ord + nsub) {
                const int pc = want - ord;
                seg[0] = lseg > 0 ? t + pc * lseg : t; seg[1] = lseg > 0 ? min(lseg, e - seg[0]) : e - t; seg[2] = rec[t]; seg[3] = pc == nsub - 1;
                break;
            }
            ord += nsub;
        }
    }
    __syncthreads();
    const int first = seg[0], len = seg[1], word = seg[2], last = seg[3];
    if (len == 0 || word < 0 || (mode == 1 && last)) return;
    const int slot = word & ~CM_FRESH;
    const int cols = blockDim.x / R;
    const int ext = RULE == 0 ? dim : 1;                              // extra columns of mode 1
    const int ncol = mode == 1 ? vdim + ext : vdim, sw = vdim + ext;   // columns this launch walks; row stride of a piece's block in scratch
    const int j = blockIdx.y * cols + tid / R, sp = tid % R;
    const bool col_ok = j < ncol;
    const int hq = h / hpg;                                            // the q / k head this head reads
    float * S_hbm = state + ((int64_t) slot * heads + h) * dim * vdim;
    float * S_scr = scratch ? scratch + ((int64_t) blockIdx.z * heads + h) * dim * sw : nullptr;
    float S[DPT];
#pragma unroll
    for (int ii = 0; ii < DPT; ii++) {
        const int i = sp * DPT + ii;
        float s0 = 0.0f;
        if (col_ok && i < dim) {
            if (mode == 1) s0 = j >= vdim && (RULE == 1 || i == j - vdim) ? 1.0f : 0.0f;
            else if (mode == 2) s0 = S_scr[(int64_t) i * sw + j];
            else if (!(word & CM_FRESH)) s0 = S_hbm[(int64_t) i * vdim + j];
        }
        S[ii] = s0;
    }
    const int dp = R * (DPT + 4);
    float * qt = lds, * kt = qt + tb * dp, * gt = kt + tb * dp, * vt = gt + tb * dp;        // tb <= CR_TB tokens at a time (fewer where the keys are very wide)
    const float ah = decay_mode == 2 ? expf(a_log[h]) : 0.0f;
    for (int t0 = 0; t0 < len; t0 += tb) {
        const int nt = min(tb, len - t0);
        __syncthreads();
        for (int idx = tid; idx < nt * R * DPT; idx += blockDim.x) {
            const int tt = idx / (R * DPT), i = idx % (R * DPT);
            const int64_t tok = first + t0 + tt;
            float qv = 0.0f, kv = 0.0f, d = 0.0f;
            if (i < dim) {
                qv = q[tok * qs + (int64_t) hq * dim + i];
                kv = k[tok * ks + (int64_t) hq * dim + i];
                d = draw[tok * ds + (int64_t) h * dim + i];
                if (decay_mode == 1) d = expf(-expf(d + (dbias ? dbias[h * dim + i] : 0.0f)));
                else if (decay_mode == 2) d = expf(-ah * cm_softplus(d + (dbias ? dbias[h * dim + i] : 0.0f)));
            }
            const int at = tt * dp + i / DPT * (DPT + 4) + i % DPT;
            qt[at] = qv; kt[at] = kv; gt[at] = d;
        }
        if (tid < nt) beta_t[tid] = braw ? cm_sigmoid(braw[(int64_t) (first + t0 + tid) * bs + h]) : 1.0f;
        for (int idx = tid; idx < nt * cols; idx += blockDim.x) {
            const int tt = idx / cols, jj = blockIdx.y * cols + idx % cols;
            vt[idx] = jj < vdim ? v[(int64_t) (first + t0 + tt) * vs + (int64_t) h * vdim + jj] : 0.0f;       // (the extra columns of mode 1 carry v = 0)
        }
        __syncthreads();
        for (int tt = wave; tt < nt; tt += nw) {                          // a wave per token: unit vectors, then the token's scalar (k . q, or sum q b k)
            float * qr = qt + tt * dp, * kr = kt + tt * dp;
            auto at = [&](int i) { return i / DPT * (DPT + 4) + i % DPT; };
            if (qk_unit) {
                float sq = 0.0f, sk = 0.0f;
                for (int i = lane; i < dim; i += 64) { sq = fmaf(qr[at(i)], qr[at(i)], sq); sk = fmaf(kr[at(i)], kr[at(i)], sk); }
                const float iq = q_mult / sqrtf(pi_lanes_sum<64>(sq) + 1e-6f), ik = 1.0f / sqrtf(pi_lanes_sum<64>(sk) + 1e-6f);
                for (int i = lane; i < dim; i += 64) { qr[at(i)] *= iq; kr[at(i)] *= ik; }
            } else if (q_mult != 1.0f) for (int i = lane; i < dim; i += 64) qr[at(i)] *= q_mult;
            float d = 0.0f;
            for (int i = lane; i < dim; i += 64) d = fmaf(RULE == 1 && bonus ? qr[at(i)] * bonus[h * dim + i] : qr[at(i)], kr[at(i)], d);      // (a lane re-reads only what it wrote itself)
            d = pi_lanes_sum<64>(d);
            if (lane == 0) dot_t[tt] = d;
        }
        __syncthreads();
        for (int tt = 0; tt < nt; tt++) {
            const float vj = vt[tt * cols + tid / R];
            const float * kr = kt + tt * dp + sp * (DPT + 4), * qr = qt + tt * dp + sp * (DPT + 4), * gr = gt + tt * dp + sp * (DPT + 4);
            float a = 0.0f, c = 0.0f, o;
            float4 k4[DPT / 4], q4[DPT / 4], g4[DPT / 4];                 // 16-byte LDS reads, no bounds (rows beyond dim: k = q = g = 0, their S stays 0): all of a token's reads go out before the first use
#pragma unroll
            for (int ii = 0; ii < DPT / 4; ii++) { k4[ii] = *(const float4 *) (kr + 4 * ii); q4[ii] = *(const float4 *) (qr + 4 * ii); g4[ii] = *(const float4 *) (gr + 4 * ii); }
            float a2 = 0.0f, c2 = 0.0f;                                   // (two chains each: half the depth of the dependent sums)
#pragma unroll
            for (int ii = 0; ii < DPT / 4; ii++) {
                const float4 kv = k4[ii], qv = q4[ii], gv = g4[ii];
                float * Sq = S + 4 * ii;
                if (RULE == 0) {
                    Sq[0] *= gv.x; Sq[1] *= gv.y; Sq[2] *= gv.z; Sq[3] *= gv.w;
                    a = fmaf(Sq[0], kv.x, a); a2 = fmaf(Sq[1], kv.y, a2); a = fmaf(Sq[2], kv.z, a); a2 = fmaf(Sq[3], kv.w, a2);
                }
                c = fmaf(Sq[0], qv.x, c); c2 = fmaf(Sq[1], qv.y, c2); c = fmaf(Sq[2], qv.z, c); c2 = fmaf(Sq[3], qv.w, c2);
                if (RULE == 1) { Sq[0] *= gv.x; Sq[1] *= gv.y; Sq[2] *= gv.z; Sq[3] *= gv.w; }
            }
            a += a2; c += c2;
            if (R == 2) { if (RULE == 0) a += pi_partner<1>(a); c += pi_partner<1>(c); }
            else if (R == 4) { if (RULE == 0) { a += pi_partner<2>(a); a += pi_partner<1>(a); } c += pi_partner<2>(c); c += pi_partner<1>(c); }
            else for (int d = R >> 1; d > 0; d >>= 1) { if (RULE == 0) a += __shfl_xor(a, d, PI_WAVE); c += __shfl_xor(c, d, PI_WAVE); }
            const float u = RULE == 0 ? beta_t[tt] * (vj - a) : vj;       // what the token writes under its key
            o = fmaf(u, dot_t[tt], c);
#pragma unroll
            for (int ii = 0; ii < DPT / 4; ii++) { S[4 * ii] = fmaf(k4[ii].x, u, S[4 * ii]); S[4 * ii + 1] = fmaf(k4[ii].y, u, S[4 * ii + 1]); S[4 * ii + 2] = fmaf(k4[ii].z, u, S[4 * ii + 2]); S[4 * ii + 3] = fmaf(k4[ii].w, u, S[4 * ii + 3]); }
            if (mode != 1 && col_ok && sp == 0) out[(int64_t) (first + t0 + tt) * os + (int64_t) h * vdim + j] = o;
        }
    }
    if (!col_ok) return;
    if (mode == 1) {
#pragma unroll
        for (int ii = 0; ii < DPT; ii++) { const int i = sp * DPT + ii; if (i < dim) S_scr[(int64_t) i * sw + j] = S[ii]; }
    } else if (last) {
#pragma unroll
        for (int ii = 0; ii < DPT; ii++) { const int i = sp * DPT + ii; if (i < dim) S_hbm[(int64_t) i * vdim + j] = S[ii]; }
    }
}

// grid (head, blocks of CR_SCAN_COLS value columns, run): per piece p of the run, in order: scratch[p] holds [L_p | T_p] coming in and S_in(p) (in L_p's place) going out.
// A workgroup keeps its columns of S in LDS (two buffers) and T_p transposed ([c][i], so that a thread's rows are neighbours); a thread owns a tile of 8 rows x 4 columns: per column c of T_p
// three 16-byte LDS reads feed 32 multiply-adds.
template <int CR_SCAN_COLS>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 4))) k_channel_state_scan(int heads, int dim, int vdim, int piece, const float * __restrict__ state, const int32_t * __restrict__ rec, int n_tok,
                                                                                                     float * __restrict__ scratch, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    extern __shared__ float lds[];                // T^T [dim][tp] | S [2][dim][CR_SCAN_COLS]
    __shared__ int seg[3], bnd[CR_MAXRUNS], sorted[CR_MAXRUNS], nbnd;      // slot word, first piece ordinal, pieces of the run (0: no such run)
    const int tid = threadIdx.x, h = blockIdx.x, j0 = blockIdx.y * CR_SCAN_COLS;
    const int n_runs = cr_runs(rec, n_tok, bnd, sorted, &nbnd);
    if (tid == 0) {
        int ord = 0;
        seg[0] = -1; seg[2] = 0;
        for (int r = 0; r < n_runs; r++) {
            const int t = sorted[r], e = r + 1 < n_runs ? sorted[r + 1] : n_tok;
            const int ns = (e - t + piece - 1) / piece;
            if (r == (int) blockIdx.z) { seg[0] = rec[t]; seg[1] = ord; seg[2] = ns; break; }
            ord += ns;
        }
    }
    __syncthreads();
    const int word = seg[0], sub0 = seg[1], nsub = seg[2];
    if (nsub == 0 || word < 0) return;
    const int slot = word & ~CM_FRESH, sw = vdim + dim, tp = (dim + 3) / 4 * 4 + 4;       // (rows of T^T start 16-byte aligned)
    float * Tt = lds, * Sb = Tt + dim * tp;
    constexpr int CG = CR_SCAN_COLS / 4;                               // column groups of 4
    const int jg = tid % CG, part = tid / CG, jl = jg * 4, pstep = 8 * (256 / CG);      // row parts of 8 rows
    const float * S0 = state + ((int64_t) slot * heads + h) * dim * vdim;
    for (int idx = tid; idx < dim * CR_SCAN_COLS; idx += 256) {
        const int i = idx / CR_SCAN_COLS, jj = j0 + idx % CR_SCAN_COLS;
        Sb[idx] = (jj < vdim && !(word & CM_FRESH)) ? S0[(int64_t) i * vdim + jj] : 0.0f;
    }
    int cur = 0;
    for (int p = 0; p < nsub; p++) {
        float * blk = scratch + ((int64_t) (sub0 + p) * heads + h) * dim * sw;
        const bool more = p + 1 < nsub;
        __syncthreads();                                               // (S of this piece is complete, T of the last one is no longer read)
        if (more) for (int idx = tid; idx < dim * dim; idx += 256) { const int i = idx / dim, c = idx % dim; Tt[c * tp + i] = blk[(int64_t) i * sw + vdim + c]; }
        __syncthreads();
        const float * Sc = Sb + cur * dim * CR_SCAN_COLS;
        float * Sn = Sb + (cur ^ 1) * dim * CR_SCAN_COLS;
        for (int i0 = part * 8; i0 < dim; i0 += pstep) {
            float acc[8][4];
#pragma unroll
            for (int r = 0; r < 8; r++)
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const bool ok = i0 + r < dim && j0 + jl + u < vdim;
                    acc[r][u] = (more && ok) ? blk[(int64_t) (i0 + r) * sw + j0 + jl + u] : 0.0f;                                     // L_p, read before S_in(p) takes its place
                    if (ok) blk[(int64_t) (i0 + r) * sw + j0 + jl + u] = Sc[(i0 + r) * CR_SCAN_COLS + jl + u];
                }
            if (!more) continue;
            for (int c = 0; c < dim; c++) {
                const float4 sv = *(const float4 *) (Sc + c * CR_SCAN_COLS + jl);
                const float4 ta = *(const float4 *) (Tt + c * tp + i0), tb = *(const float4 *) (Tt + c * tp + i0 + 4);      // (rows beyond dim read the pad or the next row of T^T: their sums are dropped)
                const float tv[8] = { ta.x, ta.y, ta.z, ta.w, tb.x, tb.y, tb.z, tb.w };
#pragma unroll
                for (int r = 0; r < 8; r++) { acc[r][0] = fmaf(tv[r], sv.x, acc[r][0]); acc[r][1] = fmaf(tv[r], sv.y, acc[r][1]); acc[r][2] = fmaf(tv[r], sv.z, acc[r][2]); acc[r][3] = fmaf(tv[r], sv.w, acc[r][3]); }
            }
#pragma unroll
            for (int r = 0; r < 8; r++) if (i0 + r < dim) *(float4 *) (Sn + (i0 + r) * CR_SCAN_COLS + jl) = make_float4(acc[r][0], acc[r][1], acc[r][2], acc[r][3]);
        }
        cur ^= 1;
    }
}

// the same chain where T_p is diagonal (bonus rule): scratch[p] holds [L_p | diag T_p] ([dim][vdim + 1]).  grid (head, blocks over dim * vdim, run): eight pieces' loads in flight, the chain in registers
__global__ void __launch_bounds__(256) k_channel_state_scan_diag(int heads, int dim, int vdim, int piece, const float * __restrict__ state, const int32_t * __restrict__ rec, int n_tok, float * __restrict__ scratch,
                                                                 const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    __shared__ int seg[3], bnd[CR_MAXRUNS], sorted[CR_MAXRUNS], nbnd;
    const int tid = threadIdx.x, h = blockIdx.x;
    const int n_runs = cr_runs(rec, n_tok, bnd, sorted, &nbnd);
    if (tid == 0) {
        int ord = 0;
        seg[0] = -1; seg[2] = 0;
        for (int r = 0; r < n_runs; r++) {
            const int t = sorted[r], e = r + 1 < n_runs ? sorted[r + 1] : n_tok;
            const int ns = (e - t + piece - 1) / piece;
            if (r == (int) blockIdx.z) { seg[0] = rec[t]; seg[1] = ord; seg[2] = ns; break; }
            ord += ns;
        }
    }
    __syncthreads();
    const int word = seg[0], sub0 = seg[1], nsub = seg[2];
    if (nsub == 0 || word < 0) return;
    const int64_t per = (int64_t) dim * vdim, idx = (int64_t) blockIdx.y * 256 + tid;
    if (idx >= per) return;
    const int i = (int) (idx / vdim), j = (int) (idx % vdim), sw = vdim + 1;
    float run = (word & CM_FRESH) ? 0.0f : state[((int64_t) (word & ~CM_FRESH) * heads + h) * per + idx];
    for (int p0 = 0; p0 < nsub; p0 += 8) {
        float lp[8], tp[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const float * blk = scratch + ((int64_t) (sub0 + p0 + u) * heads + h) * dim * sw + (int64_t) i * sw;
            const bool more = p0 + u < nsub - 1;
            lp[u] = more ? blk[j] : 0.0f; tp[u] = more ? blk[vdim] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 8; u++)
            if (p0 + u < nsub) {
                scratch[((int64_t) (sub0 + p0 + u) * heads + h) * dim * sw + (int64_t) i * sw + j] = run;
                run = fmaf(tp[u], run, lp[u]);
            }
    }
}

#define CR_LDS_MAX (150 * 1024)
template <int DPT, int RULE> static int cr_reserve_one() { PI_CHECK_HIP(hipFuncSetAttribute((const void *) k_channel_recurrence<DPT, RULE>, hipFuncAttributeMaxDynamicSharedMemorySize, CR_LDS_MAX)); return 0; }
extern "C" int pi_op_channel_recurrence_reserve(void) {
    static bool done = false;
    if (done) return 0;
    if (cr_reserve_one<8, 0>() || cr_reserve_one<16, 0>() || cr_reserve_one<32, 0>() || cr_reserve_one<8, 1>() || cr_reserve_one<16, 1>() || cr_reserve_one<32, 1>()) return -1;
    PI_CHECK_HIP(hipFuncSetAttribute((const void *) k_channel_state_scan<8>, hipFuncAttributeMaxDynamicSharedMemorySize, CR_LDS_MAX));
    PI_CHECK_HIP(hipFuncSetAttribute((const void *) k_channel_state_scan<16>, hipFuncAttributeMaxDynamicSharedMemorySize, CR_LDS_MAX));
    PI_CHECK_HIP(hipFuncSetAttribute((const void *) k_channel_state_scan<32>, hipFuncAttributeMaxDynamicSharedMemorySize, CR_LDS_MAX));
    done = true;
    return 0;
}
static int cr_max_pieces(int n_tok, int max_segments, int piece = CR_TB) { return n_tok / piece + std::min(n_tok, std::max(1, max_segments)) + 1; }
// passes of more than 32 tokens cut the runs into pieces that run side by side: floats of scratch they need (0: such a pass is walked in one piece per run)
extern "C" size_t pi_op_channel_recurrence_scratch_floats(int heads, int dim, int vdim, int n_tok, int max_segments) {      // (sized for the delta rule, which needs more)
    return (n_tok <= CR_TB || dim > CR_SCAN_MAXDIM) ? 0 : (size_t) cr_max_pieces(n_tok, max_segments) * heads * dim * (vdim + dim);
}
extern "C" int pi_op_channel_recurrence(int rule, const float * q, int64_t q_stride, const float * k, int64_t k_stride, const float * v, int64_t v_stride, const float * decay_raw, int64_t decay_stride, int decay_mode,
                                        const float * decay_bias_dev, const float * a_log_dev, const float * beta_raw, int64_t beta_stride, const float * bonus_dev, int qk_unit, float q_mult,
                                        int heads, int qk_heads, int dim, int vdim, float * state_dev, const int32_t * rec_dev, int n_tok, int max_segments, float * scratch_dev, size_t scratch_floats,
                                        float * out, int64_t out_stride, void * stream) {
    if (n_tok <= 0) return 0;
    if (rule != PI_RULE_DELTA && rule != PI_RULE_BONUS) { pi_set_error("pi_op_channel_recurrence: rule %d is unknown", rule); return -1; }
    if (qk_heads < 1 || heads % qk_heads) { pi_set_error("pi_op_channel_recurrence: %d heads do not divide over %d query / key heads", heads, qk_heads); return -1; }
    if (dim <= 0 || vdim <= 0 || heads <= 0 || dim > 1024) { pi_set_error("pi_op_channel_recurrence: head sizes %d x %d outside the kernel's range (key width <= 1024)", dim, vdim); return -1; }
    if (decay_mode < 0 || decay_mode > 2 || (decay_mode == 2 && !a_log_dev) || !decay_raw) { pi_set_error("pi_op_channel_recurrence: decays (mode %d) are missing a part", decay_mode); return -1; }
    if (max_segments > CR_MAXRUNS) { pi_set_error("pi_op_channel_recurrence: at most %d sequences in a pass", CR_MAXRUNS); return -1; }
    const int dpt = dim <= 8 ? 8 : dim <= 16 ? 16 : 32;                // state values a thread keeps in registers
    int R = 1; while (R * dpt < dim) R *= 2;
    const size_t need = pi_op_channel_recurrence_scratch_floats(heads, dim, vdim, n_tok, max_segments);
    const bool pieces = need > 0 && scratch_dev && scratch_floats >= need;       // (without scratch a long pass is still right, only serial)
    const int runs = std::max(1, std::min(n_tok, max_segments));
    const double bytes = 4.0 * n_tok * heads * (3.0 * dim + 2.0 * vdim) + 8.0 * heads * dim * vdim;
    hipStream_t s = (hipStream_t) stream;
    const int nta = std::min(n_tok, PI_KT_MAXNT - 1);
    // delta rule: the scan's work grows with the number of pieces, so pieces of 64 tokens where that still leaves a workgroup per compute unit; bonus rule (a scan of no weight): 32
    const int cols0 = std::min(256, (vdim * R + 63) / 64 * 64) / R;
    const int piece = (rule == PI_RULE_DELTA && (int64_t) heads * ((vdim + cols0 - 1) / cols0) * (n_tok / CR_PIECE) >= 256) ? CR_PIECE : CR_TB;
    auto launch = [&](int mode) -> int {
        const int ncol = mode == 1 ? vdim + (rule == PI_RULE_DELTA ? dim : 1) : vdim;
        const int threads = std::min(256, (ncol * R + 63) / 64 * 64);
        const int cols = threads / R;
        const dim3 grid((unsigned) heads, (unsigned) ((ncol + cols - 1) / cols), (unsigned) (mode ? cr_max_pieces(n_tok, max_segments, piece) : runs));
        int tb = CR_TB;                                                 // tokens staged at a time: as many as the LDS takes
        auto lds_of = [&](int n) { return ((size_t) 3 * n * R * (dpt + 4) + (size_t) n * cols) * sizeof(float); };
        while (tb > 1 && lds_of(tb) > CR_LDS_MAX) tb >>= 1;
        const size_t lds = lds_of(tb);
        if (lds > CR_LDS_MAX) { pi_set_error("pi_op_channel_recurrence: a key width of %d needs %zu bytes of LDS (at most %d)", dim, lds, CR_LDS_MAX); return -1; }
        if (lds > 48 * 1024 && pi_op_channel_recurrence_reserve() != 0) return -1;
#define CR_GO(D, RL) PI_KT_LAUNCH(PI_KT_ATT, 0, nta, bytes, (k_channel_recurrence<D, RL>), grid, dim3(threads), lds, s, q, q_stride, k, k_stride, v, v_stride, decay_raw, decay_stride, decay_mode, decay_bias_dev, a_log_dev, \
                                  beta_raw, beta_stride, bonus_dev, qk_unit, q_mult, heads, heads / qk_heads, dim, vdim, R, state_dev, rec_dev, n_tok, mode, tb, piece, scratch_dev, out, out_stride, pi_abort_word())
        if (rule == PI_RULE_DELTA) { if (dpt == 8) CR_GO(8, 0); else if (dpt == 16) CR_GO(16, 0); else CR_GO(32, 0); }
        else                       { if (dpt == 8) CR_GO(8, 1); else if (dpt == 16) CR_GO(16, 1); else CR_GO(32, 1); }
#undef CR_GO
        PI_CHECK_LAUNCH(); return 0;
    };
    if (!pieces) return launch(0);
    if (launch(1) != 0) return -1;
    const int n_pieces = cr_max_pieces(n_tok, max_segments, piece);
    if (rule == PI_RULE_BONUS) {
        PI_KT_LAUNCH(PI_KT_ATT, 0, nta, 12.0 * n_pieces * heads * dim * vdim, k_channel_state_scan_diag, dim3((unsigned) heads, (unsigned) (((int64_t) dim * vdim + 255) / 256), (unsigned) runs), dim3(256), 0, s,
                     heads, dim, vdim, piece, state_dev, rec_dev, n_tok, scratch_dev, pi_abort_word());
    } else {
        // columns per workgroup: as few as it takes to put a workgroup on every compute unit (each one re-reads the transition matrices, which the others' reads keep in L2)
        int sc = 32;
        while (sc > 8 && (int64_t) heads * ((vdim + sc - 1) / sc) < 256) sc >>= 1;           // (a pass usually carries one run, whatever the slots allow)
        const size_t scan_lds = ((size_t) dim * ((dim + 3) / 4 * 4 + 4) + (size_t) 2 * dim * sc + 8) * sizeof(float);
        if (scan_lds > 48 * 1024 && pi_op_channel_recurrence_reserve() != 0) return -1;
        const dim3 sgrid((unsigned) heads, (unsigned) ((vdim + sc - 1) / sc), (unsigned) runs);
        const double sbytes = 4.0 * n_pieces * heads * dim * (2.0 * vdim + dim);
#define CR_SCAN(C) PI_KT_LAUNCH(PI_KT_ATT, 0, nta, sbytes, k_channel_state_scan<C>, sgrid, dim3(256), scan_lds, s, heads, dim, vdim, piece, state_dev, rec_dev, n_tok, scratch_dev, pi_abort_word())
        if (sc == 8) CR_SCAN(8); else if (sc == 16) CR_SCAN(16); else CR_SCAN(32);
#undef CR_SCAN
    }
    PI_CHECK_LAUNCH();
    return launch(2);
}

// ---- per-head RMS norm, weight, gate ------------------------------------------------------------------------------------------------------------------------------
// out[t][h][i] = y[t][h][i] / sqrt(mean_i(y[t][h]^2) + eps) * w[(w_per_head ? h * n : 0) + i] * act(gate[t][h][i]);  a wave per (token, head); out may be y
__global__ void __launch_bounds__(256) k_head_norm_gate(const float * __restrict__ y, int64_t ys, int heads, int n, const float * __restrict__ w, int w_per_head, const float * __restrict__ gate, int64_t gs, int gate_act,
                                                        float eps, float * __restrict__ out, int64_t os, const int32_t * __restrict__ abort_w) {
    if (pi_aborted(abort_w)) return;
    const int t = blockIdx.x, h = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (h >= heads) return;
    const float * yr = y + (int64_t) t * ys + (int64_t) h * n;
    float ss = 0.0f;
    for (int i = lane; i < n; i += 64) ss = fmaf(yr[i], yr[i], ss);
    const float inv = 1.0f / sqrtf(pi_lanes_sum<64>(ss) / (float) n + eps);
    for (int i = lane; i < n; i += 64) {
        float g = gate ? gate[(int64_t) t * gs + (int64_t) h * n + i] : 1.0f;
        if (gate && gate_act == PI_ACT_SIGMOID) g = cm_sigmoid(g);
        else if (gate && gate_act == PI_ACT_SILU) g = g / (1.0f + expf(-g));
        out[(int64_t) t * os + (int64_t) h * n + i] = yr[i] * inv * w[(w_per_head ? h * n : 0) + i] * g;
    }
}
extern "C" int pi_op_head_norm_gate(const float * y, int64_t y_stride, int heads, int n, const float * w_dev, int w_per_head, const float * gate, int64_t gate_stride, int gate_act, float eps, int n_tok,
                                    float * out, int64_t out_stride, void * stream) {
    if (n_tok <= 0 || heads <= 0 || n <= 0) return 0;
    PI_KT_LAUNCH(PI_KT_OTHER, 0, 1, 12.0 * n_tok * heads * n, k_head_norm_gate, dim3((unsigned) n_tok, (unsigned) ((heads + 3) / 4)), dim3(256), 0, (hipStream_t) stream, y, y_stride, heads, n, w_dev, w_per_head,
                 gate, gate_stride, gate_act, eps, out, out_stride, pi_abort_word());
    PI_CHECK_LAUNCH(); return 0;
}
