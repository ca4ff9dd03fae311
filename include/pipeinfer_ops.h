/* pipeinfer_ops.h — C ABI of the MI355X hot-path operators (libpipeinfer_amd.so).
 *
 * One entry point per reference operator on the per-token path.  Every pointer named *_dev is a device
 * (HBM) pointer; `stream` is a hipStream_t passed as void* (NULL = the default stream).  All functions return 0 on
 * success and a negative value on error (pi_last_error() has the text).  There is NO CPU fallback: without a GPU the
 * compute entry points fail loudly.
 *
 * Reference interface each one replaces (file:line under the reference tree):
 *   pi_weight_upload        ggml tensor data as laid out by the GGUF loader             llama.cpp:1805-2134, ggml-quants.h:10-166
 *   pi_op_get_rows          ggml_compute_forward_get_rows_q                             ggml.c:10161-10188
 *   pi_op_norm              ggml_compute_forward_rms_norm_f32 / _norm_f32 + ggml_mul/add ggml.c:9028-9074, 8959-9008; llama.cpp:3579-3609
 *   pi_op_quantize          quantize_row_q8_K / quantize_row_q8_0 (mul_mat INIT phase)   ggml-quants.c:2329-2364, 702-760; ggml.c:9493-9506
 *   pi_op_mul_mat           ggml_compute_forward_mul_mat + ggml_vec_dot_{q4_0,q8_0,q4_K,q5_K,q6_K}_q8_*  ggml.c:9388-9597; ggml-quants.c:2426,3521,5216,5864,6594
 *   pi_op_rope_kv_store     ggml_compute_forward_rope_f32 + llm_build_kv_store           ggml.c:11006-11168; llama.cpp:3546-3577
 *   pi_op_attention         llm_build_kqv (KQ, scale, mask, soft_max, KQV)               llama.cpp:3698-3764; ggml.c:10551-10620, 1193-1228
 *   pi_op_silu_mul/_gelu/_add  ggml_silu / ggml_gelu / ggml_mul / ggml_add               ggml.c:1418-1498, 7583, 6803
 *   pi_op_topk              llama_sample_softmax / llama_sample_token_greedy             llama.cpp:7019-7046, 7496-7510
 */
#ifndef PIPEINFER_OPS_H
#define PIPEINFER_OPS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PI_API __attribute__((visibility("default")))

/* ggml tensor type ids (ggml.h enum ggml_type) */
enum pi_type { PI_F32 = 0, PI_F16 = 1, PI_Q4_0 = 2, PI_Q4_1 = 3, PI_Q5_0 = 6, PI_Q5_1 = 7, PI_Q8_0 = 8, PI_Q8_1 = 9, PI_Q2_K = 10, PI_Q3_K = 11, PI_Q4_K = 12, PI_Q5_K = 13, PI_Q6_K = 14, PI_Q8_K = 15, PI_BF16 = 30 /* bfloat16 rows as a safetensors checkpoint holds them (dense operators below) */ };

typedef struct pi_weight pi_weight;    /* a weight matrix resident in HBM in the kernel-friendly layout */

PI_API const char * pi_last_error(void);
PI_API int     pi_device_count(void);
PI_API int     pi_device_init(int device);            /* selects the GPU, builds + uploads the fp16 lookup tables */

PI_API void *  pi_malloc(size_t bytes);
PI_API void    pi_free(void * p_dev);
PI_API int     pi_memcpy_h2d(void * dst_dev, const void * src, size_t bytes, void * stream);
PI_API int     pi_memcpy_d2h(void * dst, const void * src_dev, size_t bytes, void * stream);
PI_API int     pi_memset(void * dst_dev, int value, size_t bytes, void * stream);
PI_API int     pi_stream_sync(void * stream);
PI_API int     pi_device_sync(void);

/* Kernel-granular early cancellation (reference: the abort callback polled between graph nodes, ggml.c:15748-15811, llama.cpp:5614-5628, 5665-5687).
 * word_dev: the first int32 of a 64-byte block in device memory (zeroed by the owner) holding (run id << 1 | aborted); words 8..14 of the block count, per kernel family
 * (enum order of pi_kt_row.family), the launches that found the run aborted and returned on entry.  Every hot-path kernel launched — or captured into a
 * graph — by the calling thread after pi_set_abort_word(word_dev) reads it on entry and returns at once when bit 0 is set (NULL: no check).
 *   pi_op_abort_begin   (in stream order, ahead of a run's kernels)  word = run_id << 1 | (*host_flag != 0); host_flag: pinned host memory, nullable
 *   pi_op_abort_cancel  (any stream, any time)                        if word == run_id << 1 then word |= 1: only the run that is executing NOW is hit */
PI_API void    pi_set_abort_word(const int32_t * word_dev);
/* launch accounting only: the attention launches of the calling thread are priced with n_kv cells from now on (0: with the n_kv they are launched with) */
PI_API void    pi_set_account_n_kv(int n_kv);
/* launches of the calling thread from now on go to a stream restricted to `n` compute units (hipExtStreamCreateWithCUMask): the launchers size "one round of workgroups" for it (0 / 256: the whole chip) */
PI_API void    pi_set_cu_count(int n);
PI_API int     pi_op_abort_begin(int32_t * word_dev, int32_t run_id, const int32_t * host_flag, void * stream);
PI_API int     pi_op_abort_cancel(int32_t * word_dev, int32_t run_id, void * stream);
/* Arrival flags of the stage transport (reference: the blocking MPI_Recv of the activations, ggml-mpi.c:451-487): a 16-byte record {ticket << 1 | aborted, -, realtime stamp}
 * in page-locked host memory mapped by the producing and the consuming process.
 *   pi_op_flag_publish      (producer's stream, behind its peer store)  flag = ticket << 1 | (abort word & 1 | force_abort), stamped with the device's 100 MHz clock
 *   pi_op_abort_begin_wait  (consumer's stream, ahead of the run)       polls the flag from the device until it carries `ticket` (at most timeout_us: then the run is marked
 *                           aborted and *timeout_flag_dev = 1), then arms the abort word like pi_op_abort_begin, with the producer's abort bit or-ed in;
 *                           hop_ticks_dev (nullable) accumulates {flag written -> seen, time waited, runs} in 10 ns ticks */
/* A run's results (logits rows, top-8 ids / values, soft-max sums) written into the caller's PAGE-LOCKED host buffers by a kernel on the run's stream, instead of
 * hipMemcpyAsync: on this runtime a device -> host copy of the logits' size does not complete while another stream's kernels keep the device busy (runtime.hip). */
PI_API int     pi_op_copy_out(const float * logits_dev, float * logits_host, int64_t n_logits, const int32_t * ids_dev, int32_t * ids_host, const float * vals_dev, float * vals_host,
                              const float * sum_dev, float * sum_host, int n_tok, void * stream);
PI_API int     pi_op_flag_publish(void * flag_dev, uint32_t ticket, const int32_t * abort_word_dev, int force_abort, void * stream);
PI_API int     pi_op_abort_begin_wait(int32_t * word_dev, int32_t run_id, const int32_t * host_flag, const void * flag_dev, uint32_t ticket, int64_t timeout_us,
                                      int32_t * timeout_flag_dev, uint64_t * hop_ticks_dev, void * stream);

/* Launch accounting for the roofline report.  An instance = (family, weight type, tokens of the launch); families: 0 VALU mat-vec (k_mmvq_*), 1 matrix-core mat-mat
 * (k_mmq_kq), 2 norm + quantise, 3 quantise, 4 activation + quantise, 5 attention, 6 everything else (get_rows, RoPE + KV store, norms, adds, top-k).
 * pi_kernel_timing(1, N) opens a window: every eager launch is counted with its algorithmic bytes and every Nth launch of an instance is timed (HIP events of
 * hipExtLaunchKernelGGL = the kernel's own begin / end timestamps); pi_kernel_timing_rows reads the window after a device sync.  Launches captured into a HIP graph are
 * counted per graph instead (pipeinfer_get_launch_rows in pipeinfer.h: graph contents x replays). */
struct pi_kt_row { int32_t family, type, n_tok, sampled_dropped; /* timed launches left out of avg_us: below a third of the median (they found their run aborted) */ uint64_t shape_bytes; /* mat launches: algorithmic bytes of this launch shape (0 for the other families) */
                   uint64_t launches; double bytes_total; uint64_t sampled; double avg_us, avg_sampled_bytes; };
PI_API void    pi_kernel_timing(int on, int sample_every);
PI_API int     pi_kernel_timing_rows(struct pi_kt_row * out, int cap);
PI_API int     pi_kernel_lifetime_rows(struct pi_kt_row * out, int cap);   /* every eager launch since the process started (counts and bytes, never reset): what a PMC pass of the process sees */

/* host_blocks: ne1 rows of ne0 elements in the GGUF/ggml block format of `type` (row-major, rows contiguous) */
PI_API pi_weight * pi_weight_upload(int type, int64_t ne0, int64_t ne1, const void * host_blocks, void * stream);
PI_API void    pi_weight_free(pi_weight * w);
PI_API size_t  pi_weight_nbytes(const pi_weight * w);  /* HBM bytes == ggml_nbytes of the tensor */
PI_API size_t  pi_weight_copy_nbytes(const pi_weight * w); /* HBM bytes of the second, tile-major copy the matrix-core kernel reads (0 without one) */
/* uploads of the calling thread from now on do (1, default) / do not (0) make that copy: a context that never decodes more than two tokens at once has no use for it */
PI_API void    pi_weight_set_mq_copies(int on);
/* gives a weight that was uploaded without the copy its tile-major copy now, from the same GGUF bytes (no-op when it has one or its type has no matrix-core kernel); 0 ok
   (also when HBM is short: the weight then stays on the VALU kernel), < 0 on a failed copy */
PI_API int     pi_weight_ensure_mq_copy(pi_weight * w, const void * host_blocks, void * stream);
PI_API const void * pi_weight_data(const pi_weight * w); /* device address of the (repacked) tensor bytes */
/* reads [p, p + bytes) once with up to `workgroups` workgroups (0: as many as the bytes need): warms the memory-side Infinity Cache */
PI_API int     pi_op_prefetch(const void * p, size_t bytes, int workgroups, void * stream);
PI_API int     pi_weight_type(const pi_weight * w);

/* type the activations must be quantised to for this weight type (type_traits[].vec_dot_type, ggml.c:415-600) */
PI_API int     pi_vec_dot_type(int weight_type);
/* bytes of the device activation buffer for n_tok rows of k values quantised to vdt (PI_Q8_K, PI_Q8_0 or PI_Q8_1) */
PI_API size_t  pi_q8_nbytes(int vdt, int64_t k, int n_tok);
/* byte offsets of the planes inside that buffer: qs (int8 [n_tok][k]), d (f32 [n_tok][k/256] | f16 [n_tok][k/32] | Q8_1: f32 [n_tok][k/32]), third plane: bsums (int16 [n_tok][k/16], Q8_K) or s = d * sum(qs) (f32 [n_tok][k/32], Q8_1) */
PI_API void    pi_q8_layout(int vdt, int64_t k, int n_tok, size_t * off_qs, size_t * off_d, size_t * off_bsums);
/* Q8_K, n_tok >= 2: byte offsets of the MFMA operand planes the quantisers also write (f16 copies of qs in the lane order of
 * v_mfma_f32_16x16x32_f16, two sub-block pairings, and per-token block sums / scales as floats); layout in runtime.hip */
PI_API void    pi_q8_frag_layout(int64_t k, int n_tok, size_t * off_frag_a, size_t * off_frag_b, size_t * off_aux);

PI_API int pi_op_get_rows(const pi_weight * w, const int32_t * tokens_dev, int n_tok, float * out_dev, void * stream);
PI_API int pi_op_norm(const float * x_dev, const float * w_dev, const float * b_dev, float * y_dev, int n, int n_tok, float eps, int rms, void * stream);
PI_API int pi_op_quantize(int vdt, const float * x_dev, int64_t k, int n_tok, void * q8_dev, void * stream);
/* fusions of the above (same arithmetic, same rounding points): norm -> quantised planes (y_f32_dev nullable: also keep the fp32 result);
 * which = 0: silu(gate) * up, 1: gelu(gate), 2: relu(gate)^2 (LLM_FFN_RELU_SQR) -> quantised planes */
PI_API int pi_op_norm_quantize(const float * x_dev, const float * w_dev, const float * b_dev, float * y_f32_dev, int n, int n_tok, float eps, int rms, int vdt, void * q8_dev, void * stream);
PI_API int pi_op_act_quantize(const float * gate_dev, const float * up_dev, int which, int64_t n, int n_tok, int vdt, void * q8_dev, void * stream);
/* out[t][row] = (residual ? residual[t][row] : 0) + W[row] . act[t]      out/residual: f32 [n_tok][ne1] */
PI_API int pi_op_mul_mat(const pi_weight * w, const void * q8_dev, int n_tok, float * out_dev, const float * residual_dev, void * stream);
/* up to 3 weights of one type and width applied to the same activations in ONE launch (wq/wk/wv, ffn_up/ffn_gate); same results as separate calls */
/* attention projections with RoPE and the KV-cache writes as the mat-vec's epilogue (Llama-style RoPE, K-quant weights):
 *   q16[t][n_head*hd] = f16(rope(Wq.act)),  kc[(kv_head+t)][n_head_kv*hd] = f16(rope(Wk.act)),  vc[(kv_head+t)][..] = f16(Wv.act)
 * == pi_op_mul_mat x3 + pi_op_rope_kv_store, same bytes.  dyn_dev (optional): {kv_head, n_kv} in device memory, as for pi_op_rope_kv_store. */
PI_API int pi_op_mul_mat_qkv_rope_ok(const pi_weight * wq, const pi_weight * wk, const pi_weight * wv, int neox, int head_dim);
PI_API int pi_op_mul_mat_qkv_rope(const pi_weight * wq, const pi_weight * wk, const pi_weight * wv, const void * q8_dev, int n_tok, const int32_t * pos_dev, const void * rope_table,
                                  int head_dim, int n_head, int n_head_kv, int kv_head, const int32_t * dyn_dev, uint16_t * q16_dev, uint16_t * k_cache_dev, uint16_t * v_cache_dev, void * stream);
PI_API int pi_op_mul_mat_multi(int n_w, const pi_weight * const * ws, const void * q8_dev, int n_tok, float * const * outs_dev, const float * const * residuals_dev, void * stream);

/* RoPE tables as the reference iterates them: cos/sin [n_pos][head_dim/2] f32, built on the host (theta *= theta_scale) */
PI_API void *  pi_rope_table_create(int n_pos, int head_dim, float freq_base, float freq_scale, int neox);
/* NeoX mode with n_rot < head_dim (StableLM, llama.cpp:4860-4871): the reference walks head_dim / n_rot blocks of n_rot values, pairs (i, i + n_rot/2) inside a block,
 * theta_scale = freq_base^(-2/n_rot) and theta keeps advancing across the blocks (ggml.c:11133-11160) */
PI_API void *  pi_rope_table_create_ex(int n_pos, int head_dim, int n_rot, float freq_base, float freq_scale, int neox);
PI_API void    pi_rope_table_free(void * table);
/* q/k/v: f32 rows of n_head*hd / n_head_kv*hd values per token, *_stride floats apart (a fused QKV output is passed as three
 * views); writes roped Q as f16 [n_tok][n_head*hd]; K and V as f16 rows of the layer's cache at cells kv_head..
 * (k_cache/v_cache: [n_ctx][n_head_kv*hd] f16 each) */
PI_API int pi_op_rope_kv_store(const float * q_dev, const float * k_dev, const float * v_dev, int64_t q_stride, int64_t k_stride, int64_t v_stride,
                               const int32_t * pos_dev, const void * rope_table,
                               int neox, int head_dim, int n_head, int n_head_kv, int n_tok, int kv_head,
                               uint16_t * q16_dev, uint16_t * k_cache_dev, uint16_t * v_cache_dev, const int32_t * dyn_dev, void * stream);
/* build_persimmon's attention inputs (llama.cpp:4372-4460): qkv_dev rows are [head][q | k | v][64] (fused projection + bias); per-head LayerNorm of Q and K
 * (attn_q_norm / attn_k_norm), NeoX RoPE over the first 32 values of a head (rope_table: pi_rope_table_create_ex(n_pos, 32, 32, ...)), f16 Q and cache rows */
PI_API int pi_op_persimmon_qkv_store(const float * qkv_dev, int n_head, int head_dim, const float * q_norm_w, const float * q_norm_b, const float * k_norm_w, const float * k_norm_b,
                                     float eps, const int32_t * pos_dev, const void * rope_table, int n_tok, int kv_head,
                                     uint16_t * q16_dev, uint16_t * k_cache_dev, uint16_t * v_cache_dev, const int32_t * dyn_dev, void * stream);
/* mask_dev: uint32 bitmap [n_tok][ceil(n_kv/32)], bit i set <=> cell i visible to the token; out f32 [n_tok][n_head*hd].
 * dyn_dev (nullable): int32 {kv_head, n_kv} in device memory that overrides the scalar arguments at run time, so that a
 * captured HIP graph can be replayed for every call (n_kv then only sizes LDS and the mask row stride). */
PI_API int pi_op_attention(const uint16_t * q16_dev, const uint16_t * k_cache_dev, const uint16_t * v_cache_dev, const uint32_t * mask_dev,
                           int head_dim, int n_head, int n_head_kv, int n_tok, int n_kv, float * out_dev, const int32_t * dyn_dev, void * stream);
/* the same for a pass that may carry several runs (per_token_kv != 0): dyn_dev = {kv_head, n_kv of the widest run, n_tok, has_table, cell[n_tok], n_kv[n_tok]}; with
 * has_table set every token attends over the n_kv of ITS run (kv_self.n at that run's start, llama.cpp:5571) */
PI_API int pi_op_attention_ex(const uint16_t * q16_dev, const uint16_t * k_cache_dev, const uint16_t * v_cache_dev, const uint32_t * mask_dev,
                              int head_dim, int n_head, int n_head_kv, int n_tok, int n_kv, float * out_dev, const int32_t * dyn_dev, int per_token_kv, void * stream);
/* ... with ALiBi (llm_build_kqv with max_alibi_bias > 0, llama.cpp:3735-3740; ggml_compute_forward_alibi_f32, ggml.c:10736-10793): score = i * m_k + kq * scale, i the cell's index in
 * the n_kv view, m_k the slope of query head k.  alibi_slopes_dev: f32 [n_head] (pi_alibi_slopes writes the host values), nullable = no bias */
PI_API void pi_alibi_slopes(int n_head, float max_bias, float * out_host);
PI_API int pi_op_attention_alibi(const uint16_t * q16_dev, const uint16_t * k_cache_dev, const uint16_t * v_cache_dev, const uint32_t * mask_dev,
                                 int head_dim, int n_head, int n_head_kv, int n_tok, int n_kv, float * out_dev, const int32_t * dyn_dev, int per_token_kv,
                                 const float * alibi_slopes_dev, void * stream);
PI_API int pi_op_mmq_min_tokens(void);                             /* narrowest batch that pi_op_mul_mat sends to the matrix-core kernel (and its tile-major weight copies) */
PI_API int pi_op_mul_mat_reserve(void);                            /* once per process, outside graph capture: dynamic-LDS limits of the matrix-core kernels */
PI_API int pi_op_attention_max_cells(void);                       /* longest context the attention kernel serves (one score row per workgroup in LDS): 36 200 cells */
PI_API int pi_op_attention_reserve(int head_dim, int n_kv_max);   /* once per context, outside graph capture: LDS limit for long contexts */
PI_API int pi_op_silu_mul(const float * gate_dev, const float * up_dev, float * out_dev, int64_t n, void * stream);
PI_API int pi_op_gelu(const float * x_dev, float * out_dev, int64_t n, void * stream);
PI_API int pi_op_add(const float * a_dev, const float * b_dev, float * out_dev, int64_t n, void * stream);
/* ggml_add with a row broadcast (the bias of a projection, llama.cpp:3628-3630, 3770-3772): x[t][i] += b[i] */
PI_API int pi_op_add_bias(float * x_dev, const float * b_dev, int64_t n, int n_tok, void * stream);
/* ggml_clamp (ggml.c:10893-10931: MAX(MIN(x, max), min); MPT's clamp_kqv, llama.cpp:4755-4757) in place */
PI_API int pi_op_clamp(float * x_dev, float lo, float hi, int64_t n, void * stream);
/* per token: ids/logits of the k largest (logit desc, id asc), max logit and sum_i expf(l_i - max) over the full vocab */
PI_API size_t pi_op_topk_scratch_bytes(int n_tok);                  /* caller-owned scratch, one per stream */
PI_API int pi_op_topk(const float * logits_dev, int n_vocab, int n_tok, int k, int32_t * ids_dev, float * vals_dev, float * sumexp_dev, void * scratch_dev, void * stream);

/* ---- dense bfloat16 matrices and the operators of hybrid blocks (recurrent / low-rank-attention mixers, routed feed-forwards) --------------------------------------
 * Weights are PI_BF16 pi_weights ([rows][K] as stored, pi_weight_upload(PI_BF16, K, rows, ...)); activations, norms, scores, states and outputs are fp32.
 * exact = 0: activations are rounded to bfloat16 where they enter a matrix product (fp32 accumulation); exact = 1: nothing is rounded, every product is an fp32 fma. */
enum pi_act { PI_ACT_NONE = 0, PI_ACT_SILU = 1, PI_ACT_SIGMOID = 2, PI_ACT_RELU_SQR = 3, PI_ACT_TANH = 4, PI_ACT_GELU_TANH = 5 /* 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))) */,
              PI_ACT_GELU_ERF = 6 /* 0.5 z (1 + erf(z / sqrt 2)) */ };
/* out[t][:] = widen(table[tokens[t]]) * scale */
PI_API int pi_op_embed(const pi_weight * table, const int32_t * tokens_dev, int n_tok, float scale, float * out_dev, void * stream);
/* out[t][r] = act(W[r] . x[t]); rows [0, rows_a) take act_a, the others act_b (projections that share their input are one matrix and one launch); strides in floats */
PI_API int pi_op_dense(const pi_weight * w, const float * x_dev, int64_t x_stride, int n_tok, float * out_dev, int64_t out_stride, int act_a, int64_t rows_a, int act_b, int exact, void * stream);
/* y = x / sqrt(mean(x^2) + eps) * (w + w_offset) [* gate]; out = [residual +] mult * y.  to_cells != 0: row t is written to row cell(t) of `out` (dyn_dev as for pi_op_attention_ex) */
PI_API int pi_op_rms_scale(const float * x_dev, int64_t x_stride, const float * w_dev, float w_offset, float eps, int n, int n_tok, const float * gate_dev, int64_t gate_stride,
                           const float * residual_dev, int64_t residual_stride, float mult, float * out_dev, int64_t out_stride, const int32_t * dyn_dev, int to_cells, void * stream);
/* Linear attention with a per-head decay: S <- decay[h] * S + k v^T, o = S^T q, token by token.  q / k: [n_tok][heads * dim], v: [n_tok][heads * vdim], all `stride` floats apart;
 * state_dev: [slots][heads][dim][vdim] fp32; rec_dev[t]: the slot of token t's sequence, | 1 << 30 on a token whose sequence starts from a zero state; tokens of one slot are
 * consecutive and at most max_segments slots occur in a pass */
PI_API int pi_op_linear_attention(const float * q_dev, const float * k_dev, const float * v_dev, int64_t stride, int heads, int dim, int vdim, const float * decay_dev, float * state_dev,
                                  const int32_t * rec_dev, int n_tok, int max_segments, float * scratch_dev, size_t scratch_floats, float * out_dev, int64_t out_stride, void * stream);
/* passes of more than 32 tokens cut the sequences into pieces that run side by side (the recurrence is linear in the state): floats of scratch they need (0 for shorter passes) */
PI_API size_t pi_op_linear_attention_scratch_floats(int heads, int dim, int vdim, int n_tok, int max_segments);
PI_API int pi_op_linear_attention_reserve(void);                   /* once per process, outside graph capture: the LDS limit wide keys need */
PI_API int pi_op_copy_f32(const float * src_dev, float * dst_dev, int64_t n, void * stream);
/* Attention over a cache of latents c [cells][rank] fp32 shared by all heads: k = W_uk c, v = W_uv c per head, never materialised (W_uk is folded into the query, W_uv applied to
 * the weighted sum of latents); score = q . k * scale; soft-max whose denominator also holds exp(sink[h]).  mask_dev / n_kv / dyn_dev as for pi_op_attention_ex (single run).
 * scratch_dev: pi_op_latent_attention_scratch_floats(heads, rank, widest pass, n_kv) floats (folded queries and the partial results of the cell-range splits) */
PI_API int pi_op_latent_attention(const float * q_dev, int64_t q_stride, const float * cache_dev, const uint32_t * mask_dev, const pi_weight * w_uk, const pi_weight * w_uv, const float * sink_dev,
                                  float scale, int heads, int dim, int vdim, int rank, int n_tok, int n_kv, float * scratch_dev, size_t scratch_floats, float * out_dev, int64_t out_stride,
                                  const int32_t * dyn_dev, void * stream);
PI_API size_t pi_op_latent_attention_scratch_floats(int heads, int rank, int n_tok, int n_kv);
PI_API int pi_op_latent_attention_reserve(void);                   /* once per process, outside graph capture: LDS limit of the score kernels */
PI_API int pi_op_latent_attention_max_cells(int rank);             /* longest context the kernels serve */
/* Router of a mixture of experts: scores = softmax(W_router x) over all outputs; the `top` outputs with the largest score + correction are chosen (lowest index wins a tie); their
 * weights are the scores themselves.  sel_dev / selw_dev: [n_tok][top] */
PI_API int pi_op_moe_route(const pi_weight * router, const float * correction_dev, const float * x_dev, int64_t x_stride, int n_tok, int top, int exact, int32_t * sel_dev, float * selw_dev, void * stream);
/* out[t] = sum over the chosen outputs e of weight * (e < n_exp ? W_down[e] relu(W_up[e] x[t])^2 : x[t]); w_up: [n_exp * ff][width], w_down: [n_exp * width][ff]; up_dev: scratch [n_tok][top][ff] */
PI_API int pi_op_moe_experts(const pi_weight * w_up, const pi_weight * w_down, int n_exp, int ff, const float * x_dev, int64_t x_stride, const int32_t * sel_dev, const float * selw_dev, int n_tok, int top,
                             int exact, float * up_dev, float * out_dev, int64_t out_stride, void * stream);
/* the same result for a prompt's worth of tokens, serving precision: the (token, choice) slots are sorted by expert on the device and every expert's run goes through the
 * matrix cores 64 slots at a time.  up_dev: [n_tok * top][ff], dn_dev: [n_tok * top][width], idx_dev: pi_op_moe_grouped_index_ints(n_tok, top, n_exp) int32 */
PI_API int pi_op_moe_grouped_ok(const pi_weight * w_up, const pi_weight * w_down, int n_exp, int ff, int glu, int n_tok, int top, int exact);
PI_API size_t pi_op_moe_grouped_index_ints(int n_tok, int top, int n_exp);
PI_API int pi_op_moe_experts_grouped(const pi_weight * w_up, const pi_weight * w_down, int n_exp, int ff, const float * x_dev, int64_t x_stride, const int32_t * sel_dev, const float * selw_dev, int n_tok, int top,
                                     float * up_dev, float * dn_dev, int32_t * idx_dev, float * out_dev, int64_t out_stride, void * stream);

/* ---- operators of blocks with pre- and post-norms, a learned average over depth, and a mixer of two branches (chunked sigmoid attention beside a selective recurrence) ---- */
/* y = LayerNorm(ca * a + cb * b) * w + bias (b nullable: one input; the variance is the mean of squared deviations, eps inside the root); out = [residual +] y */
PI_API int pi_op_layer_norm_mix(const float * a_dev, int64_t a_stride, float ca, const float * b_dev, int64_t b_stride, float cb, const float * w_dev, const float * bias_dev, float eps, int n, int n_tok,
                                const float * residual_dev, int64_t residual_stride, float * out_dev, int64_t out_stride, void * stream);
/* the end of a block in one launch: v = [residual +] LayerNorm(ca * a + cb * b) * w + bias -> out_a;  n_hist > 0: v = sum_(j < n_hist - 1) coef[j] * hist[j] + coef[n_hist - 1] * v -> out_mix
 * (out_a must be the history's last entry, rows n floats apart);  w_next != NULL: LayerNorm(v) * w_next + bias_next -> out_next.  In place (out_a == residual, out_mix == residual) is allowed */
PI_API int pi_op_norm_chain(const float * a_dev, int64_t a_stride, float ca, const float * b_dev, int64_t b_stride, float cb, const float * w_dev, const float * bias_dev, float eps, int n, int n_tok,
                            const float * residual_dev, int64_t residual_stride, float * out_a_dev, int64_t out_a_stride, const float * hist_dev, int64_t hist_stride, int n_hist, const float * coef_dev,
                            float * out_mix_dev, int64_t out_mix_stride, const float * w_next, const float * bias_next, float * out_next_dev, int64_t out_next_stride, void * stream);
/* out[t] = sum_j coef[j] * hist[j][t], j = 0 .. n_hist - 1 in this order; hist: n_hist arrays of n_tok rows of n floats, hist_stride floats apart; coef_dev: fp32 [n_hist] */
PI_API int pi_op_depth_mix(const float * hist_dev, int64_t hist_stride, int n_hist, const float * coef_dev, int n, int n_tok, float * out_dev, int64_t out_stride, void * stream);
/* x <- cap * tanh(x / cap), in place */
PI_API int pi_op_softcap(float * x_dev, int64_t n, float cap, void * stream);
/* out[t][f] = in[t][f] * in[t][ff + f] */
PI_API int pi_op_glu_mul(const float * in_dev, int64_t in_stride, int ff, int n_tok, float * out_dev, int64_t out_stride, void * stream);
/* pi_op_linear_attention with its options: qk_heads query / key heads shared by heads / qk_heads neighbouring heads each; tdecay_dev / tscale_dev (nullable): fp32 [n_tok][heads]
 * rows t_stride floats apart, S <- tdecay[t][h] * S + tscale[t][h] * k v^T (tdecay replaces decay_dev); skip_dev (nullable, [heads]): o += skip[h] * v */
PI_API int pi_op_linear_attention_ex(const float * q_dev, const float * k_dev, const float * v_dev, int64_t stride, int heads, int qk_heads, int dim, int vdim, const float * decay_dev, const float * tdecay_dev,
                                     const float * tscale_dev, int64_t t_stride, const float * skip_dev, float * state_dev, const int32_t * rec_dev, int n_tok, int max_segments, float * scratch_dev,
                                     size_t scratch_floats, float * out_dev, int64_t out_stride, void * stream);
/* cos / sin of p * base^(-2i / dims), p < n_pos, i < dims / 2 (angles formed in double precision on the host) */
PI_API void * pi_rotary_table_create(int n_pos, int dims, float base);
PI_API int    pi_rotary_table_positions(const void * table);
PI_API void   pi_rotary_table_free(void * table);
/* per token: q and k heads RMS-normed over dim with a weight shared by the heads (eps inside the root), then their first `dims` dimensions rotated by the token's position (dimension i
 * pairs with i + dims / 2); v heads divided by their root mean square.  q goes to q_out, k and v to the token's cell of k_cache [cells][kv_heads * dim] / v_cache [cells][kv_heads * vdim]
 * (fp32), and cell_pos_dev [cells] learns the cell's position.  q / k / v rows are `stride` floats apart; dyn_dev as for pi_op_attention_ex */
PI_API int pi_op_qkv_prepare(const float * q_dev, const float * k_dev, const float * v_dev, int64_t stride, const float * q_norm_w, const float * k_norm_w, float eps, int heads, int kv_heads, int dim, int vdim,
                             const void * rotary_table, const int32_t * pos_dev, int n_tok, float * q_out_dev, int64_t q_out_stride, float * k_cache_dev, float * v_cache_dev, int32_t * cell_pos_dev,
                             const int32_t * dyn_dev, void * stream);
/* out[t][h] = out_mult * gate[t][h] * sum over the cells c that token t sees of sigmoid(q[t][h] . K[c][h / (heads / kv_heads)] * scale + head_bias[h]) * V[c][..]: no soft-max, no normalisation.
 * A cell is seen when its bit of the pass's mask is set AND (chunk > 0) its position is not below the start of the chunk of `chunk` positions that holds the token's position.
 * head_bias_dev, gate_dev nullable (0 and 1); gate_act: PI_ACT_SIGMOID when the gate values are still raw */
PI_API int pi_op_chunk_attention(const float * q_dev, int64_t q_stride, const float * k_cache_dev, const float * v_cache_dev, const int32_t * cell_pos_dev, const uint32_t * mask_dev, const int32_t * pos_dev,
                                 const float * head_bias_dev, const float * gate_dev, int64_t gate_stride, int gate_act, float scale, float out_mult, int chunk, int heads, int kv_heads, int dim, int vdim, int n_tok, int n_kv,
                                 float * out_dev, int64_t out_stride, const int32_t * dyn_dev, void * stream);
/* out[t][c] = act(bias[c] + sum_l w[c][l] * input(t - (taps - 1 - l))[c]) over the tokens of each sequence (rec_dev as for pi_op_linear_attention); inputs from before the pass come from
 * state_dev [slots][taps - 1][channels] (oldest first; zeros for a sequence that starts), which then takes the sequence's last taps - 1 inputs.  w_dev: fp32 [channels][taps] */
PI_API int pi_op_causal_conv(const float * x_dev, int64_t x_stride, int channels, int taps, const float * w_dev, const float * bias_dev, float * state_dev, const int32_t * rec_dev, int n_tok, int act,
                             float * out_dev, int64_t out_stride, void * stream);
/* pi_op_causal_conv and pi_op_ssd_steps together: ONE launch where the pass has at most 32 tokens and the convolution at most 8 taps (a sequence's tokens are then walked by one
 * thread per channel, which also leaves the new state), the separate launches otherwise */
PI_API int pi_op_causal_conv_steps(const float * x_dev, int64_t x_stride, int channels, int taps, const float * w_dev, const float * bias_dev, float * state_dev, const int32_t * rec_dev, int n_tok, int act,
                                   float * out_dev, int64_t out_stride, const float * raw_dev, int64_t raw_stride, const float * dt_bias_dev, const float * a_log_dev, int heads, float * dt_out_dev,
                                   float * decay_out_dev, void * stream);
/* dt[t][h] = softplus(raw[t][h] + dt_bias[h]); decay[t][h] = exp(-exp(a_log[h]) * dt[t][h]); outputs [n_tok][heads] */
PI_API int pi_op_ssd_steps(const float * raw_dev, int64_t raw_stride, const float * dt_bias_dev, const float * a_log_dev, int heads, int n_tok, float * dt_out_dev, float * decay_out_dev, void * stream);
/* u = y * silu(z); out = u / rms(u over each of `groups` equal parts) * w * mult */
PI_API int pi_op_gate_group_norm(const float * y_dev, int64_t y_stride, const float * z_dev, int64_t z_stride, const float * w_dev, float eps, float mult, int n, int groups, int n_tok, float * out_dev, int64_t out_stride, void * stream);
/* router with sigmoid scores and a group-restricted choice: consecutive outputs are bundled into n_groups groups of equal size, a group is ranked by top1 + top2 of its members' scores, the
 * choice is restricted to members of the `keep` highest-ranked groups; among them the `top` highest scores win, and those scores themselves are the mixing weights */
PI_API int pi_op_moe_route_groups(const pi_weight * router, const float * x_dev, int64_t x_stride, int n_tok, int top, int n_groups, int keep, int exact, int32_t * sel_dev, float * selw_dev, void * stream);
/* the grouped path with the expert's activation as a parameter (glu as for pi_op_moe_experts_act; up_dev is then [n_tok * top][2 * ff]) */
PI_API int pi_op_moe_experts_grouped_act(const pi_weight * w_up, const pi_weight * w_down, int n_exp, int ff, int glu, const float * x_dev, int64_t x_stride, const int32_t * sel_dev, const float * selw_dev, int n_tok, int top,
                                         float * up_dev, float * dn_dev, int32_t * idx_dev, float * out_dev, int64_t out_stride, void * stream);
/* pi_op_moe_experts with the expert's activation as a parameter: glu = 0: relu(W_up x)^2; glu = 1: w_up holds [gate (ff rows) | up (ff rows)] per expert and the hidden values are silu(gate) * up */
PI_API int pi_op_moe_experts_act(const pi_weight * w_up, const pi_weight * w_down, int n_exp, int ff, int glu, const float * x_dev, int64_t x_stride, const int32_t * sel_dev, const float * selw_dev, int n_tok, int top,
                                 int exact, float * up_dev, float * out_dev, int64_t out_stride, void * stream);

/* ---- operators of blocks whose norm comes after the sum, of recurrences with a decay per key channel, and of soft-max attention inside chunks -------------------------------- */
/* out[t][:] = widen(table[tokens[t]]) * scale + widen(table2[rows2[t]]) (a row outside its table counts as zeros) */
PI_API int pi_op_embed_pair(const pi_weight * table, const int32_t * tokens_dev, int n_tok, float scale, const pi_weight * table2, const int32_t * rows2_dev, float * out_dev, void * stream);
/* pi_op_dense over a matrix whose rows fall into n_seg segments that each read an input of their own: rows [g * seg_rows, (g + 1) * seg_rows) read x + g * seg_off, the last segment takes the
 * remaining rows (projections of DIFFERENT inputs of one width in one launch where the pass has few tokens) */
PI_API int pi_op_dense_segments(const pi_weight * w, const float * x_dev, int64_t x_stride, int64_t seg_rows, int64_t seg_off, int n_seg, int n_tok, float * out_dev, int64_t out_stride, int act_a, int64_t rows_a,
                                int act_b, int exact, void * stream);
/* the end of a sublayer, R(y) = y / sqrt(mean(y^2) + eps):  m = b ? mean_mult * (R(a) * wa + R(b) * wb) : a;  out = R(alpha * x + layer_scale * m) * w  (layer_scale nullable: 1);
 * w_next != NULL: out_next = R(out) * w_next (the norm of whatever reads the stream next).  out may be x.  Rows of at most 8192 values */
PI_API int pi_op_rms_post(const float * a_dev, int64_t a_stride, const float * wa_dev, const float * b_dev, int64_t b_stride, const float * wb_dev, float mean_mult, const float * layer_scale_dev,
                          const float * x_dev, int64_t x_stride, float alpha, const float * w_dev, float eps, int n, int n_tok, float * out_dev, int64_t out_stride, const float * w_next_dev, float * out_next_dev,
                          int64_t out_next_stride, void * stream);
/* out[t][s][:] = h[t] + (h_prev - h[t]) * mu[s], s < n_mix (rows out_stride >= n_mix * n floats apart); h_prev: the sequence's previous token — the row before inside the pass, state_dev [slots][n] at a
 * sequence's first token of the pass (zeros on a fresh slot); the sequence's last token of the pass becomes its state.  rec_dev as for pi_op_linear_attention */
PI_API int pi_op_token_shift(const float * h_dev, int64_t h_stride, int n, const float * mu_dev, int n_mix, float * state_dev, const int32_t * rec_dev, int n_tok, float * out_dev, int64_t out_stride, void * stream);
/* Recurrence over a [dim][vdim] state per head and sequence with a decay g[t][h][i] per token and key channel (state_dev [slots][heads][dim][vdim], rec_dev as for pi_op_linear_attention):
 *   PI_RULE_DELTA  S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q              beta[t][h] = sigmoid(beta_raw) (nullable: 1)
 *   PI_RULE_BONUS  o = (S + diag(bonus_h) k v^T)^T q;  S <- diag(g) S + k v^T                       bonus_dev [heads][dim] (nullable: 0)
 * decay_mode 0: g = decay_raw; 1: g = exp(-exp(decay_raw + decay_bias[h][i])); 2: g = exp(-exp(a_log[h]) * softplus(decay_raw + decay_bias[h][i])).  qk_unit: q and k are divided by their length
 * (sqrt(sum of squares + 1e-6)) per head first; q is then multiplied by q_mult.  q / k: [n_tok][qk_heads * dim] (head h reads q / k head h / (heads / qk_heads)), v: [n_tok][heads * vdim] */
enum pi_recurrence_rule { PI_RULE_DELTA = 0, PI_RULE_BONUS = 1 };
PI_API int pi_op_channel_recurrence(int rule, const float * q_dev, int64_t q_stride, const float * k_dev, int64_t k_stride, const float * v_dev, int64_t v_stride, const float * decay_raw_dev, int64_t decay_stride,
                                    int decay_mode, const float * decay_bias_dev, const float * a_log_dev, const float * beta_raw_dev, int64_t beta_stride, const float * bonus_dev, int qk_unit, float q_mult,
                                    int heads, int qk_heads, int dim, int vdim, float * state_dev, const int32_t * rec_dev, int n_tok, int max_segments, float * scratch_dev, size_t scratch_floats,
                                    float * out_dev, int64_t out_stride, void * stream);
/* passes of more than 32 tokens cut the sequences into pieces that run side by side (a column's step is affine in the column): floats of scratch they need; with less the pass is walked token by token */
PI_API size_t pi_op_channel_recurrence_scratch_floats(int heads, int dim, int vdim, int n_tok, int max_segments);
PI_API int pi_op_channel_recurrence_reserve(void);                 /* once per process, outside graph capture: the LDS limit wide keys need */
/* out[t][h][i] = y[t][h][i] / sqrt(mean_i(y[t][h]^2) + eps) * w[(w_per_head ? h * n : 0) + i] * act(gate[t][h][i]) (gate nullable; gate_act PI_ACT_NONE, _SIGMOID or _SILU); out may be y */
PI_API int pi_op_head_norm_gate(const float * y_dev, int64_t y_stride, int heads, int n, const float * w_dev, int w_per_head, const float * gate_dev, int64_t gate_stride, int gate_act, float eps, int n_tok,
                                float * out_dev, int64_t out_stride, void * stream);
/* pi_op_qkv_prepare with its order and pairing as parameters: norm_first != 0: R(.) * w then the rotation, else the rotation first and R(.) * w over the rotated head (weights nullable: 1);
 * pairing: dimension i with i + dims / 2, or 2i with 2i + 1; v_norm = 0: value heads are cached as they are */
enum pi_rot_pairing { PI_PAIR_HALVES = 0, PI_PAIR_NEIGHBOURS = 1 };
PI_API int pi_op_qkv_prepare_ex(const float * q_dev, const float * k_dev, const float * v_dev, int64_t stride, const float * q_norm_w, const float * k_norm_w, float eps, int heads, int kv_heads, int dim, int vdim,
                                const void * rotary_table, int norm_first, int pairing, int v_norm, const int32_t * pos_dev, int n_tok, float * q_out_dev, int64_t q_out_stride, float * k_cache_dev, float * v_cache_dev,
                                int32_t * cell_pos_dev, const int32_t * dyn_dev, void * stream);
/* pi_op_chunk_attention with the kind of weights as a parameter.  s = q . k * scale + head_bias[h], softcap > 0: s <- softcap * tanh(s / softcap) (soft-max kinds);
 * PI_WEIGHTS_SIGMOID: sigmoid(s), nothing normalised; PI_WEIGHTS_SOFTMAX: exp(s) / sum exp(s) over the visible cells; PI_WEIGHTS_SOFTMAX_SINK: exp(s) / (1 + sum exp(s)) */
enum pi_attention_weights { PI_WEIGHTS_SIGMOID = 0, PI_WEIGHTS_SOFTMAX = 1, PI_WEIGHTS_SOFTMAX_SINK = 2 };
PI_API int pi_op_chunk_attention_ex(const float * q_dev, int64_t q_stride, const float * k_cache_dev, const float * v_cache_dev, const int32_t * cell_pos_dev, const uint32_t * mask_dev, const int32_t * pos_dev,
                                    const float * head_bias_dev, const float * gate_dev, int64_t gate_stride, int gate_act, float scale, float out_mult, int weights, float softcap, int chunk, int heads, int kv_heads,
                                    int dim, int vdim, int n_tok, int n_kv, float * out_dev, int64_t out_stride, const int32_t * dyn_dev, void * stream);

/* ---- operators of layers whose mixer and feed-forward read ONE tanh norm, of sliding-window attention with pooled far blocks, and of clipped gated experts ------------------- */
/* rows of n floats, strides in floats */
PI_API int pi_op_copy_rows(const float * src_dev, int64_t src_stride, float * dst_dev, int64_t dst_stride, int n, int n_tok, void * stream);
/* the end of a layer and the norm of what reads the stream next, in one launch:  x_out = x + a + b + c (a, b, c nullable; x_out may be x);  w != NULL: h_out = tanh(alpha * x_out) * w + bias
 * (a norm without statistics; alpha_dev: one float on the device).  x_out may be NULL when only the norm is wanted (then a, b, c are still added for h) */
PI_API int pi_op_sum_tanh_norm(const float * x_dev, int64_t x_stride, const float * a_dev, int64_t a_stride, const float * b_dev, int64_t b_stride, const float * c_dev, int64_t c_stride, int n, int n_tok,
                               float * x_out_dev, int64_t x_out_stride, const float * alpha_dev, const float * w_dev, const float * bias_dev, float * h_out_dev, int64_t h_out_stride, void * stream);
/* pi_op_sum_tanh_norm and, of its norm output, pi_op_token_shift with one mix: m_out = h + (h_prev - h) * mu; one launch for passes of at most 32 tokens */
PI_API int pi_op_sum_tanh_norm_shift(const float * x_dev, int64_t x_stride, const float * a_dev, int64_t a_stride, const float * b_dev, int64_t b_stride, const float * c_dev, int64_t c_stride, int n, int n_tok,
                                     float * x_out_dev, int64_t x_out_stride, const float * alpha_dev, const float * w_dev, const float * bias_dev, float * h_out_dev, int64_t h_out_stride,
                                     const float * mu_dev, float * state_dev, const int32_t * rec_dev, float * m_out_dev, int64_t m_out_stride, void * stream);
/* pi_rotary_table_create with angle steps stretched by wavelength l = 2 pi / f against `original` positions: f stays where l < original / high, becomes f / factor where l > original / low, and
 * (1 - s) f / factor + s f with s = (original / l - low) / (high - low) between the two */
PI_API void * pi_rotary_table_create_scaled(int n_pos, int dims, float base, float factor, float low, float high, int original);
/* pi_op_qkv_prepare_ex's norm_first takes these: rotation first, then R(.) * w over the rotated head; R(.) * w, then the rotation; the rotation alone */
enum pi_qk_norm { PI_QK_NORM_LAST = 0, PI_QK_NORM_FIRST = 1, PI_QK_NORM_NONE = 2 };
/* which cells of its sequence a token sees besides "not later": those of its own block of `size` positions (blocks start at multiples of size), or the last `size` positions up to itself */
enum pi_mask_kind { PI_MASK_CHUNK = 0, PI_MASK_WINDOW = 1 };
/* Pooled far blocks.  The caches hold two rows per cell: row c the token's own key / value, row pooled_row_offset + c — on the cell of a block's LAST position, (pos + 1) % pool == 0 — the means of the
 * keys / values of the block's `pool` positions as the cache holds them, summed in position order.  This writes those rows for the tokens of the pass that complete a block (their block mates are the
 * visible cells of the `pool - 1` positions before them); call it behind pi_op_qkv_prepare(_ex) and ahead of the attention.  k_cache: [2 * offset.. rows][kv_heads * dim], v_cache likewise */
PI_API int pi_op_pool_blocks(float * k_cache_dev, float * v_cache_dev, const int32_t * cell_pos_dev, const uint32_t * mask_dev, const int32_t * pos_dev, int pool, int64_t pooled_row_offset, int kv_heads, int dim, int vdim,
                             int n_tok, int n_kv, const int32_t * dyn_dev, void * stream);
/* pi_op_chunk_attention_ex with the mask kind as a parameter and two more sources of weight.  mask_kind PI_MASK_WINDOW: a token at position p sees the cells of its sequence at positions (p - size, p]
 * (size 0: all up to p); pool > 0 (windows only): and for every block of `pool` positions that ends at or before p - size the pooled row (pi_op_pool_blocks) of the block's last cell, in the same soft-max.
 * sink_dev (nullable, fp32 [heads]; soft-max kinds): exp(sink[h]) joins the denominator, without a value and without the scale (PI_WEIGHTS_SOFTMAX_SINK alone is sink = 0).
 * pool_here != 0: an extra slice of workgroups does pi_op_pool_blocks' work in the same launch — allowed where no token of the pass can read a row that the pass writes, n_tok <= size */
PI_API int pi_op_window_attention(const float * q_dev, int64_t q_stride, float * k_cache_dev, float * v_cache_dev, const int32_t * cell_pos_dev, const uint32_t * mask_dev, const int32_t * pos_dev,
                                  const float * head_bias_dev, const float * sink_dev, const float * gate_dev, int64_t gate_stride, int gate_act, float scale, float out_mult, int weights, float softcap, int mask_kind, int size,
                                  int pool, int64_t pooled_row_offset, int pool_here, int heads, int kv_heads, int dim, int vdim, int n_tok, int n_kv, float * scratch_dev, size_t scratch_floats, float * out_dev, int64_t out_stride,
                                  const int32_t * dyn_dev, void * stream);
/* scratch_dev (nullable): with pi_op_window_attention_scratch_floats(heads, vdim, n_tok) floats a pass of few tokens cuts the cell range into splits that run side by side and merges them in a second launch */
PI_API size_t pi_op_window_attention_scratch_floats(int heads, int vdim, int n_tok);
/* router by logits: z = W x + bias (bias nullable), the `top` largest z win (lowest index on a tie), their weights are the soft-max over the chosen z alone */
PI_API int pi_op_moe_route_top_logits(const pi_weight * router, const float * bias_dev, const float * x_dev, int64_t x_stride, int n_tok, int top, int exact, int32_t * sel_dev, float * selw_dev, void * stream);
/* the expert operators with one more kind of hidden layer.  PI_GLU_OFF / PI_GLU_SILU are glu = 0 / 1 of pi_op_moe_experts_act; PI_GLU_CLIPPED: g = min(gate, limit), u = clip(up, -limit, limit)
 * (limit <= 0: no bounds), hidden = g * sigmoid(1.702 g) * (u + 1) */
enum pi_glu_kind { PI_GLU_OFF = 0, PI_GLU_SILU = 1, PI_GLU_CLIPPED = 2 };
PI_API int pi_op_moe_experts_glu(const pi_weight * w_up, const pi_weight * w_down, int n_exp, int ff, int glu, float limit, const float * x_dev, int64_t x_stride, const int32_t * sel_dev, const float * selw_dev, int n_tok,
                                 int top, int exact, float * up_dev, float * out_dev, int64_t out_stride, void * stream);
PI_API int pi_op_moe_experts_grouped_glu(const pi_weight * w_up, const pi_weight * w_down, int n_exp, int ff, int glu, float limit, const float * x_dev, int64_t x_stride, const int32_t * sel_dev, const float * selw_dev,
                                         int n_tok, int top, float * up_dev, float * dn_dev, int32_t * idx_dev, float * out_dev, int64_t out_stride, void * stream);
/* out[t][f] = hidden(in[t][f], in[t][ff + f]) [* sigmoid(in[t][gate_col])]: a gated hidden layer whose halves [gate | up] a projection left raw (glu / limit as above, PI_GLU_OFF: the plain product of
 * pi_op_glu_mul); gate_col >= 0: one more column of the same rows holds a per-token gate */
PI_API int pi_op_glu_mul_ex(const float * in_dev, int64_t in_stride, int ff, int glu, float limit, int64_t gate_col, int n_tok, float * out_dev, int64_t out_stride, void * stream);

#ifdef __cplusplus
}
#endif
#endif
