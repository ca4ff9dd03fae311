"""ctypes loader for libpipeinfer_amd.so (HIP kernels + engine, C ABI in include/*.h).

There is no fallback: if the shared library is missing or no MI355X is visible, the compute entry points raise."""
import ctypes as C
import os
import re
import subprocess

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
SO = os.environ.get("PIPEINFER_LIB") or os.path.join(PKG, "libpipeinfer_amd.so")        # (override: A/B runs of two builds on one box, tools_dev/)

SO_DENSE = os.path.join(PKG, "libpipeinfer_amd_dense.so")     # `make dense`: the engine with the dense-weight kernels only (hybrid safetensors models need no more)

_lib = None


class PipeInferError(RuntimeError):
    pass


def build(force=False):
    """compile the HIP extension in-tree (hipcc cross-compiles gfx950 without a GPU)"""
    if force or not os.path.exists(SO) or _stale():
        subprocess.check_call(["make", "-C", os.path.join(PKG, "csrc"), "-j8"], stdout=subprocess.DEVNULL)
    return SO


def build_dense():
    """the library a model of dense bfloat16 weights needs, where the full one is not there: the engine + the dense / hybrid kernels (a fraction of the full build's time)"""
    if os.path.exists(SO) and not _stale():
        return SO
    if not os.path.exists(SO_DENSE) or _stale(SO_DENSE):
        subprocess.check_call(["make", "-C", os.path.join(PKG, "csrc"), "-j8", "dense"], stdout=subprocess.DEVNULL)
    return SO_DENSE


def _stale(so=None):
    t = os.path.getmtime(so or SO)
    for d in (os.path.join(PKG, "csrc", "kernels"), os.path.join(PKG, "csrc", "engine"), os.path.join(ROOT, "include")):
        if os.path.isdir(d):
            for f in os.listdir(d):
                if os.path.getmtime(os.path.join(d, f)) > t:
                    return os.path.exists("/opt/rocm/bin/hipcc")
    return False


def declared_symbols():
    """every PI_API / LLAMA_API / GGML_API function name declared in include/*.h"""
    names = []
    inc = os.path.join(ROOT, "include")
    for f in sorted(os.listdir(inc)):
        if f.endswith(".h"):
            text = open(os.path.join(inc, f)).read()
            text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
            text = re.sub(r"//[^\n]*", "", text)
            text = re.sub(r"#define[^\n]*", "", text)
            text = text.replace("DEPRECATED(", "")
            names += re.findall(r"(?:PI_API|LLAMA_API|GGML_API)\s+[^;{]*?\b(\w+)\s*\(", text)
    return sorted(set(names))


def load(dense_ok=False):
    """dense_ok: the caller only runs dense-weight (safetensors) models, so where the full library is missing the dense-only build will do"""
    global _lib
    if _lib is None:
        so = SO
        if not os.path.exists(SO):
            if not os.path.exists("/opt/rocm/bin/hipcc") and not (dense_ok and os.path.exists(SO_DENSE)):
                raise PipeInferError(f"{SO} is missing and hipcc is not available: the MI355X path has no fallback")
            so = build_dense() if dense_ok else build()
        lib = C.CDLL(so)
        _declare(lib)
        _lib = lib
    return _lib


def check(rc, what=""):
    if rc != 0:
        raise PipeInferError(f"{what} failed: {load().pi_last_error().decode()}")


def _declare(lib):
    vp, i32, i64, f32, sz = C.c_void_p, C.c_int, C.c_int64, C.c_float, C.c_size_t
    lib.pi_last_error.restype = C.c_char_p
    lib.pi_device_count.restype = i32
    lib.pi_device_init.argtypes = [i32]
    lib.pi_malloc.restype = vp
    lib.pi_malloc.argtypes = [sz]
    lib.pi_free.argtypes = [vp]
    lib.pi_memcpy_h2d.argtypes = [vp, vp, sz, vp]
    lib.pi_memcpy_d2h.argtypes = [vp, vp, sz, vp]
    lib.pi_memset.argtypes = [vp, i32, sz, vp]
    lib.pi_stream_sync.argtypes = [vp]
    lib.pi_set_abort_word.argtypes = [vp]; lib.pi_set_abort_word.restype = None
    lib.pi_op_abort_begin.argtypes = [vp, i32, vp, vp]
    lib.pi_op_abort_cancel.argtypes = [vp, i32, vp]
    lib.pi_op_copy_out.argtypes = [vp, vp, C.c_int64, vp, vp, vp, vp, vp, vp, i32, vp]
    lib.pi_kernel_timing.argtypes = [i32, i32]
    lib.pi_kernel_timing_rows.argtypes = [vp, i32]
    lib.pi_kernel_timing_rows.restype = i32
    lib.pi_kernel_lifetime_rows.argtypes = [vp, i32]
    lib.pi_kernel_lifetime_rows.restype = i32
    lib.pi_weight_upload.restype = vp
    lib.pi_weight_upload.argtypes = [i32, i64, i64, vp, vp]
    lib.pi_weight_free.argtypes = [vp]
    lib.pi_weight_nbytes.restype = sz
    lib.pi_weight_nbytes.argtypes = [vp]
    lib.pi_weight_type.argtypes = [vp]
    lib.pi_vec_dot_type.argtypes = [i32]
    lib.pi_q8_nbytes.restype = sz
    lib.pi_q8_nbytes.argtypes = [i32, i64, i32]
    lib.pi_q8_layout.argtypes = [i32, i64, i32, C.POINTER(sz), C.POINTER(sz), C.POINTER(sz)]
    lib.pi_op_get_rows.argtypes = [vp, vp, i32, vp, vp]
    lib.pi_op_norm.argtypes = [vp, vp, vp, vp, i32, i32, f32, i32, vp]
    lib.pi_op_quantize.argtypes = [i32, vp, i64, i32, vp, vp]
    lib.pi_op_norm_quantize.argtypes = [vp, vp, vp, vp, i32, i32, f32, i32, i32, vp, vp]
    lib.pi_op_act_quantize.argtypes = [vp, vp, i32, i64, i32, i32, vp, vp]
    lib.pi_op_mul_mat.argtypes = [vp, vp, i32, vp, vp, vp]
    lib.pi_op_mul_mat_multi.argtypes = [i32, vp, vp, i32, vp, vp, vp]
    lib.pi_op_mul_mat_qkv_rope_ok.argtypes = [vp, vp, vp, i32, i32]
    lib.pi_op_mul_mat_qkv_rope.argtypes = [vp, vp, vp, vp, i32, vp, vp, i32, i32, i32, i32, vp, vp, vp, vp, vp]
    lib.pi_rope_table_create.restype = vp
    lib.pi_rope_table_create.argtypes = [i32, i32, f32, f32, i32]
    lib.pi_rope_table_create_ex.restype = vp
    lib.pi_rope_table_create_ex.argtypes = [i32, i32, i32, f32, f32, i32]
    lib.pi_rope_table_free.argtypes = [vp]
    lib.pi_alibi_slopes.argtypes = [i32, f32, vp]; lib.pi_alibi_slopes.restype = None
    lib.pi_op_attention_alibi.argtypes = [vp, vp, vp, vp, i32, i32, i32, i32, i32, vp, vp, i32, vp, vp]
    lib.pi_op_persimmon_qkv_store.argtypes = [vp, i32, i32, vp, vp, vp, vp, f32, vp, vp, i32, i32, vp, vp, vp, vp, vp]
    lib.pi_op_add_bias.argtypes = [vp, vp, i64, i32, vp]
    lib.pi_op_clamp.argtypes = [vp, f32, f32, i64, vp]
    lib.pi_op_rope_kv_store.argtypes = [vp, vp, vp, i64, i64, i64, vp, vp, i32, i32, i32, i32, i32, i32, vp, vp, vp, vp, vp]
    lib.pi_op_attention.argtypes = [vp, vp, vp, vp, i32, i32, i32, i32, i32, vp, vp, vp]
    lib.pi_op_attention_reserve.argtypes = [i32, i32]
    lib.pi_op_silu_mul.argtypes = [vp, vp, vp, i64, vp]
    lib.pi_op_gelu.argtypes = [vp, vp, i64, vp]
    lib.pi_op_add.argtypes = [vp, vp, vp, i64, vp]
    lib.pi_op_topk_scratch_bytes.argtypes = [i32]; lib.pi_op_topk_scratch_bytes.restype = C.c_size_t
    lib.pi_op_topk.argtypes = [vp, i32, i32, i32, vp, vp, vp, vp, vp]
    # dense bfloat16 matrices and the operators of hybrid blocks
    lib.pi_op_embed.argtypes = [vp, vp, i32, f32, vp, vp]
    lib.pi_op_dense.argtypes = [vp, vp, i64, i32, vp, i64, i32, i64, i32, i32, vp]
    lib.pi_op_rms_scale.argtypes = [vp, i64, vp, f32, f32, i32, i32, vp, i64, vp, i64, f32, vp, i64, vp, i32, vp]
    lib.pi_op_linear_attention.argtypes = [vp, vp, vp, i64, i32, i32, i32, vp, vp, vp, i32, i32, vp, sz, vp, i64, vp]
    lib.pi_op_linear_attention_scratch_floats.argtypes = [i32, i32, i32, i32, i32]; lib.pi_op_linear_attention_scratch_floats.restype = sz
    lib.pi_op_copy_f32.argtypes = [vp, vp, i64, vp]
    lib.pi_op_latent_attention.argtypes = [vp, i64, vp, vp, vp, vp, vp, f32, i32, i32, i32, i32, i32, i32, vp, sz, vp, i64, vp, vp]
    lib.pi_op_latent_attention_scratch_floats.argtypes = [i32, i32, i32, i32]; lib.pi_op_latent_attention_scratch_floats.restype = sz
    lib.pi_op_latent_attention_max_cells.argtypes = [i32]
    lib.pi_op_moe_route.argtypes = [vp, vp, vp, i64, i32, i32, i32, vp, vp, vp]
    lib.pi_op_moe_experts.argtypes = [vp, vp, i32, i32, vp, i64, vp, vp, i32, i32, i32, vp, vp, i64, vp]
    lib.pi_op_moe_grouped_ok.argtypes = [vp, vp, i32, i32, i32, i32, i32, i32]
    lib.pi_op_moe_grouped_index_ints.argtypes = [i32, i32, i32]; lib.pi_op_moe_grouped_index_ints.restype = sz
    lib.pi_op_moe_experts_grouped.argtypes = [vp, vp, i32, i32, vp, i64, vp, vp, i32, i32, vp, vp, vp, vp, i64, vp]
    # blocks with pre- and post-norms, the depth average, the parallel mixer's two branches, grouped routing and gated experts
    lib.pi_op_layer_norm_mix.argtypes = [vp, i64, f32, vp, i64, f32, vp, vp, f32, i32, i32, vp, i64, vp, i64, vp]
    lib.pi_op_depth_mix.argtypes = [vp, i64, i32, vp, i32, i32, vp, i64, vp]
    lib.pi_op_softcap.argtypes = [vp, i64, f32, vp]
    lib.pi_op_glu_mul.argtypes = [vp, i64, i32, i32, vp, i64, vp]
    lib.pi_op_linear_attention_ex.argtypes = [vp, vp, vp, i64, i32, i32, i32, i32, vp, vp, vp, i64, vp, vp, vp, i32, i32, vp, sz, vp, i64, vp]
    lib.pi_rotary_table_create.restype = vp
    lib.pi_rotary_table_create.argtypes = [i32, i32, f32]
    lib.pi_rotary_table_positions.argtypes = [vp]
    lib.pi_rotary_table_free.argtypes = [vp]; lib.pi_rotary_table_free.restype = None
    lib.pi_op_qkv_prepare.argtypes = [vp, vp, vp, i64, vp, vp, f32, i32, i32, i32, i32, vp, vp, i32, vp, i64, vp, vp, vp, vp, vp]
    lib.pi_op_chunk_attention.argtypes = [vp, i64, vp, vp, vp, vp, vp, vp, vp, i64, i32, f32, f32, i32, i32, i32, i32, i32, i32, i32, vp, i64, vp, vp]
    lib.pi_op_causal_conv.argtypes = [vp, i64, i32, i32, vp, vp, vp, vp, i32, i32, vp, i64, vp]
    lib.pi_op_ssd_steps.argtypes = [vp, i64, vp, vp, i32, i32, vp, vp, vp]
    lib.pi_op_gate_group_norm.argtypes = [vp, i64, vp, i64, vp, f32, f32, i32, i32, i32, vp, i64, vp]
    lib.pi_op_norm_chain.argtypes = [vp, i64, f32, vp, i64, f32, vp, vp, f32, i32, i32, vp, i64, vp, i64, vp, i64, i32, vp, vp, i64, vp, vp, vp, i64, vp]
    lib.pi_op_causal_conv_steps.argtypes = [vp, i64, i32, i32, vp, vp, vp, vp, i32, i32, vp, i64, vp, i64, vp, vp, i32, vp, vp, vp]
    lib.pi_op_moe_route_groups.argtypes = [vp, vp, i64, i32, i32, i32, i32, i32, vp, vp, vp]
    lib.pi_op_moe_experts_act.argtypes = [vp, vp, i32, i32, i32, vp, i64, vp, vp, i32, i32, i32, vp, vp, i64, vp]
    lib.pi_op_moe_experts_grouped_act.argtypes = [vp, vp, i32, i32, i32, vp, i64, vp, vp, i32, i32, vp, vp, vp, vp, i64, vp]
    # blocks with the norm after the sum, recurrences with a decay per key channel, soft-max attention in chunks
    lib.pi_op_dense_segments.argtypes = [vp, vp, i64, i64, i64, i32, i32, vp, i64, i32, i64, i32, i32, vp]
    lib.pi_op_embed_pair.argtypes = [vp, vp, i32, f32, vp, vp, vp, vp]
    lib.pi_op_rms_post.argtypes = [vp, i64, vp, vp, i64, vp, f32, vp, vp, i64, f32, vp, f32, i32, i32, vp, i64, vp, vp, i64, vp]
    lib.pi_op_token_shift.argtypes = [vp, i64, i32, vp, i32, vp, vp, i32, vp, i64, vp]
    lib.pi_op_channel_recurrence.argtypes = [i32, vp, i64, vp, i64, vp, i64, vp, i64, i32, vp, vp, vp, i64, vp, i32, f32, i32, i32, i32, i32, vp, vp, i32, i32, vp, sz, vp, i64, vp]
    lib.pi_op_channel_recurrence_scratch_floats.argtypes = [i32, i32, i32, i32, i32]; lib.pi_op_channel_recurrence_scratch_floats.restype = sz
    lib.pi_op_head_norm_gate.argtypes = [vp, i64, i32, i32, vp, i32, vp, i64, i32, f32, i32, vp, i64, vp]
    lib.pi_op_qkv_prepare_ex.argtypes = [vp, vp, vp, i64, vp, vp, f32, i32, i32, i32, i32, vp, i32, i32, i32, vp, i32, vp, i64, vp, vp, vp, vp, vp]
    lib.pi_op_chunk_attention_ex.argtypes = [vp, i64, vp, vp, vp, vp, vp, vp, vp, i64, i32, f32, f32, i32, f32, i32, i32, i32, i32, i32, i32, i32, vp, i64, vp, vp]
    # layers with one tanh norm, sliding-window attention with pooled far blocks, clipped gated experts
    lib.pi_op_copy_rows.argtypes = [vp, i64, vp, i64, i32, i32, vp]
    lib.pi_op_sum_tanh_norm.argtypes = [vp, i64, vp, i64, vp, i64, vp, i64, i32, i32, vp, i64, vp, vp, vp, vp, i64, vp]
    lib.pi_op_sum_tanh_norm_shift.argtypes = [vp, i64, vp, i64, vp, i64, vp, i64, i32, i32, vp, i64, vp, vp, vp, vp, i64, vp, vp, vp, vp, i64, vp]
    lib.pi_rotary_table_create_scaled.restype = vp
    lib.pi_rotary_table_create_scaled.argtypes = [i32, i32, f32, f32, f32, f32, i32]
    lib.pi_op_pool_blocks.argtypes = [vp, vp, vp, vp, vp, i32, i64, i32, i32, i32, i32, i32, vp, vp]
    lib.pi_op_window_attention.argtypes = [vp, i64, vp, vp, vp, vp, vp, vp, vp, vp, i64, i32, f32, f32, i32, f32, i32, i32, i32, i64, i32, i32, i32, i32, i32, i32, i32, vp, sz, vp, i64, vp, vp]
    lib.pi_op_window_attention_scratch_floats.argtypes = [i32, i32, i32]; lib.pi_op_window_attention_scratch_floats.restype = sz
    lib.pi_op_moe_route_top_logits.argtypes = [vp, vp, vp, i64, i32, i32, i32, vp, vp, vp]
    lib.pi_op_moe_experts_glu.argtypes = [vp, vp, i32, i32, i32, f32, vp, i64, vp, vp, i32, i32, i32, vp, vp, i64, vp]
    lib.pi_op_moe_experts_grouped_glu.argtypes = [vp, vp, i32, i32, i32, f32, vp, i64, vp, vp, i32, i32, vp, vp, vp, vp, i64, vp]
    lib.pi_op_glu_mul_ex.argtypes = [vp, i64, i32, i32, f32, i64, i32, vp, i64, vp]
