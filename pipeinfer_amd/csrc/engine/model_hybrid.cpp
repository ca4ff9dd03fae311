// Hybrid models described by a folder: config.json (the layer list with every size and constant) + model.safetensors (bfloat16 tensors, linear weights [out][in]).
//
// config.json:  architecture, vocab, width, embedding.scale, norm.eps, residual_mult, layers[]: { type: "latent_attention" | "lightning", mixer: { heads, dim, vdim,
// kv_rank + scale | decay[] }, mlp: null | { kind: "moe", expert.ff, router.experts / identity / top }, weights_of: j (optional: the layer has no tensors, it uses layer j's) }.
// Tensors: embed, final.norm, l<i>.norm1 / norm2, l<i>.mix.{q, dkv, dkv.norm, uk, uv, sink, o} or l<i>.mix.{q, k, v, g, o, norm}, l<i>.mlp.{router, correction, e<k>.up, e<k>.down}.
// Projections that read the same input are uploaded as ONE matrix (rows one after the other) so that they are one launch; vectors go up as fp32.
//
// Vikarax (same files, other keys): vocab, width, norm.eps, logit_softcap, layers[]: { type: "parallel", mixer: { left: { heads, kv_heads, dim, vdim, scale, rot.dims / rot.base,
// mask.size }, right: { heads, vdim, state, groups, conv, norm_groups }, left_scale, right_scale }, mlp: null | { kind: "dense", ff } | { kind: "moe", expert.ff, router.experts /
// top / groups.count / groups.keep, shared.ff } }.  Tensors: embed, head, final.norm (+ .b), l<i>.norm1 / norm1b / norm2 / norm2b (+ .b), l<i>.dwa, l<i>.mix.left.{q, k, v, q.norm,
// k.norm, pb, g, o}, l<i>.mix.right.{in, conv, conv.b, dt_bias, A_log, D, norm, o}, l<i>.mlp.{up, down} or l<i>.mlp.{router, e<k>.{gate, up, down}, shared.{gate, up, down}}.
//
// Rafusun (same files, other keys): vocab, width, norm.eps, postln_alpha, embedding.scale, embedding.bigram.{buckets, mul_prev, mul_cur}, layers[]: { type: "channel_delta", mixer: { heads, kv_heads, dim, vdim, conv } }
// or { type: "parallel", mixer: { left: { heads, kv_heads, dim, vdim, scale, softcap, rot.dims / rot.base, mask.size }, right: { heads, dim } } }, mlp: null | { kind: "dense", ff }.  The ranks of the low-rank
// projections are the tensors' own.  Tensors: embed, bigram, head, final.norm, l<i>.norm1 / norm2, l<i>.ls1 / ls2, l<i>.mix.{q, k, v (+ .conv), b, A_log, dt_bias, a1, a2, g1, g2, norm, o} or
// l<i>.mix.left.{q, k, v, o, out}, l<i>.mix.right.{mu.{r, k, v, g, w}, r, k, v, g, w1, w2, w0, u, norm, o, out}, l<i>.mlp.{gate, up, down}.
//
// Rarevik (same files, other keys): vocab, width, norm.eps, loop.{start, stop, times} (optional: layers [start, stop) run `times` times in a row with the same tensors, each run with a cache and state of
// its own), layers[]: { type: "attention", mixer: { heads, kv_heads, dim, vdim, scale, conv, rot.dims / rot.base, mask.size / mask.pool } } or { type: "attention_2", mixer: { heads, kv_heads, dim, vdim,
// scale, rot.dims / rot.base / rot.scaling.{factor, low, high, original}, mask.size } }, mlp: null | { kind: "dense", ff } | { kind: "moe", expert.ff / expert.limit, router.experts / router.top,
// shared.ff / shared.limit }.  Tensors: embed, loop.in, final.norm (+ .b, .alpha), l<i>.norm1 (+ .b, .alpha), l<i>.shift, l<i>.mix.{q, k, v, o} with {q.conv, k.conv, v.conv, q.norm, k.norm, sink} or {g},
// l<i>.mlp.{up, down} or l<i>.mlp.{router, router.b, e<k>.{gate, up, down}, shared.{gate, up, down, sg}}.
#include "engine.h"
#include "json.h"

#include <cmath>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <sstream>
#include <sys/stat.h>

namespace {

bool num_at(const pi::json & j, const char * path, double & out) { const pi::json * v = j.at(path); if (!v || !v->is_num()) return false; out = v->num; return true; }
bool int_at(const pi::json & j, const char * path, int & out) { double d; if (!num_at(j, path, d) || d != std::floor(d) || d < 0 || d > 1e9) return false; out = (int) d; return true; }

float bf16_to_f32(uint16_t b) { const uint32_t u = (uint32_t) b << 16; float f; memcpy(&f, &u, 4); return f; }

struct loader {
    llama_model & m; std::string & err;
    const pi::st_tensor * get(const std::string & name, std::initializer_list<int64_t> shape) {
        const pi::st_tensor * t = m.st_file.tensor(name);
        if (!t) { err = "missing tensor " + name; return nullptr; }
        if (t->dtype != "BF16") { err = "tensor " + name + " is " + t->dtype + ", expected BF16"; return nullptr; }
        if (t->shape != std::vector<int64_t>(shape)) {
            std::string got, want;
            for (int64_t d : t->shape) got += (got.empty() ? "" : ",") + std::to_string(d);
            for (int64_t d : shape) want += (want.empty() ? "" : ",") + std::to_string(d);
            err = "tensor " + name + " has shape [" + got + "], expected [" + want + "]"; return nullptr;
        }
        return t;
    }
    // rows of several [rows_i][k] tensors one after the other as one bfloat16 matrix
    pi_weight * matrix(const std::vector<std::pair<std::string, int64_t>> & parts, int64_t k) {
        std::vector<uint16_t> host; int64_t rows = 0;
        const uint8_t * single = nullptr;
        for (const auto & p : parts) {
            const pi::st_tensor * t = get(p.first, { p.second, k });
            if (!t) return nullptr;
            if (parts.size() == 1) single = t->data;
            else { const size_t at = host.size(); host.resize(at + (size_t) p.second * k); memcpy(host.data() + at, t->data, t->nbytes); }
            rows += p.second;
        }
        pi_weight * w = pi_weight_upload(PI_BF16, k, rows, single ? (const void *) single : (const void *) host.data(), nullptr);
        if (!w) { err = "upload of " + parts[0].first + " failed: " + pi_last_error(); return nullptr; }
        m.hbm_bytes += pi_weight_nbytes(w);
        m.matrices.push_back({ w, nullptr, -1 });
        return w;
    }
    // columns of several [rows][k_i] tensors side by side as one bfloat16 matrix [rows][sum k_i] (projections whose outputs are summed: one product over the concatenated inputs)
    pi_weight * matrix_cols(const std::vector<std::pair<std::string, int64_t>> & parts, int64_t rows) {
        int64_t k = 0;
        for (const auto & p : parts) k += p.second;
        std::vector<uint16_t> host((size_t) (rows * k));
        int64_t at = 0;
        for (const auto & p : parts) {
            const pi::st_tensor * t = get(p.first, { rows, p.second });
            if (!t) return nullptr;
            for (int64_t r = 0; r < rows; r++) memcpy(host.data() + r * k + at, (const uint16_t *) t->data + r * p.second, (size_t) p.second * 2);
            at += p.second;
        }
        pi_weight * w = pi_weight_upload(PI_BF16, k, rows, host.data(), nullptr);
        if (!w) { err = "upload of " + parts[0].first + " failed: " + pi_last_error(); return nullptr; }
        m.hbm_bytes += pi_weight_nbytes(w);
        m.matrices.push_back({ w, nullptr, -1 });
        return w;
    }
    float * vector_f32(const std::vector<float> & v) {
        float * d = (float *) pi_malloc(std::max<size_t>(v.size(), 1) * 4);
        if (!d || (!v.empty() && (pi_memcpy_h2d(d, v.data(), v.size() * 4, nullptr) || pi_stream_sync(nullptr)))) { err = std::string("upload of a vector failed: ") + pi_last_error(); return nullptr; }
        m.f32_allocs.push_back(d); m.hbm_bytes += v.size() * 4;
        return d;
    }
    float * vector2(const std::string & name, int64_t rows, int64_t cols) {      // a small [rows][cols] table widened to fp32, as stored
        const pi::st_tensor * t = get(name, { rows, cols });
        if (!t) return nullptr;
        std::vector<float> v((size_t) (rows * cols));
        for (size_t i = 0; i < v.size(); i++) v[i] = bf16_to_f32(((const uint16_t *) t->data)[i]);
        return vector_f32(v);
    }
    // several vectors (or [rows][cols] tables of equal cols) one after the other, widened to fp32
    float * vectors(const std::vector<std::pair<std::string, int64_t>> & parts, int64_t cols) {
        std::vector<float> v;
        for (const auto & p : parts) {
            const pi::st_tensor * t = cols > 0 ? get(p.first, { p.second, cols }) : get(p.first, { p.second });
            if (!t) return nullptr;
            const size_t n = (size_t) (p.second * std::max<int64_t>(cols, 1)), at = v.size();
            v.resize(at + n);
            for (size_t i = 0; i < n; i++) v[at + i] = bf16_to_f32(((const uint16_t *) t->data)[i]);
        }
        return vector_f32(v);
    }
    float * scalar(const std::string & name) {                                  // a tensor without dimensions: one float on the device
        const pi::st_tensor * t = get(name, {});
        if (!t) return nullptr;
        return vector_f32({ bf16_to_f32(((const uint16_t *) t->data)[0]) });
    }
    float * vector(const std::string & name, int64_t n) {
        const pi::st_tensor * t = get(name, { n });
        if (!t) return nullptr;
        std::vector<float> v((size_t) n);
        for (int64_t i = 0; i < n; i++) v[(size_t) i] = bf16_to_f32(((const uint16_t *) t->data)[i]);
        return vector_f32(v);
    }
};


// Vikarax: every layer is a parallel mixer (attention branch + recurrence) with an optional dense or routed feed-forward
static bool read_vikarax_config(const pi::json & cfg, pi_hparams & hp, std::string & what) {
    using pi::json;
    double d;
    if (!num_at(cfg, "norm.eps", d)) { what = "no 'norm.eps'"; return false; }
    hp.f_norm_eps = hp.f_norm_rms_eps = (float) d;
    hp.logit_softcap = num_at(cfg, "logit_softcap", d) ? (float) d : 0.0f;
    hp.pre_post_norm = hp.depth_average = hp.own_head = true;
    const json * layers = cfg.find("layers");
    if (!layers || !layers->is_arr() || layers->arr.empty()) { what = "'layers' must be a non-empty list"; return false; }
    hp.n_layer = (int) layers->arr.size();
    hp.n_head = hp.n_head_kv = 1; hp.n_ctx_train = 0;
    int n_cache = 0, n_state = 0;
    for (int i = 0; i < hp.n_layer; i++) {
        const json & jl = layers->arr[(size_t) i];
        const std::string where = "layers[" + std::to_string(i) + "]: ";
        auto bad = [&](const std::string & w) { what = where + w; return false; };
        pi_hybrid_layer H;
        const json * type = jl.find("type");
        if (!type || !type->is_str() || type->str != "parallel") return bad("mixer type must be 'parallel'");
        H.mixer = PI_MIXER_PARALLEL; H.weights = i;
        pi_gate_attention & A = H.left; pi_ssd & R = H.right;
        if (!int_at(jl, "mixer.left.heads", A.heads) || !int_at(jl, "mixer.left.kv_heads", A.kv_heads) || !int_at(jl, "mixer.left.dim", A.dim) || !int_at(jl, "mixer.left.vdim", A.vdim) ||
            A.heads < 1 || A.kv_heads < 1 || A.heads % A.kv_heads || A.dim < 1 || A.vdim < 1) return bad("mixer.left needs positive 'heads', 'kv_heads' (a divisor of heads), 'dim', 'vdim'");
        if (!num_at(jl, "mixer.left.scale", d)) return bad("mixer.left needs 'scale'");
        A.scale = (float) d;
        if (jl.at("mixer.left.rot") && !jl.at("mixer.left.rot")->is_null()) {
            if (!int_at(jl, "mixer.left.rot.dims", A.rot_dims) || !num_at(jl, "mixer.left.rot.base", d) || (A.rot_dims & 1) || A.rot_dims > A.dim) return bad("mixer.left.rot needs an even 'dims' <= dim and 'base'");
            A.rot_base = (float) d;
        }
        if (jl.at("mixer.left.mask") && !jl.at("mixer.left.mask")->is_null() && (!int_at(jl, "mixer.left.mask.size", A.chunk) || A.chunk < 1)) return bad("mixer.left.mask needs a positive 'size'");
        if (!int_at(jl, "mixer.right.heads", R.heads) || !int_at(jl, "mixer.right.vdim", R.vdim) || !int_at(jl, "mixer.right.state", R.state) || !int_at(jl, "mixer.right.groups", R.groups) ||
            !int_at(jl, "mixer.right.conv", R.conv) || R.heads < 1 || R.vdim < 1 || R.state < 1 || R.groups < 1 || R.heads % R.groups || R.conv < 1 || R.conv > 64)
            return bad("mixer.right needs positive 'heads', 'vdim', 'state', 'groups' (a divisor of heads) and 'conv' (1..64)");
        if (R.state > 1024) return bad("mixer.right.state above 1024");
        R.norm_groups = 1;
        if (jl.at("mixer.right.norm_groups") && (!int_at(jl, "mixer.right.norm_groups", R.norm_groups) || R.norm_groups < 1 || R.inner() % R.norm_groups)) return bad("mixer.right.norm_groups must divide heads * vdim");
        if (!num_at(jl, "mixer.left_scale", d)) return bad("mixer needs 'left_scale'");
        H.left_scale = (float) d;
        if (!num_at(jl, "mixer.right_scale", d)) return bad("mixer needs 'right_scale'");
        H.right_scale = (float) d;
        H.heads = A.heads; H.dim = A.dim; H.vdim = A.vdim;
        H.cache_index = n_cache++; H.state_index = n_state++;
        if (jl.has("mlp")) {
            const json * kind = jl.at("mlp.kind");
            if (!kind || !kind->is_str()) return bad("mlp needs 'kind'");
            if (kind->str == "dense") {
                if (!int_at(jl, "mlp.ff", H.ff) || H.ff < 1) return bad("a dense mlp needs 'ff'");
                H.mlp = PI_MLP_DENSE_RELU_SQR;
            } else if (kind->str == "moe") {
                if (!int_at(jl, "mlp.router.experts", H.n_expert) || !int_at(jl, "mlp.router.top", H.top) || !int_at(jl, "mlp.expert.ff", H.ff) || H.n_expert < 1 || H.ff < 1 || H.top < 1) return bad("a routed mlp needs 'router.experts', 'router.top', 'expert.ff'");
                H.route_groups = H.route_keep = 1;
                if (jl.at("mlp.router.groups") && !jl.at("mlp.router.groups")->is_null() && (!int_at(jl, "mlp.router.groups.count", H.route_groups) || !int_at(jl, "mlp.router.groups.keep", H.route_keep))) return bad("mlp.router.groups needs 'count' and 'keep'");
                if (H.route_groups < 1 || H.n_expert % H.route_groups || H.route_keep < 1 || H.route_keep > H.route_groups || H.top > H.route_keep * (H.n_expert / H.route_groups)) return bad("the router's groups must divide the experts, and the kept groups must hold at least 'top' experts");
                if (jl.at("mlp.shared") && !jl.at("mlp.shared")->is_null() && (!int_at(jl, "mlp.shared.ff", H.shared_ff) || H.shared_ff < 1)) return bad("mlp.shared needs 'ff'");
                H.mlp = PI_MLP_MOE_GLU;
            } else return bad("feed-forward kind '" + kind->str + "' is unknown (dense, moe)");
            H.has_mlp = true;
        }
        hp.hybrid.push_back(std::move(H));
    }
    return true;
}

// Rafusun: layers of two kinds (a delta-rule mixer, or attention beside time mixing), an optional gated dense feed-forward, the norm after the sum
static bool read_rafusun_config(const pi::json & cfg, const pi::safetensors_file * st, pi_hparams & hp, std::string & what) {
    using pi::json;
    double d;
    if (!num_at(cfg, "norm.eps", d)) { what = "no 'norm.eps'"; return false; }
    hp.f_norm_eps = hp.f_norm_rms_eps = (float) d;
    if (!num_at(cfg, "postln_alpha", d)) { what = "no 'postln_alpha'"; return false; }
    hp.post_alpha = (float) d; hp.post_norm = hp.own_head = true;
    hp.embed_scale = num_at(cfg, "embedding.scale", d) ? (float) d : 1.0f;
    if (cfg.at("embedding.bigram") && !cfg.at("embedding.bigram")->is_null()) {
        if (!int_at(cfg, "embedding.bigram.buckets", hp.pair_buckets) || !int_at(cfg, "embedding.bigram.mul_prev", hp.pair_mul_prev) || !int_at(cfg, "embedding.bigram.mul_cur", hp.pair_mul_cur) || hp.pair_buckets < 1) { what = "embedding.bigram needs a positive 'buckets', 'mul_prev' and 'mul_cur'"; return false; }
    }
    const json * layers = cfg.find("layers");
    if (!layers || !layers->is_arr() || layers->arr.empty()) { what = "'layers' must be a non-empty list"; return false; }
    hp.n_layer = (int) layers->arr.size();
    hp.n_head = hp.n_head_kv = 1; hp.n_ctx_train = 0;
    int n_cache = 0, n_state = 0;
    // the rank of a low-rank projection is the first size of its first matrix [rank][width]
    auto rank_of = [&](const std::string & name, int & out) { out = 0; if (!st) return true; const pi::st_tensor * t = st->tensor(name); if (!t || t->shape.size() != 2 || t->shape[0] < 1 || t->shape[1] != hp.n_embd) return false; out = (int) t->shape[0]; return true; };
    for (int i = 0; i < hp.n_layer; i++) {
        const json & jl = layers->arr[(size_t) i];
        const std::string where = "layers[" + std::to_string(i) + "]: ", p = "l" + std::to_string(i) + ".mix.";
        auto bad = [&](const std::string & w) { what = where + w; return false; };
        pi_hybrid_layer H;
        H.weights = i;
        const json * type = jl.find("type");
        if (!type || !type->is_str()) return bad("no 'type'");
        if (type->str == "channel_delta") {
            H.mixer = PI_MIXER_CHANNEL_DELTA;
            pi_channel_delta & D = H.delta;
            if (!int_at(jl, "mixer.heads", D.heads) || !int_at(jl, "mixer.kv_heads", D.kv_heads) || !int_at(jl, "mixer.dim", D.dim) || !int_at(jl, "mixer.vdim", D.vdim) || !int_at(jl, "mixer.conv", D.conv) ||
                D.heads < 1 || D.kv_heads < 1 || D.heads % D.kv_heads || D.dim < 1 || D.vdim < 1 || D.conv < 1 || D.conv > 64) return bad("channel_delta needs positive 'heads', 'kv_heads' (a divisor of heads), 'dim', 'vdim' and 'conv' (1..64)");
            if (D.dim > 1024) return bad("channel_delta key width above 1024");
            if (!rank_of(p + "a1", D.decay_rank) || !rank_of(p + "g1", D.gate_rank)) return bad("tensors mix.a1 / mix.g1 [rank][width] are missing");
            H.heads = D.heads; H.dim = D.dim; H.vdim = D.vdim;
            H.state_index = n_state++;
        } else if (type->str == "parallel") {
            H.mixer = PI_MIXER_PARALLEL_SHIFT;
            pi_gate_attention & A = H.left; pi_time_mix & R = H.shift;
            if (!int_at(jl, "mixer.left.heads", A.heads) || !int_at(jl, "mixer.left.kv_heads", A.kv_heads) || !int_at(jl, "mixer.left.dim", A.dim) || !int_at(jl, "mixer.left.vdim", A.vdim) ||
                A.heads < 1 || A.kv_heads < 1 || A.heads % A.kv_heads || A.dim < 1 || A.vdim < 1) return bad("mixer.left needs positive 'heads', 'kv_heads' (a divisor of heads), 'dim', 'vdim'");
            if (!num_at(jl, "mixer.left.scale", d)) return bad("mixer.left needs 'scale'");
            A.scale = (float) d; A.gated = false; A.weights = PI_WEIGHTS_SOFTMAX_SINK;
            if (jl.at("mixer.left.softcap") && !jl.at("mixer.left.softcap")->is_null()) { if (!num_at(jl, "mixer.left.softcap", d) || d <= 0) return bad("mixer.left.softcap must be positive"); A.softcap = (float) d; }
            if (jl.at("mixer.left.rot") && !jl.at("mixer.left.rot")->is_null()) {
                if (!int_at(jl, "mixer.left.rot.dims", A.rot_dims) || !num_at(jl, "mixer.left.rot.base", d) || (A.rot_dims & 1) || A.rot_dims > A.dim) return bad("mixer.left.rot needs an even 'dims' <= dim and 'base'");
                A.rot_base = (float) d;
            }
            if (jl.at("mixer.left.mask") && !jl.at("mixer.left.mask")->is_null() && (!int_at(jl, "mixer.left.mask.size", A.chunk) || A.chunk < 1)) return bad("mixer.left.mask needs a positive 'size'");
            if (!int_at(jl, "mixer.right.heads", R.heads) || !int_at(jl, "mixer.right.dim", R.dim) || R.heads < 1 || R.dim < 1 || R.dim > 1024) return bad("mixer.right needs positive 'heads' and 'dim' (at most 1024)");
            if (!rank_of(p + "right.w1", R.decay_rank)) return bad("tensor mix.right.w1 [rank][width] is missing");
            R.width = hp.n_embd;
            H.heads = A.heads; H.dim = A.dim; H.vdim = A.vdim;
            H.cache_index = n_cache++; H.state_index = n_state++;
        } else return bad("mixer type '" + type->str + "' is unknown (channel_delta, parallel)");
        if (jl.has("mlp")) {
            const json * kind = jl.at("mlp.kind");
            if (!kind || !kind->is_str() || kind->str != "dense") return bad("feed-forward kind must be 'dense'");
            if (!int_at(jl, "mlp.ff", H.ff) || H.ff < 1) return bad("a dense mlp needs 'ff'");
            H.mlp = PI_MLP_DENSE_GEGLU; H.has_mlp = true;
        }
        hp.hybrid.push_back(std::move(H));
    }
    return true;
}

// Rarevik: every layer has ONE tanh norm that its mixer (through a token shift) and its feed-forward read; the mixers are sliding-window attentions of two kinds; a run of layers may repeat
static bool read_rarevik_config(const pi::json & cfg, pi_hparams & hp, std::string & what) {
    using pi::json;
    double d;
    if (!num_at(cfg, "norm.eps", d)) { what = "no 'norm.eps'"; return false; }
    hp.f_norm_eps = hp.f_norm_rms_eps = (float) d;
    hp.shared_tanh_norm = true;
    const json * layers = cfg.find("layers");
    if (!layers || !layers->is_arr() || layers->arr.empty()) { what = "'layers' must be a non-empty list"; return false; }
    const int n_desc = (int) layers->arr.size();
    std::vector<pi_hybrid_layer> desc;
    for (int i = 0; i < n_desc; i++) {
        const json & jl = layers->arr[(size_t) i];
        const std::string where = "layers[" + std::to_string(i) + "]: ";
        auto bad = [&](const std::string & w) { what = where + w; return false; };
        pi_hybrid_layer H;
        H.mixer = PI_MIXER_WINDOW_ATTENTION; H.name_index = i;
        pi_gate_attention & A = H.left;
        const json * type = jl.find("type");
        if (!type || !type->is_str()) return bad("no 'type'");
        const bool pooled_kind = type->str == "attention";
        if (!pooled_kind && type->str != "attention_2") return bad("mixer type '" + type->str + "' is unknown (attention, attention_2)");
        if (!int_at(jl, "mixer.heads", A.heads) || !int_at(jl, "mixer.kv_heads", A.kv_heads) || !int_at(jl, "mixer.dim", A.dim) || !int_at(jl, "mixer.vdim", A.vdim) ||
            A.heads < 1 || A.kv_heads < 1 || A.heads % A.kv_heads || A.dim < 1 || A.vdim < 1) return bad("mixer needs positive 'heads', 'kv_heads' (a divisor of heads), 'dim', 'vdim'");
        if (!num_at(jl, "mixer.scale", d)) return bad("mixer needs 'scale'");
        A.scale = (float) d; A.weights = PI_WEIGHTS_SOFTMAX; A.v_norm = false; A.mask_kind = PI_MASK_WINDOW;
        if (jl.at("mixer.rot") && !jl.at("mixer.rot")->is_null()) {
            if (!int_at(jl, "mixer.rot.dims", A.rot_dims) || !num_at(jl, "mixer.rot.base", d) || (A.rot_dims & 1) || A.rot_dims > A.dim || d <= 0) return bad("mixer.rot needs an even 'dims' <= dim and a positive 'base'");
            A.rot_base = (float) d;
        }
        if (jl.at("mixer.mask") && !jl.at("mixer.mask")->is_null() && (!int_at(jl, "mixer.mask.size", A.chunk) || A.chunk < 1)) return bad("mixer.mask needs a positive 'size'");
        if (pooled_kind) {                                                  // a short convolution behind the projections, normed q / k turned in halves, pooled far blocks, a learned sink
            A.gated = false; A.qk_norm = PI_QK_NORM_FIRST; A.pairing = PI_PAIR_HALVES;
            if (jl.at("mixer.conv") && !jl.at("mixer.conv")->is_null() && (!int_at(jl, "mixer.conv", A.conv) || A.conv < 1 || A.conv > 64)) return bad("mixer.conv must lie between 1 and 64");
            if (A.chunk > 0 && jl.at("mixer.mask.pool") && !jl.at("mixer.mask.pool")->is_null() && (!int_at(jl, "mixer.mask.pool", A.pool) || A.pool < 1 || A.pool > 8192)) return bad("mixer.mask.pool must lie between 1 and 8192");
        } else {                                                            // q / k turned in neighbouring pairs by (possibly stretched) angle steps, no norms, a sigmoid gate per head
            A.gated = true; A.qk_norm = PI_QK_NORM_NONE; A.pairing = PI_PAIR_NEIGHBOURS;
            if (A.rot_dims > 0 && jl.at("mixer.rot.scaling") && !jl.at("mixer.rot.scaling")->is_null()) {
                double f, lo, hi;
                if (!num_at(jl, "mixer.rot.scaling.factor", f) || !num_at(jl, "mixer.rot.scaling.low", lo) || !num_at(jl, "mixer.rot.scaling.high", hi) || !int_at(jl, "mixer.rot.scaling.original", A.rot_original) ||
                    f <= 0 || lo <= 0 || hi <= 0 || A.rot_original < 1) return bad("mixer.rot.scaling needs positive 'factor', 'low', 'high' and 'original'");
                A.rot_factor = (float) f; A.rot_low = (float) lo; A.rot_high = (float) hi;
            }
        }
        H.heads = A.heads; H.dim = A.dim; H.vdim = A.vdim; H.shift.width = hp.n_embd;
        if (jl.has("mlp")) {
            const json * kind = jl.at("mlp.kind");
            if (!kind || !kind->is_str()) return bad("mlp needs 'kind'");
            if (kind->str == "dense") {
                if (!int_at(jl, "mlp.ff", H.ff) || H.ff < 1) return bad("a dense mlp needs 'ff'");
                H.mlp = PI_MLP_DENSE_GELU;
            } else if (kind->str == "moe") {
                if (!int_at(jl, "mlp.router.experts", H.n_expert) || !int_at(jl, "mlp.router.top", H.top) || !int_at(jl, "mlp.expert.ff", H.ff) || H.n_expert < 1 || H.ff < 1 || H.top < 1 || H.top > H.n_expert)
                    return bad("a routed mlp needs 'router.experts', 'router.top' (at most the experts), 'expert.ff'");
                if (num_at(jl, "mlp.expert.limit", d)) { if (d <= 0) return bad("mlp.expert.limit must be positive"); H.glu_limit = (float) d; }
                if (jl.at("mlp.shared") && !jl.at("mlp.shared")->is_null()) {
                    if (!int_at(jl, "mlp.shared.ff", H.shared_ff) || H.shared_ff < 1) return bad("mlp.shared needs 'ff'");
                    if (num_at(jl, "mlp.shared.limit", d)) { if (d <= 0) return bad("mlp.shared.limit must be positive"); H.shared_limit = (float) d; }
                }
                H.mlp = PI_MLP_MOE_CLIPPED;
            } else return bad("feed-forward kind '" + kind->str + "' is unknown (dense, moe)");
            H.has_mlp = true;
        }
        desc.push_back(std::move(H));
    }
    // the order the layers run in: [0, start) once, [start, stop) `times` times, [stop, n) once.  Every entry of the run list is a layer of its own to the context (cache, state); its tensors are those of
    // the first run of the same description
    int start = n_desc, stop = n_desc, times = 1;
    if (cfg.at("loop") && !cfg.at("loop")->is_null()) {
        if (!int_at(cfg, "loop.start", start) || !int_at(cfg, "loop.stop", stop) || !int_at(cfg, "loop.times", times) || start > stop || stop > n_desc || times > 4096) { what = "'loop' needs 0 <= start <= stop <= layers and 'times'"; return false; }
    }
    std::vector<int> first_run((size_t) n_desc, -1);
    auto add = [&](int i, bool entry) {
        pi_hybrid_layer H = desc[(size_t) i];
        const int r = (int) hp.hybrid.size();
        if (first_run[(size_t) i] < 0) first_run[(size_t) i] = r;
        H.weights = first_run[(size_t) i]; H.loop_entry = entry; H.cache_index = r; H.state_index = r;
        hp.hybrid.push_back(std::move(H));
    };
    for (int i = 0; i < start; i++) add(i, false);
    for (int k = 0; k < times; k++) for (int i = start; i < stop; i++) add(i, i == start);
    for (int i = stop; i < n_desc; i++) add(i, false);
    if (hp.hybrid.empty()) { what = "no layer runs"; return false; }
    hp.n_layer = (int) hp.hybrid.size();
    hp.n_head = hp.n_head_kv = 1; hp.n_ctx_train = 0;
    return true;
}

}  // namespace

bool llama_model::ensure_loaded_hybrid(int n_positions, std::string & err) {
    const pi_hparams & hp = hparams;
    loader L{ *this, err };
    pi_weight_set_mq_copies(0);
    struct restore { ~restore() { pi_weight_set_mq_copies(1); } } r;
    const int64_t width = hp.n_embd;
    if (!tok_embd) {
        if (!(tok_embd = L.matrix({ { "embed", hp.n_vocab } }, width))) return false;
        if (!(output_norm = L.vector("final.norm", width))) return false;
    }
    if (hp.own_head && !output) {
        if (!(output = L.matrix({ { "head", hp.n_vocab } }, width))) return false;
        if (!hp.post_norm && !(output_norm_b = L.vector("final.norm.b", width))) return false;
    }
    if (hp.shared_tanh_norm && !output_norm_alpha && (!(output_norm_b = L.vector("final.norm.b", width)) || !(output_norm_alpha = L.scalar("final.norm.alpha")))) return false;
    if (hp.pair_buckets > 0 && !pair_embd && !(pair_embd = L.matrix({ { "bigram", (int64_t) hp.pair_buckets + 1 } }, width))) return false;
    for (size_t i = 0; i < hp.hybrid.size(); i++) {
        const pi_hybrid_layer & H = hp.hybrid[i];
        pi_hybrid_weights & W = hweights[i];
        if (H.weights == (int) i && W.loaded && W.rotary && pi_rotary_table_positions(W.rotary) < n_positions) {        // a later context is longer than the table
            void * t = pi_rotary_table_create_scaled(n_positions, H.left.rot_dims, H.left.rot_base, H.left.rot_factor, H.left.rot_low, H.left.rot_high, H.left.rot_original);
            if (!t) { err = std::string("rotation table: ") + pi_last_error(); return false; }
            retired_tables.push_back(W.rotary); W.rotary = t;
        }
        if (H.weights != (int) i || W.loaded) continue;
        const std::string p = "l" + std::to_string(H.name_index >= 0 ? H.name_index : (int) i) + ".";
        if (hp.shared_tanh_norm) {                                         // one tanh norm per layer; window attention; dense or routed clipped feed-forward
            if (H.mixer != PI_MIXER_WINDOW_ATTENTION) { err = "a block with one shared tanh norm has no mixer of kind " + std::to_string((int) H.mixer); return false; }
            const pi_gate_attention & A = H.left;
            const std::string m = p + "mix.";
            const int64_t hd = (int64_t) A.heads * A.dim, gd = (int64_t) A.kv_heads * A.dim, gv = (int64_t) A.kv_heads * A.vdim;
            if (!(W.norm1 = L.vector(p + "norm1", width)) || !(W.norm1_b = L.vector(p + "norm1.b", width)) || !(W.norm1_alpha = L.scalar(p + "norm1.alpha")) || !(W.mu = L.vector(p + "shift", width))) return false;
            std::vector<std::pair<std::string, int64_t>> in_parts = { { m + "q", hd }, { m + "k", gd }, { m + "v", gv } };
            if (A.gated) in_parts.push_back({ m + "g", A.heads });
            if (!(W.w_in = L.matrix(in_parts, width)) || !(W.w_o = L.matrix({ { m + "o", width } }, (int64_t) A.heads * A.vdim))) return false;
            if (A.conv > 0 && !(W.conv_w = L.vectors({ { m + "q.conv", hd }, { m + "k.conv", gd }, { m + "v.conv", gv } }, A.conv))) return false;
            if (A.qk_norm != PI_QK_NORM_NONE && (!(W.q_norm = L.vector(m + "q.norm", A.dim)) || !(W.k_norm = L.vector(m + "k.norm", A.dim)))) return false;
            if (!A.gated && !(W.sink = L.vector(m + "sink", A.heads))) return false;
            if (!(W.rotary = pi_rotary_table_create_scaled(std::max(n_positions, 32), A.rot_dims, A.rot_base, A.rot_factor, A.rot_low, A.rot_high, A.rot_original))) { err = std::string("rotation table: ") + pi_last_error(); return false; }
            if (H.mlp == PI_MLP_DENSE_GELU) {
                if (!(W.ff_up = L.matrix({ { p + "mlp.up", H.ff } }, width)) || !(W.ff_down = L.matrix({ { p + "mlp.down", width } }, H.ff))) return false;
            } else if (H.mlp == PI_MLP_MOE_CLIPPED) {
                if (!(W.router = L.matrix({ { p + "mlp.router", H.n_expert } }, width)) || !(W.correction = L.vector(p + "mlp.router.b", H.n_expert))) return false;
                std::vector<std::pair<std::string, int64_t>> ups, downs;
                for (int e = 0; e < H.n_expert; e++) {
                    const std::string q = p + "mlp.e" + std::to_string(e) + ".";
                    ups.push_back({ q + "gate", H.ff }); ups.push_back({ q + "up", H.ff }); downs.push_back({ q + "down", width });
                }
                if (!(W.e_up = L.matrix(ups, width)) || !(W.e_down = L.matrix(downs, H.ff))) return false;
                // the shared expert's per-token gate is one more row of its first matrix: [gate | up | sg]
                if (H.shared_ff > 0 && (!(W.ff_up = L.matrix({ { p + "mlp.shared.gate", H.shared_ff }, { p + "mlp.shared.up", H.shared_ff }, { p + "mlp.shared.sg", 1 } }, width)) ||
                                        !(W.ff_down = L.matrix({ { p + "mlp.shared.down", width } }, H.shared_ff)))) return false;
            }
            if (H.loop_entry && !(W.w_loop = L.matrix({ { "loop.in", width } }, 2 * width))) return false;
            W.loaded = true;
            continue;
        }
        if (hp.post_norm) {                                                // the norm after the sum: per sublayer a norm and a layer scale
            if (!(W.norm1 = L.vector(p + "norm1", width)) || !(W.ls1 = L.vector(p + "ls1", width))) return false;
            if (H.has_mlp && (!(W.norm2 = L.vector(p + "norm2", width)) || !(W.ls2 = L.vector(p + "ls2", width)))) return false;
            if (H.mixer == PI_MIXER_CHANNEL_DELTA) {
                const pi_channel_delta & D = H.delta;
                const std::string m = p + "mix.";
                const int64_t gd = (int64_t) D.kv_heads * D.dim, hd = (int64_t) D.heads * D.dim, hv = (int64_t) D.heads * D.vdim;
                if (!(W.w_in = L.matrix({ { m + "q", gd }, { m + "k", gd }, { m + "v", hv }, { m + "a1", D.decay_rank }, { m + "g1", D.gate_rank }, { m + "b", D.heads } }, width))) return false;
                // the second halves of the two low-rank projections: one matrix [a2 | g2] in two segments where their ranks are equal (one launch), two matrices otherwise
                if (D.decay_rank == D.gate_rank) { if (!(W.w_a2 = L.matrix({ { m + "a2", hd }, { m + "g2", hv } }, D.decay_rank))) return false; }
                else if (!(W.w_a2 = L.matrix({ { m + "a2", hd } }, D.decay_rank)) || !(W.w_g2 = L.matrix({ { m + "g2", hv } }, D.gate_rank))) return false;
                if (!(W.w_o = L.matrix({ { m + "o", width } }, hv))) return false;
                if (!(W.conv_w = L.vectors({ { m + "q.conv", gd }, { m + "k.conv", gd }, { m + "v.conv", hv } }, D.conv))) return false;
                if (!(W.a_log = L.vector(m + "A_log", D.heads)) || !(W.dt_bias = L.vector(m + "dt_bias", hd)) || !(W.mix_norm = L.vector(m + "norm", D.vdim))) return false;
            } else if (H.mixer == PI_MIXER_PARALLEL_SHIFT) {
                const pi_gate_attention & A = H.left; const pi_time_mix & R = H.shift;
                const std::string l = p + "mix.left.", r = p + "mix.right.";
                if (!(W.w_in = L.matrix({ { l + "q", (int64_t) A.heads * A.dim }, { l + "k", (int64_t) A.kv_heads * A.dim }, { l + "v", (int64_t) A.kv_heads * A.vdim } }, width))) return false;
                if (!(W.w_o = L.matrix({ { l + "o", width } }, (int64_t) A.heads * A.vdim)) || !(W.left_out = L.vector(l + "out", width))) return false;
                if (!(W.rotary = pi_rotary_table_create(std::max(n_positions, 32), A.rot_dims, A.rot_base))) { err = std::string("rotation table: ") + pi_last_error(); return false; }
                const int64_t inner = R.inner();
                if (!(W.mu = L.vectors({ { r + "mu.r", width }, { r + "mu.k", width }, { r + "mu.v", width }, { r + "mu.g", width }, { r + "mu.w", width } }, 0))) return false;
                if (!(W.w_r = L.matrix({ { r + "r", inner }, { r + "k", inner }, { r + "v", inner }, { r + "g", inner }, { r + "w1", R.decay_rank } }, width))) return false;      // one matrix, five inputs (pi_op_dense_segments)
                if (!(W.w_w2 = L.matrix({ { r + "w2", inner } }, R.decay_rank)) || !(W.w_o2 = L.matrix({ { r + "o", width } }, inner))) return false;
                if (!(W.w0 = L.vector(r + "w0", inner)) || !(W.bonus = L.vector2(r + "u", R.heads, R.dim)) || !(W.mix_norm = L.vector(r + "norm", inner)) || !(W.right_out = L.vector(r + "out", width))) return false;
            } else { err = "a block with the norm after the sum has no mixer of kind " + std::to_string((int) H.mixer); return false; }
            if (H.mlp == PI_MLP_DENSE_GEGLU && (!(W.ff_up = L.matrix({ { p + "mlp.gate", H.ff }, { p + "mlp.up", H.ff } }, width)) || !(W.ff_down = L.matrix({ { p + "mlp.down", width } }, H.ff)))) return false;
            W.loaded = true;
            continue;
        }
        if (H.mixer == PI_MIXER_PARALLEL) {
            const pi_gate_attention & A = H.left; const pi_ssd & R = H.right;
            const std::string l = p + "mix.left.", r = p + "mix.right.";
            struct { float ** w, ** b; const char * name; bool need; } norms[] = { { &W.norm1, &W.norm1_b, "norm1", true }, { &W.post1, &W.post1_b, "norm1b", true },
                                                                                   { &W.norm2, &W.norm2_b, "norm2", H.has_mlp }, { &W.post2, &W.post2_b, "norm2b", H.has_mlp } };
            for (auto & n : norms) if (n.need && (!(*n.w = L.vector(p + n.name, width)) || !(*n.b = L.vector(p + n.name + ".b", width)))) return false;
            if (hp.depth_average && !(W.depth = L.vector(p + "dwa", (int64_t) i + 2))) return false;
            if (!(W.w_in = L.matrix({ { l + "q", (int64_t) A.heads * A.dim }, { l + "k", (int64_t) A.kv_heads * A.dim }, { l + "v", (int64_t) A.kv_heads * A.vdim }, { l + "g", A.heads }, { r + "in", R.in_rows() } }, width))) return false;
            if (!(W.q_norm = L.vector(l + "q.norm", A.dim)) || !(W.k_norm = L.vector(l + "k.norm", A.dim)) || !(W.head_bias = L.vector(l + "pb", A.heads))) return false;
            if (!(W.w_o = L.matrix_cols({ { l + "o", (int64_t) A.heads * A.vdim }, { r + "o", R.inner() } }, width))) return false;      // [W_o | W_o']: both branches' outputs enter one product
            if (!(W.conv_w = L.vector2(r + "conv", R.channels(), R.conv)) || !(W.conv_b = L.vector(r + "conv.b", R.channels()))) return false;
            if (!(W.dt_bias = L.vector(r + "dt_bias", R.heads)) || !(W.a_log = L.vector(r + "A_log", R.heads)) || !(W.skip = L.vector(r + "D", R.heads)) || !(W.mix_norm = L.vector(r + "norm", R.inner()))) return false;
            if (!(W.rotary = pi_rotary_table_create(std::max(n_positions, 32), A.rot_dims, A.rot_base))) { err = std::string("rotation table: ") + pi_last_error(); return false; }
            if (H.mlp == PI_MLP_DENSE_RELU_SQR) {
                if (!(W.ff_up = L.matrix({ { p + "mlp.up", H.ff } }, width)) || !(W.ff_down = L.matrix({ { p + "mlp.down", width } }, H.ff))) return false;
            } else if (H.mlp == PI_MLP_MOE_GLU) {
                if (!(W.router = L.matrix({ { p + "mlp.router", H.n_expert } }, width))) return false;
                std::vector<std::pair<std::string, int64_t>> ups, downs;
                for (int e = 0; e < H.n_expert; e++) {
                    const std::string q = p + "mlp.e" + std::to_string(e) + ".";
                    ups.push_back({ q + "gate", H.ff }); ups.push_back({ q + "up", H.ff }); downs.push_back({ q + "down", width });
                }
                if (!(W.e_up = L.matrix(ups, width)) || !(W.e_down = L.matrix(downs, H.ff))) return false;
                if (H.shared_ff > 0 && (!(W.ff_up = L.matrix({ { p + "mlp.shared.gate", H.shared_ff }, { p + "mlp.shared.up", H.shared_ff } }, width)) || !(W.ff_down = L.matrix({ { p + "mlp.shared.down", width } }, H.shared_ff)))) return false;
            }
            W.loaded = true;
            continue;
        }
        const int64_t hd = (int64_t) H.heads * H.dim, hv = (int64_t) H.heads * H.vdim;
        if (!(W.norm1 = L.vector(p + "norm1", width))) return false;
        if (H.mixer == PI_MIXER_LIGHTNING) {
            if (!(W.w_in = L.matrix({ { p + "mix.q", hd }, { p + "mix.k", hd }, { p + "mix.v", hv }, { p + "mix.g", hv } }, width))) return false;
            if (!(W.mix_norm = L.vector(p + "mix.norm", hv))) return false;
            if (!(W.decay = L.vector_f32(H.decay))) return false;
        } else {
            if (!(W.w_in = L.matrix({ { p + "mix.q", hd }, { p + "mix.dkv", H.kv_rank } }, width))) return false;
            if (!(W.mix_norm = L.vector(p + "mix.dkv.norm", H.kv_rank))) return false;
            if (!(W.w_uk = L.matrix({ { p + "mix.uk", hd } }, H.kv_rank)) || !(W.w_uv = L.matrix({ { p + "mix.uv", hv } }, H.kv_rank))) return false;
            if (!(W.sink = L.vector(p + "mix.sink", H.heads))) return false;
        }
        if (!(W.w_o = L.matrix({ { p + "mix.o", width } }, hv))) return false;
        if (H.has_mlp) {
            if (!(W.norm2 = L.vector(p + "norm2", width))) return false;
            const int n_out = H.n_expert + H.n_identity;
            if (!(W.router = L.matrix({ { p + "mlp.router", n_out } }, width)) || !(W.correction = L.vector(p + "mlp.correction", n_out))) return false;
            if (H.n_expert > 0) {
                std::vector<std::pair<std::string, int64_t>> ups, downs;
                for (int e = 0; e < H.n_expert; e++) { ups.push_back({ p + "mlp.e" + std::to_string(e) + ".up", H.ff }); downs.push_back({ p + "mlp.e" + std::to_string(e) + ".down", width }); }
                if (!(W.e_up = L.matrix(ups, width)) || !(W.e_down = L.matrix(downs, H.ff))) return false;
            }
        }
        W.loaded = true;
    }
    return true;
}

namespace pi {

// path: the folder, or its config.json / model.safetensors
bool is_hybrid_model_path(const std::string & path, std::string & folder) {
    struct stat st;
    if (stat(path.c_str(), &st) != 0) return false;
    if (S_ISDIR(st.st_mode)) { folder = path; return stat((path + "/config.json").c_str(), &st) == 0; }
    const size_t slash = path.find_last_of('/');
    const std::string base = slash == std::string::npos ? path : path.substr(slash + 1);
    if (base != "config.json" && base != "model.safetensors") return false;
    folder = slash == std::string::npos ? "." : path.substr(0, slash);
    return true;
}

llama_model * load_hybrid_model(const std::string & folder, const llama_model_params & params) {
    std::unique_ptr<llama_model> m(new llama_model());
    m->path = folder; m->device = params.main_gpu;
    auto fail = [&](const std::string & what) { fprintf(stderr, "llama_load_model_from_file: %s/config.json: %s\n", folder.c_str(), what.c_str()); return (llama_model *) nullptr; };
    std::ifstream in(folder + "/config.json");
    if (!in) return fail("cannot be read");
    std::stringstream ss; ss << in.rdbuf();
    json cfg; std::string err;
    if (!json::parse(ss.str(), cfg, err) || !cfg.is_obj()) return fail(err.empty() ? "not a JSON object" : err);
    const json * arch = cfg.find("architecture");
    if (!arch || !arch->is_str()) return fail("no 'architecture'");
    pi_hparams & hp = m->hparams;
    // the registry of folder-described architectures (GGUF files name theirs in general.architecture, model.cpp)
    if (arch->str == "Fasovik") hp.arch = PI_ARCH_FASOVIK;
    else if (arch->str == "Vikarax") hp.arch = PI_ARCH_VIKARAX;
    else if (arch->str == "Rafusun") hp.arch = PI_ARCH_RAFUSUN;
    else if (arch->str == "Rarevik") hp.arch = PI_ARCH_RAREVIK;
    else return fail("architecture '" + arch->str + "' is not one this engine builds (Fasovik, Vikarax, Rafusun, Rarevik)");
    m->name = arch->str;
    double d;
    if (!int_at(cfg, "vocab", hp.n_vocab) || !int_at(cfg, "width", hp.n_embd) || hp.n_vocab < 1 || hp.n_embd < 1) return fail("'vocab' and 'width' must be positive integers");
    if (hp.arch == PI_ARCH_VIKARAX || hp.arch == PI_ARCH_RAFUSUN || hp.arch == PI_ARCH_RAREVIK) {
        std::string what;
        if (!params.vocab_only && !m->st_file.open(folder + "/model.safetensors", err)) { fprintf(stderr, "llama_load_model_from_file: %s\n", err.c_str()); return nullptr; }
        if (hp.arch == PI_ARCH_VIKARAX ? !read_vikarax_config(cfg, hp, what) : hp.arch == PI_ARCH_RAREVIK ? !read_rarevik_config(cfg, hp, what) : !read_rafusun_config(cfg, params.vocab_only ? nullptr : &m->st_file, hp, what)) return fail(what);
        m->hweights.resize((size_t) hp.n_layer);
        if (!params.vocab_only) {
            for (const auto & kv : m->st_file.tensors) { m->n_elements += (uint64_t) kv.second.elements(); m->n_bytes += kv.second.nbytes; }
            const st_tensor * e = m->st_file.tensor("embed"), * h = m->st_file.tensor("head");
            if (!e || e->shape != std::vector<int64_t>{ hp.n_vocab, hp.n_embd } || (hp.arch != PI_ARCH_RAREVIK && (!h || h->shape != e->shape))) return fail("tensors 'embed' and 'head' are missing or not [vocab][width]");
        }
        return m.release();
    }
    if (!num_at(cfg, "embedding.scale", d)) return fail("no 'embedding.scale'");
    hp.embed_scale = (float) d;
    if (!num_at(cfg, "norm.eps", d)) return fail("no 'norm.eps'");
    hp.f_norm_rms_eps = (float) d;
    if (!num_at(cfg, "residual_mult", d)) return fail("no 'residual_mult'");
    hp.residual_mult = (float) d;
    const json * layers = cfg.find("layers");
    if (!layers || !layers->is_arr() || layers->arr.empty()) return fail("'layers' must be a non-empty list");
    hp.n_layer = (int) layers->arr.size();
    hp.n_head = hp.n_head_kv = 1; hp.n_ctx_train = 0;
    int n_cache = 0, n_state = 0;
    for (int i = 0; i < hp.n_layer; i++) {
        const json & jl = layers->arr[(size_t) i];
        const std::string where = "layers[" + std::to_string(i) + "]: ";
        pi_hybrid_layer H;
        const json * type = jl.find("type");
        if (!type || !type->is_str()) return fail(where + "no 'type'");
        if (type->str == "latent_attention") H.mixer = PI_MIXER_LATENT_ATTENTION;
        else if (type->str == "lightning") H.mixer = PI_MIXER_LIGHTNING;
        else return fail(where + "mixer type '" + type->str + "' is unknown (latent_attention, lightning)");
        if (!int_at(jl, "mixer.heads", H.heads) || !int_at(jl, "mixer.dim", H.dim) || !int_at(jl, "mixer.vdim", H.vdim) || H.heads < 1 || H.dim < 1 || H.vdim < 1) return fail(where + "mixer needs positive 'heads', 'dim', 'vdim'");
        if (H.mixer == PI_MIXER_LATENT_ATTENTION) {
            if (!int_at(jl, "mixer.kv_rank", H.kv_rank) || H.kv_rank < 1 || !num_at(jl, "mixer.scale", d)) return fail(where + "latent_attention needs 'kv_rank' and 'scale'");
            H.scale = (float) d;
            H.cache_index = n_cache++;
        } else {
            const json * dec = jl.at("mixer.decay");
            if (!dec || !dec->is_arr() || (int) dec->arr.size() != H.heads) return fail(where + "lightning needs 'decay' with one value per head");
            for (const json & v : dec->arr) { if (!v.is_num()) return fail(where + "'decay' holds a non-number"); H.decay.push_back((float) v.num); }
            if (H.dim > 1024) return fail(where + "lightning key width above 1024");
            H.state_index = n_state++;
        }
        H.weights = i;
        if (jl.has("weights_of")) {
            if (!int_at(jl, "weights_of", H.weights) || H.weights >= hp.n_layer) return fail(where + "'weights_of' names no layer");
        }
        if (jl.has("mlp")) {
            const json * kind = jl.at("mlp.kind");
            if (!kind || !kind->is_str() || kind->str != "moe") return fail(where + "feed-forward kind must be 'moe'");
            if (!int_at(jl, "mlp.router.experts", H.n_expert) || !int_at(jl, "mlp.router.identity", H.n_identity) || !int_at(jl, "mlp.router.top", H.top)) return fail(where + "mlp.router needs 'experts', 'identity', 'top'");
            if (H.n_expert > 0 && (!int_at(jl, "mlp.expert.ff", H.ff) || H.ff < 1)) return fail(where + "mlp.expert needs 'ff'");
            if (H.top < 1 || H.top > H.n_expert + H.n_identity) return fail(where + "'top' must lie between 1 and the number of router outputs");
            H.has_mlp = true; H.mlp = PI_MLP_MOE_RELU_SQR;
        }
        hp.hybrid.push_back(std::move(H));
    }
    for (int i = 0; i < hp.n_layer; i++) {                                   // (a borrowed layer may itself borrow: follow to the layer that owns the tensors)
        int w = hp.hybrid[(size_t) i].weights, hops = 0;
        while (hp.hybrid[(size_t) w].weights != w && hops++ <= hp.n_layer) w = hp.hybrid[(size_t) w].weights;
        if (hp.hybrid[(size_t) w].weights != w) return fail("layers[" + std::to_string(i) + "]: 'weights_of' runs in a circle");
        hp.hybrid[(size_t) i].weights = w;
    }
    for (int i = 0; i < hp.n_layer; i++) {                                   // a layer that borrows tensors must be the same kind of layer with the same sizes
        const pi_hybrid_layer & a = hp.hybrid[(size_t) i], & b = hp.hybrid[(size_t) a.weights];
        if (a.mixer != b.mixer || a.heads != b.heads || a.dim != b.dim || a.vdim != b.vdim || a.kv_rank != b.kv_rank || a.has_mlp != b.has_mlp || a.n_expert != b.n_expert || a.n_identity != b.n_identity || a.ff != b.ff)
            return fail("layers[" + std::to_string(i) + "]: its sizes differ from those of the layer whose tensors it uses");
    }
    m->hweights.resize((size_t) hp.n_layer);
    if (!params.vocab_only) {
        if (!m->st_file.open(folder + "/model.safetensors", err)) { fprintf(stderr, "llama_load_model_from_file: %s\n", err.c_str()); return nullptr; }
        for (const auto & kv : m->st_file.tensors) { m->n_elements += (uint64_t) kv.second.elements(); m->n_bytes += kv.second.nbytes; }
        const st_tensor * e = m->st_file.tensor("embed");
        if (!e || e->shape != std::vector<int64_t>{ hp.n_vocab, hp.n_embd }) return fail("tensor 'embed' is missing or not [vocab][width]");
    }
    return m.release();
}

}  // namespace pi
