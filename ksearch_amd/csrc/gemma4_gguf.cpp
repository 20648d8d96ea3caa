// Gemma-4 from a GGUF file: the configuration from the metadata table and the
// weights onto the device in the forms the decode loop takes.
//
// Mirrors GemmaConfig::from_gguf (crates/ksearch_gemma/src/lib.rs:39-122) and
// the load path of GemmaPrimModel (crates/ksearch_gemma/src/gemma_prim.rs:
// 146-410): Q4_K tensors go up as they are; Q6_K ffn_down / attn_v are
// requantized to Q4_K like the reference does (:418-433; flag
// KSH_LOAD_KEEP_Q6K keeps them); any other type is dequantized and packed to
// Q4_K (:437-447); per_layer_model_proj is scaled by 1/sqrt(hidden) before it is
// packed (:341-352).  Differences: norm vectors stay f32 (the reference rounds
// them to f16 for its f16 activations), a Q6_K embedding table stays Q6_K (the
// reference expands it to f16), and the quantizers run on the device.
#include <cmath>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

#include "ksh_internal.hpp"

namespace {

using namespace ksh;

bool ends_with(const std::string &s, const char *suffix)
{
    const size_t n = strlen(suffix);
    return s.size() >= n && s.compare(s.size() - n, n, suffix) == 0;
}

struct Loader {
    ksh_ctx *ctx;
    const ksh_gguf *g;
    int flags;
    std::vector<ksh_buf *> made;   // released on failure, adopted by the model on success

    ~Loader()
    {
        for (ksh_buf *b : made) ksh_buffer_release(b);
    }

    int kernel(int kind, int64_t n, int dt, ksh_kernel **out)
    {
        ksh_kernel_desc d;
        memset(&d, 0, sizeof(d));
        d.kind = kind;
        d.dims[0] = n;
        d.dtypes[0] = dt;
        return ksh_kernel_get(ctx, &d, out);
    }

    int upload(const void *src, size_t bytes, ksh_buf **out)
    {
        if (ksh_buffer_alloc(ctx, bytes, src, out)) return 1;
        made.push_back(*out);
        return 0;
    }

    void drop(ksh_buf *b)
    {
        for (size_t i = 0; i < made.size(); i++)
            if (made[i] == b) { made.erase(made.begin() + (long)i); break; }
        ksh_buffer_release(b);
    }

    struct T {
        int32_t type = 0, n_dims = 0;
        int64_t dims[4] = {1, 1, 1, 1};
        const void *data = nullptr;
        size_t bytes = 0;
        int64_t cols() const { return dims[0]; }
        int64_t rows() const { return dims[1] * dims[2] * dims[3]; }
        int64_t elems() const { return cols() * rows(); }
    };

    int tensor(const std::string &name, T &t)
    {
        return ksh_gguf_tensor(g, name.c_str(), &t.type, t.dims, &t.n_dims, &t.data, &t.bytes);
    }

    static int ksh_dtype(int32_t ggml)
    {
        switch (ggml) {
        case KSH_GGML_Q4_K: return KSH_Q4K;
        case KSH_GGML_Q5_K: return KSH_Q5K;
        case KSH_GGML_Q6_K: return KSH_Q6K;
        case KSH_GGML_Q4_0: return KSH_Q40;
        }
        return -1;
    }

    // the whole tensor as f32 on the host (dequant_to_f32, gguf_impl.rs:424-432)
    int to_f32(const std::string &name, const T &t, std::vector<float> &out)
    {
        out.resize((size_t)t.elems());
        const int kdt = ksh_dtype(t.type);
        if (kdt == KSH_Q4K || kdt == KSH_Q5K || kdt == KSH_Q6K) {
            ksh_buf *raw = nullptr, *f = nullptr;
            ksh_kernel *k = nullptr;
            if (upload(t.data, t.bytes, &raw) || upload(nullptr, out.size() * 4, &f) || kernel(KSH_DEQUANT, t.elems(), kdt, &k)) return 1;
            ksh_buf *in[1] = {raw}, *ob[1] = {f};
            if (ksh_encode(ctx, k, in, nullptr, 1, ob, nullptr, 1) || ksh_buffer_read(ctx, f, 0, out.data(), out.size() * 4, 1)) return 1;
            drop(raw);
            drop(f);
            return 0;
        }
        if (ksh_gguf_dequant_host(t.type, t.data, out.size(), out.data())) return set_error("%s: ggml type %d cannot be converted", name.c_str(), t.type);
        return 0;
    }

    int pack(const std::vector<float> &f, int dt, ksh_buf **out)
    {
        if (f.size() % 256) return set_error("elems %zu not multiple of 256", f.size());
        ksh_buf *src = nullptr;
        ksh_kernel *k = nullptr;
        if (upload(f.data(), f.size() * 4, &src) || upload(nullptr, f.size() / 256 * (dt == KSH_Q4K ? 144 : 210), out) ||
            kernel(KSH_QUANTIZE_K, (int64_t)f.size(), dt, &k))
            return 1;
        ksh_buf *in[1] = {src}, *ob[1] = {*out};
        if (ksh_encode(ctx, k, in, nullptr, 1, ob, nullptr, 1) || ksh_synchronize(ctx)) return 1;
        drop(src);
        return 0;
    }

    // ensure_weight (gemma_prim.rs:414-450), plus an optional scale applied before packing
    int weight(const std::string &name, int64_t rows, int64_t cols, float scale, ksh_buf **out, int32_t *dt)
    {
        T t;
        if (tensor(name, t)) return 1;
        if (t.cols() != cols || t.rows() != rows)
            return set_error("%s is [%lld, %lld], the configuration needs [%lld, %lld]", name.c_str(), (long long)t.rows(), (long long)t.cols(),
                             (long long)rows, (long long)cols);
        const bool requant6 = t.type == KSH_GGML_Q6_K && !(flags & KSH_LOAD_KEEP_Q6K) &&
                              (ends_with(name, "ffn_down.weight") || ends_with(name, "attn_v.weight"));
        if (scale == 1.0f && (t.type == KSH_GGML_Q4_K || (t.type == KSH_GGML_Q6_K && !requant6))) {
            *dt = t.type == KSH_GGML_Q4_K ? KSH_Q4K : KSH_Q6K;
            return upload(t.data, t.bytes, out);
        }
        std::vector<float> f;
        if (to_f32(name, t, f)) return 1;
        if (scale != 1.0f)
            for (float &v : f) v *= scale;
        *dt = KSH_Q4K;
        return pack(f, KSH_Q4K, out);
    }

    int vector(const std::string &name, int64_t n, ksh_buf **out, float *first = nullptr)
    {
        T t;
        if (tensor(name, t)) return 1;
        if (t.elems() != n) return set_error("%s has %lld elements, the configuration needs %lld", name.c_str(), (long long)t.elems(), (long long)n);
        std::vector<float> f;
        if (to_f32(name, t, f)) return 1;
        if (first) *first = f[0];
        return out ? upload(f.data(), f.size() * 4, out) : 0;
    }
};

}  // namespace

extern "C" {

int ksh_gemma4_config_from_gguf(const ksh_gguf *g, int max_seq, ksh_gemma4_cfg *cfg, int32_t *ffn, int32_t *is_swa, int cap)
{
    if (!g || !cfg) return set_error("ksh_gemma4_config_from_gguf: bad arguments");
    char arch[64];
    if (!ksh_gguf_get_str(g, "general.architecture", arch, sizeof(arch)) && strcmp(arch, "gemma4"))
        return set_error("unsupported GGUF architecture `%s` (expected gemma4)", arch);
    uint32_t u = 0;
    if (!ksh_gguf_get_u32(g, "gemma4.expert_count", &u) && u > 0) return set_error("Gemma 4 MoE (A4B) is not supported");
    memset(cfg, 0, sizeof(*cfg));
    if (ksh_gguf_get_u32(g, "gemma4.block_count", &u)) return set_error("block_count");
    cfg->n_layers = (int32_t)u;
    if (ksh_gguf_get_u32(g, "gemma4.embedding_length", &u)) return set_error("embedding_length");
    cfg->hidden = (int32_t)u;
    if (ksh_gguf_get_u32(g, "gemma4.attention.head_count", &u)) return set_error("attention.head_count");
    cfg->n_q = (int32_t)u;
    uint32_t kvl[4] = {1, 0, 0, 0};
    int nk = 1;
    if (!ksh_gguf_get_arr_u32(g, "gemma4.attention.head_count_kv", kvl, 4, &nk) && nk > 1)
        return set_error("per-layer head_count_kv is not supported (A4B/MoE)");
    cfg->n_kv = nk >= 1 && kvl[0] > 0 ? (int32_t)kvl[0] : 1;
    if (cfg->n_q % cfg->n_kv) return set_error("head_count %d not divisible by head_count_kv %d", cfg->n_q, cfg->n_kv);
    auto u32_or = [&](const char *key, uint32_t dflt) { uint32_t v; return ksh_gguf_get_u32(g, key, &v) ? dflt : v; };
    auto f32_or = [&](const char *key, float dflt) { float v; return ksh_gguf_get_f32(g, key, &v) ? dflt : v; };
    cfg->hd_full = (int32_t)u32_or("gemma4.attention.key_length", 512);
    cfg->hd_swa = (int32_t)u32_or("gemma4.attention.key_length_swa", 256);
    cfg->sliding_window = (int32_t)u32_or("gemma4.attention.sliding_window", 512);
    cfg->shared_kv_layers = (int32_t)u32_or("gemma4.attention.shared_kv_layers", 0);
    cfg->eps = f32_or("gemma4.attention.layer_norm_rms_epsilon", 1e-6f);
    cfg->softcap = f32_or("gemma4.final_logit_softcapping", 30.0f);
    cfg->ple_dim = (int32_t)u32_or("gemma4.embedding_length_per_layer_input", 256);
    if (!ksh_gguf_has_tensor(g, "per_layer_model_proj.weight")) cfg->ple_dim = 0;   // a file without the per-layer tables
    cfg->rope_theta_full = f32_or("gemma4.rope.freq_base", 1000000.0f);
    cfg->rope_theta_swa = f32_or("gemma4.rope.freq_base_swa", 10000.0f);
    cfg->partial_rotary = 0.25f;
    cfg->attn_scale = 1.0f;   // the reference's attention is unscaled (crates/ksearch_codegen/src/lower.rs:5152-5299)
    cfg->max_seq = max_seq;
    int64_t dims[4];
    int32_t nd = 0, ty = 0;
    cfg->vocab = 262144;
    if (!ksh_gguf_tensor(g, "token_embd.weight", &ty, dims, &nd, nullptr, nullptr)) cfg->vocab = (int32_t)(dims[1] * dims[2] * dims[3]);
    const int n = cfg->n_layers;
    if (n <= 0 || n > 4096) return set_error("block_count=%d", n);
    if (ffn || is_swa) {
        if (cap < n) return set_error("ksh_gemma4_config_from_gguf: room for %d layers, the file has %d", cap, n);
        std::vector<uint32_t> fl((size_t)n, 0), sp((size_t)n, 0);
        int nf = 0, ns = 0;
        // a scalar on some checkpoints, a per-layer list on others; anything else falls back to 6144 (lib.rs:79-91)
        if (ksh_gguf_get_arr_u32(g, "gemma4.feed_forward_length", fl.data(), n, &nf)) nf = 0;
        for (int i = 0; i < n && ffn; i++) ffn[i] = nf == 1 ? (int32_t)fl[0] : nf == n ? (int32_t)fl[(size_t)i] : 6144;
        const bool have = ksh_gguf_arr_is_bool(g, "gemma4.attention.sliding_window_pattern") &&
                          !ksh_gguf_get_arr_u32(g, "gemma4.attention.sliding_window_pattern", sp.data(), n, &ns);
        for (int i = 0; i < n && is_swa; i++) is_swa[i] = have ? (i < ns ? (sp[(size_t)i] != 0) : 1) : ((i + 1) % 6 != 0);
    }
    return 0;
}

int ksh_gemma4_load_gguf(ksh_ctx *ctx, const ksh_gguf *g, int max_seq, int flags, ksh_gemma4 **out)
{
    if (!ctx || !g || !out) return set_error("ksh_gemma4_load_gguf: bad arguments");
    *out = nullptr;
    ksh_gemma4_cfg c;
    std::vector<int32_t> ffn(4096), swa(4096);
    if (ksh_gemma4_config_from_gguf(g, max_seq, &c, ffn.data(), swa.data(), 4096)) return 1;
    Loader L{ctx, g, flags, {}};
    const int64_t h = c.hidden;
    std::vector<ksh_gemma4_layer> layers((size_t)c.n_layers);
    for (int i = 0; i < c.n_layers; i++) {
        ksh_gemma4_layer &w = layers[(size_t)i];
        memset(&w, 0, sizeof(w));
        w.is_swa = swa[(size_t)i];
        w.ffn = ffn[(size_t)i];
        w.layer_scale = 1.0f;
        const int64_t hd = w.is_swa ? c.hd_swa : c.hd_full, qd = c.n_q * hd, kvd = c.n_kv * hd;
        const bool owns = i < c.n_layers - c.shared_kv_layers;
        const std::string p = "blk." + std::to_string(i) + ".";
        if (L.weight(p + "attn_q.weight", qd, h, 1.f, &w.wq, &w.dt_q) || L.weight(p + "attn_output.weight", h, qd, 1.f, &w.wo, &w.dt_o) ||
            L.weight(p + "ffn_gate.weight", w.ffn, h, 1.f, &w.wgate, &w.dt_gate) || L.weight(p + "ffn_up.weight", w.ffn, h, 1.f, &w.wup, &w.dt_up) ||
            L.weight(p + "ffn_down.weight", h, w.ffn, 1.f, &w.wdown, &w.dt_down))
            return 1;
        if (owns && (L.weight(p + "attn_k.weight", kvd, h, 1.f, &w.wk, &w.dt_k) || L.weight(p + "attn_v.weight", kvd, h, 1.f, &w.wv, &w.dt_v)))
            return 1;
        if (L.vector(p + "attn_norm.weight", h, &w.attn_norm) || L.vector(p + "attn_q_norm.weight", hd, &w.q_norm) ||
            L.vector(p + "post_attention_norm.weight", h, &w.post_attn_norm) || L.vector(p + "ffn_norm.weight", h, &w.ffn_norm) ||
            L.vector(p + "post_ffw_norm.weight", h, &w.post_ffw_norm))
            return 1;
        // (layers that reuse a cache normalise no keys, but the files carry the vector for every layer)
        if ((owns || ksh_gguf_has_tensor(g, (p + "attn_k_norm.weight").c_str())) && L.vector(p + "attn_k_norm.weight", hd, &w.k_norm)) return 1;
        if (c.ple_dim > 0) {
            if (L.weight(p + "inp_gate.weight", c.ple_dim, h, 1.f, &w.inp_gate, &w.dt_inp_gate) ||
                L.weight(p + "proj.weight", h, c.ple_dim, 1.f, &w.proj, &w.dt_proj) || L.vector(p + "post_norm.weight", h, &w.post_norm) ||
                L.vector(p + "layer_output_scale.weight", 1, nullptr, &w.layer_scale))
                return 1;
            if (w.dt_inp_gate != KSH_Q4K) {
                // the gate GEMV with its gelu(.)*ctx epilogue is built for Q4_K
                Loader::T t;
                std::vector<float> f;
                if (L.tensor(p + "inp_gate.weight", t) || L.to_f32(p + "inp_gate.weight", t, f)) return 1;
                L.drop(w.inp_gate);
                if (L.pack(f, KSH_Q4K, &w.inp_gate)) return 1;
                w.dt_inp_gate = KSH_Q4K;
            }
        }
    }
    ksh_gemma4_globals G;
    memset(&G, 0, sizeof(G));
    {
        Loader::T t;
        if (L.tensor("token_embd.weight", t)) return 1;
        if (t.cols() != h) return set_error("token_embd.weight has %lld columns, the configuration needs %lld", (long long)t.cols(), (long long)h);
        if (t.type == KSH_GGML_Q4_K || t.type == KSH_GGML_Q6_K) {
            G.dt_embd = t.type == KSH_GGML_Q4_K ? KSH_Q4K : KSH_Q6K;
            if (L.upload(t.data, t.bytes, &G.token_embd)) return 1;
        } else {
            std::vector<float> f;
            if (L.to_f32("token_embd.weight", t, f) || L.pack(f, KSH_Q6K, &G.token_embd)) return 1;
            G.dt_embd = KSH_Q6K;
        }
    }
    if (L.vector("output_norm.weight", h, &G.output_norm)) return 1;
    if (c.ple_dim > 0) {
        const int64_t pt = (int64_t)c.n_layers * c.ple_dim;
        // gemma_prim.rs:341-352: the model projection is scaled by 1/sqrt(hidden) before it is packed
        if (L.weight("per_layer_model_proj.weight", pt, h, 1.0f / std::sqrt((float)h), &G.ple_model_proj, &G.dt_ple_proj) ||
            L.vector("per_layer_proj_norm.weight", c.ple_dim, &G.ple_proj_norm))
            return 1;
        Loader::T t;
        if (L.tensor("per_layer_token_embd.weight", t)) return 1;
        if (t.cols() != pt || t.rows() != c.vocab)
            return set_error("per_layer_token_embd.weight is [%lld, %lld], the configuration needs [%d, %lld]", (long long)t.rows(), (long long)t.cols(),
                             c.vocab, (long long)pt);
        const int kdt = Loader::ksh_dtype(t.type);
        if (kdt == KSH_Q4K || kdt == KSH_Q5K || kdt == KSH_Q6K || t.type == KSH_GGML_F16 || t.type == KSH_GGML_F32) {
            G.dt_ple = kdt >= 0 ? kdt : t.type == KSH_GGML_F16 ? KSH_F16 : KSH_F32;
            if (L.upload(t.data, t.bytes, &G.ple_embd)) return 1;
        } else {
            std::vector<float> f;
            if (L.to_f32("per_layer_token_embd.weight", t, f) || L.upload(f.data(), f.size() * 4, &G.ple_embd)) return 1;
            G.dt_ple = KSH_F32;
        }
    }
    if (ksh_synchronize(ctx)) return 1;
    ksh_gemma4 *m = nullptr;
    if (ksh_gemma4_create(ctx, &c, layers.data(), &G, &m)) return 1;
    for (ksh_buf *b : L.made) ksh_gemma4_adopt(m, b);
    L.made.clear();
    *out = m;
    return 0;
}

}  // extern "C"
