// Greedy decode loop with the layer features of the real Gemma-4 checkpoints,
// above the C ABI: sliding-window and full-attention layers with their own head
// dims, rope tables and windows, layers that reuse an earlier layer's KV cache,
// per-layer embeddings, Q4_K or Q6_K per weight tensor.
//
// Mirrors GemmaPrimModel::forward_token (crates/ksearch_gemma/src/gemma_prim.rs:
// 881-1275) with GemmaConfig's layer rules (crates/ksearch_gemma/src/lib.rs:
// 136-167).  As in the loop for the synthetic shape, norms ride in the GEMV that
// consumes them, the position lives on the device and a token is one HIP graph.
// A residual add stays "pending" (y, norm weight) until the next GEMV folds it
// into its prologue: the feed-forward block's into the per-layer-embedding gate,
// the layer-closing one (with the layer's output scale) into the next layer's
// QKV or the LM head.
#include <chrono>
#include <cmath>
#include <cstdlib>
#include <algorithm>
#include <map>
#include <memory>
#include <vector>

#include "ksh_device.hpp"
#include "ksh_internal.hpp"
#include "section_timer.hpp"

namespace {

// end of token: remember the id, advance the position and both attended ranges
// (full attention: rows [0, pos]; sliding window: the last `window` of them,
// gemma_prim.rs:1010-1017), and put the next position's rows of the two rope
// tables where the attention launches read them
__global__ void advance4_kernel(float *meta_full, float *meta_swa, const float *tok, float *history, int max_hist,
                                const float *rope_full, float *cur_full, int hd_full, const float *rope_swa,
                                float *cur_swa, int hd_swa, int window)
{
    const int pos = (int)meta_full[3];
    __syncthreads();   // every thread has read the position before thread 0 moves it
    if (pos + 1 < max_hist) {
        for (int i = threadIdx.x; i < hd_full; i += blockDim.x) cur_full[i] = rope_full[(size_t)(pos + 1) * hd_full + i];
        for (int i = threadIdx.x; i < hd_swa; i += blockDim.x) cur_swa[i] = rope_swa[(size_t)(pos + 1) * hd_swa + i];
    }
    if (threadIdx.x == 0) {
        if (history && pos < max_hist) history[pos] = tok[0];
        const int kv_len = pos + 2;   // the next token attends up to and including its own row
        const int start = kv_len > window ? kv_len - window : 0;
        meta_full[3] = meta_swa[3] = (float)(pos + 1);
        meta_full[0] = (float)kv_len;
        meta_swa[0] = (float)(kv_len - start);
        meta_swa[1] = (float)start;
    }
}

// points the device-side state at position `pos` (a model that is bound to another sequence's KV slot)
__global__ void seek4_kernel(float *meta_full, float *meta_swa, int pos, const float *rope_full, float *cur_full, int hd_full,
                             const float *rope_swa, float *cur_swa, int hd_swa, int window)
{
    for (int i = threadIdx.x; i < hd_full; i += blockDim.x) cur_full[i] = rope_full[(size_t)pos * hd_full + i];
    for (int i = threadIdx.x; i < hd_swa; i += blockDim.x) cur_swa[i] = rope_swa[(size_t)pos * hd_swa + i];
    if (threadIdx.x == 0) {
        const int kv_len = pos + 1, start = kv_len > window ? kv_len - window : 0;
        meta_full[0] = (float)kv_len; meta_full[1] = 0.f; meta_full[2] = 0.f; meta_full[3] = (float)pos;
        meta_swa[0] = (float)(kv_len - start); meta_swa[1] = (float)start; meta_swa[2] = (float)window; meta_swa[3] = (float)pos;
    }
}

// start of a prompt chunk: the records the batched attention reads ({rows the first token attends, -, window}), from
// the device-side position; full-attention layers see everything up to the token, sliding-window layers the last
// `window` rows (gemma_prim.rs:1426-1436)
__global__ void chunk_begin4_kernel(const float *meta_full, float *bmeta_full, float *bmeta_swa, int max_seq, int window)
{
    if (threadIdx.x == 0) {
        const float tlen0 = meta_full[3] + 1.0f;
        bmeta_full[0] = tlen0; bmeta_full[1] = 0.f; bmeta_full[2] = (float)max_seq; bmeta_full[3] = 0.f;
        bmeta_swa[0] = tlen0; bmeta_swa[1] = 0.f; bmeta_swa[2] = (float)window; bmeta_swa[3] = 0.f;
    }
}

__global__ void set_token4_kernel(float *tok, float value)
{
    if (threadIdx.x == 0 && blockIdx.x == 0) tok[0] = value;
}

struct Bufs {
    std::vector<ksh_buf *> owned;
    ~Bufs()
    {
        for (ksh_buf *b : owned) ksh_buffer_release(b);
    }
};

// the kernels of one layer, bound when the model is built
struct LayerPlan {
    int hd = 0, qd = 0, kvd = 0, src = 0;
    bool swa = false, owns = false;
    bool fused_qkv = false, fused_gate_up = false, attend = false, attend_parts = false;
    ksh_kernel *qkv[2] = {nullptr, nullptr};       // [pending add folded in?]; fused QKV, or q alone
    ksh_kernel *kmat[2] = {nullptr, nullptr};      // k and v one by one (mixed weight types), on the materialised stream
    ksh_kernel *head = nullptr, *sdpa = nullptr, *k_attend = nullptr;
    ksh_kernel *oproj = nullptr;
    ksh_kernel *gate_up = nullptr, *gate = nullptr, *up = nullptr, *gelu = nullptr;
    ksh_kernel *down = nullptr;
    ksh_kernel *ple_gate = nullptr, *ple_proj = nullptr;
};

}  // namespace

struct ksh_gemma4 {
    std::vector<float> host_logits;   // decode_token_sampled's read-back
    ksh_ctx *ctx = nullptr;
    ksh_gemma4_cfg c{};
    ksh_gemma4_globals g{};
    std::vector<ksh_gemma4_layer> layers;
    std::vector<LayerPlan> plan;
    Bufs bufs;
    ksh_buf *embd_rows = nullptr;
    ksh_buf *x = nullptr, *xb = nullptr, *y = nullptr, *hidden = nullptr, *tq = nullptr, *tk = nullptr, *tv = nullptr, *to = nullptr,
            *ff = nullptr, *ff2 = nullptr, *logits = nullptr, *tok = nullptr, *meta_full = nullptr, *meta_swa = nullptr,
            *rope_full = nullptr, *rope_swa = nullptr, *cur_full = nullptr, *cur_swa = nullptr, *attn_tmp = nullptr,
            *history = nullptr, *ple_tok = nullptr, *ple_tmp = nullptr, *ple_ctx = nullptr, *ple_u = nullptr;
    std::vector<ksh_buf *> kv_k, kv_v;   // per layer; null where the layer reads another layer's cache
    ksh_kernel *k_embed = nullptr, *k_ple_gather = nullptr, *k_ple_proj = nullptr, *k_ple_norm = nullptr, *k_ple_mix = nullptr,
               *k_lm_head[2] = {nullptr, nullptr}, *k_argmax = nullptr;
    ksh_graph *g_body = nullptr, *g_full = nullptr;   // the graphs of the caches in use (own or a pool slot's)
    ksh_graph *g_span = nullptr;                      // kSpan decode steps with logits as one graph (generate's loop)
    std::vector<float> rope0_full, rope0_swa;
    int pos = 0, launches_full = 0;
    // serving: the model's own caches, and the graphs captured for each slot of the pool it was last bound to
    std::vector<ksh_buf *> own_k, own_v;
    struct SlotGraphs { ksh_graph *body = nullptr, *full = nullptr, *span = nullptr; };
    ksh_kvpool *pool = nullptr;
    uint64_t pool_uid = 0;   // (a new pool can be allocated where a destroyed one lay: the address alone does not identify it)
    std::vector<SlotGraphs> slot_graphs;
    SlotGraphs own_graphs;
    int bound_slot = -1;
    // prompt chunks (allocated at the first chunk): [kChunk, .] activations of the batched layer pass
    ksh_buf *c_tok = nullptr, *c_x = nullptr, *c_x2 = nullptr, *c_y = nullptr, *c_q = nullptr, *c_k = nullptr, *c_v = nullptr, *c_o = nullptr,
            *c_g = nullptr, *c_u = nullptr, *c_ff = nullptr, *c_tmp = nullptr, *c_meta_full = nullptr, *c_meta_swa = nullptr,
            *c_po = nullptr, *c_pg = nullptr,   // unfolded partial sums of the o and the gate | up projection of a chunk
            *c_ple_tok = nullptr, *c_ple_tmp = nullptr, *c_ple_ctx = nullptr, *c_ple_u = nullptr;
    // decode rounds over several KV slots (allocated at the first round): the per-token table (ids, slots, attended
    // ranges of the two layer kinds), the logits of every token of the round, the greedy ids
    ksh_buf *r_tab = nullptr, *r_logits = nullptr, *r_next = nullptr, *r_xp = nullptr, *r_xp2 = nullptr;   // (r_xp, r_xp2: a round's prepared GEMM operands)
    // a round of t sequences is one graph per t, tied to the pool whose buffers it was captured over
    ksh_graph *round_graphs[17] = {};
    bool round_bound[17] = {};     // a width's kernels are bound (a first round launched kernel by kernel)
    ksh_kvpool *round_pool = nullptr;
    uint64_t round_pool_uid = 0;   // a new pool can come up at a destroyed pool's address: the graphs are tied to the pool's uid as well
    bool round_graph = true;       // KSEARCH_ROUND_GRAPH, read when the model is created
    ksh::SectionTimer prof;        // KSEARCH_PROFILE (read when the model is created): per-section times of every decode step
    int r_count = 0;
};

namespace {

using namespace ksh;

constexpr int kAttendPartitions = 16;
constexpr int kShortPartitions = 8;     // sliding-window layers: the o-projection merges the partitions
constexpr int kShortWindow = 640;

int alloc(ksh_gemma4 *m, size_t bytes, ksh_buf **out)
{
    if (ksh_buffer_alloc(m->ctx, bytes ? bytes : 16, nullptr, out)) return 1;
    m->bufs.owned.push_back(*out);
    return 0;
}

int get(ksh_gemma4 *m, int kind, std::initializer_list<int64_t> dims, std::initializer_list<int> dtypes,
        std::initializer_list<float> params, ksh_kernel **out)
{
    ksh_kernel_desc d;
    memset(&d, 0, sizeof(d));
    d.kind = kind;
    int i = 0;
    for (int64_t v : dims) d.dims[i++] = v;
    i = 0;
    for (int v : dtypes) d.dtypes[i++] = v;
    i = 0;
    for (float v : params) d.params[i++] = v;
    return ksh_kernel_get(m->ctx, &d, out);
}

int enc(ksh_gemma4 *m, ksh_kernel *k, std::initializer_list<ksh_buf *> in, std::initializer_list<ksh_buf *> out, int &count)
{
    ksh_buf *ib[kMaxIn], *ob[kMaxOut];
    int ni = 0, no = 0;
    for (ksh_buf *b : in) ib[ni++] = b;
    for (ksh_buf *b : out) ob[no++] = b;
    count += 1;
    return ksh_encode(m->ctx, k, ib, nullptr, ni, ob, nullptr, no);
}

int enc_off(ksh_gemma4 *m, ksh_kernel *k, std::initializer_list<ksh_buf *> in, std::initializer_list<size_t> in_off,
            std::initializer_list<ksh_buf *> out, int &count)
{
    ksh_buf *ib[kMaxIn], *ob[kMaxOut];
    size_t io[kMaxIn];
    int ni = 0, no = 0, nf = 0;
    for (ksh_buf *b : in) ib[ni++] = b;
    for (size_t o : in_off) io[nf++] = o;
    for (ksh_buf *b : out) ob[no++] = b;
    count += 1;
    return ksh_encode(m->ctx, k, ib, io, ni, ob, nullptr, no);
}

bool packed_ok(int dt) { return dt == KSH_Q4K || dt == KSH_Q6K; }

// the residual stream while a token is encoded: `cur` holds x; if `y` is set, the
// stream is really cur + rms(y)*w and the add has not been written anywhere yet
struct Stream {
    ksh_buf *cur, *other;
    ksh_buf *y = nullptr, *w = nullptr;
};

// norm(x)*w_norm -> GEMV, folding a pending add in (the fused kinds write the new stream themselves)
int enc_norm_gemv(ksh_gemma4 *m, ksh_kernel *const k[2], std::initializer_list<ksh_buf *> weights, ksh_buf *w_norm, Stream &s,
                  std::initializer_list<ksh_buf *> outs, int &n)
{
    ksh_buf *ib[kMaxIn], *ob[kMaxOut];
    int ni = 0, no = 0;
    for (ksh_buf *b : weights) ib[ni++] = b;
    for (ksh_buf *b : outs) ob[no++] = b;
    if (s.y) {
        ib[ni++] = s.y; ib[ni++] = w_norm; ib[ni++] = s.w; ib[ni++] = s.cur;
        ob[no++] = s.other;
        n += 1;
        if (ksh_encode(m->ctx, k[1], ib, nullptr, ni, ob, nullptr, no)) return 1;
        std::swap(s.cur, s.other);
        s.y = s.w = nullptr;
        return 0;
    }
    ib[ni++] = s.cur; ib[ni++] = w_norm;
    n += 1;
    return ksh_encode(m->ctx, k[0], ib, nullptr, ni, ob, nullptr, no);
}

int encode_token(ksh_gemma4 *m, bool want_logits, int &launches)
{
    const ksh_gemma4_cfg &c = m->c;
    launches = 0;
    Stream s{m->x, m->xb};
    if (enc(m, m->k_embed, {m->g.token_embd, m->tok}, {s.cur}, launches)) return 1;
    m->prof.mark(SectionTimer::kEmbed);
    if (c.ple_dim > 0) {
        // ple_from_idx + ple_prepass (gemma_prim.rs:712-728, 845-878)
        if (enc(m, m->k_ple_gather, {m->g.ple_embd, m->tok}, {m->ple_tok}, launches) ||
            enc(m, m->k_ple_proj, {m->g.ple_model_proj, s.cur}, {m->ple_tmp}, launches) ||
            enc(m, m->k_ple_norm, {m->ple_tmp, m->g.ple_proj_norm}, {m->ple_ctx}, launches) ||
            enc(m, m->k_ple_mix, {m->ple_ctx, m->ple_tok}, {m->ple_ctx}, launches))
            return 1;
        m->prof.mark(SectionTimer::kPrepass);
    }
    for (int l = 0; l < c.n_layers; l++) {
        const ksh_gemma4_layer &L = m->layers[l];
        const LayerPlan &P = m->plan[l];
        ksh_buf *meta = P.swa ? m->meta_swa : m->meta_full;
        ksh_buf *rope_cur = P.swa ? m->cur_swa : m->cur_full, *rope_tab = P.swa ? m->rope_swa : m->rope_full;
        ksh_buf *kc = m->kv_k[P.src], *vc = m->kv_v[P.src];
        // -- q, k, v of the normalised stream
        if (P.owns && P.fused_qkv) {
            if (enc_norm_gemv(m, P.qkv, {L.wq, L.wk, L.wv}, L.attn_norm, s, {m->tq, m->tk, m->tv}, launches)) return 1;
        } else {
            if (enc_norm_gemv(m, P.qkv, {L.wq}, L.attn_norm, s, {m->tq}, launches)) return 1;
            if (P.owns &&
                (enc(m, P.kmat[0], {L.wk, s.cur, L.attn_norm}, {m->tk}, launches) ||
                 enc(m, P.kmat[1], {L.wv, s.cur, L.attn_norm}, {m->tv}, launches)))
                return 1;
        }
        // -- per-head norm, RoPE, cache append, attention
        bool parts = false;
        if (P.attend && !P.owns) {
            parts = P.attend_parts;
            if (parts ? enc(m, P.k_attend, {m->tq, L.q_norm, rope_cur, kc, vc, meta}, {m->attn_tmp}, launches)
                      : enc(m, P.k_attend, {m->tq, L.q_norm, rope_cur, kc, vc, meta}, {m->attn_tmp, m->to}, launches))
                return 1;
        } else if (P.attend) {
            parts = P.attend_parts;
            if (parts ? enc(m, P.k_attend, {m->tq, L.q_norm, rope_cur, m->tk, L.k_norm, m->tv, meta}, {kc, vc, m->attn_tmp}, launches)
                      : enc(m, P.k_attend, {m->tq, L.q_norm, rope_cur, m->tk, L.k_norm, m->tv, meta}, {kc, vc, m->attn_tmp, m->to}, launches))
                return 1;
        } else {
            if (P.owns ? enc(m, P.head, {m->tq, L.q_norm, rope_tab, m->tk, L.k_norm, m->tv, meta}, {m->tq, kc, vc}, launches)
                       : enc(m, P.head, {m->tq, L.q_norm, rope_tab, meta}, {m->tq}, launches))   // gemma_prim.rs:989-1008
                return 1;
            if (enc(m, P.sdpa, {m->tq, kc, vc, meta}, {m->attn_tmp, m->to}, launches)) return 1;
        }
        if (enc(m, P.oproj, {L.wo, parts ? m->attn_tmp : m->to}, {m->y}, launches)) return 1;
        m->prof.mark(SectionTimer::kAttn);
        // -- feed-forward on norm(x + rms(o)*post_attn_norm)
        s.y = m->y;
        s.w = L.post_attn_norm;
        if (P.fused_gate_up) {
            ksh_kernel *const k2[2] = {nullptr, P.gate_up};
            if (enc_norm_gemv(m, k2, {L.wgate, L.wup}, L.ffn_norm, s, {m->ff}, launches)) return 1;
        } else {
            ksh_kernel *const k2[2] = {nullptr, P.gate};
            if (enc_norm_gemv(m, k2, {L.wgate}, L.ffn_norm, s, {m->ff}, launches) ||
                enc(m, P.up, {L.wup, s.cur, L.ffn_norm}, {m->ff2}, launches) ||
                enc(m, P.gelu, {m->ff, m->ff2}, {m->ff}, launches))
                return 1;
        }
        if (enc(m, P.down, {L.wdown, m->ff}, {m->y}, launches)) return 1;
        m->prof.mark(SectionTimer::kMlp);
        s.y = m->y;
        s.w = L.post_ffw_norm;
        if (c.ple_dim > 0) {
            // gemma_prim.rs:1150-1200: x += rms(down)*post_ffw_norm; u = gelu(Wg x) * ctx_l; x = (x + rms(Wp u)*post_norm) * scale.
            // The first add rides in the gate GEMV; the last one stays pending, with the scale, for the next layer's
            // QKV (or the LM head).
            if (enc_off(m, P.ple_gate, {L.inp_gate, s.y, m->ple_ctx, s.w, s.cur}, {0, 0, (size_t)l * c.ple_dim * 4, 0, 0}, {m->ple_u, s.other},
                        launches))
                return 1;
            std::swap(s.cur, s.other);
            if (enc(m, P.ple_proj, {L.proj, m->ple_u}, {m->y}, launches)) return 1;
            m->prof.mark(SectionTimer::kPle);
            s.y = m->y;
            s.w = L.post_norm;
        }
    }
    if (want_logits) {
        if (enc_norm_gemv(m, m->k_lm_head, {m->embd_rows ? m->embd_rows : m->g.token_embd}, m->g.output_norm, s, {m->logits}, launches))
            return 1;
        if (enc(m, m->k_argmax, {m->logits}, {m->tok}, launches)) return 1;
        launches += 1;   // two passes
    }
    // (a pending add of the last layer of a logits-free token is never needed, and the test hook follows the
    // tokens that produce logits: the two captured graphs end in different buffers)
    if (want_logits) m->hidden = s.cur;
    hipStream_t st = (hipStream_t)ksh_stream(m->ctx);
    hipLaunchKernelGGL(advance4_kernel, dim3(1), dim3(64), 0, st, (float *)ksh_buffer_device_ptr(m->meta_full),
                       (float *)ksh_buffer_device_ptr(m->meta_swa), (const float *)ksh_buffer_device_ptr(m->tok),
                       want_logits ? (float *)ksh_buffer_device_ptr(m->history) : nullptr, c.max_seq,
                       (const float *)ksh_buffer_device_ptr(m->rope_full), (float *)ksh_buffer_device_ptr(m->cur_full), c.hd_full,
                       (const float *)ksh_buffer_device_ptr(m->rope_swa), (float *)ksh_buffer_device_ptr(m->cur_swa), c.hd_swa,
                       c.sliding_window);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e, "advance launch");
    launches += 1;
    m->prof.mark(SectionTimer::kLogits);
    return 0;
}

int run_token(ksh_gemma4 *m, bool want_logits, bool use_graph)
{
    if (m->pos >= m->c.max_seq) return set_error("max_seq exceeded");   // gemma_prim.rs:882-884
    int n = 0;
    if (m->prof.on) {
        // gemma_prim.rs:885: with KSEARCH_PROFILE every step is timed section by section (launched kernel by kernel)
        m->prof.begin((hipStream_t)ksh_stream(m->ctx));
        if (encode_token(m, want_logits, n)) return 1;
        m->prof.report(want_logits ? "decode" : "prefill", m->pos);
    } else if (!use_graph) {
        if (encode_token(m, want_logits, n)) return 1;
    } else {
        ksh_graph *&g = want_logits ? m->g_full : m->g_body;
        if (!g) {
            if (ksh_synchronize(m->ctx)) return 1;
            if (ksh_graph_begin(m->ctx)) return 1;
            if (encode_token(m, want_logits, n)) {
                ksh_graph *dead = nullptr;
                ksh_graph_end(m->ctx, &dead);
                ksh_graph_destroy(dead);
                return 1;
            }
            if (ksh_graph_end(m->ctx, &g)) return 1;
            if (want_logits) m->launches_full = n;
        }
        if (ksh_graph_launch(m->ctx, g)) return 1;
    }
    if (want_logits && (!use_graph || m->prof.on)) m->launches_full = n;
    m->pos += 1;
    return 0;
}

// Several decode steps as one graph launch: positions, attended ranges, rope rows and the token live on the device
// and are advanced by the step's last kernel, so a token's graph repeated kSpan times is kSpan tokens (what it saves
// is the time between two graph launches, ~6 us each).
constexpr int kSpan = 8;

int run_span(ksh_gemma4 *m)
{
    ksh_graph *&g = m->g_span;
    if (!g) {
        int n = 0;
        if (ksh_synchronize(m->ctx)) return 1;
        if (ksh_graph_begin(m->ctx)) return 1;
        for (int i = 0; i < kSpan; i++) {
            if (encode_token(m, true, n)) {
                ksh_graph *dead = nullptr;
                ksh_graph_end(m->ctx, &dead);
                ksh_graph_destroy(dead);
                return 1;
            }
        }
        if (ksh_graph_end(m->ctx, &g)) return 1;
        m->launches_full = n;   // (the count of one step: every step starts its own)
    }
    if (ksh_graph_launch(m->ctx, g)) return 1;
    m->pos += kSpan;
    return 0;
}

int write_token(ksh_gemma4 *m, uint32_t token)
{
    hipLaunchKernelGGL(set_token4_kernel, dim3(1), dim3(64), 0, (hipStream_t)ksh_stream(m->ctx),
                       (float *)ksh_buffer_device_ptr(m->tok), (float)token);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, "set_token launch");
}

// gemma_prim.rs:33-56: per position cos[0..hd/2) || sin[0..hd/2); pairs past `angles` are the identity
// prefill_chunk's chunk length (gemma_prim.rs:16)
constexpr int kChunk4 = 1024;
constexpr int kChunkPartitions4 = 8;
constexpr int kPartsRows4 = 4;      // room for the unfolded partial sums of a hidden-wide projection: this many chunks of rows

int chunk_buffers4(ksh_gemma4 *m)
{
    if (m->c_tok) return 0;
    const ksh_gemma4_cfg &c = m->c;
    const size_t T = kChunk4, max_hd = (size_t)std::max(c.hd_swa, c.hd_full), qd = c.n_q * max_hd, kvd = c.n_kv * max_hd;
    size_t max_ff = 0;
    for (const ksh_gemma4_layer &L : m->layers) max_ff = std::max(max_ff, (size_t)L.ffn);
    const size_t pt = (size_t)c.n_layers * c.ple_dim;
    if (alloc(m, T * 4, &m->c_tok) || alloc(m, T * c.hidden * 4, &m->c_x) || alloc(m, T * c.hidden * 4, &m->c_x2) ||
        alloc(m, T * c.hidden * 4, &m->c_y) || alloc(m, T * qd * 4, &m->c_q) || alloc(m, T * kvd * 4, &m->c_k) ||
        alloc(m, T * kvd * 4, &m->c_v) || alloc(m, T * qd * 4, &m->c_o) || alloc(m, T * max_ff * 4, &m->c_g) ||
        alloc(m, T * max_ff * 4, &m->c_u) || alloc(m, T * max_ff * 4, &m->c_ff) ||
        alloc(m, T * c.n_q * kChunkPartitions4 * (max_hd + 2) * 4, &m->c_tmp) || alloc(m, 16, &m->c_meta_full) || alloc(m, 16, &m->c_meta_swa) ||
        alloc(m, kPartsRows4 * T * c.hidden * 4, &m->c_po) || alloc(m, 2 * T * 2 * max_ff * 4, &m->c_pg))
        return 1;
    if (c.ple_dim > 0 && (alloc(m, T * pt * 4, &m->c_ple_tok) || alloc(m, T * pt * 4, &m->c_ple_tmp) || alloc(m, T * pt * 4, &m->c_ple_ctx) ||
                          alloc(m, T * c.ple_dim * 4, &m->c_ple_u)))
        return 1;
    return 0;
}

// forward_prefill_chunk (gemma_prim.rs:1317-1607) for 2 <= t <= kChunk4 validated tokens: every layer as matrices
// of t rows, with the layer kinds' own head sizes, rope tables and windows, cache-reading layers attending over their
// source layer's rows, and the per-layer-embedding block.  The GEMMs run on the batch rounded up to 32 rows.
int forward_prefill_chunk4(ksh_gemma4 *m, const uint32_t *tokens, int t)
{
    const ksh_gemma4_cfg &c = m->c;
    if (chunk_buffers4(m)) return 1;
    const int64_t h = c.hidden, tp = (t + 31) / 32 * 32, pt = (int64_t)c.n_layers * c.ple_dim;
    float ids[kChunk4];
    for (int i = 0; i < t; i++) ids[i] = (float)tokens[i];
    if (ksh_synchronize(m->ctx)) return 1;                                   // c_tok may still be read by the previous chunk
    if (ksh_buffer_write(m->ctx, m->c_tok, 0, ids, (size_t)t * 4, 1)) return 1;
    hipStream_t st = (hipStream_t)ksh_stream(m->ctx);
    hipLaunchKernelGGL(chunk_begin4_kernel, dim3(1), dim3(64), 0, st, (const float *)ksh_buffer_device_ptr(m->meta_full),
                       (float *)ksh_buffer_device_ptr(m->c_meta_full), (float *)ksh_buffer_device_ptr(m->c_meta_swa), c.max_seq, c.sliding_window);
    if (hipGetLastError() != hipSuccess) return set_error("chunk_begin launch failed");
    int n = 0;
    ksh_kernel *k = nullptr, *k_norm = nullptr, *k_add = nullptr, *k_add_then = nullptr;
    auto mm = [&](int dt, int64_t rows, int64_t cols, ksh_buf *w, ksh_buf *x, ksh_buf *y) {
        ksh_kernel *kk = nullptr;
        return get(m, KSH_MATVEC_BATCH, {rows, cols, tp}, {dt, KSH_F32, KSH_F32}, {}, &kk) || enc(m, kk, {w, x}, {y}, n);
    };
    // matrices of one dtype over the same rows (q | k | v, gate | up) are one launch of the tile over one preparation
    // of the rows
    auto mm2 = [&](int dt, int64_t rows, int64_t cols, ksh_buf *w0, ksh_buf *w1, ksh_buf *x, ksh_buf *y0, ksh_buf *y1) {
        ksh_kernel *kk = nullptr;
        return get(m, KSH_MATVEC_BATCH, {rows, cols, tp, rows}, {dt, KSH_F32, KSH_F32}, {}, &kk) || enc(m, kk, {w0, x, w1}, {y0, y1}, n);
    };
    auto mm3 = [&](int dt, int64_t rows0, int64_t rows12, int64_t cols, ksh_buf *w0, ksh_buf *w1, ksh_buf *w2, ksh_buf *x, ksh_buf *y0, ksh_buf *y1,
                   ksh_buf *y2) {
        ksh_kernel *kk = nullptr;
        return get(m, KSH_MATVEC_BATCH, {rows0, cols, tp, rows12, rows12}, {dt, KSH_F32, KSH_F32}, {}, &kk) ||
               enc(m, kk, {w0, x, w1, w2}, {y0, y1, y2}, n);
    };
    const bool merged = true;
    // ... with the rows' producers inside the GEMMs' preparations (dims[5]: the attention norm in q | k | v's,
    // add-then-norm in gate | up's, gelu(gate) * up in the down projection's)
    const bool inside = merged && h % 512 == 0 && h <= 8192;
    auto mm_pro = [&](int dt, std::initializer_list<int64_t> dims, std::initializer_list<ksh_buf *> ins, std::initializer_list<ksh_buf *> outs) {
        ksh_kernel *kk = nullptr;
        return get(m, KSH_MATVEC_BATCH, dims, {dt, KSH_F32, KSH_F32}, {c.eps}, &kk) || enc(m, kk, ins, outs, n);
    };
    if (get(m, KSH_COPY_SCALE_INDEXED, {h, c.vocab, t}, {m->g.dt_embd}, {std::sqrt((float)c.hidden)}, &k) ||
        enc(m, k, {m->g.token_embd, m->c_tok}, {m->c_x}, n))
        return 1;
    if (c.ple_dim > 0) {
        // ple_from_idx_batch + ple_prepass_batch (gemma_prim.rs:1333-1358)
        ksh_kernel *kg = nullptr, *kn = nullptr, *kmix = nullptr;
        if (get(m, KSH_COPY_SCALE_INDEXED, {pt, c.vocab, t}, {m->g.dt_ple}, {std::sqrt((float)c.ple_dim)}, &kg) ||
            enc(m, kg, {m->g.ple_embd, m->c_tok}, {m->c_ple_tok}, n) ||
            mm(m->g.dt_ple_proj, pt, h, m->g.ple_model_proj, m->c_x, m->c_ple_tmp) ||
            get(m, KSH_RMSNORM_PER_HEAD, {(int64_t)t * c.n_layers, c.ple_dim, 0}, {}, {c.eps}, &kn) ||
            enc(m, kn, {m->c_ple_tmp, m->g.ple_proj_norm}, {m->c_ple_ctx}, n) ||
            get(m, KSH_ADD_SCALE, {(int64_t)t * pt}, {}, {0.70710678118654752440f}, &kmix) ||
            enc(m, kmix, {m->c_ple_ctx, m->c_ple_tok}, {m->c_ple_ctx}, n))
            return 1;
    }
    if (get(m, KSH_RMSNORM, {h, 0, 0, t}, {}, {c.eps}, &k_norm) || get(m, KSH_RMSNORM, {h, 1, 0, t}, {}, {c.eps}, &k_add) ||
        get(m, KSH_RMSNORM_ADD_THEN_RMSNORM, {h, t}, {}, {c.eps}, &k_add_then))
        return 1;
    for (int l = 0; l < c.n_layers; l++) {
        const ksh_gemma4_layer &L = m->layers[l];
        const LayerPlan &P = m->plan[l];
        ksh_buf *rope_tab = P.swa ? m->rope_swa : m->rope_full;
        ksh_buf *kc = m->kv_k[P.src], *vc = m->kv_v[P.src];
        ksh_kernel *k_head = nullptr, *k_sdpa = nullptr, *k_gelu = nullptr;
        const bool qkv_merged = merged && P.owns && L.dt_q == L.dt_k && L.dt_q == L.dt_v;
        const bool q_inside = inside && (qkv_merged || !P.owns);
        if (q_inside) {
            if (qkv_merged ? mm_pro(L.dt_q, {P.qd, h, tp, P.kvd, P.kvd, 1}, {L.wq, m->c_x, L.wk, L.wv, L.attn_norm}, {m->c_q, m->c_k, m->c_v})
                           : mm_pro(L.dt_q, {P.qd, h, tp, 0, 0, 1}, {L.wq, m->c_x, L.attn_norm}, {m->c_q}))
                return 1;
        } else {
            if (enc(m, k_norm, {m->c_x, L.attn_norm}, {m->c_x2}, n)) return 1;
            if (qkv_merged ? mm3(L.dt_q, P.qd, P.kvd, h, L.wq, L.wk, L.wv, m->c_x2, m->c_q, m->c_k, m->c_v) : mm(L.dt_q, P.qd, h, L.wq, m->c_x2, m->c_q)) return 1;
        }
        if (P.owns) {
            if ((!qkv_merged && (mm(L.dt_k, P.kvd, h, L.wk, m->c_x2, m->c_k) || mm(L.dt_v, P.kvd, h, L.wv, m->c_x2, m->c_v))) ||
                get(m, KSH_RMSNORM_PER_HEAD_QKV_Q40, {c.n_q, c.n_kv, P.hd, c.max_seq, t}, {}, {c.eps}, &k_head) ||
                enc(m, k_head, {m->c_q, L.q_norm, rope_tab, m->c_k, L.k_norm, m->c_v, m->meta_full}, {m->c_q, kc, vc}, n))
                return 1;
        } else {
            if (get(m, KSH_RMSNORM_PER_HEAD, {(int64_t)t * c.n_q, P.hd, 2, c.max_seq, c.n_q}, {}, {c.eps}, &k_head) ||
                enc(m, k_head, {m->c_q, L.q_norm, rope_tab, m->meta_full}, {m->c_q}, n))
                return 1;
        }
        // (heads of 256 or 512 in chunks of more than 16 tokens take the attention's matrix-core form: one partition per token)
        if (get(m, KSH_SDPA_BATCH, {c.n_q, c.n_kv, P.hd, c.max_seq, t, t > 16 && (P.hd == 256 || P.hd == 512) && c.n_q / c.n_kv <= 8 ? 1 : kChunkPartitions4}, {KSH_Q40, KSH_F32}, {c.attn_scale}, &k_sdpa) ||
            enc(m, k_sdpa, {m->c_q, kc, vc, P.swa ? m->c_meta_swa : m->c_meta_full}, {m->c_tmp, m->c_o}, n))
            return 1;
        // With the producers inside, the o and the gate | up projection leave their K slices' partial sums unfolded
        // for the preparation that reads them (dims[6], dims[7]); the down projection folds (a plain norm reads it).
        ksh_kernel *u_o = nullptr, *u_gu = nullptr;
        bool travel = false;
        if (inside && L.dt_gate == L.dt_up) {
            const size_t T = kChunk4;
            if (get(m, KSH_MATVEC_BATCH, {h, P.qd, tp, 0, 0, 0, 1}, {L.dt_o, KSH_F32, KSH_F32}, {c.eps}, &u_o) ||
                get(m, KSH_MATVEC_BATCH, {L.ffn, h, tp, L.ffn, 0, 2, 1, (int64_t)u_o->info.grid[2]}, {L.dt_gate, KSH_F32, KSH_F32}, {c.eps}, &u_gu))
                return 1;
            travel = u_o->out_bytes[0] <= kPartsRows4 * T * c.hidden * 4 && u_gu->out_bytes[0] <= ksh_buffer_size(m->c_pg);
        }
        if (travel) {
            if (enc(m, u_o, {L.wo, m->c_o}, {m->c_po}, n) ||
                enc(m, u_gu, {L.wgate, m->c_po, L.wup, L.post_attn_norm, m->c_x, L.ffn_norm}, {m->c_pg, m->c_x}, n) ||
                mm_pro(L.dt_down, {h, L.ffn, tp, 0, 0, 3, 0, (int64_t)u_gu->info.grid[2]}, {L.wdown, m->c_pg}, {m->c_y}))
                return 1;
        } else if (
            mm(L.dt_o, h, P.qd, L.wo, m->c_o, m->c_y) ||
            (inside && L.dt_gate == L.dt_up
                 ? mm_pro(L.dt_gate, {L.ffn, h, tp, L.ffn, 0, 2}, {L.wgate, m->c_y, L.wup, L.post_attn_norm, m->c_x, L.ffn_norm}, {m->c_g, m->c_u, m->c_x})
                 : (enc(m, k_add_then, {m->c_y, L.post_attn_norm, m->c_x, L.ffn_norm}, {m->c_x, m->c_x2}, n) ||
                    (merged && L.dt_gate == L.dt_up ? mm2(L.dt_gate, L.ffn, h, L.wgate, L.wup, m->c_x2, m->c_g, m->c_u)
                                                    : (mm(L.dt_gate, L.ffn, h, L.wgate, m->c_x2, m->c_g) || mm(L.dt_up, L.ffn, h, L.wup, m->c_x2, m->c_u))))) ||
            (inside ? mm_pro(L.dt_down, {h, L.ffn, tp, 0, 0, 3}, {L.wdown, m->c_g, m->c_u}, {m->c_y})
                    : (get(m, KSH_GELU_MUL, {(int64_t)t * L.ffn}, {}, {}, &k_gelu) || enc(m, k_gelu, {m->c_g, m->c_u}, {m->c_ff}, n) ||
                       mm(L.dt_down, h, L.ffn, L.wdown, m->c_ff, m->c_y))))
            return 1;
        if (enc(m, k_add, {m->c_y, L.post_ffw_norm, m->c_x}, {m->c_x}, n)) return 1;
        if (c.ple_dim > 0) {
            // gemma_prim.rs:1558-1600: u = gelu(Wg x) * ctx_l; x = (x + rms(Wp u) * post_norm) * layer_scale
            ksh_kernel *k_gs = nullptr, *k_as = nullptr;
            if (mm(L.dt_inp_gate, c.ple_dim, h, L.inp_gate, m->c_x, m->c_ple_u) ||
                get(m, KSH_GELU_MUL, {(int64_t)t * c.ple_dim, c.ple_dim, pt}, {}, {}, &k_gs) ||
                enc_off(m, k_gs, {m->c_ple_u, m->c_ple_ctx}, {0, (size_t)l * c.ple_dim * 4}, {m->c_ple_u}, n) ||
                mm(L.dt_proj, h, c.ple_dim, L.proj, m->c_ple_u, m->c_y) ||
                get(m, KSH_RMSNORM, {h, 1, 1, t}, {}, {c.eps, L.layer_scale}, &k_as) ||
                enc(m, k_as, {m->c_y, L.post_norm, m->c_x}, {m->c_x}, n))
                return 1;
        }
    }
    m->pos += t;
    const int at = std::min(m->pos, c.max_seq - 1);
    hipLaunchKernelGGL(seek4_kernel, dim3(1), dim3(64), 0, st, (float *)ksh_buffer_device_ptr(m->meta_full),
                       (float *)ksh_buffer_device_ptr(m->meta_swa), at, (const float *)ksh_buffer_device_ptr(m->rope_full),
                       (float *)ksh_buffer_device_ptr(m->cur_full), c.hd_full, (const float *)ksh_buffer_device_ptr(m->rope_swa),
                       (float *)ksh_buffer_device_ptr(m->cur_swa), c.hd_swa, c.sliding_window);
    return hipGetLastError() == hipSuccess ? 0 : set_error("seek launch failed");
}

int make_rope(ksh_gemma4 *m, int hd, float theta, int angles, ksh_buf **table, ksh_buf **cur, std::vector<float> &row0)
{
    const int half = hd / 2, max_seq = m->c.max_seq;
    angles = std::min(angles, half);
    std::vector<float> tab((size_t)max_seq * hd);
    for (int pos = 0; pos < max_seq; pos++)
        for (int i = 0; i < half; i++) {
            float cs = 1.0f, sn = 0.0f;
            if (i < angles) {
                const float freq = (float)(1.0 / std::pow((double)theta, (double)(2 * i) / (double)hd));
                const float ang = (float)pos * freq;
                cs = std::cos(ang);
                sn = std::sin(ang);
            }
            tab[(size_t)pos * hd + i] = cs;
            tab[(size_t)pos * hd + half + i] = sn;
        }
    if (ksh_buffer_alloc(m->ctx, tab.size() * 4, tab.data(), table)) return 1;
    m->bufs.owned.push_back(*table);
    row0.assign(tab.begin(), tab.begin() + hd);
    return alloc(m, (size_t)hd * 4, cur);
}

int plan_layer(ksh_gemma4 *m, int l)
{
    const ksh_gemma4_cfg &c = m->c;
    const ksh_gemma4_layer &L = m->layers[l];
    LayerPlan &P = m->plan[l];
    const int64_t h = c.hidden;
    P.swa = L.is_swa != 0;
    P.hd = P.swa ? c.hd_swa : c.hd_full;
    P.qd = c.n_q * P.hd;
    P.kvd = c.n_kv * P.hd;
    P.owns = l < c.n_layers - c.shared_kv_layers;
    P.src = l;
    if (!P.owns) {
        // kv_source, crates/ksearch_gemma/src/lib.rs:151-162
        P.src = 0;
        for (int i = l - 1; i >= 0; i--)
            if (i < c.n_layers - c.shared_kv_layers && (m->layers[i].is_swa != 0) == P.swa) { P.src = i; break; }
        if ((m->layers[P.src].is_swa != 0) != P.swa)
            return set_error("layer %d reuses the cache of layer %d, which has another head dim", l, P.src);
    }
    {
        // every buffer the layer's launches will bind
        const ksh_buf *need[] = {L.wq, L.wo, L.wgate, L.wup, L.wdown, L.attn_norm, L.q_norm, L.post_attn_norm, L.ffn_norm, L.post_ffw_norm};
        for (const ksh_buf *b : need)
            if (!b) return set_error("layer %d: a weight or norm buffer is missing", l);
        if (P.owns && (!L.wk || !L.wv || !L.k_norm)) return set_error("layer %d owns its KV cache and needs k / v weights and the key norm", l);
        if (c.ple_dim > 0 && (!L.inp_gate || !L.proj || !L.post_norm)) return set_error("layer %d: per-layer-embedding weights are missing", l);
    }
    const int dts[] = {L.dt_q, L.dt_o, L.dt_gate, L.dt_up, L.dt_down};
    for (int dt : dts)
        if (!packed_ok(dt)) return set_error("layer %d: weight dtype %d is not built (Q4_K and Q6_K are)", l, dt);
    if (P.owns && (!packed_ok(L.dt_k) || !packed_ok(L.dt_v))) return set_error("layer %d: k/v weight dtype is not built", l);
    if (L.ffn <= 0 || L.ffn % 256) return set_error("layer %d: ffn=%d is not a positive multiple of 256", l, L.ffn);

    P.fused_qkv = P.owns && L.dt_q == KSH_Q4K && L.dt_k == KSH_Q4K && L.dt_v == KSH_Q4K;
    // the add that this layer's first GEMV folds in closes the previous layer: with per-layer embeddings it carries
    // that layer's output scale
    const float prev_scale = c.ple_dim > 0 && l > 0 ? m->layers[l - 1].layer_scale : 0.f;
    if (P.fused_qkv) {
        for (int r = 0; r < 2; r++)
            if (get(m, KSH_RMSNORM_MATVEC_QKV, {P.qd, P.kvd, h, r}, {KSH_Q4K, KSH_F32}, {c.eps, r ? prev_scale : 0.f}, &P.qkv[r])) return 1;
    } else {
        for (int r = 0; r < 2; r++)
            if (get(m, KSH_RMSNORM_MATVEC, {P.qd, h, r}, {L.dt_q, KSH_F32}, {c.eps, r ? prev_scale : 0.f}, &P.qkv[r])) return 1;
        if (P.owns && (get(m, KSH_RMSNORM_MATVEC, {P.kvd, h, 0}, {L.dt_k, KSH_F32}, {c.eps}, &P.kmat[0]) ||
                       get(m, KSH_RMSNORM_MATVEC, {P.kvd, h, 0}, {L.dt_v, KSH_F32}, {c.eps}, &P.kmat[1])))
            return 1;
    }
    // attention: one launch where the fused kind is built for the shape (appending, or reading another layer's cache)
    const bool short_form = P.swa && c.sliding_window <= kShortWindow && L.dt_o == KSH_Q4K && P.qd <= 2048 && (P.hd & (P.hd - 1)) == 0;
    P.attend = sdpa_lanes_supports(c.n_q, c.n_kv, P.hd);
    P.attend_parts = P.attend && short_form;
    if (P.attend) {
        if (get(m, KSH_ATTEND_DECODE,
                {c.n_q, c.n_kv, P.hd, c.max_seq, P.attend_parts ? kShortPartitions : kAttendPartitions, P.attend_parts ? 1 : 0, 1, P.owns ? 0 : 1},
                {KSH_Q40, KSH_F32}, {c.eps, c.attn_scale}, &P.k_attend))
            return 1;
    } else {
        if (P.owns ? get(m, KSH_RMSNORM_PER_HEAD_QKV_Q40, {c.n_q, c.n_kv, P.hd, c.max_seq}, {}, {c.eps}, &P.head)
                   : get(m, KSH_RMSNORM_PER_HEAD, {c.n_q, P.hd, 2, c.max_seq}, {}, {c.eps}, &P.head))
            return 1;
        if (get(m, KSH_SDPA_SLOTS, {c.n_q, c.n_kv, P.hd, c.max_seq, 1, kAttendPartitions}, {KSH_Q40, KSH_F32}, {c.attn_scale}, &P.sdpa)) return 1;
    }
    if (P.attend_parts ? get(m, KSH_ATTN_MERGE_MATVEC, {h, c.n_q, P.hd, kShortPartitions}, {KSH_Q4K, KSH_F32}, {}, &P.oproj)
                       : get(m, KSH_MATVEC, {h, P.qd}, {L.dt_o, KSH_F32}, {}, &P.oproj))
        return 1;
    P.fused_gate_up = L.dt_gate == KSH_Q4K && L.dt_up == KSH_Q4K;
    if (P.fused_gate_up) {
        if (get(m, KSH_RMSNORM_MATVEC_GATE_UP_GELU, {L.ffn, h, 1}, {KSH_Q4K, KSH_F32}, {c.eps}, &P.gate_up)) return 1;
    } else {
        if (get(m, KSH_RMSNORM_MATVEC, {L.ffn, h, 1}, {L.dt_gate, KSH_F32}, {c.eps}, &P.gate) ||
            get(m, KSH_RMSNORM_MATVEC, {L.ffn, h, 0}, {L.dt_up, KSH_F32}, {c.eps}, &P.up) ||
            get(m, KSH_GELU_MUL, {L.ffn}, {}, {}, &P.gelu))
            return 1;
    }
    if (get(m, KSH_MATVEC, {h, L.ffn}, {L.dt_down, KSH_F32}, {}, &P.down)) return 1;
    if (c.ple_dim > 0) {
        if (L.dt_inp_gate != KSH_Q4K || !packed_ok(L.dt_proj))
            return set_error("layer %d: per-layer-embedding weights must be Q4_K (gate) and Q4_K or Q6_K (projection)", l);
        if (get(m, KSH_MATVEC_GELU_MUL, {c.ple_dim, h, 1}, {KSH_Q4K, KSH_F32}, {c.eps}, &P.ple_gate) ||
            get(m, KSH_MATVEC, {h, c.ple_dim}, {L.dt_proj, KSH_F32}, {}, &P.ple_proj))
            return 1;
    }
    return 0;
}

// Schedule searches at model load (Eng::warm_matvec_plans, gemma_prim.rs:254-290), one per distinct GEMV shape of the
// layers: the candidates run as the decode step runs them, a graph of one launch per layer of that shape over the
// layer's own weights.  Kinds whose partition count the loop fixes (attention) keep their defaults.
void warm_plans(ksh_gemma4 *m)
{
    const ksh_gemma4_cfg &c = m->c;
    struct Group {
        ksh_kernel_desc d;
        std::vector<ksh_buf *> in, out;
        int n_in = 0, n_out = 0, n_sets = 0;
    };
    std::map<std::vector<int64_t>, Group> groups;
    auto add = [&](int kind, std::initializer_list<int64_t> dims, int wdt, std::initializer_list<ksh_buf *> in, std::initializer_list<ksh_buf *> out) {
        std::vector<int64_t> key{kind, wdt};
        key.insert(key.end(), dims.begin(), dims.end());
        Group &g = groups[key];
        if (!g.n_sets) {
            memset(&g.d, 0, sizeof(g.d));
            g.d.kind = kind;
            int i = 0;
            for (int64_t v : dims) g.d.dims[i++] = v;
            g.d.dtypes[0] = wdt;
            g.d.dtypes[1] = KSH_F32;
            g.d.params[0] = c.eps;
            g.n_in = (int)in.size();
            g.n_out = (int)out.size();
        }
        g.in.insert(g.in.end(), in.begin(), in.end());
        g.out.insert(g.out.end(), out.begin(), out.end());
        g.n_sets++;
    };
    const int64_t h = c.hidden;
    for (int l = 0; l < c.n_layers; l++) {
        const ksh_gemma4_layer &L = m->layers[l];
        const int hd = L.is_swa ? c.hd_swa : c.hd_full;
        const int64_t qd = (int64_t)c.n_q * hd, kvd = (int64_t)c.n_kv * hd;
        const bool owns = l < c.n_layers - c.shared_kv_layers;
        // (a layer that plan_layer is about to refuse takes no part)
        if (!L.wq || !L.wo || !L.wgate || !L.wup || !L.wdown || !L.attn_norm || !L.post_attn_norm || !L.ffn_norm || !L.post_ffw_norm ||
            L.ffn <= 0 || L.ffn % 256 || (owns && (!L.wk || !L.wv)))
            continue;
        if (owns && L.dt_q == KSH_Q4K && L.dt_k == KSH_Q4K && L.dt_v == KSH_Q4K)
            add(KSH_RMSNORM_MATVEC_QKV, {qd, kvd, h, 1}, KSH_Q4K, {L.wq, L.wk, L.wv, m->y, L.attn_norm, L.post_ffw_norm, m->x}, {m->tq, m->tk, m->tv, m->xb});
        else
            add(KSH_RMSNORM_MATVEC, {qd, h, 1}, L.dt_q, {L.wq, m->y, L.attn_norm, L.post_ffw_norm, m->x}, {m->tq, m->xb});
        add(KSH_MATVEC, {h, qd}, L.dt_o, {L.wo, m->to}, {m->y});
        if (L.dt_gate == KSH_Q4K && L.dt_up == KSH_Q4K)
            add(KSH_RMSNORM_MATVEC_GATE_UP_GELU, {L.ffn, h, 1}, KSH_Q4K, {L.wgate, L.wup, m->y, L.ffn_norm, L.post_attn_norm, m->x}, {m->ff, m->xb});
        add(KSH_MATVEC, {h, L.ffn}, L.dt_down, {L.wdown, m->ff}, {m->y});
    }
    for (auto &kv : groups) {
        Group &g = kv.second;
        ksh_sched best;
        double ms = 0.0;
        int cached = 0;
        (void)ksh_beam_search_chain(m->ctx, &g.d, g.n_sets, g.in.data(), g.n_in, g.out.data(), g.n_out, 4, 0, &best, &ms, &cached);
    }
    (void)ksh_synchronize(m->ctx);
}

// puts the graphs in use back where they belong (they are tied to the cache buffers they were captured with)
void stash_graphs(ksh_gemma4 *m)
{
    ksh_gemma4::SlotGraphs &g = m->bound_slot >= 0 ? m->slot_graphs[(size_t)m->bound_slot] : m->own_graphs;
    g.body = m->g_body;
    g.full = m->g_full;
    g.span = m->g_span;
    m->g_body = m->g_full = m->g_span = nullptr;
}

}  // namespace

extern "C" {

int ksh_gemma4_create(ksh_ctx *ctx, const ksh_gemma4_cfg *cfg, const ksh_gemma4_layer *layers, const ksh_gemma4_globals *globals,
                      ksh_gemma4 **out)
{
    if (!ctx || !cfg || !layers || !globals || !out || !globals->token_embd || !globals->output_norm)
        return set_error("ksh_gemma4_create: bad arguments");
    *out = nullptr;
    const ksh_gemma4_cfg &c = *cfg;
    if (c.n_layers <= 0 || c.hidden <= 0 || c.hidden % 256 || c.n_q <= 0 || c.n_kv <= 0 || c.n_q % c.n_kv || c.hd_swa <= 0 ||
        c.hd_full <= 0 || c.vocab <= 0 || c.vocab >= (1 << 24) || c.max_seq <= 0 || c.sliding_window <= 0 ||
        c.shared_kv_layers < 0 || c.shared_kv_layers >= c.n_layers || c.ple_dim < 0 || c.ple_dim % 256)
        return set_error("ksh_gemma4_create: invalid configuration");
    if (c.ple_dim > 0 && (!globals->ple_embd || !globals->ple_model_proj || !globals->ple_proj_norm))
        return set_error("ksh_gemma4_create: per-layer embeddings need their table, projection and norm");
    auto mp = std::make_unique<ksh_gemma4>();
    ksh_gemma4 *m = mp.get();
    m->ctx = ctx;
    m->c = c;
    m->g = *globals;
    m->layers.assign(layers, layers + c.n_layers);
    m->plan.resize(c.n_layers);
    if (const char *e = std::getenv("KSEARCH_ROUND_GRAPH")) m->round_graph = e[0] != '0';
    m->prof.on = std::getenv("KSEARCH_PROFILE") != nullptr;
    const int max_hd = std::max(c.hd_swa, c.hd_full);
    int max_ff = 0;
    for (const ksh_gemma4_layer &L : m->layers) max_ff = std::max(max_ff, (int)L.ffn);
    const size_t h4 = (size_t)c.hidden * 4, pt = (size_t)c.n_layers * c.ple_dim;
    if (alloc(m, h4, &m->x) || alloc(m, h4, &m->xb) || alloc(m, h4, &m->y) || alloc(m, (size_t)c.n_q * max_hd * 4, &m->tq) ||
        alloc(m, (size_t)c.n_kv * max_hd * 4, &m->tk) || alloc(m, (size_t)c.n_kv * max_hd * 4, &m->tv) ||
        alloc(m, (size_t)c.n_q * max_hd * 4, &m->to) || alloc(m, (size_t)max_ff * 4, &m->ff) || alloc(m, (size_t)max_ff * 4, &m->ff2) ||
        alloc(m, (size_t)c.vocab * 4, &m->logits) || alloc(m, 16, &m->tok) || alloc(m, 16, &m->meta_full) || alloc(m, 16, &m->meta_swa) ||
        alloc(m, (size_t)c.max_seq * 4, &m->history) || alloc(m, pt * 4, &m->ple_tok) || alloc(m, pt * 4, &m->ple_tmp) ||
        alloc(m, pt * 4, &m->ple_ctx) || alloc(m, (size_t)c.ple_dim * 4, &m->ple_u) ||
        alloc(m, (size_t)c.n_q * kAttendPartitions * (max_hd + 2) * 4, &m->attn_tmp))
        return 1;
    if (make_rope(m, c.hd_swa, c.rope_theta_swa, c.hd_swa / 2, &m->rope_swa, &m->cur_swa, m->rope0_swa) ||
        make_rope(m, c.hd_full, c.rope_theta_full, (int)((float)c.hd_full * c.partial_rotary) / 2, &m->rope_full, &m->cur_full,
                  m->rope0_full))
        return 1;
    m->kv_k.assign(c.n_layers, nullptr);
    m->kv_v.assign(c.n_layers, nullptr);
    if (!getenv("KSEARCH_SKIP_BEAM")) warm_plans(m);
    for (int l = 0; l < c.n_layers; l++) {
        if (plan_layer(m, l)) return 1;
        if (!m->plan[l].owns) continue;
        const size_t kvb = (size_t)c.max_seq * c.n_kv * (m->plan[l].hd / 32) * 18;   // gemma_prim.rs:199-207
        if (alloc(m, kvb, &m->kv_k[l]) || alloc(m, kvb, &m->kv_v[l])) return 1;
    }
    const int de = globals->dt_embd;
    if (!packed_ok(de)) return set_error("ksh_gemma4_create: embedding dtype %d is not built (Q4_K and Q6_K are)", de);
    int lm_dt = de;
    if (de == KSH_Q6K && (c.hidden == 1536 || c.hidden == 2048 || c.hidden == 4096)) {
        // the LM head streams the whole table every token: it gets a copy with each row's fields grouped
        ksh_kernel *rp = nullptr;
        if (alloc(m, (size_t)c.vocab * (((size_t)(c.hidden / 256) * 210 + 15) / 16 * 16), &m->embd_rows) ||
            get(m, KSH_REPACK_ROWS, {c.vocab, c.hidden}, {KSH_Q6K, KSH_Q6K_ROWS}, {}, &rp))
            return 1;
        int n = 0;
        if (enc(m, rp, {m->g.token_embd}, {m->embd_rows}, n) || ksh_synchronize(ctx)) return 1;
        lm_dt = KSH_Q6K_ROWS;
    }
    if (get(m, KSH_COPY_SCALE_INDEXED, {c.hidden, c.vocab}, {de}, {std::sqrt((float)c.hidden)}, &m->k_embed) ||
        get(m, KSH_RMSNORM_MATVEC, {c.vocab, c.hidden, 0}, {lm_dt, KSH_F32}, {c.eps}, &m->k_lm_head[0]) ||
        get(m, KSH_RMSNORM_MATVEC, {c.vocab, c.hidden, 1}, {lm_dt, KSH_F32}, {c.eps, c.ple_dim > 0 ? m->layers[c.n_layers - 1].layer_scale : 0.f},
            &m->k_lm_head[1]) ||
        get(m, KSH_SOFTCAP_ARGMAX, {c.vocab}, {}, {c.softcap}, &m->k_argmax))
        return 1;
    if (c.ple_dim > 0) {
        if (!packed_ok(globals->dt_ple_proj)) return set_error("ksh_gemma4_create: per-layer projection dtype %d is not built", globals->dt_ple_proj);
        if (get(m, KSH_COPY_SCALE_INDEXED, {(int64_t)pt, c.vocab}, {globals->dt_ple}, {std::sqrt((float)c.ple_dim)}, &m->k_ple_gather) ||
            get(m, KSH_MATVEC, {(int64_t)pt, c.hidden}, {globals->dt_ple_proj, KSH_F32}, {}, &m->k_ple_proj) ||
            get(m, KSH_RMSNORM_PER_HEAD, {c.n_layers, c.ple_dim, 0}, {}, {c.eps}, &m->k_ple_norm) ||
            get(m, KSH_ADD_SCALE, {(int64_t)pt}, {}, {0.70710678118654752440f}, &m->k_ple_mix))
            return 1;
    }
    if (ksh_gemma4_reset(m)) return 1;
    *out = mp.release();
    return 0;
}

void ksh_gemma4_destroy(ksh_gemma4 *m)
{
    if (!m) return;
    ksh_synchronize(m->ctx);
    stash_graphs(m);
    ksh_graph_destroy(m->own_graphs.body);
    ksh_graph_destroy(m->own_graphs.full);
    ksh_graph_destroy(m->own_graphs.span);
    for (auto &g : m->slot_graphs) { ksh_graph_destroy(g.body); ksh_graph_destroy(g.full); ksh_graph_destroy(g.span); }
    for (ksh_graph *g : m->round_graphs) ksh_graph_destroy(g);
    delete m;
}

int ksh_gemma4_reset(ksh_gemma4 *m)
{
    if (!m) return set_error("ksh_gemma4_reset: null model");
    if (ksh_synchronize(m->ctx)) return 1;
    const float full[4] = {1.f, 0.f, 0.f, 0.f};                              // tlen, start, window, pos
    const float swa[4] = {1.f, 0.f, (float)m->c.sliding_window, 0.f};
    if (ksh_buffer_write(m->ctx, m->meta_full, 0, full, 16, 1) || ksh_buffer_write(m->ctx, m->meta_swa, 0, swa, 16, 1) ||
        ksh_buffer_write(m->ctx, m->cur_full, 0, m->rope0_full.data(), m->rope0_full.size() * 4, 1) ||
        ksh_buffer_write(m->ctx, m->cur_swa, 0, m->rope0_swa.data(), m->rope0_swa.size() * 4, 1))
        return 1;
    m->pos = 0;
    return 0;
}

int ksh_gemma4_forward_token(ksh_gemma4 *m, uint32_t token, int want_logits, int use_graph, uint32_t *next_id)
{
    if (!m) return set_error("ksh_gemma4_forward_token: null model");
    if (token >= (uint32_t)m->c.vocab) return set_error("token id %u is outside the vocabulary", token);
    if (write_token(m, token)) return 1;
    if (run_token(m, want_logits != 0, use_graph != 0)) return 1;
    if (next_id && want_logits) {
        float f = 0.f;
        if (ksh_buffer_read(m->ctx, m->tok, 0, &f, 4, 1)) return 1;
        *next_id = (uint32_t)f;
    }
    return 0;
}

int ksh_gemma4_generate(ksh_gemma4 *m, const uint32_t *prompt, int n_prompt, int n_new, int use_graph, uint32_t *out_ids,
                        double *prefill_ms, double *decode_ms)
{
    if (!m || !prompt || n_prompt < 1 || n_new < 0 || (n_new && !out_ids)) return set_error("ksh_gemma4_generate: bad arguments");
    if (m->pos + n_prompt - 1 + n_new > m->c.max_seq) return set_error("max_seq exceeded");
    for (int i = 0; i < n_prompt; i++)
        if (prompt[i] >= (uint32_t)m->c.vocab) return set_error("token id %u is outside the vocabulary", prompt[i]);
    using clk = std::chrono::steady_clock;
    const auto t0 = clk::now();
    // all prompt tokens but the last go through without logits (gemma_prim.rs:1670-1675)
    if (ksh_gemma4_prefill_chunk(m, prompt, n_prompt - 1, use_graph)) return 1;   // (use_graph & 2: token by token)
    if (write_token(m, prompt[n_prompt - 1])) return 1;
    if (ksh_synchronize(m->ctx)) return 1;
    const auto t1 = clk::now();
    const int first = m->pos;
    for (int i = 0; i < n_new;) {
        if ((use_graph & 1) && n_new - i >= kSpan && !m->prof.on && m->pos + kSpan <= m->c.max_seq) {
            if (run_span(m)) return 1;
            i += kSpan;
        } else {
            if (run_token(m, true, (use_graph & 1) != 0)) return 1;
            i += 1;
        }
    }
    if (ksh_synchronize(m->ctx)) return 1;
    const auto t2 = clk::now();
    if (prefill_ms) *prefill_ms = std::chrono::duration<double, std::milli>(t1 - t0).count();
    if (decode_ms) *decode_ms = std::chrono::duration<double, std::milli>(t2 - t1).count();
    if (n_new) {
        std::vector<float> ids((size_t)n_new);
        if (ksh_buffer_read(m->ctx, m->history, (size_t)first * 4, ids.data(), (size_t)n_new * 4, 1)) return 1;
        for (int i = 0; i < n_new; i++) out_ids[i] = (uint32_t)ids[i];
    }
    return 0;
}

// generate_timed's stop rule (gemma_prim.rs:1683-1710): the id of step i-1 is read while step i runs, and an id
// from `eos` ends the run with that id as the last output (the step already in flight is discarded; the model's
// position has moved past it, as the reference's has).
int ksh_gemma4_generate_until(ksh_gemma4 *m, const uint32_t *prompt, int n_prompt, int n_new, const uint32_t *eos, int n_eos,
                              int use_graph, uint32_t *out_ids, int *n_out, double *prefill_ms, double *decode_ms)
{
    if (!m || !prompt || n_prompt < 1 || n_new < 0 || (n_new && !out_ids) || !n_out || n_eos < 0 || (n_eos && !eos))
        return set_error("ksh_gemma4_generate_until: bad arguments");
    *n_out = 0;
    if (m->pos + n_prompt - 1 + n_new > m->c.max_seq) return set_error("max_seq exceeded");
    for (int i = 0; i < n_prompt; i++)
        if (prompt[i] >= (uint32_t)m->c.vocab) return set_error("token id %u is outside the vocabulary", prompt[i]);
    using clk = std::chrono::steady_clock;
    const auto t0 = clk::now();
    if (ksh_gemma4_prefill_chunk(m, prompt, n_prompt - 1, use_graph)) return 1;   // (use_graph & 2: token by token)
    if (write_token(m, prompt[n_prompt - 1])) return 1;
    if (ksh_synchronize(m->ctx)) return 1;
    const auto t1 = clk::now();
    const int first = m->pos;
    auto is_eos = [&](uint32_t id) {
        for (int e = 0; e < n_eos; e++)
            if (eos[e] == id) return true;
        return false;
    };
    auto take = [&](int step) -> int {   // the id step `step` produced (that step has completed)
        float f = 0.f;
        if (ksh_buffer_read(m->ctx, m->history, (size_t)(first + step) * 4, &f, 4, 0)) return -1;
        out_ids[(*n_out)++] = (uint32_t)f;
        return is_eos((uint32_t)f) ? 1 : 0;
    };
    bool stopped = false;
    for (int i = 0; i < n_new && !stopped; i++) {
        if (run_token(m, true, (use_graph & 1) != 0) || ksh_flush_async(m->ctx)) return 1;
        if (i > 0) {
            if (ksh_wait_inflight_at_most(m->ctx, 1)) return 1;
            const int r = take(i - 1);
            if (r < 0) return 1;
            stopped = r == 1;
        }
    }
    if (ksh_synchronize(m->ctx)) return 1;
    if (!stopped && n_new > 0 && take(n_new - 1) < 0) return 1;
    const auto t2 = clk::now();
    if (prefill_ms) *prefill_ms = std::chrono::duration<double, std::milli>(t1 - t0).count();
    if (decode_ms) *decode_ms = std::chrono::duration<double, std::milli>(t2 - t1).count();
    return 0;
}

// GemmaPrimModel::decode_token_sampled (gemma_prim.rs:1614-1635): one token with logits; below a temperature of 1e-6
// the device argmax decides, else the logits are read back and the host sampler draws (gemma_prim.rs:1239-1261).
int ksh_gemma4_decode_token_sampled(ksh_gemma4 *m, uint32_t token, float temperature, float min_p, uint32_t seed, int use_graph,
                                    uint32_t *next_id)
{
    if (!m || !next_id) return set_error("ksh_gemma4_decode_token_sampled: bad arguments");
    if (temperature < 1e-6f) return ksh_gemma4_forward_token(m, token, 1, use_graph, next_id);
    if (ksh_gemma4_forward_token(m, token, 1, use_graph, nullptr)) return 1;
    std::vector<float> &logits = m->host_logits;   // (kept: a megabyte at the real vocabulary, every token)
    logits.resize((size_t)m->c.vocab);
    if (ksh_buffer_read(m->ctx, m->logits, 0, logits.data(), logits.size() * 4, 1)) return 1;
    return ksh_sample_softcap_min_p(logits.data(), logits.size(), m->c.softcap, temperature, min_p, seed, next_id);
}

// GemmaPrimModel::prefill_chunk (gemma_prim.rs:1305-1315): the tokens go through without logits, then one
// synchronisation.  Chunks of up to 256 tokens go through the batched layer pass (forward_prefill_chunk,
// gemma_prim.rs:1317-1607), a chunk of one token through the decode step; use_graph & 2 feeds every token through
// the decode step instead (use_graph & 1: from its captured graph).
int ksh_gemma4_prefill_chunk(ksh_gemma4 *m, const uint32_t *tokens, int n, int use_graph)
{
    if (!m || (n > 0 && !tokens) || n < 0) return set_error("ksh_gemma4_prefill_chunk: bad arguments");
    if (m->pos + n > m->c.max_seq) return set_error("max_seq exceeded");
    for (int i = 0; i < n; i++)
        if (tokens[i] >= (uint32_t)m->c.vocab) return set_error("token id %u is outside the vocabulary", tokens[i]);
    for (int i = 0; i < n;) {
        const int t = (use_graph & 2) ? 1 : std::min(kChunk4, n - i);
        if (t == 1) {
            if (write_token(m, tokens[i])) return 1;
            if (run_token(m, false, (use_graph & 1) != 0)) return 1;
        } else if (forward_prefill_chunk4(m, tokens + i, t)) {
            return 1;
        }
        i += t;
    }
    return ksh_synchronize(m->ctx);
}

}  // extern "C"

// One decode step for several sequences at once: the reference's decode round (crates/ksearch_cli/src/scheduler.rs:
// 163-231) runs decode_token_sampled once per decoding request, each a full pass over the weights; here the round's
// tokens go through the layers together as a matrix of n rows (the batched layer pass of forward_prefill_chunk,
// gemma_prim.rs:1317-1607, with one position, one attended range and one KV slot per row), so the weights are read
// once per round.  Row i appends to and attends the caches of pool slot slots[i] at that slot's sequence length.
namespace {
constexpr int kRoundMax = 16;         // the attention launch shares its partitions among up to 16 entries by length
constexpr int kRoundPartitions = 16;
constexpr int kRoundStride = 16;      // floats per field of the table: ids | slots | full-attention records | sliding-window records

int pool_fits(const ksh_gemma4 *m, const ksh_kvpool *pool, int *max_batch, int *pool_hd)
{
    const ksh_gemma4_cfg &c = m->c;
    int max_seq, n_kv_layers, n_kv;
    if (ksh_kvpool_dims(pool, max_batch, &max_seq, &n_kv_layers, pool_hd, &n_kv)) return 1;
    const int owners = c.n_layers - c.shared_kv_layers;
    if (n_kv_layers != owners) return set_error("kv layer mismatch: model=%d pool=%d", owners, n_kv_layers);
    if (max_seq != c.max_seq || n_kv != c.n_kv || *pool_hd < std::max(c.hd_swa, c.hd_full))
        return set_error("KvPool(max_seq=%d, n_kv=%d, hd=%d) does not fit the model (max_seq=%d, n_kv=%d, hd=%d)", max_seq, n_kv, *pool_hd,
                         c.max_seq, c.n_kv, std::max(c.hd_swa, c.hd_full));
    return 0;
}

int encode_round4(ksh_gemma4 *m, ksh_kvpool *pool, int t, int max_batch, int pool_hd);

void drop_round_graphs(ksh_gemma4 *m)
{
    for (ksh_graph *&g : m->round_graphs) { ksh_graph_destroy(g); g = nullptr; }
    for (bool &b : m->round_bound) b = false;
    m->round_pool = nullptr;
    m->round_pool_uid = 0;
}

int forward_decode_round4(ksh_gemma4 *m, ksh_kvpool *pool, const int32_t *slots, const uint32_t *tokens, int t)
{
    const ksh_gemma4_cfg &c = m->c;
    int max_batch = 0, pool_hd = 0;
    if (pool_fits(m, pool, &max_batch, &pool_hd)) return 1;
    if (chunk_buffers4(m)) return 1;
    int64_t widest = std::max<int64_t>(c.hidden, c.ple_dim);
    for (int l = 0; l < c.n_layers; l++) widest = std::max<int64_t>(widest, std::max<int64_t>(m->layers[l].ffn, m->plan[l].qd));
    widest = (widest + 255) / 256 * 256;
    if (!m->r_tab && (alloc(m, (size_t)kRoundStride * 10 * 4, &m->r_tab) || alloc(m, (size_t)kRoundMax * c.vocab * 4, &m->r_logits) ||
                      alloc(m, (size_t)kRoundMax * 4, &m->r_next) || alloc(m, (size_t)(64 * widest + 2048 * (widest / 256)), &m->r_xp) ||
                      alloc(m, (size_t)(64 * widest + 2048 * (widest / 256)), &m->r_xp2)))
        return 1;
    float tab[kRoundStride * 10] = {};
    for (int i = 0; i < t; i++) {
        const int pos = ksh_kvpool_seq_len(pool, slots[i]);
        const int kv_len = pos + 1, start = kv_len > c.sliding_window ? kv_len - c.sliding_window : 0;
        tab[i] = (float)tokens[i];
        tab[kRoundStride + i] = (float)slots[i];
        float *full = tab + 2 * kRoundStride + 4 * i, *swa = tab + 6 * kRoundStride + 4 * i;
        full[0] = (float)kv_len; full[3] = (float)pos;
        swa[0] = (float)(kv_len - start); swa[1] = (float)start; swa[2] = (float)c.sliding_window; swa[3] = (float)pos;
    }
    if (ksh_synchronize(m->ctx)) return 1;   // the table may still be read by the previous round
    if (ksh_buffer_write(m->ctx, m->r_tab, 0, tab, sizeof(tab), 1)) return 1;
    m->r_count = t;
    // The launches of a round depend on its width alone (tokens, slots and positions are in the table): one graph per
    // width, captured at its second round (the first binds the width's kernels, which allocates, and a capture must
    // not).  KSEARCH_ROUND_GRAPH=0 (read when the model is created) launches every round kernel by kernel.
    if (!m->round_graph) return encode_round4(m, pool, t, max_batch, pool_hd);
    // the graphs hold the pool's device addresses: another pool, or a new pool at a destroyed one's address, drops them
    if (m->round_pool != pool || m->round_pool_uid != ksh_kvpool_uid(pool)) {
        drop_round_graphs(m);
        m->round_pool = pool;
        m->round_pool_uid = ksh_kvpool_uid(pool);
    }
    ksh_graph *&g = m->round_graphs[t];
    if (!g && !m->round_bound[t]) {
        // bound only once every kernel of the width has been looked up: a capture must find nothing left to allocate
        if (encode_round4(m, pool, t, max_batch, pool_hd)) return 1;
        m->round_bound[t] = true;
        return 0;
    }
    if (!g) {
        if (ksh_graph_begin(m->ctx)) return 1;
        if (encode_round4(m, pool, t, max_batch, pool_hd)) {
            ksh_graph *dead = nullptr;
            ksh_graph_end(m->ctx, &dead);
            ksh_graph_destroy(dead);
            return 1;
        }
        if (ksh_graph_end(m->ctx, &g)) return 1;
    }
    return ksh_graph_launch(m->ctx, g);
}

// every launch of a round of t sequences, behind the table's upload
int encode_round4(ksh_gemma4 *m, ksh_kvpool *pool, int t, int max_batch, int pool_hd)
{
    const ksh_gemma4_cfg &c = m->c;
    const size_t o_ids = 0, o_slots = (size_t)kRoundStride * 4, o_full = (size_t)2 * kRoundStride * 4, o_swa = (size_t)6 * kRoundStride * 4;
    const int64_t h = c.hidden, tp = 32, pt = (int64_t)c.n_layers * c.ple_dim;
    const size_t slot_stride = (size_t)c.max_seq * c.n_kv * (pool_hd / 32) * 18;
    int n = 0;
    ksh_kernel *k = nullptr, *k_norm = nullptr, *k_add = nullptr, *k_add_then = nullptr;
    auto run = [&](ksh_kernel *kk, std::initializer_list<ksh_buf *> in, std::initializer_list<size_t> in_off, std::initializer_list<ksh_buf *> out,
                   std::initializer_list<size_t> out_off) {
        ksh_buf *ib[kMaxIn], *ob[kMaxOut];
        uint64_t io[kMaxIn] = {}, oo[kMaxOut] = {};
        int ni = 0, no = 0, j = 0;
        for (ksh_buf *b : in) ib[ni++] = b;
        for (size_t o : in_off) io[j++] = o;
        j = 0;
        for (ksh_buf *b : out) ob[no++] = b;
        for (size_t o : out_off) oo[j++] = o;
        n += 1;
        return ksh_encode(m->ctx, kk, ib, io, ni, ob, oo, no);
    };
    // Q4_K matrices: the small-batch GEMM on exact integer codes (the GEMV's accuracy).  Q6_K matrices (files loaded
    // with their Q6_K tensors kept): the GEMM's f16 operand rounds sc * q above 2048 to even integers, 2^-11 on those
    // weights, which a step that must equal the serial one to 1e-3 through every layer cannot afford: row by row
    // through the GEMV instead.
    auto mm = [&](int dt, int64_t rows, int64_t cols, ksh_buf *w, ksh_buf *x, ksh_buf *y) -> int {
        ksh_kernel *kk = nullptr;
        if (dt != KSH_Q6K) return get(m, KSH_MATVEC_BATCH, {rows, cols, tp}, {dt, KSH_F32, KSH_F32}, {}, &kk) || enc(m, kk, {w, x}, {y}, n);
        if (get(m, KSH_MATVEC, {rows, cols}, {dt, KSH_F32}, {}, &kk)) return 1;
        for (int i = 0; i < t; i++)
            if (run(kk, {w, x}, {0, (size_t)i * cols * 4}, {y}, {(size_t)i * rows * 4})) return 1;
        return 0;
    };
    // Q4_K matrices of a round share one prepared operand per distinct input (KSH_ROUND_PREP) and go several to a
    // launch where they read the same rows (q | k | v; gate | up with the GELU in the epilogue)
    auto prep = [&](int64_t cols, ksh_buf *x) -> int {
        ksh_kernel *kk = nullptr;
        return get(m, KSH_ROUND_PREP, {cols, t}, {KSH_F32}, {}, &kk) || enc(m, kk, {x}, {m->r_xp}, n);
    };
    // (a norm whose only readers are such GEMMs writes the operand itself)
    auto prep_norm = [&](int64_t cols, ksh_buf *x, ksh_buf *w) -> int {
        ksh_kernel *kk = nullptr;
        return get(m, KSH_ROUND_PREP, {cols, t, 1}, {KSH_F32}, {c.eps}, &kk) || enc(m, kk, {x, w}, {m->r_xp}, n);
    };
    auto mm1 = [&](int dt, int64_t rows, int64_t cols, ksh_buf *w, ksh_buf *x, ksh_buf *y) -> int {
        ksh_kernel *kk = nullptr;
        if (dt != KSH_Q4K) return mm(dt, rows, cols, w, x, y);
        return prep(cols, x) || get(m, KSH_MATVEC_ROUND, {rows, cols, t, 0, 0, 0}, {KSH_Q4K}, {}, &kk) || enc(m, kk, {w, m->r_xp}, {y}, n);
    };
    if (get(m, KSH_COPY_SCALE_INDEXED, {h, c.vocab, t}, {m->g.dt_embd}, {std::sqrt((float)c.hidden)}, &k) ||
        run(k, {m->g.token_embd, m->r_tab}, {0, o_ids}, {m->c_x}, {0}))
        return 1;
    if (c.ple_dim > 0) {
        ksh_kernel *kg = nullptr, *kn = nullptr, *kmix = nullptr;
        if (get(m, KSH_COPY_SCALE_INDEXED, {pt, c.vocab, t}, {m->g.dt_ple}, {std::sqrt((float)c.ple_dim)}, &kg) ||
            run(kg, {m->g.ple_embd, m->r_tab}, {0, o_ids}, {m->c_ple_tok}, {0}) ||
            mm1(m->g.dt_ple_proj, pt, h, m->g.ple_model_proj, m->c_x, m->c_ple_tmp) ||
            get(m, KSH_RMSNORM_PER_HEAD, {(int64_t)t * c.n_layers, c.ple_dim, 0}, {}, {c.eps}, &kn) ||
            enc(m, kn, {m->c_ple_tmp, m->g.ple_proj_norm}, {m->c_ple_ctx}, n) ||
            get(m, KSH_ADD_SCALE, {(int64_t)t * pt}, {}, {0.70710678118654752440f}, &kmix) ||
            enc(m, kmix, {m->c_ple_ctx, m->c_ple_tok}, {m->c_ple_ctx}, n))
            return 1;
    }
    if (get(m, KSH_RMSNORM, {h, 0, 0, t}, {}, {c.eps}, &k_norm) || get(m, KSH_RMSNORM, {h, 1, 0, t}, {}, {c.eps}, &k_add) ||
        get(m, KSH_RMSNORM_ADD_THEN_RMSNORM, {h, t}, {}, {c.eps}, &k_add_then))
        return 1;
    ksh_buf *lm_w = m->embd_rows ? m->embd_rows : m->g.token_embd;
    // the LM head once for all rows where the table is kept row-grouped (the matrix cores on exact codes, the int8
    // scales applied in f32); row by row through the GEMV otherwise
    const bool lm_batched = m->embd_rows && h % 256 == 0 && h <= 2048;
    // a layer whose q | k | v read the prepared operand of the normed residual stream
    auto qkv_prepared = [&](int l) {
        const ksh_gemma4_layer &L = m->layers[l];
        return L.dt_q == KSH_Q4K && (!m->plan[l].owns || (L.dt_k == KSH_Q4K && L.dt_v == KSH_Q4K));
    };
    // The norm that closes a layer also writes the operand the next layer's q | k | v (or the LM head) start from, where
    // those take one: x_new = [scale *] (res + norm(y) * w), xp = norm(x_new) * w_next (KSH_ROUND_PREP mode 2).
    bool xp_ready = false;
    auto close_layer = [&](int l, ksh_buf *w, float scale, ksh_kernel *k_plain) -> int {
        const bool last = l + 1 == c.n_layers;
        const bool fuse = h <= 8192 && (last ? lm_batched : qkv_prepared(l + 1));
        if (!fuse) return enc(m, k_plain, {m->c_y, w, m->c_x}, {m->c_x}, n);
        ksh_kernel *kk = nullptr;
        if (get(m, KSH_ROUND_PREP, {h, t, 2}, {KSH_F32}, {c.eps, scale}, &kk) ||
            enc(m, kk, {m->c_y, w, m->c_x, last ? m->g.output_norm : m->layers[l + 1].attn_norm}, {m->r_xp, m->c_x}, n))
            return 1;
        xp_ready = true;
        return 0;
    };
    for (int l = 0; l < c.n_layers; l++) {
        const ksh_gemma4_layer &L = m->layers[l];
        const LayerPlan &P = m->plan[l];
        ksh_buf *rope_tab = P.swa ? m->rope_swa : m->rope_full;
        ksh_buf *kc = ksh_kvpool_layer_k(pool, P.src), *vc = ksh_kvpool_layer_v(pool, P.src);
        const size_t o_meta = P.swa ? o_swa : o_full;
        ksh_kernel *k_head = nullptr, *k_sdpa = nullptr, *k_gelu = nullptr;
        if (!sdpa_lanes_supports(c.n_q, c.n_kv, P.hd))
            return set_error("ksh_gemma4_decode_round: attention over several slots is built for heads of 128 / 256 / 512 with up to 8 q heads per kv head");
        const bool qkv_q4k = qkv_prepared(l);
        if (!qkv_q4k && enc(m, k_norm, {m->c_x, L.attn_norm}, {m->c_x2}, n)) return 1;
        if (qkv_q4k) {
            ksh_kernel *kq = nullptr;
            if (!xp_ready && prep_norm(h, m->c_x, L.attn_norm)) return 1;   // (ready: the previous layer's last norm wrote it)
            xp_ready = false;
            if (P.owns ? (get(m, KSH_MATVEC_ROUND, {P.qd, h, t, P.kvd, P.kvd, 0}, {KSH_Q4K}, {}, &kq) ||
                          enc(m, kq, {L.wq, m->r_xp, L.wk, L.wv}, {m->c_q, m->c_k, m->c_v}, n))
                       : (get(m, KSH_MATVEC_ROUND, {P.qd, h, t, 0, 0, 0}, {KSH_Q4K}, {}, &kq) || enc(m, kq, {L.wq, m->r_xp}, {m->c_q}, n)))
                return 1;
        } else if (mm(L.dt_q, P.qd, h, L.wq, m->c_x2, m->c_q) ||
                   (P.owns && (mm(L.dt_k, P.kvd, h, L.wk, m->c_x2, m->c_k) || mm(L.dt_v, P.kvd, h, L.wv, m->c_x2, m->c_v)))) {
            return 1;
        }
        if (P.owns) {
            if (get(m, KSH_RMSNORM_PER_HEAD_QKV_Q40, {c.n_q, c.n_kv, P.hd, c.max_seq, t, max_batch, (int64_t)slot_stride}, {}, {c.eps}, &k_head) ||
                run(k_head, {m->c_q, L.q_norm, rope_tab, m->c_k, L.k_norm, m->c_v, m->r_tab, m->r_tab}, {0, 0, 0, 0, 0, 0, o_meta, o_slots},
                    {m->c_q, kc, vc}, {0, 0, 0}))
                return 1;
        } else {
            if (get(m, KSH_RMSNORM_PER_HEAD, {(int64_t)t * c.n_q, P.hd, 2, c.max_seq, c.n_q, 1}, {}, {c.eps}, &k_head) ||
                run(k_head, {m->c_q, L.q_norm, rope_tab, m->r_tab}, {0, 0, 0, o_meta}, {m->c_q}, {0}))
                return 1;
        }
        // the attention's merge writes the o projection's prepared operand itself where that projection takes one
        const bool o_chain = t >= 2 && L.dt_o == KSH_Q4K && P.qd % 256 == 0;
        if (get(m, KSH_SDPA_SLOTS, {c.n_q, c.n_kv, P.hd, c.max_seq, t, kRoundPartitions, max_batch, (int64_t)slot_stride}, {KSH_Q40, KSH_F32},
                {c.attn_scale, o_chain ? 1.0f : 0.0f}, &k_sdpa) ||
            run(k_sdpa, {m->c_q, kc, vc, m->r_tab, m->r_tab}, {0, 0, 0, o_meta, o_slots}, {m->c_tmp, o_chain ? m->r_xp : m->c_o}, {0, 0}))
            return 1;
        if (o_chain) {
            ksh_kernel *k_o = nullptr;
            if (get(m, KSH_MATVEC_ROUND, {h, P.qd, t, 0, 0, 0}, {KSH_Q4K}, {}, &k_o) || enc(m, k_o, {L.wo, m->r_xp}, {m->c_y}, n)) return 1;
        } else if (mm1(L.dt_o, h, P.qd, L.wo, m->c_o, m->c_y)) {
            return 1;
        }
        const bool gu_q4k = L.dt_gate == KSH_Q4K && L.dt_up == KSH_Q4K && h <= 8192;
        const bool ple_q4k = c.ple_dim > 0 && L.dt_inp_gate == KSH_Q4K && L.dt_proj == KSH_Q4K && c.ple_dim % 256 == 0 && h <= 2048;
        // a down projection whose columns are split leaves its slices' partial sums (in c_g) to the closing norm where
        // that norm is the kind that adds them up
        const int down_slices = (int)((L.ffn / 256 + 7) / 8);
        const bool down_unfolded = L.dt_down == KSH_Q4K && ple_q4k && down_slices > 1;
        bool down_done = false;
        if (!gu_q4k && enc(m, k_add_then, {m->c_y, L.post_attn_norm, m->c_x, L.ffn_norm}, {m->c_x, m->c_x2}, n)) return 1;
        if (gu_q4k) {
            ksh_kernel *k_gu = nullptr, *k_pn = nullptr;
            if (get(m, KSH_ROUND_PREP, {h, t, 2}, {KSH_F32}, {c.eps}, &k_pn) ||
                enc(m, k_pn, {m->c_y, L.post_attn_norm, m->c_x, L.ffn_norm}, {m->r_xp, m->c_x}, n))
                return 1;
            // gelu(gate) * up leaves as the prepared operand of the down projection where that one takes it
            const bool chain = L.dt_down == KSH_Q4K && L.ffn % 256 == 0 && h <= 2048;
            if (get(m, KSH_MATVEC_ROUND, {L.ffn, h, t, 0, 0, 1, chain ? 1 : 0}, {KSH_Q4K}, {}, &k_gu) ||
                enc(m, k_gu, {L.wgate, m->r_xp, L.wup}, {chain ? m->r_xp2 : m->c_ff}, n))
                return 1;
            if (chain) {
                ksh_kernel *k_dn = nullptr;
                if (get(m, KSH_MATVEC_ROUND, {h, L.ffn, t, 0, 0, 0, down_unfolded ? 2 : 0}, {KSH_Q4K}, {}, &k_dn) ||
                    enc(m, k_dn, {L.wdown, m->r_xp2}, {down_unfolded ? m->c_g : m->c_y}, n))
                    return 1;
                down_done = true;
            }
        } else if (mm(L.dt_gate, L.ffn, h, L.wgate, m->c_x2, m->c_g) || mm(L.dt_up, L.ffn, h, L.wup, m->c_x2, m->c_u) ||
                   get(m, KSH_GELU_MUL, {(int64_t)t * L.ffn}, {}, {}, &k_gelu) || enc(m, k_gelu, {m->c_g, m->c_u}, {m->c_ff}, n)) {
            return 1;
        }
        if (!down_done && down_unfolded) {
            ksh_kernel *k_dn = nullptr;
            if (prep(L.ffn, m->c_ff) || get(m, KSH_MATVEC_ROUND, {h, L.ffn, t, 0, 0, 0, 2}, {KSH_Q4K}, {}, &k_dn) || enc(m, k_dn, {L.wdown, m->r_xp}, {m->c_g}, n))
                return 1;
            down_done = true;
        }
        if (!down_done && mm1(L.dt_down, h, L.ffn, L.wdown, m->c_ff, m->c_y)) return 1;
        // the feed-forward block's closing norm + add
        if (c.ple_dim == 0) {
            if (close_layer(l, L.post_ffw_norm, 0.f, k_add)) return 1;
        } else if (ple_q4k) {
            // ... which also prepares the new residual stream for the per-layer-embedding gate (mode 3); the gate's
            // gelu(W x) * context leaves as the projection's prepared operand
            ksh_kernel *k_pa = nullptr, *k_pg = nullptr, *k_pp = nullptr, *k_as = nullptr;
            if (get(m, KSH_ROUND_PREP, {h, t, 3, down_unfolded ? down_slices : 0}, {KSH_F32}, {c.eps}, &k_pa) ||
                enc(m, k_pa, {down_unfolded ? m->c_g : m->c_y, L.post_ffw_norm, m->c_x}, {m->r_xp, m->c_x}, n) ||
                get(m, KSH_MATVEC_ROUND, {c.ple_dim, h, t, 0, 0, 0, 1, pt}, {KSH_Q4K}, {}, &k_pg) ||
                enc_off(m, k_pg, {L.inp_gate, m->r_xp, m->c_ple_ctx}, {0, 0, (size_t)l * c.ple_dim * 4}, {m->r_xp2}, n) ||
                get(m, KSH_MATVEC_ROUND, {h, c.ple_dim, t, 0, 0, 0}, {KSH_Q4K}, {}, &k_pp) || enc(m, k_pp, {L.proj, m->r_xp2}, {m->c_y}, n) ||
                get(m, KSH_RMSNORM, {h, 1, 1, t}, {}, {c.eps, L.layer_scale}, &k_as))
                return 1;
            if (L.layer_scale != 0.f ? close_layer(l, L.post_norm, L.layer_scale, k_as) : enc(m, k_as, {m->c_y, L.post_norm, m->c_x}, {m->c_x}, n)) return 1;
        } else {
            ksh_kernel *k_gs = nullptr, *k_as = nullptr;
            if (enc(m, k_add, {m->c_y, L.post_ffw_norm, m->c_x}, {m->c_x}, n) ||
                mm1(L.dt_inp_gate, c.ple_dim, h, L.inp_gate, m->c_x, m->c_ple_u) ||
                get(m, KSH_GELU_MUL, {(int64_t)t * c.ple_dim, c.ple_dim, pt}, {}, {}, &k_gs) ||
                enc_off(m, k_gs, {m->c_ple_u, m->c_ple_ctx}, {0, (size_t)l * c.ple_dim * 4}, {m->c_ple_u}, n) ||
                mm1(L.dt_proj, h, c.ple_dim, L.proj, m->c_ple_u, m->c_y) ||
                get(m, KSH_RMSNORM, {h, 1, 1, t}, {}, {c.eps, L.layer_scale}, &k_as))
                return 1;
            if (L.layer_scale != 0.f ? close_layer(l, L.post_norm, L.layer_scale, k_as) : enc(m, k_as, {m->c_y, L.post_norm, m->c_x}, {m->c_x}, n)) return 1;
        }
    }
    // logits and the greedy id of every row: the output norm rides in the LM head's prologue, as in the decode step
    if (lm_batched) {
        ksh_kernel *k_lm = nullptr;
        if ((!xp_ready && prep_norm(h, m->c_x, m->g.output_norm)) ||
            get(m, KSH_MATVEC_ROUND, {c.vocab, h, t, 0, 0, 0}, {KSH_Q6K_ROWS}, {}, &k_lm) || enc(m, k_lm, {lm_w, m->r_xp}, {m->r_logits}, n))
            return 1;
    }
    for (int i = 0; i < t && !lm_batched; i++)
        if (run(m->k_lm_head[0], {lm_w, m->c_x, m->g.output_norm}, {0, (size_t)i * h * 4, 0}, {m->r_logits}, {(size_t)i * c.vocab * 4})) return 1;
    ksh_kernel *k_arg = nullptr;
    if (get(m, KSH_SOFTCAP_ARGMAX, {c.vocab, t}, {}, {c.softcap}, &k_arg) || enc(m, k_arg, {m->r_logits}, {m->r_next}, n)) return 1;
    return 0;
}
}  // namespace

extern "C" {

int ksh_gemma4_decode_round(ksh_gemma4 *m, ksh_kvpool *pool, const int32_t *slots, const uint32_t *tokens, int n, const float *temperature,
                            const float *min_p, const uint32_t *seed, uint32_t *next_ids)
{
    if (!m || !pool || !slots || !tokens || !next_ids) return set_error("ksh_gemma4_decode_round: bad arguments");
    if (n < 1 || n > kRoundMax) return set_error("ksh_gemma4_decode_round: %d sequences (1 to %d at once)", n, kRoundMax);
    if (temperature && (!min_p || !seed)) return set_error("ksh_gemma4_decode_round: sampling needs min_p and seed");
    int max_batch = 0, pool_hd = 0;
    if (pool_fits(m, pool, &max_batch, &pool_hd)) return 1;
    for (int i = 0; i < n; i++) {
        if (slots[i] < 0 || slots[i] >= max_batch) return set_error("bad SlotId");
        if (ksh_kvpool_occupied(pool, slots[i]) != 1) return set_error("slot not occupied");
        for (int j = 0; j < i; j++)
            if (slots[j] == slots[i]) return set_error("ksh_gemma4_decode_round: slot %d is named twice", slots[i]);
        if (ksh_kvpool_seq_len(pool, slots[i]) >= m->c.max_seq) return set_error("max_seq exceeded");   // gemma_prim.rs:882-884
        if (tokens[i] >= (uint32_t)m->c.vocab) return set_error("token id %u is outside the vocabulary", tokens[i]);
    }
    if (forward_decode_round4(m, pool, slots, tokens, n)) return 1;
    float ids[kRoundMax];
    if (ksh_buffer_read(m->ctx, m->r_next, 0, ids, (size_t)n * 4, 1)) return 1;
    for (int i = 0; i < n; i++) {
        next_ids[i] = (uint32_t)ids[i];
        if (temperature && temperature[i] >= 1e-6f) {   // decode_token_sampled's other branch (gemma_prim.rs:1614-1635)
            std::vector<float> &logits = m->host_logits;
            logits.resize((size_t)m->c.vocab);
            if (ksh_buffer_read(m->ctx, m->r_logits, (size_t)i * m->c.vocab * 4, logits.data(), logits.size() * 4, 0) ||
                ksh_sample_softcap_min_p(logits.data(), logits.size(), m->c.softcap, temperature[i], min_p[i], seed[i], &next_ids[i]))
                return 1;
        }
    }
    return 0;
}

ksh_buf *ksh_gemma4_round_logits(ksh_gemma4 *m) { return m ? m->r_logits : nullptr; }

}  // extern "C"

extern "C" {

// GemmaPrimModel::bind_slot (gemma_prim.rs:1277-1292): the model's K / V caches become the slot's and its position the
// slot's sequence length.  pool == NULL goes back to the model's own caches at position `slot` (0 after a reset).
int ksh_gemma4_bind_slot(ksh_gemma4 *m, ksh_kvpool *pool, int slot)
{
    if (!m) return set_error("ksh_gemma4_bind_slot: null model");
    const ksh_gemma4_cfg &c = m->c;
    const int owners = c.n_layers - c.shared_kv_layers;
    int pos = slot;
    if (pool) {
        int max_batch, max_seq, n_kv_layers, hd, n_kv;
        if (ksh_kvpool_dims(pool, &max_batch, &max_seq, &n_kv_layers, &hd, &n_kv)) return 1;
        if (n_kv_layers != owners) return set_error("kv layer mismatch: model=%d pool=%d", owners, n_kv_layers);
        if (max_seq != c.max_seq || n_kv != c.n_kv || hd < std::max(c.hd_swa, c.hd_full))
            return set_error("KvPool(max_seq=%d, n_kv=%d, hd=%d) does not fit the model (max_seq=%d, n_kv=%d, hd=%d)", max_seq, n_kv, hd,
                             c.max_seq, c.n_kv, std::max(c.hd_swa, c.hd_full));
        if (slot < 0 || slot >= max_batch) return set_error("bad SlotId");
        pos = ksh_kvpool_seq_len(pool, slot);
    }
    if (pos < 0 || pos > c.max_seq) return set_error("ksh_gemma4_bind_slot: position %d", pos);
    // the slot it is bound to already, at the position the model has reached by itself: the device-side state is
    // in place (a scheduler with one decoding request asks for this before every token)
    const bool same_pool = pool && pool == m->pool && ksh_kvpool_uid(pool) == m->pool_uid;
    if (same_pool && slot == m->bound_slot && pos == m->pos) return 0;
    stash_graphs(m);
    if (pool && !same_pool) {
        // graphs captured over another pool's buffers are of no use any more
        if (ksh_synchronize(m->ctx)) return 1;
        for (auto &g : m->slot_graphs) { ksh_graph_destroy(g.body); ksh_graph_destroy(g.full); ksh_graph_destroy(g.span); }
        int max_batch = 0;
        ksh_kvpool_dims(pool, &max_batch, nullptr, nullptr, nullptr, nullptr);
        m->slot_graphs.assign((size_t)max_batch, ksh_gemma4::SlotGraphs{});
        m->pool = pool;
        m->pool_uid = ksh_kvpool_uid(pool);
    }
    if (m->own_k.empty()) { m->own_k = m->kv_k; m->own_v = m->kv_v; }
    for (int l = 0; l < owners; l++) {
        m->kv_k[l] = pool ? ksh_kvpool_k(pool, slot, l) : m->own_k[l];
        m->kv_v[l] = pool ? ksh_kvpool_v(pool, slot, l) : m->own_v[l];
    }
    m->bound_slot = pool ? slot : -1;
    const ksh_gemma4::SlotGraphs &g = pool ? m->slot_graphs[(size_t)slot] : m->own_graphs;
    m->g_body = g.body;
    m->g_full = g.full;
    m->g_span = g.span;
    m->pos = pos;
    // the device-side position, attended ranges and rope rows, ordered behind whatever is still running
    const int at = std::min(pos, c.max_seq - 1);
    hipLaunchKernelGGL(seek4_kernel, dim3(1), dim3(64), 0, (hipStream_t)ksh_stream(m->ctx), (float *)ksh_buffer_device_ptr(m->meta_full),
                       (float *)ksh_buffer_device_ptr(m->meta_swa), at, (const float *)ksh_buffer_device_ptr(m->rope_full),
                       (float *)ksh_buffer_device_ptr(m->cur_full), c.hd_full, (const float *)ksh_buffer_device_ptr(m->rope_swa),
                       (float *)ksh_buffer_device_ptr(m->cur_swa), c.hd_swa, c.sliding_window);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, "seek launch");
}

ksh_buf *ksh_gemma4_logits(ksh_gemma4 *m) { return m ? m->logits : nullptr; }
ksh_buf *ksh_gemma4_hidden(ksh_gemma4 *m) { return m ? (m->hidden ? m->hidden : m->x) : nullptr; }
int ksh_gemma4_kv_source(ksh_gemma4 *m, int layer) { return (!m || layer < 0 || layer >= m->c.n_layers) ? -1 : m->plan[layer].src; }
ksh_buf *ksh_gemma4_kv(ksh_gemma4 *m, int layer, int which)
{
    if (!m || layer < 0 || layer >= m->c.n_layers) return nullptr;
    const int src = m->plan[layer].src;
    return which ? m->kv_v[src] : m->kv_k[src];
}
int ksh_gemma4_pos(ksh_gemma4 *m) { return m ? m->pos : -1; }
int ksh_gemma4_launches_per_token(ksh_gemma4 *m) { return m ? m->launches_full : -1; }
int ksh_gemma4_config(ksh_gemma4 *m, ksh_gemma4_cfg *cfg)
{
    if (!m || !cfg) return set_error("ksh_gemma4_config: bad arguments");
    *cfg = m->c;
    return 0;
}
void ksh_gemma4_adopt(ksh_gemma4 *m, ksh_buf *b)
{
    if (m && b) m->bufs.owned.push_back(b);
}

}  // extern "C"
