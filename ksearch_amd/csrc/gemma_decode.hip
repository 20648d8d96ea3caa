// Greedy decode loop for the synthetic Gemma-4-E2B shape, above the C ABI.
//
// Mirrors GemmaPrimModel::forward_token and generate_timed
// (crates/ksearch_gemma/src/gemma_prim.rs:881-1275, 1658-1768) without the
// parts that shape lacks (per-layer embeddings, sliding-window layers, shared
// KV).  The reference's per-layer sequence is
//   rmsnorm -> fused QKV GEMV -> per-head RMS + RoPE + Q4_0 KV append ->
//   split-KV attention -> o-proj GEMV -> add-then-rmsnorm ->
//   fused gate||up + GELU GEMV -> down GEMV -> rmsnorm_add
// then the output norm, the Q6_K LM head and the soft-capped argmax.  Here every
// normalisation rides in the GEMV that consumes it (RmsNormMatvecQkv,
// RmsNormMatvecGateUpGelu with the preceding residual add folded in), so a
// layer is
//   [add+]rmsnorm+QKV -> per-head RMS + RoPE + KV append + attention + merge
//   (AttendDecode) -> o-proj -> add+rmsnorm+gate||up+GELU -> down
// and the layer-closing rmsnorm_add becomes the prologue of the next layer's
// QKV (or of the output norm).  The residual stream ping-pongs between two
// buffers because the fused prologue may not overwrite the vector that other
// workgroups of the same launch still read.
//
// What differs from the reference's host loop, and why:
//   - the position lives in a device buffer (meta = {tlen, start, window,
//     pos}) that a one-thread kernel advances at the end of each token, so the
//     whole token is one HIP graph that is replayed unchanged; the reference
//     re-encodes every token with host-side offsets (:941, :976, :1017);
//   - the next token id never leaves the device: argmax writes it where the
//     embedding gather of the next step reads it (the reference ping-pongs two
//     buffers for the same purpose, :1237-1241) and a history array keeps
//     every id for one read-back at the end.
#include <chrono>
#include <cmath>
#include <cstdlib>
#include <algorithm>
#include <memory>
#include <functional>
#include <vector>

#include "ksh_device.hpp"
#include "ksh_internal.hpp"
#include "section_timer.hpp"

namespace {

// end of token: remember the id, advance position and attended length, and put the next position's row of the
// rope table where the attention launches read it (they then fetch it without first waiting for the position)
__global__ void advance_kernel(float *meta, const float *tok, float *history, int max_hist, const float *rope,
                               float *rope_cur, int hd)
{
    const int pos = (int)meta[3];
    __syncthreads();   // every thread has read the position before thread 0 moves it
    if (pos + 1 < max_hist)
        for (int i = threadIdx.x; i < hd; i += blockDim.x) rope_cur[i] = rope[(size_t)(pos + 1) * hd + i];
    if (threadIdx.x == 0) {
        if (history && pos < max_hist) history[pos] = tok[0];
        meta[3] = (float)(pos + 1);
        meta[0] = (float)(pos + 2);   // the next token attends rows [0, pos+1]
    }
}

// the id the next embedding gather reads; a kernel rather than a copy so that
// it is ordered behind the previous token's work on the same stream
__global__ void set_token_kernel(float *tok, float value)
{
    if (threadIdx.x == 0 && blockIdx.x == 0) tok[0] = value;
}

// start of a prompt chunk: the record the batched attention reads ({rows the first token attends, -, window}),
// derived on the stream from the device-side position
__global__ void chunk_begin_kernel(const float *meta, float *bmeta, int max_seq)
{
    if (threadIdx.x == 0) {
        bmeta[0] = meta[3] + 1.0f;
        bmeta[1] = 0.f;
        bmeta[2] = (float)max_seq;
        bmeta[3] = 0.f;
    }
}

// end of a prompt chunk: position and attended length move on by n tokens, and the new position's rope row is put
// where the decode step's attention reads it
__global__ void chunk_end_kernel(float *meta, int n, int max_seq, const float *rope, float *rope_cur, int hd)
{
    const int pos = (int)meta[3] + n;
    __syncthreads();
    if (pos < max_seq)
        for (int i = threadIdx.x; i < hd; i += blockDim.x) rope_cur[i] = rope[(size_t)pos * hd + i];
    if (threadIdx.x == 0) {
        meta[3] = (float)pos;
        meta[0] = (float)(pos + 1);
    }
}

struct Bufs {
    std::vector<ksh_buf *> owned;
    ~Bufs()
    {
        for (ksh_buf *b : owned) ksh_buffer_release(b);
    }
};

}  // namespace

struct ksh_gemma {
    ksh_ctx *ctx = nullptr;
    ksh_gemma_cfg c{};
    std::vector<ksh_gemma_layer> layers;
    ksh_buf *embd = nullptr, *output_norm = nullptr;
    ksh_buf *embd_rows = nullptr;   // the LM head's copy of the embedding table, rows regrouped by field (KSH_Q6K_ROWS)
    Bufs bufs;
    ksh_buf *x = nullptr, *xb = nullptr, *y = nullptr, *x2 = nullptr, *hidden = nullptr, *tq = nullptr, *tk = nullptr, *tv = nullptr, *to = nullptr, *ff = nullptr,
            *logits = nullptr, *tok = nullptr, *meta = nullptr, *rope = nullptr, *rope_cur = nullptr, *attn_tmp = nullptr,
            *history = nullptr;
    std::vector<ksh_buf *> kv_k, kv_v;
    ksh_kernel *k_embed = nullptr, *k_qkv_first = nullptr, *k_qkv = nullptr, *k_head = nullptr, *k_sdpa = nullptr, *k_attend = nullptr,
               *k_attend_parts = nullptr, *k_oproj_merge = nullptr,   // short contexts: the o-projection merges the partitions
               *k_oproj = nullptr, *k_add_then = nullptr, *k_gate_up = nullptr, *k_down = nullptr,
               *k_lm_head = nullptr, *k_argmax = nullptr;
    ksh_graph *g_body[2] = {nullptr, nullptr}, *g_full[2] = {nullptr, nullptr};   // [1]: the short-context form
    ksh_graph *g_span[2] = {nullptr, nullptr};   // kSpan decode steps with logits in one graph (generate's loop)
    int pos = 0;
    int launches_full = 0;
    int nwg = 16;
    int sdpa_launches = 2;
    int short_context = 0;   // positions below this use the short-context graph
    std::vector<float> rope0;   // row 0 of the rope table, for reset
    // prompt chunks (allocated at the first chunk): [kChunk, .] activations of the batched layer pass
    ksh_buf *c_tok = nullptr, *c_x = nullptr, *c_x2 = nullptr, *c_y = nullptr, *c_q = nullptr, *c_k = nullptr, *c_v = nullptr, *c_o = nullptr,
            *c_g = nullptr, *c_u = nullptr, *c_ff = nullptr, *c_tmp = nullptr, *c_meta = nullptr,
            *c_po = nullptr, *c_pg = nullptr, *c_pd = nullptr;   // unfolded partial sums of the o, gate | up and down projections
    int c_nwg = 0;
    ksh::SectionTimer prof;   // KSEARCH_PROFILE (read when the model is created): per-section times of every decode step
};

namespace {

using namespace ksh;

int alloc(ksh_gemma *m, size_t bytes, ksh_buf **out)
{
    if (ksh_buffer_alloc(m->ctx, bytes, nullptr, out)) return 1;
    m->bufs.owned.push_back(*out);
    return 0;
}

int get(ksh_gemma *m, int kind, std::initializer_list<int64_t> dims, std::initializer_list<int> dtypes,
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

int enc(ksh_gemma *m, ksh_kernel *k, std::initializer_list<ksh_buf *> in, std::initializer_list<ksh_buf *> out,
        int &count)
{
    ksh_buf *ib[kMaxIn], *ob[kMaxOut];
    int ni = 0, no = 0;
    for (ksh_buf *b : in) ib[ni++] = b;
    for (ksh_buf *b : out) ob[no++] = b;
    count += 1;
    return ksh_encode(m->ctx, k, ib, nullptr, ni, ob, nullptr, no);
}

// Schedule search at load (Eng::warm_matvec_plans + beam_matvec, gemma_prim.rs:254-290, ksearch_kernels/src/lib.rs:
// 1985-2080): the kind is timed on the model's own buffers over its candidate schedules and the winner saved in the
// plan cache, where the kernel lookups that follow find it; a plan that is there already is taken as it is.  A kind
// without a schedule space, or whose search fails, keeps the library default.
// One schedule search at model load: the candidate kernels run as the decode step runs them, a graph of one launch
// per layer over that layer's own weights (Eng::warm_matvec_plans, gemma_prim.rs:254-290).
void warm_plan(ksh_gemma *m, int kind, std::initializer_list<int64_t> dims, std::initializer_list<int> dtypes,
               std::initializer_list<float> params, int n_sets, const std::function<void(int, std::vector<ksh_buf *> &, std::vector<ksh_buf *> &)> &set)
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
    std::vector<ksh_buf *> in, out, one_in, one_out;
    for (int l = 0; l < n_sets; l++) {
        one_in.clear();
        one_out.clear();
        set(l, one_in, one_out);
        in.insert(in.end(), one_in.begin(), one_in.end());
        out.insert(out.end(), one_out.begin(), one_out.end());
    }
    ksh_sched best;
    double ms = 0.0;
    int cached = 0;
    (void)ksh_beam_search_chain(m->ctx, &d, n_sets, in.data(), (int)one_in.size(), out.data(), (int)one_out.size(), 4, 0, &best, &ms, &cached);
}

// Up to this many cached positions the attention launch leaves its (then 8) partitions unmerged and the
// o-projection folds them in its prologue: 0.8 us per layer less at 320 positions, 1.5 us more at 1500,
// where 16 partitions and the merge inside the attention launch win.
// (KSEARCH_SHORT_CONTEXT overrides the limit when the model is built; 0 switches the short form off.)
constexpr int kShortContext = 640;
constexpr int kShortPartitions = 8;

// one token: embedding gather -> layers (-> logits -> argmax) -> advance
int encode_token(ksh_gemma *m, bool want_logits, bool short_ctx, int &launches)
{
    const ksh_gemma_cfg &c = m->c;
    launches = 0;
    ksh_buf *cur = m->x, *other = m->xb;   // the residual stream and its next home
    // (the token's embedding row is in m->x already: write_token put it there, or the previous step's last launch)
    for (int l = 0; l < c.n_layers; l++) {
        const ksh_gemma_layer &L = m->layers[l];
        if (l == 0) {
            if (enc(m, m->k_qkv_first, {L.wq, L.wk, L.wv, cur, L.attn_norm}, {m->tq, m->tk, m->tv}, launches)) return 1;
        } else {
            // closes layer l-1 (x += rmsnorm(down, post_ffw_norm), gemma_prim.rs:1150-1160) and opens layer l
            if (enc(m, m->k_qkv, {L.wq, L.wk, L.wv, m->y, L.attn_norm, m->layers[l - 1].post_ffw_norm, cur},
                    {m->tq, m->tk, m->tv, other}, launches))
                return 1;
            std::swap(cur, other);
        }
        if (short_ctx) {
            if (enc(m, m->k_attend_parts, {m->tq, L.q_norm, m->rope_cur, m->tk, L.k_norm, m->tv, m->meta},
                    {m->kv_k[l], m->kv_v[l], m->attn_tmp}, launches))
                return 1;
        } else if (m->k_attend) {
            if (enc(m, m->k_attend, {m->tq, L.q_norm, m->rope_cur, m->tk, L.k_norm, m->tv, m->meta},
                    {m->kv_k[l], m->kv_v[l], m->attn_tmp, m->to}, launches))
                return 1;
        } else {
            if (enc(m, m->k_head, {m->tq, L.q_norm, m->rope, m->tk, L.k_norm, m->tv, m->meta},
                    {m->tq, m->kv_k[l], m->kv_v[l]}, launches))
                return 1;
            if (enc(m, m->k_sdpa, {m->tq, m->kv_k[l], m->kv_v[l], m->meta}, {m->attn_tmp, m->to}, launches)) return 1;
            if (m->sdpa_launches == 2) launches += 1;   // partials, then the merge
        }
        if (short_ctx ? enc(m, m->k_oproj_merge, {L.wo, m->attn_tmp}, {m->y}, launches) : enc(m, m->k_oproj, {L.wo, m->to}, {m->y}, launches))
            return 1;
        m->prof.mark(SectionTimer::kAttn);
        if (enc(m, m->k_gate_up, {L.wgate, L.wup, m->y, L.ffn_norm, L.post_attn_norm, cur}, {m->ff, other}, launches)) return 1;
        std::swap(cur, other);
        if (enc(m, m->k_down, {L.wdown, m->ff}, {m->y}, launches)) return 1;
        m->prof.mark(SectionTimer::kMlp);
    }
    if (want_logits) {
        // the last layer's rmsnorm_add and the output norm ride in the LM head's prologue
        // (the final residual stream goes to a buffer of its own: the step's last launch writes the next token's
        // embedding into m->x)
        if (enc(m, m->k_lm_head, {m->embd_rows ? m->embd_rows : m->embd, m->y, m->output_norm, m->layers[c.n_layers - 1].post_ffw_norm, cur},
                {m->logits, m->x2}, launches))
            return 1;
        m->hidden = m->x2;
        // argmax (first pass), then one launch for its second pass, the position update and the next embedding row
        DecodeTail t{};
        t.tok = (float *)ksh_buffer_device_ptr(m->tok);
        t.history = (float *)ksh_buffer_device_ptr(m->history);
        t.max_hist = c.max_seq;
        t.meta = (float *)ksh_buffer_device_ptr(m->meta);
        t.rope = (const float *)ksh_buffer_device_ptr(m->rope);
        t.rope_cur = (float *)ksh_buffer_device_ptr(m->rope_cur);
        t.hd = c.hd;
        t.embd = (const uint8_t *)ksh_buffer_device_ptr(m->embd);
        t.dtype = KSH_Q6K;
        t.n_rows = c.vocab;
        t.n = c.hidden;
        t.scale = std::sqrt((float)c.hidden);   // gemma_prim.rs:683
        t.x_out = (float *)ksh_buffer_device_ptr(m->x);
        if (launch_decode_tail(*m->k_argmax, (const float *)ksh_buffer_device_ptr(m->logits), t, (hipStream_t)ksh_stream(m->ctx))) return 1;
        ctx_mark_pending(m->ctx);
        launches += 2;
        m->prof.mark(SectionTimer::kLogits);
        return 0;
    }
    hipStream_t st = (hipStream_t)ksh_stream(m->ctx);
    hipLaunchKernelGGL(advance_kernel, dim3(1), dim3(64), 0, st, (float *)ksh_buffer_device_ptr(m->meta),
                       (const float *)ksh_buffer_device_ptr(m->tok),
                       want_logits ? (float *)ksh_buffer_device_ptr(m->history) : nullptr, c.max_seq,
                       (const float *)ksh_buffer_device_ptr(m->rope), (float *)ksh_buffer_device_ptr(m->rope_cur), c.hd);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e, "advance launch");
    launches += 1;
    m->prof.mark(SectionTimer::kLogits);
    return 0;
}

int run_token(ksh_gemma *m, bool want_logits, bool use_graph)
{
    if (m->pos >= m->c.max_seq) return set_error("max_seq exceeded");   // gemma_prim.rs:882-884
    int n = 0;
    const bool short_ctx = m->k_attend_parts && m->pos < m->short_context;
    if (m->prof.on) {
        // gemma_prim.rs:885: with KSEARCH_PROFILE every step is timed section by section (launched kernel by kernel)
        m->prof.begin((hipStream_t)ksh_stream(m->ctx));
        if (encode_token(m, want_logits, short_ctx, n)) return 1;
        m->prof.report(want_logits ? "decode" : "prefill", m->pos);
    } else if (!use_graph) {
        if (encode_token(m, want_logits, short_ctx, n)) return 1;
    } else {
        ksh_graph *&g = want_logits ? m->g_full[short_ctx] : m->g_body[short_ctx];
        if (!g) {
            if (ksh_synchronize(m->ctx)) return 1;
            if (ksh_graph_begin(m->ctx)) return 1;
            if (encode_token(m, want_logits, short_ctx, n)) {
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

// Several decode steps as one graph launch.  Position, attended length, rope row and the token itself live on the
// device and are advanced by the step's last kernel, so a token's graph repeated kSpan times is kSpan tokens; the
// generate loop uses it while the whole span stays on one form of the attention step.
constexpr int kSpan = 8;

int run_span(ksh_gemma *m)
{
    const bool short_ctx = m->k_attend_parts && m->pos < m->short_context;
    ksh_graph *&g = m->g_span[short_ctx];
    if (!g) {
        int n = 0;
        if (ksh_synchronize(m->ctx)) return 1;
        if (ksh_graph_begin(m->ctx)) return 1;
        for (int i = 0; i < kSpan; i++) {
            if (encode_token(m, true, short_ctx, n)) {
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

bool span_fits(const ksh_gemma *m, int remaining)
{
    if (remaining < kSpan || m->prof.on || m->pos + kSpan > m->c.max_seq) return false;
    if (!m->k_attend_parts) return true;
    return (m->pos < m->short_context) == (m->pos + kSpan - 1 < m->short_context);
}

// prefill_chunk's chunk length (gemma_prim.rs:16)
constexpr int kChunk = 1024;
constexpr int kPartsRows = 4;          // room for the unfolded partial sums of a hidden-wide projection: this many chunks of rows
constexpr int kChunkPartitions = 8;   // partitions per token of the batched attention (its tmp buffer is sized for this)

int chunk_buffers(ksh_gemma *m)
{
    if (m->c_tok) return 0;
    const ksh_gemma_cfg &c = m->c;
    const size_t T = kChunk, qd = (size_t)c.n_q * c.hd, kvd = (size_t)c.n_kv * c.hd;
    m->c_nwg = kChunkPartitions;
    return alloc(m, T * 4, &m->c_tok) || alloc(m, T * c.hidden * 4, &m->c_x) || alloc(m, T * c.hidden * 4, &m->c_x2) ||
           alloc(m, T * c.hidden * 4, &m->c_y) || alloc(m, T * qd * 4, &m->c_q) || alloc(m, T * kvd * 4, &m->c_k) ||
           alloc(m, T * kvd * 4, &m->c_v) || alloc(m, T * qd * 4, &m->c_o) || alloc(m, T * c.ffn * 4, &m->c_g) ||
           alloc(m, T * c.ffn * 4, &m->c_u) || alloc(m, T * c.ffn * 4, &m->c_ff) ||
           alloc(m, T * c.n_q * m->c_nwg * (c.hd + 2) * 4, &m->c_tmp) || alloc(m, 16, &m->c_meta) ||
           alloc(m, kPartsRows * T * c.hidden * 4, &m->c_po) || alloc(m, 2 * T * 2 * c.ffn * 4, &m->c_pg) || alloc(m, kPartsRows * T * c.hidden * 4, &m->c_pd);
}

// forward_prefill_chunk (gemma_prim.rs:1317-1607) for 2 <= t <= kChunk tokens already validated: the layer as
// matrices of t rows.  The GEMMs run on the batch rounded up to 32 rows (one kernel handle per 32 instead of
// one per length; the rows past t are stale and nothing reads their results).
int forward_prefill_chunk(ksh_gemma *m, const uint32_t *tokens, int t)
{
    const ksh_gemma_cfg &c = m->c;
    if (chunk_buffers(m)) return 1;
    const int64_t qd = (int64_t)c.n_q * c.hd, kvd = (int64_t)c.n_kv * c.hd, tp = (t + 31) / 32 * 32;
    float ids[kChunk];
    for (int i = 0; i < t; i++) ids[i] = (float)tokens[i];
    if (ksh_synchronize(m->ctx)) return 1;                                   // c_tok may still be read by the previous chunk
    if (ksh_buffer_write(m->ctx, m->c_tok, 0, ids, (size_t)t * 4, 1)) return 1;
    ksh_kernel *k_embed, *k_norm, *k_mm_q, *k_mm_kv, *k_head, *k_sdpa, *k_mm_o, *k_add_then, *k_mm_ff, *k_gelu, *k_mm_down, *k_add;
    // q | k | v are one launch of the tile over one preparation of x (a chunk of 4 tokens: 3.1 ms against 4.3 with a
    // small-batch GEMM per matrix)
    // (and gate | up likewise)
    // with the rows' producers inside the GEMMs' preparations: the attention norm in q | k | v's, add-then-norm in
    // gate | up's (which also stores the new residual rows), gelu(gate) * up in the down projection's
    ksh_kernel *k_mm_qkv = nullptr, *k_mm_gu = nullptr, *k_mm_down_g = nullptr;
    const bool norms_inside = c.hidden % 512 == 0 && c.hidden <= 8192 && c.ffn <= 8192;
    if ((get(m, KSH_MATVEC_BATCH, {qd, c.hidden, tp, kvd, kvd, norms_inside ? 1 : 0}, {KSH_Q4K, KSH_F32, KSH_F32}, {c.eps}, &k_mm_qkv) ||
                    get(m, KSH_MATVEC_BATCH, {c.ffn, c.hidden, tp, c.ffn, 0, norms_inside ? 2 : 0}, {KSH_Q4K, KSH_F32, KSH_F32}, {c.eps}, &k_mm_gu) ||
                    (norms_inside && get(m, KSH_MATVEC_BATCH, {c.hidden, c.ffn, tp, 0, 0, 3}, {KSH_Q4K, KSH_F32, KSH_F32}, {c.eps}, &k_mm_down_g))))
        return 1;
    const bool fused = k_mm_qkv && norms_inside;
    // ... and the o, gate | up and down projections leave their K slices' partial sums unfolded for the preparation
    // that reads them (dims[6], dims[7]): no fold launches but q | k | v's, whose reader is not a GEMM
    ksh_kernel *u_o = nullptr, *u_gu = nullptr, *u_down = nullptr, *u_down_last = nullptr, *u_qkv = nullptr;
    bool travel = false;
    if (fused && c.n_layers > 1) {
        const size_t T = kChunk;
        auto parts_of = [](ksh_kernel *kk) { return (int64_t)kk->info.grid[2]; };      // the planes of its unfolded result
        if (get(m, KSH_MATVEC_BATCH, {c.hidden, qd, tp, 0, 0, 0, 1}, {KSH_Q4K, KSH_F32, KSH_F32}, {c.eps}, &u_o) ||
            get(m, KSH_MATVEC_BATCH, {c.ffn, c.hidden, tp, c.ffn, 0, 2, 1, parts_of(u_o)}, {KSH_Q4K, KSH_F32, KSH_F32}, {c.eps}, &u_gu) ||
            get(m, KSH_MATVEC_BATCH, {c.hidden, c.ffn, tp, 0, 0, 3, 1, parts_of(u_gu)}, {KSH_Q4K, KSH_F32, KSH_F32}, {c.eps}, &u_down) ||
            get(m, KSH_MATVEC_BATCH, {c.hidden, c.ffn, tp, 0, 0, 3, 0, parts_of(u_gu)}, {KSH_Q4K, KSH_F32, KSH_F32}, {c.eps}, &u_down_last) ||
            get(m, KSH_MATVEC_BATCH, {qd, c.hidden, tp, kvd, kvd, 2, 0, parts_of(u_down)}, {KSH_Q4K, KSH_F32, KSH_F32}, {c.eps}, &u_qkv))
            return 1;
        travel = u_o->out_bytes[0] <= kPartsRows * T * c.hidden * 4 && u_gu->out_bytes[0] <= 2 * T * 2 * c.ffn * 4 &&
                 u_down->out_bytes[0] <= kPartsRows * T * c.hidden * 4;
    }
    // ... and a layer's closing norm + add with the next layer's attention norm are one add-then-norm, in that
    // layer's q | k | v preparation (the residual rows it stores are the closed layer's)
    ksh_kernel *k_mm_qkv_close = nullptr;
    if (fused && c.n_layers > 1 && get(m, KSH_MATVEC_BATCH, {qd, c.hidden, tp, kvd, kvd, 2}, {KSH_Q4K, KSH_F32, KSH_F32}, {c.eps}, &k_mm_qkv_close)) return 1;
    const float embed_scale = std::sqrt((float)c.hidden);
    if (get(m, KSH_COPY_SCALE_INDEXED, {c.hidden, c.vocab, t}, {KSH_Q6K}, {embed_scale}, &k_embed) ||
        get(m, KSH_RMSNORM, {c.hidden, 0, 0, t}, {}, {c.eps}, &k_norm) ||
        get(m, KSH_MATVEC_BATCH, {qd, c.hidden, tp}, {KSH_Q4K, KSH_F32, KSH_F32}, {}, &k_mm_q) ||
        get(m, KSH_MATVEC_BATCH, {kvd, c.hidden, tp}, {KSH_Q4K, KSH_F32, KSH_F32}, {}, &k_mm_kv) ||
        get(m, KSH_RMSNORM_PER_HEAD_QKV_Q40, {c.n_q, c.n_kv, c.hd, c.max_seq, t}, {}, {c.eps}, &k_head) ||
        // (chunks of more than 16 tokens take the attention's matrix-core form, which wants one partition per token)
        get(m, KSH_SDPA_BATCH, {c.n_q, c.n_kv, c.hd, c.max_seq, t, t > 16 && c.hd == 256 && c.n_q / c.n_kv <= 8 ? 1 : m->c_nwg}, {KSH_Q40, KSH_F32}, {c.attn_scale}, &k_sdpa) ||
        get(m, KSH_MATVEC_BATCH, {c.hidden, qd, tp}, {KSH_Q4K, KSH_F32, KSH_F32}, {}, &k_mm_o) ||
        get(m, KSH_RMSNORM_ADD_THEN_RMSNORM, {c.hidden, t}, {}, {c.eps}, &k_add_then) ||
        get(m, KSH_MATVEC_BATCH, {c.ffn, c.hidden, tp}, {KSH_Q4K, KSH_F32, KSH_F32}, {}, &k_mm_ff) ||
        get(m, KSH_GELU_MUL, {(int64_t)t * c.ffn}, {}, {}, &k_gelu) ||
        get(m, KSH_MATVEC_BATCH, {c.hidden, c.ffn, tp}, {KSH_Q4K, KSH_F32, KSH_F32}, {}, &k_mm_down) ||
        get(m, KSH_RMSNORM, {c.hidden, 1, 0, t}, {}, {c.eps}, &k_add))
        return 1;
    hipStream_t st = (hipStream_t)ksh_stream(m->ctx);
    hipLaunchKernelGGL(chunk_begin_kernel, dim3(1), dim3(64), 0, st, (const float *)ksh_buffer_device_ptr(m->meta),
                       (float *)ksh_buffer_device_ptr(m->c_meta), c.max_seq);
    if (hipGetLastError() != hipSuccess) return set_error("chunk_begin launch failed");
    int n = 0;
    if (enc(m, k_embed, {m->embd, m->c_tok}, {m->c_x}, n)) return 1;
    for (int l = 0; l < c.n_layers; l++) {
        const ksh_gemma_layer &L = m->layers[l];
        if (travel) {
            const bool last = l == c.n_layers - 1;
            if ((l > 0 ? enc(m, u_qkv, {L.wq, m->c_pd, L.wk, L.wv, m->layers[l - 1].post_ffw_norm, m->c_x, L.attn_norm}, {m->c_q, m->c_k, m->c_v, m->c_x}, n)
                       : enc(m, k_mm_qkv, {L.wq, m->c_x, L.wk, L.wv, L.attn_norm}, {m->c_q, m->c_k, m->c_v}, n)) ||
                enc(m, k_head, {m->c_q, L.q_norm, m->rope, m->c_k, L.k_norm, m->c_v, m->meta}, {m->c_q, m->kv_k[l], m->kv_v[l]}, n) ||
                enc(m, k_sdpa, {m->c_q, m->kv_k[l], m->kv_v[l], m->c_meta}, {m->c_tmp, m->c_o}, n) ||
                enc(m, u_o, {L.wo, m->c_o}, {m->c_po}, n) ||
                enc(m, u_gu, {L.wgate, m->c_po, L.wup, L.post_attn_norm, m->c_x, L.ffn_norm}, {m->c_pg, m->c_x}, n) ||
                (last ? (enc(m, u_down_last, {L.wdown, m->c_pg}, {m->c_y}, n) || enc(m, k_add, {m->c_y, L.post_ffw_norm, m->c_x}, {m->c_x}, n))
                      : enc(m, u_down, {L.wdown, m->c_pg}, {m->c_pd}, n)))
                return 1;
            continue;
        }
        if ((fused ? (l > 0 ? enc(m, k_mm_qkv_close, {L.wq, m->c_y, L.wk, L.wv, m->layers[l - 1].post_ffw_norm, m->c_x, L.attn_norm}, {m->c_q, m->c_k, m->c_v, m->c_x}, n)
                            : enc(m, k_mm_qkv, {L.wq, m->c_x, L.wk, L.wv, L.attn_norm}, {m->c_q, m->c_k, m->c_v}, n))
                   : enc(m, k_norm, {m->c_x, L.attn_norm}, {m->c_x2}, n)) ||
            (fused ? 0 : k_mm_qkv ? enc(m, k_mm_qkv, {L.wq, m->c_x2, L.wk, L.wv}, {m->c_q, m->c_k, m->c_v}, n)
                      : (enc(m, k_mm_q, {L.wq, m->c_x2}, {m->c_q}, n) || enc(m, k_mm_kv, {L.wk, m->c_x2}, {m->c_k}, n) ||
                         enc(m, k_mm_kv, {L.wv, m->c_x2}, {m->c_v}, n))) ||
            enc(m, k_head, {m->c_q, L.q_norm, m->rope, m->c_k, L.k_norm, m->c_v, m->meta}, {m->c_q, m->kv_k[l], m->kv_v[l]}, n) ||
            enc(m, k_sdpa, {m->c_q, m->kv_k[l], m->kv_v[l], m->c_meta}, {m->c_tmp, m->c_o}, n) ||
            enc(m, k_mm_o, {L.wo, m->c_o}, {m->c_y}, n) ||
            (fused ? enc(m, k_mm_gu, {L.wgate, m->c_y, L.wup, L.post_attn_norm, m->c_x, L.ffn_norm}, {m->c_g, m->c_u, m->c_x}, n)
                   : (enc(m, k_add_then, {m->c_y, L.post_attn_norm, m->c_x, L.ffn_norm}, {m->c_x, m->c_x2}, n) ||
                      (k_mm_gu ? enc(m, k_mm_gu, {L.wgate, m->c_x2, L.wup}, {m->c_g, m->c_u}, n)
                               : (enc(m, k_mm_ff, {L.wgate, m->c_x2}, {m->c_g}, n) || enc(m, k_mm_ff, {L.wup, m->c_x2}, {m->c_u}, n))))) ||
            (fused ? enc(m, k_mm_down_g, {L.wdown, m->c_g, m->c_u}, {m->c_y}, n)
                   : (enc(m, k_gelu, {m->c_g, m->c_u}, {m->c_ff}, n) || enc(m, k_mm_down, {L.wdown, m->c_ff}, {m->c_y}, n))) ||
            ((!fused || l == c.n_layers - 1) && enc(m, k_add, {m->c_y, L.post_ffw_norm, m->c_x}, {m->c_x}, n)))
            return 1;
    }
    hipLaunchKernelGGL(chunk_end_kernel, dim3(1), dim3(64), 0, st, (float *)ksh_buffer_device_ptr(m->meta), t, c.max_seq,
                       (const float *)ksh_buffer_device_ptr(m->rope), (float *)ksh_buffer_device_ptr(m->rope_cur), c.hd);
    if (hipGetLastError() != hipSuccess) return set_error("chunk_end launch failed");
    m->pos += t;
    return 0;
}

int write_token(ksh_gemma *m, uint32_t token)
{
    // ids are carried as f32 (exact below 2^24), gemma_prim.rs:893
    hipLaunchKernelGGL(set_token_kernel, dim3(1), dim3(64), 0, (hipStream_t)ksh_stream(m->ctx),
                       (float *)ksh_buffer_device_ptr(m->tok), (float)token);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e, "set_token launch");
    // its embedding row, where the decode step expects it (a step that produced its own next token has done this itself)
    int n = 0;
    return enc(m, m->k_embed, {m->embd, m->tok}, {m->x}, n);
}

}  // namespace

extern "C" {

int ksh_gemma_create(ksh_ctx *ctx, const ksh_gemma_cfg *cfg, const ksh_gemma_layer *layers, ksh_buf *token_embd_q6k,
                     ksh_buf *output_norm, ksh_gemma **out)
{
    if (!ctx || !cfg || !layers || !token_embd_q6k || !output_norm || !out) return set_error("ksh_gemma_create: bad arguments");
    *out = nullptr;
    const ksh_gemma_cfg &c = *cfg;
    if (c.n_layers <= 0 || c.hidden <= 0 || c.hidden % 256 || c.ffn <= 0 || c.ffn % 256 || c.n_q <= 0 || c.n_kv <= 0 ||
        c.n_q % c.n_kv || c.hd <= 0 || c.vocab <= 0 || c.max_seq <= 0 || c.vocab >= (1 << 24))
        return set_error("ksh_gemma_create: invalid configuration");
    auto m = std::make_unique<ksh_gemma>();
    m->ctx = ctx;
    m->c = c;
    m->layers.assign(layers, layers + c.n_layers);
    m->embd = token_embd_q6k;
    m->output_norm = output_norm;
    const int64_t qd = (int64_t)c.n_q * c.hd, kvd = (int64_t)c.n_kv * c.hd;
    const size_t kv_bytes = (size_t)c.max_seq * c.n_kv * (c.hd / 32) * 18;   // kv_pool.rs:113-116
    ksh_gemma *g = m.get();
    if (alloc(g, (size_t)c.hidden * 4, &g->x) || alloc(g, (size_t)c.hidden * 4, &g->xb) ||
        alloc(g, (size_t)c.hidden * 4, &g->y) || alloc(g, (size_t)c.hidden * 4, &g->x2) ||
        alloc(g, (size_t)qd * 4, &g->tq) || alloc(g, (size_t)kvd * 4, &g->tk) || alloc(g, (size_t)kvd * 4, &g->tv) ||
        alloc(g, (size_t)qd * 4, &g->to) || alloc(g, (size_t)c.ffn * 4, &g->ff) ||
        alloc(g, (size_t)c.vocab * 4, &g->logits) || alloc(g, 16, &g->tok) || alloc(g, 16, &g->meta) ||
        alloc(g, (size_t)c.max_seq * 4, &g->history))
        return 1;
    g->kv_k.resize(c.n_layers);
    g->kv_v.resize(c.n_layers);
    for (int l = 0; l < c.n_layers; l++)
        if (alloc(g, kv_bytes, &g->kv_k[l]) || alloc(g, kv_bytes, &g->kv_v[l])) return 1;
    // RoPE table, gemma_prim.rs:33-56: per position cos[0..hd/2) || sin[0..hd/2),
    // frequency in f64 then f32, angle = pos * freq in f32
    {
        const int half = c.hd / 2;
        std::vector<float> tab((size_t)c.max_seq * c.hd);
        for (int pos = 0; pos < c.max_seq; pos++)
            for (int i = 0; i < half; i++) {
                const float freq = (float)(1.0 / std::pow((double)c.rope_theta, (double)(2 * i) / (double)c.hd));
                const float ang = (float)pos * freq;
                tab[(size_t)pos * c.hd + i] = std::cos(ang);
                tab[(size_t)pos * c.hd + half + i] = std::sin(ang);
            }
        if (ksh_buffer_alloc(ctx, tab.size() * 4, tab.data(), &g->rope)) return 1;
        g->bufs.owned.push_back(g->rope);
        g->rope0.assign(tab.begin(), tab.begin() + c.hd);
        if (alloc(g, (size_t)c.hd * 4, &g->rope_cur)) return 1;   // the current position's row (advance_kernel keeps it so)
    }
    constexpr int kMaxPartitions = 64;   // the partials buffer holds the largest K-split a schedule may choose
    if (alloc(g, (size_t)c.n_q * kMaxPartitions * (c.hd + 2) * 4, &g->attn_tmp)) return 1;

    // The LM head streams the whole table every token: it gets a copy with each row's fields grouped (whole
    // 128-bit loads, 84 instead of 101 us at 262144 x 2048); the embedding gather keeps reading the Q6_K original.
    const bool lm_rows = c.hidden == 2048 || c.hidden == 4096;
    if (lm_rows) {
        ksh_kernel *rp = nullptr;
        if (alloc(g, (size_t)c.vocab * (c.hidden / 256) * 210, &g->embd_rows) ||
            get(g, KSH_REPACK_ROWS, {c.vocab, c.hidden}, {KSH_Q6K, KSH_Q6K_ROWS}, {}, &rp))
            return 1;
        int n = 0;
        if (enc(g, rp, {g->embd}, {g->embd_rows}, n) || ksh_synchronize(ctx)) return 1;
    }
    const bool fused_attend = sdpa_lanes_supports(c.n_q, c.n_kv, c.hd);
    if (!getenv("KSEARCH_SKIP_BEAM")) {   // gemma_prim.rs:271-286
        const ksh_gemma_layer &L = g->layers[0];
        const float T = (float)std::min(c.max_seq, 1024);
        const float meta[4] = {T, 0.f, 0.f, T - 1.f};
        if (ksh_buffer_write(ctx, g->meta, 0, meta, 16, 1)) return 1;
        ksh_buf *lm_w = g->embd_rows ? g->embd_rows : g->embd;
        using Bufs = std::vector<ksh_buf *>;
        const int nl = c.n_layers;
        auto Lw = [&](int l) -> const ksh_gemma_layer & { return g->layers[l]; };
        warm_plan(g, KSH_RMSNORM_MATVEC_QKV, {qd, kvd, c.hidden, 0}, {KSH_Q4K, KSH_F32}, {c.eps}, nl, [&](int l, Bufs &in, Bufs &out) {
            in = {Lw(l).wq, Lw(l).wk, Lw(l).wv, g->x, Lw(l).attn_norm};
            out = {g->tq, g->tk, g->tv};
        });
        warm_plan(g, KSH_RMSNORM_MATVEC_QKV, {qd, kvd, c.hidden, 1}, {KSH_Q4K, KSH_F32}, {c.eps}, nl, [&](int l, Bufs &in, Bufs &out) {
            in = {Lw(l).wq, Lw(l).wk, Lw(l).wv, g->y, Lw(l).attn_norm, Lw(l).post_ffw_norm, g->x};
            out = {g->tq, g->tk, g->tv, g->xb};
        });
        warm_plan(g, KSH_MATVEC, {c.hidden, qd}, {KSH_Q4K, KSH_F32}, {}, nl, [&](int l, Bufs &in, Bufs &out) {
            in = {Lw(l).wo, g->to};
            out = {g->y};
        });
        warm_plan(g, KSH_RMSNORM_MATVEC_GATE_UP_GELU, {c.ffn, c.hidden, 1}, {KSH_Q4K, KSH_F32}, {c.eps}, nl, [&](int l, Bufs &in, Bufs &out) {
            in = {Lw(l).wgate, Lw(l).wup, g->y, Lw(l).ffn_norm, Lw(l).post_attn_norm, g->x};
            out = {g->ff, g->xb};
        });
        warm_plan(g, KSH_MATVEC, {c.hidden, c.ffn}, {KSH_Q4K, KSH_F32}, {}, nl, [&](int l, Bufs &in, Bufs &out) {
            in = {Lw(l).wdown, g->ff};
            out = {g->y};
        });
        // the table is larger than the last-level cache: two launches over it are two cold ones
        warm_plan(g, KSH_RMSNORM_MATVEC, {c.vocab, c.hidden, 1}, {lm_rows ? KSH_Q6K_ROWS : KSH_Q6K, KSH_F32}, {c.eps}, 2, [&](int, Bufs &in, Bufs &out) {
            in = {lm_w, g->y, g->output_norm, L.post_ffw_norm, g->x};
            out = {g->logits, g->xb};
        });
        if (fused_attend)
            warm_plan(g, KSH_ATTEND_DECODE, {c.n_q, c.n_kv, c.hd, c.max_seq, 0, 0, 1}, {KSH_Q40, KSH_F32}, {c.eps, c.attn_scale}, nl,
                      [&](int l, Bufs &in, Bufs &out) {
                          in = {g->tq, Lw(l).q_norm, g->rope_cur, g->tk, Lw(l).k_norm, g->tv, g->meta};
                          out = {g->kv_k[l], g->kv_v[l], g->attn_tmp, g->to};
                      });
        if (ksh_synchronize(ctx)) return 1;
    }
    const float embed_scale = std::sqrt((float)c.hidden);   // gemma_prim.rs:683
    if (get(g, KSH_COPY_SCALE_INDEXED, {c.hidden, c.vocab}, {KSH_Q6K}, {embed_scale}, &g->k_embed) ||
        get(g, KSH_RMSNORM_MATVEC_QKV, {qd, kvd, c.hidden, 0}, {KSH_Q4K, KSH_F32}, {c.eps}, &g->k_qkv_first) ||
        get(g, KSH_RMSNORM_MATVEC_QKV, {qd, kvd, c.hidden, 1}, {KSH_Q4K, KSH_F32}, {c.eps}, &g->k_qkv) ||
        get(g, KSH_MATVEC, {c.hidden, qd}, {KSH_Q4K, KSH_F32}, {}, &g->k_oproj) ||
        get(g, KSH_RMSNORM_MATVEC_GATE_UP_GELU, {c.ffn, c.hidden, 1}, {KSH_Q4K, KSH_F32}, {c.eps}, &g->k_gate_up) ||
        get(g, KSH_MATVEC, {c.hidden, c.ffn}, {KSH_Q4K, KSH_F32}, {}, &g->k_down) ||
        get(g, KSH_RMSNORM_MATVEC, {c.vocab, c.hidden, 1}, {lm_rows ? KSH_Q6K_ROWS : KSH_Q6K, KSH_F32}, {c.eps}, &g->k_lm_head) ||
        get(g, KSH_SOFTCAP_ARGMAX, {c.vocab}, {}, {c.softcap}, &g->k_argmax))
        return 1;
    // per-head norm + RoPE + KV append + attention + merge: one launch where the fused kind is built for the
    // shape, the three reference ops otherwise
    if (fused_attend) {
        // the partition count (K-split) is the schedule's: the plan cache's, or the kind's default
        if (get(g, KSH_ATTEND_DECODE, {c.n_q, c.n_kv, c.hd, c.max_seq, 0, 0, 1}, {KSH_Q40, KSH_F32}, {c.eps, c.attn_scale},
                &g->k_attend))
            return 1;
        ksh_kernel_info info;
        if (ksh_kernel_info_get(g->k_attend, &info)) return 1;
        g->nwg = (int)info.sched.k_split;
        if (g->nwg < 1 || g->nwg > kMaxPartitions) return set_error("attend_decode: schedule with %d partitions", g->nwg);
        g->short_context = kShortContext;
        if (const char *e = getenv("KSEARCH_SHORT_CONTEXT")) g->short_context = atoi(e);
        if (g->short_context > 0 && qd <= 2048 && (c.hd & (c.hd - 1)) == 0 &&
            (get(g, KSH_ATTEND_DECODE, {c.n_q, c.n_kv, c.hd, c.max_seq, kShortPartitions, 1, 1}, {KSH_Q40, KSH_F32},
                 {c.eps, c.attn_scale}, &g->k_attend_parts) ||
             get(g, KSH_ATTN_MERGE_MATVEC, {c.hidden, c.n_q, c.hd, kShortPartitions}, {KSH_Q4K, KSH_F32}, {}, &g->k_oproj_merge)))
            return 1;
    } else {
        if (get(g, KSH_RMSNORM_PER_HEAD_QKV_Q40, {c.n_q, c.n_kv, c.hd, c.max_seq}, {}, {c.eps}, &g->k_head) ||
            get(g, KSH_SDPA_SLOTS, {c.n_q, c.n_kv, c.hd, c.max_seq, 1, g->nwg}, {KSH_Q40, KSH_F32}, {c.attn_scale}, &g->k_sdpa))
            return 1;
    }
    g->prof.on = getenv("KSEARCH_PROFILE") != nullptr;
    if (ksh_gemma_reset(g)) return 1;
    *out = m.release();
    return 0;
}

void ksh_gemma_destroy(ksh_gemma *m)
{
    if (!m) return;
    ksh_synchronize(m->ctx);
    for (int i = 0; i < 2; i++) {
        ksh_graph_destroy(m->g_body[i]);
        ksh_graph_destroy(m->g_full[i]);
        ksh_graph_destroy(m->g_span[i]);
    }
    delete m;
}

int ksh_gemma_reset(ksh_gemma *m)
{
    if (!m) return set_error("ksh_gemma_reset: null model");
    if (ksh_synchronize(m->ctx)) return 1;
    const float meta[4] = {1.f, 0.f, 0.f, 0.f};   // tlen, start, window, pos
    if (ksh_buffer_write(m->ctx, m->meta, 0, meta, 16, 1)) return 1;
    if (ksh_buffer_write(m->ctx, m->rope_cur, 0, m->rope0.data(), m->rope0.size() * 4, 1)) return 1;
    m->pos = 0;
    return 0;
}

int ksh_gemma_forward_token(ksh_gemma *m, uint32_t token, int use_graph, uint32_t *next_id)
{
    if (!m) return set_error("ksh_gemma_forward_token: null model");
    if (token >= (uint32_t)m->c.vocab) return set_error("token id %u is outside the vocabulary", token);
    if (write_token(m, token)) return 1;
    if (run_token(m, true, use_graph != 0)) return 1;
    if (next_id) {
        float f = 0.f;
        if (ksh_buffer_read(m->ctx, m->tok, 0, &f, 4, 1)) return 1;
        *next_id = (uint32_t)f;
    }
    return 0;
}

int ksh_gemma_prefill_chunk(ksh_gemma *m, const uint32_t *tokens, int n)
{
    if (!m || (n && !tokens) || n < 0) return set_error("ksh_gemma_prefill_chunk: bad arguments");
    if (m->pos + n > m->c.max_seq) return set_error("max_seq exceeded");
    for (int i = 0; i < n; i++)
        if (tokens[i] >= (uint32_t)m->c.vocab) return set_error("token id %u is outside the vocabulary", tokens[i]);
    // gemma_prim.rs:1305-1315: chunks of PREFILL_CHUNK, a remainder of one token through the decode step
    for (int i = 0; i < n; i += kChunk) {
        const int t = std::min(kChunk, n - i);
        if (t == 1) {
            if (write_token(m, tokens[i]) || run_token(m, false, false)) return 1;
        } else if (forward_prefill_chunk(m, tokens + i, t)) {
            return 1;
        }
    }
    return ksh_synchronize(m->ctx);
}

int ksh_gemma_generate(ksh_gemma *m, const uint32_t *prompt, int n_prompt, int n_new, int use_graph, uint32_t *out_ids,
                       double *prefill_ms, double *decode_ms)
{
    if (!m || !prompt || n_prompt < 1 || n_new < 0 || (n_new && !out_ids)) return set_error("ksh_gemma_generate: bad arguments");
    if (m->pos + n_prompt - 1 + n_new > m->c.max_seq) return set_error("max_seq exceeded");
    for (int i = 0; i < n_prompt; i++)
        if (prompt[i] >= (uint32_t)m->c.vocab) return set_error("token id %u is outside the vocabulary", prompt[i]);
    using clk = std::chrono::steady_clock;
    const auto t0 = clk::now();
    // all prompt tokens but the last go through without logits (gemma_prim.rs:1670-1675)
    const bool graph = (use_graph & 1) != 0;
    if (use_graph & 2) {
        for (int i = 0; i + 1 < n_prompt; i++) {
            if (write_token(m, prompt[i])) return 1;
            if (run_token(m, false, graph)) return 1;
        }
    } else if (ksh_gemma_prefill_chunk(m, prompt, n_prompt - 1)) {
        return 1;
    }
    if (write_token(m, prompt[n_prompt - 1])) return 1;
    if (ksh_synchronize(m->ctx)) return 1;
    const auto t1 = clk::now();
    const int first = m->pos;
    for (int i = 0; i < n_new;) {
        if (graph && span_fits(m, n_new - i)) {
            if (run_span(m)) return 1;
            i += kSpan;
        } else {
            if (run_token(m, true, graph)) return 1;
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

ksh_buf *ksh_gemma_logits(ksh_gemma *m) { return m ? m->logits : nullptr; }
ksh_buf *ksh_gemma_hidden(ksh_gemma *m) { return m ? (m->hidden ? m->hidden : m->x) : nullptr; }
ksh_buf *ksh_gemma_kv(ksh_gemma *m, int layer, int which)
{
    if (!m || layer < 0 || layer >= m->c.n_layers) return nullptr;
    return which ? m->kv_v[layer] : m->kv_k[layer];
}
int ksh_gemma_pos(ksh_gemma *m) { return m ? m->pos : -1; }
int ksh_gemma_launches_per_token(ksh_gemma *m) { return m ? m->launches_full : -1; }

}  // extern "C"
