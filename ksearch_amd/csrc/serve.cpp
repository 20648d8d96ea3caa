// Decode-before-prefill slot scheduler over one model and one KV pool.
//
// Mirrors spawn_scheduler and its rounds (crates/ksearch_cli/src/scheduler.rs:78-349) as a tick function the
// host drives: admission into free slots, one decode token per decoding request, then chunked prefill on the
// prefilling ones (small chunks while anything decodes, the whole budget otherwise), then the finished requests
// give their slots back.  GPU work is serial, as in the reference (one set of activation buffers); concurrency
// is the pool's slots.  What the reference does with channels is a queue of events here; what it does with the
// tokenizer (stop strings on the decoded text, scheduler.rs:207-217) is a callback the host supplies, since
// token ids are all this library sees.
#include <algorithm>
#include <deque>
#include <memory>
#include <string>
#include <vector>

#include "ksh_internal.hpp"

namespace {

struct Request {
    uint64_t id = 0;
    std::vector<uint32_t> prompt;
    size_t max_tokens = 1;
    float temperature = 0.f, min_p = 0.f;
    uint32_t seed = 1;
};

struct Active {
    uint64_t id = 0;
    int slot = -1;
    std::vector<uint32_t> prompt, generated;
    size_t max_tokens = 1;
    float temperature = 0.f, min_p = 0.f;
    uint32_t rng = 1;
    bool prefill = true;      // Phase::Prefill { cursor } / Phase::Decode { last_token }
    size_t cursor = 0;
    uint32_t last_token = 0;
    bool finished = false, cancelled = false;
};

}  // namespace

struct ksh_serve {
    ksh_gemma4 *model = nullptr;
    ksh_kvpool *pool = nullptr;
    ksh_serve_cfg cfg{};
    int max_seq = 0;
    uint64_t next_id = 1;
    std::deque<Request> waiting;
    std::vector<Active> active;
    size_t prefill_cursor = 0;
    std::deque<ksh_serve_event> events;
    std::deque<std::string> errors;   // texts of the error events, in the order of those events
};

using namespace ksh;

namespace {

void push_event(ksh_serve *s, uint64_t id, int kind, uint32_t token, int reason, size_t prompt_tokens, size_t completion_tokens)
{
    ksh_serve_event e{};
    e.request = id;
    e.kind = kind;
    e.token = token;
    e.reason = reason;
    e.prompt_tokens = (uint32_t)prompt_tokens;
    e.completion_tokens = (uint32_t)completion_tokens;
    s->events.push_back(e);
}

void push_error(ksh_serve *s, uint64_t id, const std::string &text)
{
    push_event(s, id, KSH_SERVE_ERROR, 0, KSH_FINISH_ERROR, 0, 0);
    s->errors.push_back(text);
}

// scheduler.rs:318-340: Done goes out for every reason but "error" (whose Error event went out already)
void finish(ksh_serve *s, Active &a, int reason)
{
    if (a.finished) return;
    a.finished = true;
    if (reason != KSH_FINISH_ERROR) push_event(s, a.id, KSH_SERVE_DONE, 0, reason, a.prompt.size(), a.generated.size());
}

// scheduler.rs:342-348
bool repeating_token(const std::vector<uint32_t> &ids, size_t n)
{
    if (ids.size() < n) return false;
    const uint32_t last = ids.back();
    return std::all_of(ids.end() - (long)n, ids.end(), [&](uint32_t t) { return t == last; });
}

// scheduler.rs:305-316
void enter_decode(Active &a)
{
    a.prefill = false;
    a.last_token = a.prompt.back();
}

// scheduler.rs:134-161
void admit_waiting(ksh_serve *s)
{
    while (ksh_kvpool_active_batch(s->pool, nullptr, 0) < s->cfg.slots && !s->waiting.empty()) {
        Request r = std::move(s->waiting.front());
        s->waiting.pop_front();
        if (r.prompt.empty()) {
            push_error(s, r.id, "empty prompt");
            continue;
        }
        int slot = -1;
        if (ksh_kvpool_alloc(s->pool, &slot) || ksh_kvpool_clear_slot(s->pool, slot)) {
            if (slot >= 0) ksh_kvpool_free(s->pool, slot);
            push_error(s, r.id, std::string("admit failed: ") + ksh_last_error());
            continue;
        }
        Active a;
        a.id = r.id;
        a.slot = slot;
        a.prompt = std::move(r.prompt);
        a.max_tokens = std::max<size_t>(r.max_tokens, 1);
        a.temperature = r.temperature;
        a.min_p = r.min_p;
        a.rng = r.seed | 1u;
        s->active.push_back(std::move(a));
    }
}

// what follows a decoded token (scheduler.rs:196-231)
void after_token(ksh_serve *s, Active &a, uint32_t next)
{
    a.last_token = next;
    if (next == s->cfg.eos[0] || next == s->cfg.eos[1]) { finish(s, a, KSH_FINISH_STOP); return; }
    // the reference decodes the piece and looks for its stop strings here; the host's callback stands in
    if (s->cfg.stop && s->cfg.stop(s->cfg.stop_user, a.id, next)) { finish(s, a, KSH_FINISH_STOP); return; }
    a.generated.push_back(next);
    if (repeating_token(a.generated, 24)) { finish(s, a, KSH_FINISH_STOP); return; }
    if (a.cancelled) { finish(s, a, KSH_FINISH_CANCELLED); return; }   // (the reference: the receiver is gone)
    push_event(s, a.id, KSH_SERVE_TOKEN, next, 0, 0, 0);
    if (a.generated.size() >= a.max_tokens) finish(s, a, KSH_FINISH_LENGTH);
}

// scheduler.rs:163-241.  The reference runs the round's requests one after the other, each a full pass over the
// weights; from batched_decode decoding requests on they take the step together (ksh_gemma4_decode_round, up to 16
// at a time), in the order and with the sampler sequence they would have had one by one.
void decode_round(ksh_serve *s)
{
    std::vector<Active *> ready;
    for (Active &a : s->active) {
        if (a.finished || a.prefill) continue;
        if (a.generated.size() >= a.max_tokens) { finish(s, a, KSH_FINISH_LENGTH); continue; }
        if (std::max(ksh_kvpool_seq_len(s->pool, a.slot), 0) >= s->max_seq) { finish(s, a, KSH_FINISH_LENGTH); continue; }
        a.rng += 0x9E3779B9u;
        ready.push_back(&a);
    }
    constexpr size_t kMaxRound = 16;
    for (size_t i0 = 0; i0 < ready.size();) {
        const size_t left = ready.size() - i0;
        const size_t n = s->cfg.batched_decode >= 2 && left >= (size_t)s->cfg.batched_decode ? std::min(left, kMaxRound) : 1;
        if (n == 1) {
            Active &a = *ready[i0];
            uint32_t next = 0;
            if (ksh_gemma4_bind_slot(s->model, s->pool, a.slot) ||
                ksh_gemma4_decode_token_sampled(s->model, a.last_token, a.temperature, a.min_p, a.rng, s->cfg.use_graph, &next) ||
                ksh_kvpool_bump_len_by(s->pool, a.slot, 1, nullptr)) {
                push_error(s, a.id, ksh_last_error());
                finish(s, a, KSH_FINISH_ERROR);
            } else {
                after_token(s, a, next);
            }
        } else {
            int32_t slots[kMaxRound];
            uint32_t tokens[kMaxRound], seeds[kMaxRound], next[kMaxRound];
            float temp[kMaxRound], min_p[kMaxRound];
            for (size_t i = 0; i < n; i++) {
                const Active &a = *ready[i0 + i];
                slots[i] = a.slot; tokens[i] = a.last_token; seeds[i] = a.rng; temp[i] = a.temperature; min_p[i] = a.min_p;
            }
            const bool failed = ksh_gemma4_decode_round(s->model, s->pool, slots, tokens, (int)n, temp, min_p, seeds, next) != 0;
            const std::string why = failed ? ksh_last_error() : "";
            for (size_t i = 0; i < n; i++) {
                Active &a = *ready[i0 + i];
                if (failed || ksh_kvpool_bump_len_by(s->pool, a.slot, 1, nullptr)) {
                    push_error(s, a.id, failed ? why : ksh_last_error());
                    finish(s, a, KSH_FINISH_ERROR);
                } else {
                    after_token(s, a, next[i]);
                }
            }
        }
        i0 += n;
    }
}

// scheduler.rs:243-303
void prefill_round(ksh_serve *s)
{
    const size_t n = s->active.size();
    if (!n || std::none_of(s->active.begin(), s->active.end(), [](const Active &a) { return a.prefill; })) return;
    const bool decoding = std::any_of(s->active.begin(), s->active.end(), [](const Active &a) { return !a.finished && !a.prefill; });
    size_t budget = (size_t)std::max(s->cfg.prefill_tokens_per_tick, s->cfg.prefill_chunk);
    size_t idx = s->prefill_cursor % n;
    for (size_t i = 0; i < n && budget; i++) {
        Active &a = s->active[idx];
        idx = (idx + 1) % n;
        if (a.finished || !a.prefill) continue;
        // the last prompt token is the first decode input, not a prefill step
        const size_t prefill_end = a.prompt.size() - 1;
        if (a.cursor >= prefill_end) { enter_decode(a); continue; }
        // small chunks while something decodes; otherwise the whole budget
        const size_t cap = decoding ? (size_t)s->cfg.prefill_chunk : budget;
        const size_t take = std::min({budget, cap, prefill_end - a.cursor});
        if (ksh_gemma4_bind_slot(s->model, s->pool, a.slot) ||
            ksh_gemma4_prefill_chunk(s->model, a.prompt.data() + a.cursor, (int)take, s->cfg.use_graph) ||
            ksh_kvpool_bump_len_by(s->pool, a.slot, (int)take, nullptr)) {
            push_error(s, a.id, ksh_last_error());
            finish(s, a, KSH_FINISH_ERROR);
            continue;
        }
        budget -= take;
        a.cursor += take;
        if (a.cursor >= prefill_end) enter_decode(a);
    }
    s->prefill_cursor = idx;
}

// scheduler.rs:294-303 (reap_finished)
void reap_finished(ksh_serve *s)
{
    for (Active &a : s->active)
        if (a.finished) ksh_kvpool_free(s->pool, a.slot);
    s->active.erase(std::remove_if(s->active.begin(), s->active.end(), [](const Active &a) { return a.finished; }), s->active.end());
}

}  // namespace

extern "C" {

int ksh_serve_default_cfg(ksh_serve_cfg *cfg)
{
    if (!cfg) return set_error("ksh_serve_default_cfg: null");
    *cfg = ksh_serve_cfg{};
    cfg->slots = 4;                        // SchedulerConfig::default, scheduler.rs:66-76
    cfg->prefill_chunk = 256;              // PREFILL_CHUNK_SIZE, gemma_prim.rs:16-19
    cfg->prefill_tokens_per_tick = 2048;
    cfg->eos[0] = 1;                       // EOS_IDS, scheduler.rs:14
    cfg->eos[1] = 106;
    cfg->use_graph = 1;
    cfg->batched_decode = 3;   // a joint step costs about two and a half single ones at the real checkpoints' layer layout
    return 0;
}

int ksh_serve_create(ksh_gemma4 *model, ksh_kvpool *pool, const ksh_serve_cfg *cfg, ksh_serve **out)
{
    if (!model || !pool || !cfg || !out) return set_error("ksh_serve_create: bad arguments");
    *out = nullptr;
    if (cfg->slots < 1 || cfg->prefill_chunk < 1 || cfg->prefill_tokens_per_tick < 0)
        return set_error("ksh_serve_create: slots=%d prefill_chunk=%d prefill_tokens_per_tick=%d", cfg->slots, cfg->prefill_chunk,
                         cfg->prefill_tokens_per_tick);
    ksh_gemma4_cfg mc;
    if (ksh_gemma4_config(model, &mc)) return 1;
    // a model that cannot bind the pool's slots is found here, not at the first tick
    if (ksh_gemma4_bind_slot(model, pool, 0)) return 1;
    auto s = std::make_unique<ksh_serve>();
    s->model = model;
    s->pool = pool;
    s->cfg = *cfg;
    s->max_seq = mc.max_seq;
    *out = s.release();
    return 0;
}

void ksh_serve_destroy(ksh_serve *s)
{
    if (!s) return;
    // requests still running give their slots back: the pool outlives the scheduler
    for (const Active &a : s->active) ksh_kvpool_free(s->pool, a.slot);
    delete s;
}

int ksh_serve_submit(ksh_serve *s, const uint32_t *prompt, size_t n_prompt, size_t max_tokens, float temperature, float min_p,
                     uint32_t seed, uint64_t *request)
{
    if (!s || (n_prompt && !prompt)) return set_error("ksh_serve_submit: bad arguments");
    Request r;
    r.id = s->next_id++;
    r.prompt.assign(prompt, prompt + n_prompt);
    r.max_tokens = max_tokens;
    r.temperature = temperature;
    r.min_p = min_p;
    r.seed = seed;
    if (request) *request = r.id;
    s->waiting.push_back(std::move(r));
    return 0;
}

int ksh_serve_cancel(ksh_serve *s, uint64_t request)
{
    if (!s) return set_error("ksh_serve_cancel: null");
    for (Active &a : s->active)
        if (a.id == request) { a.cancelled = true; return 0; }
    for (auto it = s->waiting.begin(); it != s->waiting.end(); ++it)
        if (it->id == request) {
            push_event(s, request, KSH_SERVE_DONE, 0, KSH_FINISH_CANCELLED, it->prompt.size(), 0);
            s->waiting.erase(it);
            return 0;
        }
    return set_error("ksh_serve_cancel: request %llu is not queued or running", (unsigned long long)request);
}

int ksh_serve_tick(ksh_serve *s)
{
    if (!s) return set_error("ksh_serve_tick: null");
    admit_waiting(s);
    if (s->active.empty()) return 0;
    decode_round(s);
    prefill_round(s);
    reap_finished(s);
    return 0;
}

size_t ksh_serve_poll(ksh_serve *s, ksh_serve_event *out, size_t cap)
{
    if (!s || !out) return 0;
    size_t n = 0;
    while (n < cap && !s->events.empty()) {
        out[n++] = s->events.front();
        s->events.pop_front();
    }
    return n;
}

const char *ksh_serve_error_text(ksh_serve *s)
{
    static thread_local std::string text;
    if (!s || s->errors.empty()) return nullptr;
    text = std::move(s->errors.front());
    s->errors.pop_front();
    return text.c_str();
}

int ksh_serve_pending(const ksh_serve *s, int *waiting, int *active)
{
    if (!s) return set_error("ksh_serve_pending: null");
    if (waiting) *waiting = (int)s->waiting.size();
    if (active) *active = (int)s->active.size();
    return 0;
}

}  // extern "C"
