// Host-only stand-ins that let the slot scheduler (ksearch_amd/csrc/serve.cpp) and the KV pool
// (ksearch_amd/csrc/kv_pool.cpp) be linked and driven without a GPU: buffers are host memory and the "model" is a
// counter with a fixed next-token rule that logs what the scheduler asks of it.  Test infrastructure only: it is
// compiled into tests/host_mock/libserve_host.so, never into the library.
#include <cstdarg>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../ksearch_amd/csrc/ksh_internal.hpp"

namespace ksh {
static thread_local std::string g_err;
int set_error(const char *fmt, ...)
{
    char b[512];
    va_list a;
    va_start(a, fmt);
    vsnprintf(b, sizeof b, fmt, a);
    va_end(a);
    g_err = b;
    return 1;
}
ksh_buf *buffer_view(ksh_buf *parent, size_t off, size_t bytes)
{
    if (!parent || off > parent->bytes || bytes > parent->bytes - off) {
        set_error("buffer_view: range outside the buffer");
        return nullptr;
    }
    ksh_buf *v = new ksh_buf;
    v->ptr = (char *)parent->ptr + off;
    v->bytes = bytes;
    v->parent = parent;
    parent->rc++;
    return v;
}
}  // namespace ksh

struct MockCall {
    int32_t kind;   // 0 bind_slot, 1 prefill_chunk, 2 decode_token_sampled, 3 one row of decode_round
    int32_t slot, pos, n;
    uint32_t token, seed;
    float temperature, min_p;
};

struct ksh_gemma4 {
    int max_seq = 64, vocab = 1000;
    int mode = 0;              // 0: next = (31 * token + 7 * pos + 1) % vocab; 1: always `constant`; 2: decode fails at position fail_pos
    uint32_t constant = 5;
    int fail_pos = -1;
    int pos = 0, slot = -1;
    ksh_kvpool *pool = nullptr;
    std::vector<MockCall> calls;
};

extern "C" {

const char *ksh_last_error(void) { return ksh::g_err.c_str(); }

int ksh_buffer_alloc(ksh_ctx *, size_t bytes, const void *init, ksh_buf **out)
{
    ksh_buf *b = new ksh_buf;
    b->ptr = malloc(bytes ? bytes : 1);
    b->bytes = bytes;
    if (init) memcpy(b->ptr, init, bytes);
    *out = b;
    return 0;
}
void ksh_buffer_release(ksh_buf *b)
{
    if (b && --b->rc == 0) {
        if (b->parent)
            ksh_buffer_release(b->parent);
        else
            free(b->ptr);
        delete b;
    }
}
int ksh_synchronize(ksh_ctx *) { return 0; }
int ksh_buffer_fill_zero(ksh_ctx *, ksh_buf *b)
{
    memset(b->ptr, 0, b->bytes);
    return 0;
}

ksh_gemma4 *mock_model_create(int max_seq, int vocab, int mode, uint32_t constant, int fail_pos)
{
    ksh_gemma4 *m = new ksh_gemma4;
    m->max_seq = max_seq;
    m->vocab = vocab;
    m->mode = mode;
    m->constant = constant;
    m->fail_pos = fail_pos;
    return m;
}
void mock_model_destroy(ksh_gemma4 *m) { delete m; }
int mock_model_calls(ksh_gemma4 *m, MockCall *out, int cap)
{
    const int n = (int)m->calls.size();
    for (int i = 0; i < n && i < cap; i++) out[i] = m->calls[(size_t)i];
    return n;
}
void mock_model_clear_calls(ksh_gemma4 *m) { m->calls.clear(); }

int ksh_gemma4_config(ksh_gemma4 *m, ksh_gemma4_cfg *cfg)
{
    memset(cfg, 0, sizeof *cfg);
    cfg->max_seq = m->max_seq;
    cfg->vocab = m->vocab;
    return 0;
}

int ksh_gemma4_bind_slot(ksh_gemma4 *m, ksh_kvpool *pool, int slot)
{
    const int len = ksh_kvpool_seq_len(pool, slot);
    if (len < 0) return ksh::set_error("bad SlotId");
    m->pool = pool;
    m->slot = slot;
    m->pos = len;
    m->calls.push_back(MockCall{0, slot, len, 0, 0, 0, 0.f, 0.f});
    return 0;
}

int ksh_gemma4_prefill_chunk(ksh_gemma4 *m, const uint32_t *tokens, int n, int)
{
    if (m->pos + n > m->max_seq) return ksh::set_error("max_seq exceeded");
    m->calls.push_back(MockCall{1, m->slot, m->pos, n, n ? tokens[0] : 0, 0, 0.f, 0.f});
    m->pos += n;
    return 0;
}

int ksh_gemma4_decode_token_sampled(ksh_gemma4 *m, uint32_t token, float temperature, float min_p, uint32_t seed, int, uint32_t *next)
{
    if (m->pos >= m->max_seq) return ksh::set_error("max_seq exceeded");
    if (m->mode == 2 && m->pos == m->fail_pos) return ksh::set_error("mock decode failure at %d", m->pos);
    m->calls.push_back(MockCall{2, m->slot, m->pos, 1, token, seed, temperature, min_p});
    *next = m->mode == 1 ? m->constant : (uint32_t)((31ull * token + 7ull * (unsigned)m->pos + 1) % (unsigned)m->vocab);
    m->pos += 1;
    return 0;
}

// one record per row; positions come from the pool, the model's own binding is left alone
int ksh_gemma4_decode_round(ksh_gemma4 *m, ksh_kvpool *pool, const int32_t *slots, const uint32_t *tokens, int n, const float *temperature,
                            const float *min_p, const uint32_t *seed, uint32_t *next_ids)
{
    if (n < 1 || n > 16) return ksh::set_error("ksh_gemma4_decode_round: %d sequences", n);
    for (int i = 0; i < n; i++) {
        const int pos = ksh_kvpool_seq_len(pool, slots[i]);
        if (pos < 0) return ksh::set_error("bad SlotId");
        if (pos >= m->max_seq) return ksh::set_error("max_seq exceeded");
        if (m->mode == 2 && pos == m->fail_pos) return ksh::set_error("mock decode failure at %d", pos);
    }
    for (int i = 0; i < n; i++) {
        const int pos = ksh_kvpool_seq_len(pool, slots[i]);
        m->calls.push_back(MockCall{3, slots[i], pos, n, tokens[i], seed ? seed[i] : 0, temperature ? temperature[i] : 0.f, min_p ? min_p[i] : 0.f});
        next_ids[i] = m->mode == 1 ? m->constant : (uint32_t)((31ull * tokens[i] + 7ull * (unsigned)pos + 1) % (unsigned)m->vocab);
    }
    return 0;
}

}  // extern "C"
