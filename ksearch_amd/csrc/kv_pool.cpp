// KV slots for serving several sequences from one set of weights: the pool owns
// the Q4_0 K / V caches of every slot, tracks occupancy and sequence length, and a
// model is pointed at one slot at a time (ksh_gemma4_bind_slot).
//
// Mirrors KvPool (crates/ksearch_gemma/src/kv_pool.rs:24-228, the Q4_0 form of
// KvPool::new): same slot rules (first free slot, freed slots are reused, a bump
// past max_seq is an error), same buffer sizes (q40_nbytes(max_seq * n_kv, hd)
// per layer and cache).  clear_slot is a fill kernel instead of a host memset.
#include <memory>
#include <vector>

#include "ksh_internal.hpp"

struct ksh_kvpool {
    ksh_ctx *ctx = nullptr;
    uint64_t uid = 0;   // never reused: a pool created where a destroyed one lay is still another pool
    int max_batch = 0, max_seq = 0, n_kv_layers = 0, hd = 0, n_kv = 0;
    std::vector<char> occupied;
    std::vector<int> seq_len;
    // One allocation per layer and cache, [slot][max_seq * n_kv * (hd / 32) * 18]: a slot's cache is a view into it
    // (what a model is bound to), and a pass over several slots' tokens addresses all of them from one base.
    std::vector<ksh_buf *> layer_k, layer_v;   // [layer]
    std::vector<ksh_buf *> k, v;               // [slot][layer] views
    size_t slot_bytes = 0;
    ~ksh_kvpool()
    {
        for (ksh_buf *b : k) ksh_buffer_release(b);
        for (ksh_buf *b : v) ksh_buffer_release(b);
        for (ksh_buf *b : layer_k) ksh_buffer_release(b);
        for (ksh_buf *b : layer_v) ksh_buffer_release(b);
    }
};

using namespace ksh;

namespace {
bool bad_slot(const ksh_kvpool *p, int slot) { return !p || slot < 0 || slot >= p->max_batch; }
}

extern "C" {

int ksh_kvpool_create(ksh_ctx *ctx, int max_batch, int max_seq, int n_kv_layers, int hd, int n_kv, ksh_kvpool **out)
{
    if (!ctx || !out) return set_error("ksh_kvpool_create: bad arguments");
    *out = nullptr;
    if (max_batch <= 0 || max_seq <= 0 || n_kv_layers <= 0 || hd <= 0 || n_kv <= 0) return set_error("KvPool dims must be non-zero");
    if (hd % 32) return set_error("KvPool: hd=%d is not a multiple of the Q4_0 block (32)", hd);
    auto p = std::make_unique<ksh_kvpool>();
    static std::atomic<uint64_t> next_uid{1};
    p->uid = next_uid.fetch_add(1);
    p->ctx = ctx;
    p->max_batch = max_batch; p->max_seq = max_seq; p->n_kv_layers = n_kv_layers; p->hd = hd; p->n_kv = n_kv;
    p->occupied.assign((size_t)max_batch, 0);
    p->seq_len.assign((size_t)max_batch, 0);
    const size_t bytes = (size_t)max_seq * n_kv * (hd / 32) * 18;   // q40_nbytes, crates/ksearch_ir/src/lib.rs:52-59
    p->slot_bytes = bytes;
    for (int l = 0; l < n_kv_layers; l++) {
        ksh_buf *kb = nullptr, *vb = nullptr;
        if (ksh_buffer_alloc(ctx, bytes * max_batch, nullptr, &kb)) return 1;
        p->layer_k.push_back(kb);
        if (ksh_buffer_alloc(ctx, bytes * max_batch, nullptr, &vb)) return 1;
        p->layer_v.push_back(vb);
    }
    for (int s = 0; s < max_batch; s++)
        for (int l = 0; l < n_kv_layers; l++) {
            ksh_buf *kb = buffer_view(p->layer_k[(size_t)l], (size_t)s * bytes, bytes), *vb = buffer_view(p->layer_v[(size_t)l], (size_t)s * bytes, bytes);
            if (kb) p->k.push_back(kb);
            if (vb) p->v.push_back(vb);
            if (!kb || !vb) return 1;
        }
    *out = p.release();
    return 0;
}

uint64_t ksh_kvpool_uid(const ksh_kvpool *p) { return p ? p->uid : 0; }

void ksh_kvpool_destroy(ksh_kvpool *p)
{
    if (!p) return;
    ksh_synchronize(p->ctx);
    delete p;
}

int ksh_kvpool_alloc(ksh_kvpool *p, int *slot)
{
    if (!p || !slot) return set_error("ksh_kvpool_alloc: bad arguments");
    for (int i = 0; i < p->max_batch; i++)
        if (!p->occupied[(size_t)i]) {
            p->occupied[(size_t)i] = 1;
            p->seq_len[(size_t)i] = 0;
            *slot = i;
            return 0;
        }
    return set_error("KvPool full (max_batch=%d)", p->max_batch);
}

int ksh_kvpool_free(ksh_kvpool *p, int slot)
{
    if (bad_slot(p, slot)) return set_error("bad SlotId");
    p->occupied[(size_t)slot] = 0;
    p->seq_len[(size_t)slot] = 0;
    return 0;
}

int ksh_kvpool_clear_slot(ksh_kvpool *p, int slot)
{
    if (bad_slot(p, slot)) return set_error("bad SlotId");
    for (int l = 0; l < p->n_kv_layers; l++)
        if (ksh_buffer_fill_zero(p->ctx, p->k[(size_t)slot * p->n_kv_layers + l]) ||
            ksh_buffer_fill_zero(p->ctx, p->v[(size_t)slot * p->n_kv_layers + l]))
            return 1;
    return 0;
}

int ksh_kvpool_seq_len(const ksh_kvpool *p, int slot) { return bad_slot(p, slot) ? -1 : p->seq_len[(size_t)slot]; }
int ksh_kvpool_occupied(const ksh_kvpool *p, int slot) { return bad_slot(p, slot) ? -1 : p->occupied[(size_t)slot]; }

int ksh_kvpool_bump_len_by(ksh_kvpool *p, int slot, int n, int *new_len)
{
    if (bad_slot(p, slot) || n < 0) return set_error("bad SlotId");
    if (!p->occupied[(size_t)slot]) return set_error("slot not occupied");
    if (p->seq_len[(size_t)slot] + n > p->max_seq) return set_error("slot seq full");
    p->seq_len[(size_t)slot] += n;
    if (new_len) *new_len = p->seq_len[(size_t)slot];
    return 0;
}

int ksh_kvpool_active_batch(const ksh_kvpool *p, int *slots, int cap)
{
    if (!p) return -1;
    int n = 0;
    for (int i = 0; i < p->max_batch; i++)
        if (p->occupied[(size_t)i]) {
            if (slots && n < cap) slots[n] = i;
            n++;
        }
    return n;
}

ksh_buf *ksh_kvpool_k(const ksh_kvpool *p, int slot, int layer)
{
    return bad_slot(p, slot) || layer < 0 || layer >= p->n_kv_layers ? nullptr : p->k[(size_t)slot * p->n_kv_layers + layer];
}
ksh_buf *ksh_kvpool_v(const ksh_kvpool *p, int slot, int layer)
{
    return bad_slot(p, slot) || layer < 0 || layer >= p->n_kv_layers ? nullptr : p->v[(size_t)slot * p->n_kv_layers + layer];
}

ksh_buf *ksh_kvpool_layer_k(const ksh_kvpool *p, int layer) { return !p || layer < 0 || layer >= p->n_kv_layers ? nullptr : p->layer_k[(size_t)layer]; }
ksh_buf *ksh_kvpool_layer_v(const ksh_kvpool *p, int layer) { return !p || layer < 0 || layer >= p->n_kv_layers ? nullptr : p->layer_v[(size_t)layer]; }

int ksh_kvpool_dims(const ksh_kvpool *p, int *max_batch, int *max_seq, int *n_kv_layers, int *hd, int *n_kv)
{
    if (!p) return set_error("ksh_kvpool_dims: null pool");
    if (max_batch) *max_batch = p->max_batch;
    if (max_seq) *max_seq = p->max_seq;
    if (n_kv_layers) *n_kv_layers = p->n_kv_layers;
    if (hd) *hd = p->hd;
    if (n_kv) *n_kv = p->n_kv;
    return 0;
}

}  // extern "C"
