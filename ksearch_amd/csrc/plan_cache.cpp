// BEAM schedule search and the on-disk plan cache, retargeted to gfx950 knobs.
// File format and keying follow crates/ksearch_codegen/src/beam.rs:67-139 and
// plan_cache.rs:9-44: one text file per (kind, dims, chip) under
// $KSEARCH_BEAM_CACHE or ~/.cache/ksearch/beam, holding key=value lines
// (tg, vec, unroll, nsg, nr0, ms; plus k_split and lds_tile, which a reader
// that does not know them skips, beam.rs:112).
#include <sys/stat.h>

#include <cerrno>
#include <cinttypes>
#include <cstdlib>
#include <functional>
#include <string>
#include <vector>

#include "ksh_internal.hpp"

namespace ksh {

int matvec_q4k_candidates(const ksh_kernel_desc &d, ksh_sched *out, int cap);
int matvec_q6k_candidates(const ksh_kernel_desc &d, ksh_sched *out, int cap);
int mul_mm_candidates(const ksh_kernel_desc &d, ksh_sched *out, int cap);

// dims that take part in a plan's key: everything up to the last non-zero entry (a zero in the middle -- a flag
// that is off, a partition count left to the schedule -- is part of the shape)
int plan_dims(const ksh_kernel_desc &d)
{
    int nd = 0;
    for (int i = 0; i < 8; i++)
        if (d.dims[i] != 0) nd = i + 1;
    return nd;
}

// Split-KV attention (sdpa_q40: KSH_SDPA_SLOTS / KSH_SDPA_BATCH with the partition count left open, and
// attend_decode_q40): K-split = partitions per sequence, waves per workgroup, and for the fused decode step the
// number of workgroups that share a kv head's rows (each with its share of the q heads).
static int sdpa_candidates(const ksh_kernel_desc &d, ksh_sched *out, int cap)
{
    const bool attend = d.kind == KSH_ATTEND_DECODE;
    const int64_t nwg_dim = attend ? d.dims[4] : d.dims[5];
    const int64_t max_t = d.dims[3], groups = d.dims[1] > 0 ? d.dims[0] / d.dims[1] : 1;
    int n = 0;
    for (uint32_t ks : {0u, 4u, 8u, 16u, 32u, 64u}) {
        if ((ks == 0) != (nwg_dim != 0)) continue;            // a fixed partition count leaves only the other knobs
        if (ks && (int64_t)ks * 32 > max_t && ks > 4) continue;   // fewer than 32 rows per partition
        for (uint32_t nsg : {4u, 8u})
            for (uint32_t hs : {1u, 2u, 4u, 8u}) {
                if (!attend && hs != 1) continue;
                if (hs > groups || groups % hs) continue;
                if (n >= cap) return n;
                ksh_sched s{};
                s.tg = 64ull * nsg; s.vec = 3; s.unroll = attend ? hs : 0; s.nsg = nsg; s.nr0 = 0; s.k_split = ks;   // vector-ALU form
                out[n++] = s;
            }
        // the matrix-core form of the row phase (several slots, heads of 256)
        const int64_t parts = ks ? ks : nwg_dim;
        if (d.dims[2] == 256 && groups <= 8 &&
            ((d.kind == KSH_SDPA_SLOTS && d.dims[4] <= 16) || (d.kind == KSH_SDPA_BATCH && d.dims[4] <= 64 && parts >= 2 && parts * d.dims[4] <= 1024)))
            for (uint32_t tile : {32u, 16u}) {                // rows per wave tile: four waves of 32 or eight of 16
                if (n >= cap) return n;
                ksh_sched s{};
                s.tg = 64ull * (128 / tile); s.vec = 2; s.unroll = 1; s.nsg = 128 / tile; s.k_split = ks; s.lds_tile = tile;
                out[n++] = s;
            }
    }
    return n;
}

namespace {

std::string cache_dir()
{
    // beam_cache_dir, beam.rs:67-79
    if (const char *p = std::getenv("KSEARCH_BEAM_CACHE")) return p;
    if (const char *h = std::getenv("HOME")) return std::string(h) + "/.cache/ksearch/beam";
    return ".ksearch_beam_cache";
}

int mkdirs(const std::string &path)
{
    std::string cur;
    for (size_t i = 0; i <= path.size(); i++) {
        if (i == path.size() || path[i] == '/') {
            if (!cur.empty() && mkdir(cur.c_str(), 0755) != 0 && errno != EEXIST) return -1;
        }
        if (i < path.size()) cur.push_back(path[i]);
    }
    return 0;
}

uint64_t fnv1a(uint64_t h, const void *data, size_t n)
{
    const unsigned char *p = (const unsigned char *)data;
    for (size_t i = 0; i < n; i++) {
        h ^= p[i];
        h *= 0x100000001b3ull;
    }
    return h;
}

std::string make_key(const char *kind, const int64_t *dims, int n_dims, const char *chip)
{
    // plan_key, plan_cache.rs:9-22: "{kind}_{d0}x{d1}.._{hash:016x}"
    uint64_t h = 0xcbf29ce484222325ull;
    h = fnv1a(h, kind, strlen(kind));
    for (int i = 0; i < n_dims; i++) {
        const uint64_t d = (uint64_t)dims[i];
        h = fnv1a(h, &d, sizeof(d));
    }
    h = fnv1a(h, chip, strlen(chip));
    std::string s = kind;
    s += "_";
    for (int i = 0; i < n_dims; i++) {
        if (i) s += "x";
        s += std::to_string((long long)dims[i]);
    }
    char hex[32];
    snprintf(hex, sizeof(hex), "_%016" PRIx64, h);
    return s + hex;
}

}  // namespace
}  // namespace ksh

using namespace ksh;

namespace {

// One candidate's time: `iters` launches timed together (weights stay in cache between them), or -- cold -- one
// launch at a time with the caches evicted in between by zero-filling `flush` (larger than the last-level cache),
// which is how a decode step meets its weights; the minimum of the single launches is taken.
int time_candidate(ksh_ctx *ctx, ksh_kernel *k, ksh_buf *const *inputs, int n_in, ksh_buf *const *outputs, int n_out, int iters,
                   ksh_buf *flush, double *ms)
{
    if (ksh_run_timed(ctx, k, inputs, nullptr, n_in, outputs, nullptr, n_out, 1, ms)) return 2;   // warm-up; a refusal shows here
    if (!flush) return ksh_run_timed(ctx, k, inputs, nullptr, n_in, outputs, nullptr, n_out, iters, ms) ? 1 : 0;
    double best = 0.0;
    for (int i = 0; i < iters; i++) {
        double t = 0.0;
        if (ksh_buffer_fill_zero(ctx, flush) || ksh_run_timed(ctx, k, inputs, nullptr, n_in, outputs, nullptr, n_out, 1, &t)) return 1;
        if (i == 0 || t < best) best = t;
    }
    *ms = best;
    return 0;
}

}  // namespace

extern "C" {

int ksh_plan_key(const char *kind, const int64_t *dims, int n_dims, const char *chip, char *dst, size_t n)
{
    if (!kind || !chip || !dst || n == 0 || n_dims < 0 || n_dims > 8 || (n_dims && !dims))
        return set_error("ksh_plan_key: bad arguments");
    snprintf(dst, n, "%s", make_key(kind, dims, n_dims, chip).c_str());
    return 0;
}

int ksh_plan_save(const char *kind, const int64_t *dims, int n_dims, const char *chip, const ksh_sched *s, double ms)
{
    if (!kind || !chip || !s || n_dims < 0 || n_dims > 8 || (n_dims && !dims))
        return set_error("ksh_plan_save: bad arguments");
    const std::string dir = cache_dir();
    if (mkdirs(dir)) return set_error("ksh_plan_save: cannot create %s", dir.c_str());
    const std::string path = dir + "/" + make_key(kind, dims, n_dims, chip) + ".txt";
    FILE *f = fopen(path.c_str(), "w");
    if (!f) return set_error("ksh_plan_save: cannot write %s", path.c_str());
    fprintf(f, "tg=%llu\nvec=%u\nunroll=%u\nnsg=%u\nnr0=%u\nms=%.6f\nk_split=%u\nlds_tile=%u\n",
            (unsigned long long)s->tg, s->vec, s->unroll, s->nsg, s->nr0, ms, s->k_split, s->lds_tile);
    fclose(f);
    return 0;
}

int ksh_plan_load(const char *kind, const int64_t *dims, int n_dims, const char *chip, ksh_sched *s, double *ms)
{
    if (!kind || !chip || !s || n_dims < 0 || n_dims > 8 || (n_dims && !dims))
        return set_error("ksh_plan_load: bad arguments");
    const std::string path = cache_dir() + "/" + make_key(kind, dims, n_dims, chip) + ".txt";
    FILE *f = fopen(path.c_str(), "r");
    if (!f) return 1;
    // load_beam_cache, beam.rs:90-123: tg, vec, unroll and ms are mandatory,
    // nsg defaults to 2 and nr0 to 4, unknown keys are skipped
    bool have_tg = false, have_vec = false, have_unroll = false, have_ms = false;
    ksh_sched r{};
    r.nsg = 2;
    r.nr0 = 4;
    double t = 0.0;
    char line[256];
    while (fgets(line, sizeof(line), f)) {
        char *eq = strchr(line, '=');
        if (!eq) continue;
        *eq = 0;
        const char *k = line, *v = eq + 1;
        char *end = nullptr;
        if (!strcmp(k, "ms")) {
            t = strtod(v, &end);
            have_ms = end != v;
            continue;
        }
        const unsigned long long u = strtoull(v, &end, 10);
        if (end == v) continue;
        if (!strcmp(k, "tg")) { r.tg = u; have_tg = true; }
        else if (!strcmp(k, "vec")) { r.vec = (uint32_t)u; have_vec = true; }
        else if (!strcmp(k, "unroll")) { r.unroll = (uint32_t)u; have_unroll = true; }
        else if (!strcmp(k, "nsg")) r.nsg = (uint32_t)u;
        else if (!strcmp(k, "nr0")) r.nr0 = (uint32_t)u;
        else if (!strcmp(k, "k_split")) r.k_split = (uint32_t)u;
        else if (!strcmp(k, "lds_tile")) r.lds_tile = (uint32_t)u;
    }
    fclose(f);
    if (!(have_tg && have_vec && have_unroll && have_ms)) return 1;
    *s = r;
    if (ms) *ms = t;
    return 0;
}

const char *ksh_plan_kind(const ksh_kernel_desc *d)
{
    if (!d) return nullptr;
    switch (d->kind) {
    case KSH_MATVEC:
        // crates/ksearch_codegen/src/lib.rs:200-205
        return d->dtypes[0] == KSH_Q4K ? "matvec_q4k" : d->dtypes[0] == KSH_Q6K ? "matvec_q6k" : d->dtypes[0] == KSH_Q6K_ROWS ? "matvec_q6krows" : nullptr;
    case KSH_RMSNORM_MATVEC:
        return d->dtypes[0] == KSH_Q4K ? "rms_matvec_q4k" : d->dtypes[0] == KSH_Q6K ? "rms_matvec_q6k" : d->dtypes[0] == KSH_Q6K_ROWS ? "rms_matvec_q6krows" : nullptr;
    case KSH_MATVEC_QKV: return "matvec_qkv_q4k";
    case KSH_RMSNORM_MATVEC_QKV: return "rms_matvec_qkv_q4k";
    case KSH_MATVEC_GATE_UP_GELU: return "matvec_gate_up_q4k";
    case KSH_RMSNORM_MATVEC_GATE_UP_GELU: return "rms_matvec_gate_up_q4k";
    case KSH_MATVEC_BATCH: return d->dtypes[0] == KSH_Q6K ? "mul_mm_q6k" : "mul_mm_q4k";
    case KSH_SDPA_SLOTS:
    case KSH_SDPA_MWG_PART: return "sdpa_q40";
    case KSH_SDPA_BATCH: return "sdpa_q40_batch";
    case KSH_ATTEND_DECODE: return "attend_decode_q40";
    case KSH_ATTN_MERGE_MATVEC: return "attn_merge_matvec_q4k";
    }
    return nullptr;
}

int ksh_beam_candidates(const ksh_kernel_desc *d, ksh_sched *out, int cap)
{
    if (!d || !out || cap <= 0) return 0;
    switch (d->kind) {
    case KSH_MATVEC:
        if (d->dtypes[0] == KSH_Q6K || d->dtypes[0] == KSH_Q6K_ROWS) return matvec_q6k_candidates(*d, out, cap);
        return matvec_q4k_candidates(*d, out, cap);
    case KSH_RMSNORM_MATVEC:
        if (d->dtypes[0] == KSH_Q6K || d->dtypes[0] == KSH_Q6K_ROWS) return matvec_q6k_candidates(*d, out, cap);
        return matvec_q4k_candidates(*d, out, cap);
    case KSH_MATVEC_QKV:
    case KSH_MATVEC_GATE_UP_GELU:
    case KSH_RMSNORM_MATVEC_QKV:
    case KSH_RMSNORM_MATVEC_GATE_UP_GELU: return matvec_q4k_candidates(*d, out, cap);
    case KSH_MATVEC_BATCH: return mul_mm_candidates(*d, out, cap);
    case KSH_SDPA_SLOTS:
    case KSH_SDPA_BATCH:
    case KSH_ATTEND_DECODE: return sdpa_candidates(*d, out, cap);
    }
    return 0;
}

// the search proper: `time_one(kernel, &ms)` returns 0, 1 (error) or 2 (this candidate cannot run: pass it over)
static int beam_search_with(ksh_ctx *ctx, const ksh_kernel_desc *desc, const std::function<int(ksh_kernel *, double *)> &time_one,
                            int force, double margin, ksh_sched *best, double *best_ms, int *from_cache)
{
    const char *pk = ksh_plan_kind(desc);
    if (!pk) return set_error("ksh_beam_search: kind %d has no schedule space", desc->kind);
    char chip[128];
    if (ksh_device_name(ctx, chip, sizeof(chip))) return 1;
    const int nd = plan_dims(*desc);
    if (from_cache) *from_cache = 0;
    // KSEARCH_BEAM_FORCE, crates/ksearch_codegen/src/lib.rs:206
    if (!(force & 1) && !std::getenv("KSEARCH_BEAM_FORCE") && ksh_plan_load(pk, desc->dims, nd, chip, best, best_ms) == 0) {
        if (from_cache) *from_cache = 1;
        return 0;
    }
    std::vector<ksh_sched> cand(128);
    const int n = ksh_beam_candidates(desc, cand.data(), (int)cand.size());
    if (n <= 0) return set_error("ksh_beam_search: no candidates for kind %d", desc->kind);
    bool found = false;
    std::string refusal;
    // The library's own default goes first: a candidate replaces it only when it is faster by the margin, so that
    // timing noise between near-equal schedules does not move a shape off the schedule its default was chosen for.
    double default_ms = 0.0;
    {
        ksh_kernel_desc d = *desc;
        memset(&d.sched, 0, sizeof(d.sched));
        d.sched.tg = ~0ull;   // the library default, whatever the plan cache holds
        ksh_kernel *k = nullptr;
        double ms = 0.0;
        if (ksh_kernel_get(ctx, &d, &k) == 0 && time_one(k, &ms) == 0) {
            ksh_kernel_info info;
            ksh_kernel_info_get(k, &info);
            found = true;
            default_ms = ms;
            *best_ms = ms;
            *best = info.sched;
        }
    }
    for (int i = 0; i < n; i++) {
        ksh_kernel_desc d = *desc;
        d.sched = cand[i];
        ksh_kernel *k = nullptr;
        if (ksh_kernel_get(ctx, &d, &k)) continue;   // a candidate the kernel family refuses
        double ms = 0.0;
        // A candidate whose bindings do not fit (a partition count the caller's scratch buffer was not sized for) is
        // passed over like a refused one.
        const int rc = time_one(k, &ms);
        if (rc == 2) {
            refusal = ksh_last_error();
            continue;
        }
        if (rc) return 1;
        if (!found || (ms < *best_ms && (default_ms == 0.0 || ms < margin * default_ms))) {
            found = true;
            *best_ms = ms;
            *best = cand[i];
        }
    }
    if (!found) return set_error("ksh_beam_search: every candidate was refused (%s)", refusal.c_str());
    return ksh_plan_save(pk, desc->dims, nd, chip, best, *best_ms);
}

int ksh_beam_search(ksh_ctx *ctx, const ksh_kernel_desc *desc, ksh_buf *const *inputs, int n_in,
                    ksh_buf *const *outputs, int n_out, int iters, int force, ksh_sched *best, double *best_ms,
                    int *from_cache)
{
    if (!ctx || !desc || !best || !best_ms) return set_error("ksh_beam_search: bad arguments");
    if (iters < 1) iters = 3;
    // force & 2: cold timing
    ksh_buf *flush = nullptr;
    if ((force & 2) && ksh_buffer_alloc(ctx, (size_t)384 << 20, nullptr, &flush)) return 1;
    struct Release {
        ksh_buf *b;
        ~Release() { if (b) ksh_buffer_release(b); }
    } release{flush};
    // 1 warm-up + timed launches, crates/ksearch_kernels/src/lib.rs:2015-2031
    auto time_one = [&](ksh_kernel *k, double *ms) { return time_candidate(ctx, k, inputs, n_in, outputs, n_out, iters, flush, ms); };
    return beam_search_with(ctx, desc, time_one, force, flush ? 0.90 : 0.97, best, best_ms, from_cache);
}

int ksh_beam_search_chain(ksh_ctx *ctx, const ksh_kernel_desc *desc, int n_sets, ksh_buf *const *input_sets, int n_in,
                          ksh_buf *const *output_sets, int n_out, int iters, int force, ksh_sched *best, double *best_ms,
                          int *from_cache)
{
    if (!ctx || !desc || !best || !best_ms || !input_sets || !output_sets || n_sets < 1 || n_in < 1 || n_out < 1) return set_error("ksh_beam_search_chain: bad arguments");
    if (iters < 1) iters = 3;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    KSH_HIP(hipEventCreate(&e0));
    KSH_HIP(hipEventCreate(&e1));
    struct Events {
        hipEvent_t a, b;
        ~Events() { (void)hipEventDestroy(a); (void)hipEventDestroy(b); }
    } events{e0, e1};
    hipStream_t st = (hipStream_t)ksh_stream(ctx);
    auto time_one = [&](ksh_kernel *k, double *ms) -> int {
        // the candidate as the decode loop runs it: one HIP graph of n_sets dependent launches, each over another
        // set of inputs (another layer's weights: cold), replayed a few times; the best replay counts
        if (ksh_synchronize(ctx) || ksh_graph_begin(ctx)) return 1;
        int rc = 0;
        for (int s2 = 0; s2 < n_sets && !rc; s2++)
            if (ksh_encode(ctx, k, input_sets + (size_t)s2 * n_in, nullptr, n_in, output_sets + (size_t)s2 * n_out, nullptr, n_out)) rc = 2;
        ksh_graph *g = nullptr;
        if (ksh_graph_end(ctx, &g)) return 1;
        double best_t = 0.0;
        if (!rc && ksh_graph_launch(ctx, g)) rc = 1;
        for (int i = 0; i < iters && !rc; i++) {
            float t = 0.f;
            if (hipEventRecord(e0, st) != hipSuccess || ksh_graph_launch(ctx, g) || hipEventRecord(e1, st) != hipSuccess ||
                hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&t, e0, e1) != hipSuccess)
                rc = 1;
            if (i == 0 || t < best_t) best_t = t;
        }
        if (ksh_synchronize(ctx)) rc = rc ? rc : 1;
        ksh_graph_destroy(g);
        *ms = best_t / n_sets;
        return rc;
    };
    return beam_search_with(ctx, desc, time_one, force, 0.97, best, best_ms, from_cache);
}

}  // extern "C"
