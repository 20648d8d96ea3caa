// libksearch_hip runtime: context, buffers, kernel handles, encode / flush /
// wait / barrier / synchronize, timed run and HIP-graph capture.  This is the
// gfx950 counterpart of crates/ksearch_metal/src/lib.rs (MetalContext); each
// entry point cites the method it stands in for in include/ksearch_hip.h.
#include <cstdlib>
#include <deque>
#include <map>
#include <memory>
#include <vector>

#include "ksh_internal.hpp"

namespace ksh {

static thread_local std::string g_err;

int set_error(const char *fmt, ...)
{
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_err = buf;
    return 1;
}

int hip_fail(hipError_t e, const char *what)
{
    return set_error("HIP error %d (%s) in %s", (int)e, hipGetErrorString(e), what);
}

int bind_matvec(ksh_kernel &k)
{
    if (k.desc.dtypes[1] != KSH_F32 && k.desc.dtypes[1] != 0)
        return set_error("matvec: activation dtype %d is not built (f32 only)", k.desc.dtypes[1]);
    switch (k.desc.dtypes[0]) {
    case KSH_Q4K: return bind_matvec_q4k(k);
    case KSH_Q6K:
    case KSH_Q6K_ROWS: return bind_matvec_q6k(k);
    }
    // unsupported dtype in lowering is an error, crates/ksearch_codegen/src/lower.rs:44-48
    return set_error("matvec: weight dtype %d is not built (Q4_K and Q6_K are)", k.desc.dtypes[0]);
}

static int bind(ksh_kernel &k)
{
    switch (k.desc.kind) {
    case KSH_MATVEC: return bind_matvec(k);
    case KSH_MATVEC_BATCH: return bind_matvec_batch(k);
    case KSH_MATVEC_QKV: return bind_matvec_qkv(k);
    case KSH_MATVEC_GATE_UP_GELU: return bind_matvec_gate_up_gelu(k);
    case KSH_RMSNORM_MATVEC: return bind_matvec(k);
    case KSH_RMSNORM_MATVEC_QKV:
    case KSH_RMSNORM_MATVEC_GATE_UP_GELU:
    case KSH_ATTN_MERGE_MATVEC: return bind_matvec_q4k_family(k);
    case KSH_SDPA_NAIVE:
    case KSH_SDPA_MWG_PART:
    case KSH_SDPA_MWG_REDUCE:
    case KSH_SDPA_SLOTS:
    case KSH_SDPA_BATCH: return bind_sdpa(k);
    case KSH_ATTEND_DECODE: return bind_attend_decode(k);
    case KSH_QUANTIZE_Q40: return bind_quantize_q40(k);
    case KSH_RMSNORM:
    case KSH_RMSNORM_ADD_THEN_RMSNORM: return bind_rmsnorm(k);
    case KSH_RMSNORM_PER_HEAD_QKV_Q40: return bind_per_head_qkv_q40(k);
    case KSH_COPY_SCALE_INDEXED:
    case KSH_GELU_MUL:
    case KSH_COPY_SLICE: return bind_glue(k);
    case KSH_SOFTCAP_ARGMAX: return bind_softcap_argmax(k);
    case KSH_DEQUANT: return bind_dequant(k);
    case KSH_REPACK_ROWS: return bind_repack_rows(k);
    case KSH_QUANTIZE_K: return bind_quantize_k(k);
    case KSH_RMSNORM_PER_HEAD:
    case KSH_ADD_SCALE:
    case KSH_MATVEC_GELU_MUL: return bind_ple_ops(k);
    case KSH_READ_FLOOR: return bind_read_floor(k);
    case KSH_ROUND_PREP: return bind_round_prep(k);
    case KSH_MATVEC_ROUND: return bind_matvec_round(k);
    }
    return set_error("unknown kernel kind %d", k.desc.kind);
}

struct DescLess {
    bool operator()(const ksh_kernel_desc &a, const ksh_kernel_desc &b) const
    {
        return memcmp(&a, &b, sizeof(a)) < 0;
    }
};

}  // namespace ksh

struct ksh_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
};

struct ksh_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    hipStream_t copy_stream = nullptr;   // host<->device copies that must not wait for queued kernels
    hipEvent_t copy_done = nullptr;
    std::string chip;
    std::map<ksh_kernel_desc, std::unique_ptr<ksh_kernel>, ksh::DescLess> kernels;
    std::deque<hipEvent_t> inflight;   // one event per flush_async
    std::vector<hipEvent_t> free_events;
    bool pending = false;              // work encoded since the last flush
    bool capturing = false;
    hipEvent_t t0 = nullptr, t1 = nullptr;
};

namespace ksh {
hipStream_t ctx_stream(ksh_ctx *ctx) { return ctx->stream; }
int ctx_device(ksh_ctx *ctx) { return ctx->device; }
ksh_buf *buffer_view(ksh_buf *parent, size_t off, size_t bytes)
{
    if (!parent || off > parent->bytes || bytes > parent->bytes - off) {
        set_error("buffer_view: range [%zu, %zu) is outside the buffer", off, off + bytes);
        return nullptr;
    }
    ksh_buf *v = new ksh_buf();
    v->ptr = (char *)parent->ptr + off;
    v->bytes = bytes;
    v->parent = parent;
    ksh_buffer_retain(parent);
    return v;
}
void ctx_mark_pending(ksh_ctx *ctx) { ctx->pending = true; }
}  // namespace ksh

using namespace ksh;

extern "C" {

const char *ksh_last_error(void) { return g_err.c_str(); }

int ksh_ctx_create(ksh_ctx **out)
{
    if (!out) return set_error("ksh_ctx_create: null out");
    *out = nullptr;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n < 1) return set_error("no HIP device is usable (%s)", hipGetErrorString(e));
    KSH_HIP(hipSetDevice(0));
    hipDeviceProp_t prop;
    KSH_HIP(hipGetDeviceProperties(&prop, 0));
    std::string arch = prop.gcnArchName;
    const size_t colon = arch.find(':');
    if (colon != std::string::npos) arch.resize(colon);
    if (arch != "gfx950")
        return set_error("device 0 is %s; this library only carries gfx950 code", arch.c_str());
    auto ctx = std::make_unique<ksh_ctx>();
    const char *chip = std::getenv("KSEARCH_CHIP");
    ctx->chip = (chip && *chip) ? chip : arch;
    KSH_HIP(hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking));
    KSH_HIP(hipStreamCreateWithFlags(&ctx->copy_stream, hipStreamNonBlocking));
    KSH_HIP(hipEventCreateWithFlags(&ctx->copy_done, hipEventDisableTiming));
    KSH_HIP(hipEventCreate(&ctx->t0));
    KSH_HIP(hipEventCreate(&ctx->t1));
    if (argmax_static_setup()) return 1;
    *out = ctx.release();
    return 0;
}

void ksh_ctx_destroy(ksh_ctx *ctx)
{
    if (!ctx) return;
    ksh_synchronize(ctx);
    for (hipEvent_t e : ctx->free_events) (void)hipEventDestroy(e);
    for (auto &kv : ctx->kernels)
        if (kv.second->scratch) (void)hipFree(kv.second->scratch);
    if (ctx->t0) (void)hipEventDestroy(ctx->t0);
    if (ctx->t1) (void)hipEventDestroy(ctx->t1);
    if (ctx->copy_done) (void)hipEventDestroy(ctx->copy_done);
    if (ctx->copy_stream) (void)hipStreamDestroy(ctx->copy_stream);
    if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

int ksh_device_name(ksh_ctx *ctx, char *dst, size_t n)
{
    if (!ctx || !dst || n == 0) return set_error("ksh_device_name: bad arguments");
    snprintf(dst, n, "%s", ctx->chip.c_str());
    return 0;
}

void *ksh_stream(ksh_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

int ksh_buffer_alloc(ksh_ctx *ctx, size_t bytes, const void *init, ksh_buf **out)
{
    if (!ctx || !out) return set_error("ksh_buffer_alloc: bad arguments");
    *out = nullptr;
    auto b = std::make_unique<ksh_buf>();
    b->bytes = bytes;
    // a zero-length buffer still gets an address, so offsets into it stay checkable
    KSH_HIP(hipMalloc(&b->ptr, bytes ? bytes : 16));
    hipError_t e = init ? hipMemcpy(b->ptr, init, bytes, hipMemcpyHostToDevice)
                        : hipMemset(b->ptr, 0, bytes ? bytes : 16);
    // hipMemset of device memory may return before the fill has run, and the fill is on the null stream, which the
    // context's non-blocking streams do not wait for: finish it here, or a kernel's output can be zeroed after the fact
    if (e == hipSuccess && !init) e = hipStreamSynchronize(nullptr);
    if (e != hipSuccess) {
        (void)hipFree(b->ptr);
        return hip_fail(e, "buffer init");
    }
    *out = b.release();
    return 0;
}

void ksh_buffer_retain(ksh_buf *buf)
{
    if (buf) buf->rc.fetch_add(1);
}

void ksh_buffer_release(ksh_buf *buf)
{
    if (buf && buf->rc.fetch_sub(1) == 1) {
        if (buf->parent)
            ksh_buffer_release(buf->parent);
        else
            (void)hipFree(buf->ptr);
        delete buf;
    }
}

size_t ksh_buffer_size(const ksh_buf *buf) { return buf ? buf->bytes : 0; }
void *ksh_buffer_device_ptr(const ksh_buf *buf) { return buf ? buf->ptr : nullptr; }

static int range_ok(const ksh_buf *buf, size_t off, size_t bytes, const char *what)
{
    if (!buf) return set_error("%s: null buffer", what);
    if (off > buf->bytes || bytes > buf->bytes - off)
        return set_error("%s: range [%zu, %zu) exceeds the buffer's %zu bytes", what, off, off + bytes, buf->bytes);
    return 0;
}

int ksh_buffer_write(ksh_ctx *ctx, ksh_buf *buf, size_t off, const void *src, size_t bytes, int sync)
{
    if (!ctx || (!src && bytes)) return set_error("ksh_buffer_write: bad arguments");
    if (range_ok(buf, off, bytes, "ksh_buffer_write")) return 1;
    if (ctx->capturing) return set_error("ksh_buffer_write: not allowed while a graph is being captured");
    if (sync && ksh_synchronize(ctx)) return 1;
    if (!bytes) return 0;
    // The copy runs on its own stream so that a nosync write does not wait for
    // kernels already queued (the reference writes straight into shared
    // memory); kernels encoded after this call are ordered behind it.
    KSH_HIP(hipMemcpyAsync((char *)buf->ptr + off, src, bytes, hipMemcpyHostToDevice, ctx->copy_stream));
    KSH_HIP(hipEventRecord(ctx->copy_done, ctx->copy_stream));
    KSH_HIP(hipStreamWaitEvent(ctx->stream, ctx->copy_done, 0));
    KSH_HIP(hipStreamSynchronize(ctx->copy_stream));
    return 0;
}

int ksh_buffer_read(ksh_ctx *ctx, ksh_buf *buf, size_t off, void *dst, size_t bytes, int sync)
{
    if (!ctx || (!dst && bytes)) return set_error("ksh_buffer_read: bad arguments");
    if (range_ok(buf, off, bytes, "ksh_buffer_read")) return 1;
    if (ctx->capturing) return set_error("ksh_buffer_read: not allowed while a graph is being captured");
    if (sync && ksh_synchronize(ctx)) return 1;
    if (!bytes) return 0;
    KSH_HIP(hipMemcpyAsync(dst, (const char *)buf->ptr + off, bytes, hipMemcpyDeviceToHost, ctx->copy_stream));
    KSH_HIP(hipStreamSynchronize(ctx->copy_stream));
    return 0;
}

// defined with the glue kernels: a plain fill kernel, safe under graph capture
int ksh_fill_zero_launch(void *ptr, size_t bytes, hipStream_t st);

int ksh_buffer_fill_zero(ksh_ctx *ctx, ksh_buf *buf)
{
    if (!ctx || !buf) return set_error("ksh_buffer_fill_zero: bad arguments");
    if (!buf->bytes) return 0;
    if (ksh_fill_zero_launch(buf->ptr, buf->bytes, ctx->stream)) return 1;
    ctx->pending = true;
    return 0;
}

int ksh_kernel_get(ksh_ctx *ctx, const ksh_kernel_desc *desc, ksh_kernel **out)
{
    if (!ctx || !desc || !out) return set_error("ksh_kernel_get: bad arguments");
    *out = nullptr;
    ksh_kernel_desc key;
    memset(&key, 0, sizeof(key));   // padding bytes take part in the map's ordering
    key.kind = desc->kind;
    memcpy(key.dtypes, desc->dtypes, sizeof(key.dtypes));
    memcpy(key.dims, desc->dims, sizeof(key.dims));
    memcpy(key.params, desc->params, sizeof(key.params));
    key.sched.tg = desc->sched.tg; key.sched.vec = desc->sched.vec; key.sched.unroll = desc->sched.unroll;
    key.sched.nsg = desc->sched.nsg; key.sched.nr0 = desc->sched.nr0; key.sched.k_split = desc->sched.k_split;
    key.sched.lds_tile = desc->sched.lds_tile;
    auto it = ctx->kernels.find(key);
    if (it != ctx->kernels.end()) {
        *out = it->second.get();
        return 0;
    }
    if (key.dtypes[1] == KSH_F16 && half_boundary_kind(key)) {
        // half activations at the boundary: the f32 handle of the same descriptor, wrapped (half_boundary.hip)
        ksh_kernel_desc f32 = *desc;
        f32.dtypes[1] = KSH_F32;
        if (key.kind == KSH_MATVEC_BATCH && f32.dtypes[2] == KSH_F16) f32.dtypes[2] = KSH_F32;
        ksh_kernel *inner = nullptr;
        if (ksh_kernel_get(ctx, &f32, &inner)) return 1;
        auto k = std::make_unique<ksh_kernel>();
        k->desc = key;
        if (bind_half_boundary(*k, *inner)) return 1;
        if (k->scratch_bytes) {
            KSH_HIP(hipMalloc(&k->scratch, k->scratch_bytes));
            KSH_HIP(hipMemset(k->scratch, 0, k->scratch_bytes));
            KSH_HIP(hipStreamSynchronize(nullptr));
        }
        *out = k.get();
        ctx->kernels[key] = std::move(k);
        return 0;
    }
    ksh_sched planned{};
    bool have_plan = false;
    // tg = all ones asks for the library's default schedule whatever the plan cache holds (the schedule search times
    // it as the incumbent); such a handle has its own cache entry
    const bool library_default = key.sched.tg == ~0ull;
    if (sched_is_zero(key.sched)) {
        // plan lookup by (kind, dims, chip), crates/ksearch_codegen/src/lib.rs:80-90
        const char *pk = ksh_plan_kind(&key);
        if (pk) {
            double ms;
            have_plan = ksh_plan_load(pk, key.dims, plan_dims(key), ctx->chip.c_str(), &planned, &ms) == 0;
        }
    }
    auto k = std::make_unique<ksh_kernel>();
    k->desc = key;
    if (have_plan) k->desc.sched = planned;
    if (library_default) memset(&k->desc.sched, 0, sizeof(k->desc.sched));
    if (bind(*k)) {
        // a stale or foreign plan must not make a kernel unusable
        if (!have_plan) return 1;
        fprintf(stderr, "[ksearch_hip] plan for kind %d refused (%s); using the default schedule\n", key.kind, ksh_last_error());
        k = std::make_unique<ksh_kernel>();
        k->desc = key;
        if (bind(*k)) return 1;
    }
    if (!k->launch) return set_error("kernel kind %d bound without a launcher", key.kind);
    if (k->scratch_bytes) {
        KSH_HIP(hipMalloc(&k->scratch, k->scratch_bytes));
        KSH_HIP(hipMemset(k->scratch, 0, k->scratch_bytes));
        KSH_HIP(hipStreamSynchronize(nullptr));   // see ksh_buffer_alloc
    }
    *out = k.get();
    ctx->kernels[key] = std::move(k);
    return 0;
}

int ksh_kernel_info_get(const ksh_kernel *k, ksh_kernel_info *info)
{
    if (!k || !info) return set_error("ksh_kernel_info_get: bad arguments");
    *info = k->info;
    return 0;
}

static int gather_args(const ksh_kernel *k, ksh_buf *const *inputs, const uint64_t *in_off, int n_in,
                       ksh_buf *const *outputs, const uint64_t *out_off, int n_out, LaunchArgs &a)
{
    // same checks, same wording, as encode_offsets_multi (ksearch_metal/src/lib.rs:280-307)
    if (n_in != k->info.n_inputs) return set_error("expected %d inputs, got %d", k->info.n_inputs, n_in);
    if (n_out != k->info.n_outputs) return set_error("expected %d outputs, got %d", k->info.n_outputs, n_out);
    if ((n_in && !inputs) || (n_out && !outputs)) return set_error("null binding array");
    memset(&a, 0, sizeof(a));
    for (int i = 0; i < n_in; i++) {
        const uint64_t off = in_off ? in_off[i] : 0;
        if (!inputs[i]) return set_error("%s: input %d is null", k->info.name, i);
        if (off > inputs[i]->bytes || k->in_bytes[i] > inputs[i]->bytes - off)
            return set_error("%s: input %d needs %zu bytes from offset %llu, buffer has %zu", k->info.name, i,
                             k->in_bytes[i], (unsigned long long)off, inputs[i]->bytes);
        const uintptr_t p = (uintptr_t)inputs[i]->ptr + off;
        if (k->in_align[i] > 1 && p % k->in_align[i])
            return set_error("%s: input %d offset %llu is not %u-byte aligned", k->info.name, i,
                             (unsigned long long)off, k->in_align[i]);
        a.in[i] = (const void *)p;
    }
    for (int i = 0; i < n_out; i++) {
        const uint64_t off = out_off ? out_off[i] : 0;
        if (!outputs[i]) return set_error("%s: output %d is null", k->info.name, i);
        if (off > outputs[i]->bytes || k->out_bytes[i] > outputs[i]->bytes - off)
            return set_error("%s: output %d needs %zu bytes from offset %llu, buffer has %zu", k->info.name, i,
                             k->out_bytes[i], (unsigned long long)off, outputs[i]->bytes);
        const uintptr_t p = (uintptr_t)outputs[i]->ptr + off;
        if (k->out_align[i] > 1 && p % k->out_align[i])
            return set_error("%s: output %d offset %llu is not %u-byte aligned", k->info.name, i,
                             (unsigned long long)off, k->out_align[i]);
        a.out[i] = (void *)p;
    }
    return 0;
}

int ksh_encode(ksh_ctx *ctx, ksh_kernel *k, ksh_buf *const *inputs, const uint64_t *in_off, int n_in,
               ksh_buf *const *outputs, const uint64_t *out_off, int n_out)
{
    if (!ctx || !k) return set_error("ksh_encode: bad arguments");
    LaunchArgs a;
    if (gather_args(k, inputs, in_off, n_in, outputs, out_off, n_out, a)) return 1;
    if (k->launch(*k, a, ctx->stream)) return 1;
    ctx->pending = true;
    return 0;
}

int ksh_run_timed(ksh_ctx *ctx, ksh_kernel *k, ksh_buf *const *inputs, const uint64_t *in_off, int n_in,
                  ksh_buf *const *outputs, const uint64_t *out_off, int n_out, int iters, double *ms)
{
    if (!ctx || !k || !ms || iters < 1) return set_error("ksh_run_timed: bad arguments");
    if (ctx->capturing) return set_error("ksh_run_timed: not allowed while a graph is being captured");
    LaunchArgs a;
    if (gather_args(k, inputs, in_off, n_in, outputs, out_off, n_out, a)) return 1;
    if (ksh_synchronize(ctx)) return 1;
    KSH_HIP(hipEventRecord(ctx->t0, ctx->stream));
    for (int i = 0; i < iters; i++)
        if (k->launch(*k, a, ctx->stream)) return 1;
    KSH_HIP(hipEventRecord(ctx->t1, ctx->stream));
    KSH_HIP(hipEventSynchronize(ctx->t1));
    float t = 0.f;
    KSH_HIP(hipEventElapsedTime(&t, ctx->t0, ctx->t1));
    *ms = (double)t / iters;
    return 0;
}

int ksh_flush_async(ksh_ctx *ctx)
{
    if (!ctx) return set_error("ksh_flush_async: null context");
    if (ctx->capturing) return set_error("ksh_flush_async: not allowed while a graph is being captured");
    if (!ctx->pending) return 0;
    // launches are already on the stream; the event is what "committed command
    // buffer" means here
    hipEvent_t ev;
    if (!ctx->free_events.empty()) {
        ev = ctx->free_events.back();
        ctx->free_events.pop_back();
    } else {
        KSH_HIP(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
    }
    KSH_HIP(hipEventRecord(ev, ctx->stream));
    ctx->inflight.push_back(ev);
    ctx->pending = false;
    return 0;
}

int ksh_wait_inflight_at_most(ksh_ctx *ctx, int n)
{
    if (!ctx || n < 0) return set_error("ksh_wait_inflight_at_most: bad arguments");
    while ((int)ctx->inflight.size() > n) {
        KSH_HIP(hipEventSynchronize(ctx->inflight.front()));
        ctx->free_events.push_back(ctx->inflight.front());
        ctx->inflight.pop_front();
    }
    // also reap what has completed already (ksearch_metal/src/lib.rs:181-191)
    while (!ctx->inflight.empty() && hipEventQuery(ctx->inflight.front()) == hipSuccess) {
        ctx->free_events.push_back(ctx->inflight.front());
        ctx->inflight.pop_front();
    }
    return 0;
}

int ksh_barrier(ksh_ctx *ctx)
{
    // one in-order stream already orders earlier launches before later ones
    return ctx ? 0 : set_error("ksh_barrier: null context");
}

int ksh_synchronize(ksh_ctx *ctx)
{
    if (!ctx) return set_error("ksh_synchronize: null context");
    if (ctx->capturing) return set_error("ksh_synchronize: not allowed while a graph is being captured");
    KSH_HIP(hipStreamSynchronize(ctx->stream));
    for (hipEvent_t e : ctx->inflight) ctx->free_events.push_back(e);
    ctx->inflight.clear();
    ctx->pending = false;
    return 0;
}

int ksh_has_gpu_work(ksh_ctx *ctx)
{
    if (!ctx) return 0;
    return (ctx->pending || !ctx->inflight.empty()) ? 1 : 0;
}

int ksh_graph_begin(ksh_ctx *ctx)
{
    if (!ctx) return set_error("ksh_graph_begin: null context");
    if (ctx->capturing) return set_error("ksh_graph_begin: a capture is already open");
    KSH_HIP(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    ctx->capturing = true;
    return 0;
}

int ksh_graph_end(ksh_ctx *ctx, ksh_graph **out)
{
    if (!ctx || !out) return set_error("ksh_graph_end: bad arguments");
    if (!ctx->capturing) return set_error("ksh_graph_end: no capture is open");
    ctx->capturing = false;
    auto g = std::make_unique<ksh_graph>();
    KSH_HIP(hipStreamEndCapture(ctx->stream, &g->graph));
    hipError_t e = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(g->graph);
        return hip_fail(e, "hipGraphInstantiate");
    }
    ctx->pending = false;
    *out = g.release();
    return 0;
}

int ksh_graph_launch(ksh_ctx *ctx, ksh_graph *g)
{
    if (!ctx || !g) return set_error("ksh_graph_launch: bad arguments");
    KSH_HIP(hipGraphLaunch(g->exec, ctx->stream));
    ctx->pending = true;
    return 0;
}

void ksh_graph_destroy(ksh_graph *g)
{
    if (!g) return;
    if (g->exec) (void)hipGraphExecDestroy(g->exec);
    if (g->graph) (void)hipGraphDestroy(g->graph);
    delete g;
}

}  // extern "C"
