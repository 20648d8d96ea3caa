// Half-precision activations at the boundary (descriptor dtypes[1] = KSH_F16).
//
// The reference's runtime keeps every activation, norm weight and the logits in half buffers and computes in f32
// inside its kernels (x_dtype, crates/ksearch_codegen/src/lower.rs:1134-1140; buffer_empty_f16,
// crates/ksearch_gemma/src/gemma_prim.rs:229-252; the norm weights :164-182).  A handle asked for with that
// activation type takes such buffers as they are: what it binds as "activation" (vectors, norm weights, logits) is
// half, everything else keeps its type -- packed weights and caches, and the buffers the reference keeps in f32
// (the rope table :33-56, the meta record :637, token ids, split-KV partials, the argmax index).
//
// Mechanics: the handle wraps the f32 handle of the same descriptor.  One launch widens all half inputs into f32
// staging that belongs to the handle, the f32 kernel runs on the staging, one launch narrows the results
// (round to nearest even, what the reference's kernels do when they store a half).  Arithmetic is therefore the
// f32 path's, bit for bit, on the widened inputs.  The decode loops inside the library keep f32 activations and do
// not pay the two conversion launches.
#include "ksh_device.hpp"
#include "ksh_internal.hpp"

namespace ksh {
namespace {

constexpr int kMaxSeg = kMaxIn;   // >= kMaxOut

struct Segments {
    const void *src[kMaxSeg];
    void *dst[kMaxSeg];
    uint32_t n[kMaxSeg];
    int count;
};

// grid = (blocks, segments): widen (WIDEN) half -> f32 or narrow f32 -> half, 8 elements per thread
template <bool WIDEN>
__global__ __launch_bounds__(256) void convert_segments_kernel(Segments s)
{
    // (a run-time index into the by-value argument: the struct is small and read once per thread)
    const int seg = blockIdx.y;
    const uint32_t n = s.n[seg];
    const size_t i0 = ((size_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (i0 >= n) return;
    if (WIDEN) {
        const __half *src = (const __half *)s.src[seg];
        float *dst = (float *)s.dst[seg];
        for (int e = 0; e < 8 && i0 + e < n; e++) dst[i0 + e] = __half2float(src[i0 + e]);
    } else {
        const float *src = (const float *)s.src[seg];
        __half *dst = (__half *)s.dst[seg];
        for (int e = 0; e < 8 && i0 + e < n; e++) dst[i0 + e] = __float2half_rn(src[i0 + e]);
    }
}

template <bool WIDEN>
int convert(const Segments &s, hipStream_t st)
{
    if (!s.count) return 0;
    uint32_t most = 0;
    for (int i = 0; i < s.count; i++) most = most > s.n[i] ? most : s.n[i];
    const unsigned blocks = (unsigned)((most + 2047) / 2048);
    hipLaunchKernelGGL(convert_segments_kernel<WIDEN>, dim3(blocks ? blocks : 1, s.count), dim3(256), 0, st, s);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, "half boundary conversion launch");
}

int launch_half(const ksh_kernel &k, const LaunchArgs &a, hipStream_t st)
{
    const ksh_kernel &in = *k.inner;
    LaunchArgs b = a;
    Segments wide{}, narrow{};
    char *stage = (char *)k.scratch;
    for (int i = 0; i < in.info.n_inputs; i++)
        if (k.half_in >> i & 1) {
            void *f = stage + k.stage_in[i];
            wide.src[wide.count] = a.in[i]; wide.dst[wide.count] = f; wide.n[wide.count] = (uint32_t)(in.in_bytes[i] / 4);
            wide.count++;
            b.in[i] = f;
        }
    for (int i = 0; i < in.info.n_outputs; i++)
        if (k.half_out >> i & 1) {
            void *f = stage + k.stage_out[i];
            narrow.src[narrow.count] = f; narrow.dst[narrow.count] = a.out[i]; narrow.n[narrow.count] = (uint32_t)(in.out_bytes[i] / 4);
            narrow.count++;
            b.out[i] = f;
        }
    if (convert<true>(wide, st)) return 1;
    if (in.launch(in, b, st)) return 1;
    return convert<false>(narrow, st);
}

// Which bindings of a kind are activations: one letter per binding, 'A' activation (half at this boundary),
// anything else keeps its type ('W' packed bytes, 'F' f32: meta, rope, token ids, partials, indices).
bool patterns(const ksh_kernel_desc &d, int n_in, int n_out, std::string &pin, std::string &pout)
{
    auto rest = [](const char *head, int n, char c) {
        std::string s(head);
        while ((int)s.size() < n) s.push_back(c);
        return s;
    };
    switch (d.kind) {
    case KSH_MATVEC: pin = "WA"; pout = "A"; return true;
    case KSH_MATVEC_QKV: pin = "WWWA"; pout = "AAA"; return true;
    case KSH_MATVEC_GATE_UP_GELU: pin = "WWA"; pout = "A"; return true;
    case KSH_MATVEC_BATCH:
        // the plain form: X (and Y when dtypes[2] asks for it) half; the producers-inside and unfolded-slice forms are the
        // library's own prompt pass
        if (d.dims[5] || d.dims[6] || d.dims[7]) return false;
        pin = rest("WA", n_in, 'W');
        pout = std::string((size_t)n_out, d.dtypes[2] == KSH_F16 ? 'A' : 'F');
        return true;
    case KSH_SDPA_NAIVE: pin = "AWWF"; pout = "A"; return true;
    case KSH_SDPA_MWG_PART: pin = "AWWF"; pout = "F"; return true;
    case KSH_SDPA_MWG_REDUCE: pin = "F"; pout = "A"; return true;
    case KSH_SDPA_SLOTS:
    case KSH_SDPA_BATCH:
        if (d.kind == KSH_SDPA_SLOTS && d.params[1] != 0.f) return false;   // the prepared operand is no activation buffer
        pin = rest("AWWF", n_in, 'F'); pout = "FA"; return true;
    case KSH_RMSNORM: pin = rest("", n_in, 'A'); pout = "A"; return true;
    case KSH_RMSNORM_ADD_THEN_RMSNORM: pin = "AAAA"; pout = "AA"; return true;
    case KSH_RMSNORM_PER_HEAD_QKV_Q40: pin = rest("AAFAAA", n_in, 'F'); pout = "AWW"; return true;
    case KSH_COPY_SCALE_INDEXED: pin = "WF"; pout = "A"; return true;
    case KSH_GELU_MUL: pin = "AA"; pout = "A"; return true;
    case KSH_COPY_SLICE: pin = "A"; pout = "A"; return true;
    case KSH_SOFTCAP_ARGMAX: pin = "A"; pout = "F"; return true;
    case KSH_RMSNORM_MATVEC: pin = rest("W", n_in, 'A'); pout = rest("", n_out, 'A'); return true;
    case KSH_RMSNORM_MATVEC_QKV: pin = rest("WWW", n_in, 'A'); pout = rest("", n_out, 'A'); return true;
    case KSH_RMSNORM_MATVEC_GATE_UP_GELU: pin = rest("WW", n_in, 'A'); pout = rest("", n_out, 'A'); return true;
    case KSH_ATTEND_DECODE:
        pin = d.dims[7] ? "AAFWWF" : "AAFAAAF";
        pout = std::string(d.dims[7] ? "" : "WW") + (d.dims[5] ? "F" : "FA");
        return true;
    case KSH_ATTN_MERGE_MATVEC: pin = "WF"; pout = "A"; return true;
    case KSH_RMSNORM_PER_HEAD: pin = rest("AA", n_in, 'F'); pout = "A"; return true;
    case KSH_ADD_SCALE: pin = "AA"; pout = "A"; return true;
    case KSH_MATVEC_GELU_MUL: pin = rest("W", n_in, 'A'); pout = rest("", n_out, 'A'); return true;
    }
    return false;
}

}  // namespace

bool half_boundary_kind(const ksh_kernel_desc &d)
{
    std::string a, b;
    return patterns(d, kMaxIn, kMaxOut, a, b);
}

// `k.desc` asks for half activations; `inner` is the bound f32 handle of the same descriptor
int bind_half_boundary(ksh_kernel &k, const ksh_kernel &inner)
{
    std::string pin, pout;
    if (!patterns(k.desc, inner.info.n_inputs, inner.info.n_outputs, pin, pout) || (int)pin.size() != inner.info.n_inputs ||
        (int)pout.size() != inner.info.n_outputs)
        return set_error("kind %d: half activations are not built for this form of the kind", k.desc.kind);
    k.inner = &inner;
    k.info = inner.info;
    size_t off = 0;
    auto take = [&](size_t bytes) {
        const size_t at = off;
        off += (bytes + 255) / 256 * 256;
        return at;
    };
    for (int i = 0; i < inner.info.n_inputs; i++) {
        k.in_bytes[i] = inner.in_bytes[i];
        k.in_align[i] = inner.in_align[i];
        if (pin[i] != 'A') continue;
        if (!inner.in_bytes[i] || inner.in_bytes[i] % 4) return set_error("%s: input %d has no known size", inner.info.name, i);
        k.half_in |= 1u << i;
        k.in_bytes[i] = inner.in_bytes[i] / 2;
        k.in_align[i] = 2;
        k.stage_in[i] = take(inner.in_bytes[i]);
    }
    for (int i = 0; i < inner.info.n_outputs; i++) {
        k.out_bytes[i] = inner.out_bytes[i];
        k.out_align[i] = inner.out_align[i];
        if (pout[i] != 'A') continue;
        if (!inner.out_bytes[i] || inner.out_bytes[i] % 4) return set_error("%s: output %d has no known size", inner.info.name, i);
        k.half_out |= 1u << i;
        k.out_bytes[i] = inner.out_bytes[i] / 2;
        k.out_align[i] = 2;
        k.stage_out[i] = take(inner.out_bytes[i]);
    }
    k.scratch_bytes = off;
    char name[sizeof(k.info.name)];
    snprintf(name, sizeof(name), "%.58s_f16", inner.info.name);
    memcpy(k.info.name, name, sizeof(name));
    k.launch = launch_half;
    return 0;
}

}  // namespace ksh
