/*
 * ksearch_oracle — CPU restatement of ksearch's quantized decode arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker the HIP path is
 * compared against (tests/, the smoke check, and the cpu_baseline leg of the
 * benchmark).  Nothing in the shipped product path may call it.
 *
 * Every function names the reference file:line it restates (paths relative to
 * the ksearch source tree).
 *
 * Pinning status (what independent evidence fixes each function):
 *   ko_f16_to_f32            all 65,536 inputs vs numpy float16
 *   ko_f32_to_f16            numpy float16 everywhere except exact ties /
 *                            the [2^-25,2^-24) band, where the reference's
 *                            add-0x1000-and-truncate rule is checked by
 *                            construction of tie inputs
 *   ko_get_scale_min_k4      bit-level brute force over the GGML layout
 *   ko_dequant_q4k           4 reference formulations agree (CPU loop, scalar
 *                            GPU helper, 16-wide mul_mm helper, coop
 *                            algebraic form via unit-vector dots) + special
 *                            cases + the reference's own round-trip unit test
 *   ko_dequant_q6k           3 reference formulations agree; no reference
 *                            test pins it beyond that
 *   ko_dequant_q40/pack_q40  2 formulations + closed-form invariants
 *   ko_matvec / ko_matmul    brute-force f64 on dequantized weights, the
 *                            check_mul_mm integer-formula inputs
 *   ko_sdpa_*                f64 brute-force softmax, partition-count
 *                            independence, needle case
 *   ko_softcap_argmax        reference unit test ([1,9,3] -> 1), tie rule
 *   ko_rmsnorm*, rope, gelu  closed forms, pos=0 identity
 *   ko_dequant (Q5_K)        the block loop vs an independent per-element
 *                            restatement of the GPU helper, reduction to Q4_K
 *                            with every fifth bit clear, +16*d*sc with all set
 *   ko_rmsnorm_per_head      f64 closed form, rope row 0 = identity, rotation
 *                            keeps the norm, equals the pinned QKV op's q half
 *   ko_add_scale,
 *   ko_matvec_gelu_mul       closed forms (f64 GELU-tanh on the f64 dot)
 *   ko_gemma4_*              bit-identical to the pinned ko_gemma_* loop when
 *                            the extras are off; kv_source vs the rule restated;
 *                            the window: equal to a wide-window run for exactly
 *                            `window` positions
 *   ko_sample_softcap_min_p  the reference's three unit tests restated (sample.rs:87-117),
 *                            the draw's distribution against the closed-form softmax
 *   ko_quantize_q4k          reference round-trip test only (output bytes of
 *                            the iterative search are PARITY UNPINNED; they
 *                            never enter a GPU-vs-oracle comparison because
 *                            both sides consume the same packed bytes)
 *   ko_quantize_q6k          not in the reference at all (build's own);
 *                            same remark
 */
#ifndef KSEARCH_ORACLE_H
#define KSEARCH_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { KO_F32 = 0, KO_F16 = 1, KO_Q4K = 2, KO_Q5K = 3, KO_Q6K = 4, KO_Q40 = 5, KO_BF16 = 6 };

/* crates/ksearch_gguf/src/lib.rs:10-75 */
float    ko_bf16_to_f32(uint16_t v);
uint16_t ko_f32_to_bf16(float v);
float    ko_f16_to_f32(uint16_t v);
uint16_t ko_f32_to_f16(float v);          /* reference rule: +0x1000, truncate */
uint16_t ko_f32_to_f16_rne(float v);      /* IEEE ties-to-even (what a GPU half() does) */

/* crates/ksearch_gguf/src/gguf_impl.rs:563-573 */
void ko_get_scale_min_k4(int j, const uint8_t *q, uint8_t *d, uint8_t *m);

/* crates/ksearch_ir/src/lib.rs:52-74, gguf_impl.rs:50-64 */
size_t ko_row_bytes(int dtype, size_t cols);

/* crates/ksearch_gguf/src/gguf_impl.rs:577-794 (dequant_blocks) */
int ko_dequant(int dtype, const uint8_t *data, size_t total_elems, float *out);

/* crates/ksearch_gguf/src/gguf_impl.rs:803-1016 */
void ko_quantize_q4k(const float *x, size_t n, uint8_t *out);
/* build's own (no reference counterpart) */
void ko_quantize_q6k(const float *x, size_t n, uint8_t *out);
/* crates/ksearch_codegen/src/render.rs:1021-1059 */
void ko_pack_q40(const float *src, size_t n, uint8_t *out, int half_roundtrip);

/* crates/ksearch_kernels/examples/check_mul_mm.rs:60-71: row-major,
 * sequential f32 `s += w*x` over the dequantized row.  threads<=0: all cores. */
int ko_matvec(int dtype, const uint8_t *w, size_t rows, size_t cols,
              const float *x, float *y, int threads);
int ko_matmul(int dtype, const uint8_t *w, size_t rows, size_t cols,
              const float *x, size_t batch, float *y, int threads); /* y[t*rows+r] */
/* f64-accumulate variant, used only to size tolerances */
int ko_matvec_f64(int dtype, const uint8_t *w, size_t rows, size_t cols,
                  const float *x, double *y, int threads);
int ko_max_threads(void);

/* crates/ksearch_codegen/src/lower.rs:4897-5359 (online), 5367-6087 (split-KV).
 * K/V: Q4_0 [max_t, n_kv, hd]; q,out: f32 [n_q*hd]; rows [start,start+tlen). */
void ko_sdpa_online(const float *q, const uint8_t *k, const uint8_t *v,
                    int n_q, int n_kv, int hd, int tlen, int start, float scale,
                    float *out);
void ko_sdpa_mwg(const float *q, const uint8_t *k, const uint8_t *v,
                 int n_q, int n_kv, int hd, int tlen, int start, float scale,
                 int nwg, float *out);
void ko_sdpa_f64(const float *q, const uint8_t *k, const uint8_t *v,
                 int n_q, int n_kv, int hd, int tlen, int start, float scale,
                 double *out);

/* crates/ksearch_codegen/src/lower.rs:6090-6156, ksearch_gemma/src/sample.rs:18-36 */
uint32_t ko_softcap_argmax(const float *x, size_t n, float cap);

/* crates/ksearch_codegen/src/lower.rs:4079-4162, 3926-4077 */
void ko_rmsnorm(const float *x, const float *w, const float *res, float eps,
                float scale, int has_scale, size_t n, float *out);
void ko_rmsnorm_add_then_rmsnorm(const float *y, const float *w_post, const float *res,
                                 const float *w_ffn, float eps, size_t n,
                                 float *out_x, float *out_x2);
/* crates/ksearch_gemma/src/gemma_prim.rs:33-56 */
void ko_rope_table(int max_seq, int hd, float theta, int rope_angles, float *out);
/* crates/ksearch_codegen/src/lower.rs:4619-4702 (n_tok<=1 branch) */
void ko_rmsnorm_per_head_qkv_q40(const float *q, const float *qw, const float *rope_row,
                                 const float *k, const float *kw, const float *v,
                                 int n_q, int n_kv, int hd, float eps,
                                 float *q_out, uint8_t *k_out, uint8_t *v_out);
/* crates/ksearch_codegen/src/lower.rs:2926-2955, 4775-4838 */
float ko_gelu_mul(float g, float u);
/* crates/ksearch_codegen/src/lower.rs:3899-3921 */
int ko_copy_scale_indexed(int dtype, const uint8_t *src, uint32_t id, size_t n,
                          float scale, float *out);

/* ---- whole-model greedy decode, following
 * crates/ksearch_gemma/src/gemma_prim.rs:881-1275 (forward_token) without the
 * Gemma-4 extras the synthetic configuration omits (PLE, SWA, shared KV). ---- */
typedef struct {
    int n_layers, hidden, ffn, n_q, n_kv, hd, vocab, max_seq;
    float eps, softcap, rope_theta, attn_scale;
} ko_gemma_cfg;

typedef struct {
    const uint8_t *wq, *wk, *wv, *wo, *wgate, *wup, *wdown; /* Q4_K */
    const float *attn_norm, *q_norm, *k_norm, *post_attn_norm, *ffn_norm, *post_ffw_norm;
} ko_gemma_layer;

/* Row adoption for whole-step comparisons with another implementation (no counterpart in the reference; it
 * removes Q4_0 rounding-boundary flips from the comparison).  When `rows` is set, every layer that appends
 * to a cache packs its own K and V rows, records how the other implementation's rows differ from them
 * (`diff_bytes[2*layer + which]`: differing bytes; `max_step[2*layer + which]`: largest difference of
 * dequantized values in units of the own block's scale, 1.0 = one code step) and then continues with the
 * other rows.  `rows` is [n_layers][2][row_stride] bytes (K then V); `diff_bytes` / `max_step` may be NULL. */
typedef struct {
    const uint8_t *rows;
    size_t row_stride;
    int *diff_bytes;
    float *max_step;
} ko_row_sync;

typedef struct ko_gemma ko_gemma;
void ko_gemma_set_row_sync(ko_gemma *m, const ko_row_sync *s);   /* NULL switches it off */
ko_gemma *ko_gemma_create(const ko_gemma_cfg *cfg, const ko_gemma_layer *layers,
                          const uint8_t *token_embd_q6k, const float *output_norm);
void ko_gemma_destroy(ko_gemma *m);
void ko_gemma_reset(ko_gemma *m);
/* one token through all layers; returns greedy next id; logits_out may be NULL */
uint32_t ko_gemma_forward(ko_gemma *m, uint32_t token, int want_logits, float *logits_out,
                          int threads);
int ko_gemma_pos(const ko_gemma *m);
/* read back layer `l`'s K (which=0) or V (which=1) Q4_0 cache bytes */
const uint8_t *ko_gemma_kv(const ko_gemma *m, int layer, int which);
/* last token's hidden state after the final layer (before output norm) */
const float *ko_gemma_hidden(const ko_gemma *m);

/* crates/ksearch_gemma/src/sample.rs:9-77 on f32 logits: soft cap, temperature, min-p, one splitmix32 draw */
uint32_t ko_sample_softcap_min_p(const float *logits, size_t n, float cap, float temperature,
                                 float min_p, uint32_t seed);

/* ---- ops the real Gemma-4 checkpoints add to the decode step ---- */
/* Eng::rmsnorm_per_head / rmsnorm_per_head_rope_off (crates/ksearch_kernels/src/lib.rs:564-625;
 * crates/ksearch_codegen/src/lower.rs:4164-4228, 4356-4435): y[h,i] = x[h,i]*inv_h*w[i], then RoPE with
 * `rope_row` (cos[0..hd/2) || sin[0..hd/2)) unless it is NULL */
void ko_rmsnorm_per_head(const float *x, const float *w, const float *rope_row, int n_heads, int hd,
                         float eps, float *out);
/* Eng::add_scale (crates/ksearch_kernels/src/lib.rs:918-937): y = scale*(a+b) */
void ko_add_scale(const float *a, const float *b, float scale, size_t n, float *out);
/* Eng::matvec_gelu_mul_at (crates/ksearch_kernels/src/lib.rs:791-822; epilogue GeluMulCtx,
 * crates/ksearch_codegen/src/lower.rs:622-643): y[r] = gelu(W[r].x) * ctx[r] */
int ko_matvec_gelu_mul(int dtype, const uint8_t *w, size_t rows, size_t cols, const float *x,
                       const float *ctx, float *y, int threads);

/* ---- whole-model greedy decode with those extras, following forward_token
 * (crates/ksearch_gemma/src/gemma_prim.rs:881-1275) and GemmaConfig (crates/ksearch_gemma/src/lib.rs:39-167):
 * sliding-window and full-attention layers with their own head dims, rope tables and windows; layers past
 * n_layers - shared_kv_layers reuse the cache of the last owning layer of their kind; per-layer embeddings
 * (ple_dim > 0).  Activations stay f32 (the reference keeps them in f16). ---- */
typedef struct {
    int n_layers, hidden, n_q, n_kv, vocab, max_seq;
    int hd_swa, hd_full, sliding_window, shared_kv_layers, ple_dim;
    float eps, softcap, rope_theta_swa, rope_theta_full, partial_rotary, attn_scale;
} ko_gemma4_cfg;

typedef struct {
    int is_swa, ffn;
    int dt_q, dt_k, dt_v, dt_o, dt_gate, dt_up, dt_down, dt_inp_gate, dt_proj;   /* KO_Q4K or KO_Q6K */
    const uint8_t *wq, *wk, *wv, *wo, *wgate, *wup, *wdown, *inp_gate, *proj;
    const float *attn_norm, *q_norm, *k_norm, *post_attn_norm, *ffn_norm, *post_ffw_norm, *post_norm;
    float layer_scale;
} ko_gemma4_layer;

typedef struct {
    const uint8_t *token_embd;      /* [vocab, hidden], also the LM head */
    int dt_embd;
    const float *output_norm;
    const uint8_t *ple_embd;        /* [vocab, n_layers*ple_dim] */
    int dt_ple;
    const uint8_t *ple_model_proj;  /* [n_layers*ple_dim, hidden] */
    int dt_ple_proj;
    const float *ple_proj_norm;     /* [ple_dim] */
} ko_gemma4_globals;

typedef struct ko_gemma4 ko_gemma4;
void ko_gemma4_set_row_sync(ko_gemma4 *m, const ko_row_sync *s);   /* layers that append nothing are skipped */
ko_gemma4 *ko_gemma4_create(const ko_gemma4_cfg *cfg, const ko_gemma4_layer *layers,
                            const ko_gemma4_globals *g);
void ko_gemma4_destroy(ko_gemma4 *m);
void ko_gemma4_reset(ko_gemma4 *m);
uint32_t ko_gemma4_forward(ko_gemma4 *m, uint32_t token, int want_logits, float *logits_out, int threads);
int ko_gemma4_pos(const ko_gemma4 *m);
/* which layer's cache layer `l` reads (crates/ksearch_gemma/src/lib.rs:151-162) */
int ko_gemma4_kv_source(const ko_gemma4 *m, int layer);
const uint8_t *ko_gemma4_kv(const ko_gemma4 *m, int layer, int which);
const float *ko_gemma4_hidden(const ko_gemma4 *m);

#ifdef __cplusplus
}
#endif
#endif
