/*
 * ksearch_hip.h — C ABI of libksearch_hip.so, the MI355X (gfx950) backend for
 * ksearch's quantized decode hot path.
 *
 * The library takes the place of two things in the ksearch tree:
 *   - crates/ksearch_metal/src/lib.rs (MetalContext: device, buffers, one open
 *     encoder, flush / wait / barrier / synchronize, timed run), and
 *   - the kernel bodies crates/ksearch_codegen/src/{lower,render}.rs emit for
 *     the Q4_K / Q6_K GEMVs, the Q4_K prefill GEMM, the Q4_0-KV attention and
 *     the glue ops of a decode step.
 * Kernels are prebuilt hand-written HIP selected by (kind, dims, dtypes,
 * schedule); there is no run-time code generation.
 *
 * Conventions
 *   - every function returns 0 on success, non-zero on failure; the message is
 *     fetched with ksh_last_error() (thread-local, valid until the next call).
 *     Count / size mismatches are errors, never aborts
 *     (crates/ksearch_metal/src/lib.rs:280-307).
 *   - a context is owned by one host thread (the reference context is !Sync).
 *   - work is appended to one in-order HIP stream; program order is execution
 *     order (the reference relies on Metal hazard tracking inside one encoder,
 *     crates/ksearch_kernels/src/lib.rs:890).
 *   - device memory is not host-visible: what the reference does through
 *     `contents()` pointers goes through ksh_buffer_write / read / fill_zero.
 */
#ifndef KSEARCH_HIP_H
#define KSEARCH_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ksh_ctx ksh_ctx;
typedef struct ksh_buf ksh_buf;
typedef struct ksh_kernel ksh_kernel;
typedef struct ksh_graph ksh_graph;

/* DType, crates/ksearch_ir/src/lib.rs:17-27 (same order).
 * KSH_Q6K_ROWS has no counterpart there: it is Q6_K with the bytes of every weight row regrouped by field
 * (all ql of the row's superblocks, then all qh, all scales, all d: the same 210 B per 256 weights, every
 * field 16-byte aligned, the row padded to a multiple of 16 bytes), which is how the LM head is kept in HBM
 * so that a wave fetches a row with whole 128-bit loads.  KSH_REPACK_ROWS makes it from Q6_K; the GEMV takes
 * rows of 1536, 2048 or 4096 columns (1264, 1680, 3360 bytes). */
enum ksh_dtype {
    KSH_F32 = 0, KSH_F16 = 1, KSH_Q4K = 2, KSH_Q5K = 3, KSH_Q6K = 4, KSH_Q40 = 5, KSH_BF16 = 6, KSH_Q6K_ROWS = 7
};

/* The KernelKind variants on the hot path (crates/ksearch_ir/src/kernel.rs:399-744).
 * Inputs/outputs are listed in binding order; "act" = activation dtype
 * (dtypes[1], F32 unless stated).
 * dtypes[1] = KSH_F16: the reference's buffer types (x_dtype, crates/ksearch_codegen/src/lower.rs:1134-1140;
 * buffer_empty_f16, crates/ksearch_gemma/src/gemma_prim.rs:229-252): every binding that is an activation vector, a
 * norm weight or the logits is half, f32 inside the kernels, results rounded to nearest even; packed weights and
 * caches, the rope table, meta records, token ids, split-KV partials and the argmax index keep their types.  Taken
 * by the kinds Eng calls (KSH_MATVEC .. KSH_GATE_UP_GELU and their RMSNORM_ forms, the RMSNORM and SDPA kinds,
 * KSH_ATTEND_DECODE, KSH_ATTN_MERGE_MATVEC, KSH_COPY_SCALE_INDEXED, KSH_GELU_MUL, KSH_ADD_SCALE,
 * KSH_MATVEC_GELU_MUL, KSH_COPY_SLICE, KSH_SOFTCAP_ARGMAX, and the plain KSH_MATVEC_BATCH, whose Y is half with
 * dtypes[2] = KSH_F16). */
enum ksh_kind {
    /* Matvec{rows,cols,weight_dtype}: y = W x.  dims: rows, cols.
     * dtypes[0] = Q4K | Q6K.  in: W, x   out: y[rows] */
    KSH_MATVEC = 1,
    /* MatvecBatch: Y[t,r] = sum_c W[r,c] X[t,c].  dims: rows, cols, batch.
     * dtypes[0] = Q4K | Q6K (GGUF byte order, blocks at 2-byte alignment),
     * dtypes[1] = BF16 (X) or F32 (X is then taken as hi + lo f16 parts, 22 bits: two passes, two sets of workgroups,
     * or -- Q4_K with a grid of at least 256 tiles -- one workgroup walking both; the form the decode loops' prompt
     * chunks use), output F32 token-major.
     * in: W, X   out: Y[batch, rows]
     * dims[3], dims[4] (0 = none): rows of a second and a third matrix of the same dtype over the same X, taken in
     * the same launch (q | k | v of a prompt chunk: one preparation of X, one grid).  in: W, X, W1[, W2]
     * out: Y, Y1[batch, rows1][, Y2[batch, rows2]].
     * dims[5] (F32 activations): the producer of the rows, run inside the preparation of X (params[0] = eps) --
     *   1: X := rmsnorm(X, w)  (in: ..., w[cols]);  2: x_new := res + rmsnorm(X, w_post), X := rmsnorm(x_new, w_norm)
     *   (in: ..., w_post[cols], res[batch, cols], w_norm[cols]; out: ..., x_new[batch, cols], which may be res);
     *   3: X := gelu(X) * up  (in: ..., up[batch, cols]).  The norms take rows of a multiple of 512 up to 8192 columns.
     *   These are the rows forms of RmsNormMatvec* / MatvecGateUpGelu's prologues (crates/ksearch_kernels/src/lib.rs:
     *   1478-1560, gemma_prim.rs:1516-1538) folded into the GEMM that reads their result.
     * dims[6] = 1: the tile's K slices stay unfolded -- out[0] is then f32[slices][batch][rows + rows1 + rows2]
     *   (slices = info.grid[2] = info.sched.k_split, the matrices' columns side by side) for a reader that adds them
     *   itself; out[1] = x_new with prologue 2.
     * dims[7] = the slices (info.grid[2]) of the GEMM whose unfolded result this one's X is (with a prologue;
     *   prologue 3 then reads gate | up from that one buffer and takes no `up` operand).  The sums are added in the
     *   fold's order, so a chain of GEMMs gives the same numbers with and without its folds.
     * F32 activations travel as hi + lo f16 parts.  The tile scales every row by its own power of two first (any
     * finite f32 row fits); the small-batch form does not: there |x| must stay below 65504.
     * sched.nr0 = 32 | 128 picks the small-batch form (Q4_K, up to 64 tokens, one matrix) or the 128 x 128 tile;
     * sched.k_split = the tile's K slices (a divisor of cols / 256; 1 = whole rows; 0 = enough to fill the chip). */
    KSH_MATVEC_BATCH = 2,
    /* MatvecQkv: three GEMVs sharing x.  dims: q_rows, kv_rows, cols.
     * in: Wq, Wk, Wv, x   out: q, k, v */
    KSH_MATVEC_QKV = 3,
    /* MatvecGateUpGelu: out[i] = gelu_tanh(clamp(Wg[i].x, +-20)) * (Wu[i].x).
     * dims: rows, cols.  in: Wg, Wu, x   out: out[rows] */
    KSH_MATVEC_GATE_UP_GELU = 4,
    /* SdpaNaive: online-softmax attention over rows [start, start+tlen).
     * dims: n_q, n_kv, hd, max_t.  params[0] = softmax scale (1.0 = reference).
     * in: q[n_q*hd], K, V (Q4_0 [max_t,n_kv,hd]), meta f32[>=3] = tlen,start,window
     * out: o[n_q*hd] */
    KSH_SDPA_NAIVE = 5,
    /* SdpaMwgPart: split-KV pass 1.  dims: n_q, n_kv, hd, max_t, nwg.
     * in: q, K, V, meta   out: tmp f32[n_q*nwg*(hd+2)] = (m, l, O[hd]) */
    KSH_SDPA_MWG_PART = 6,
    /* SdpaMwgReduce: split-KV pass 2.  dims: n_q, hd, nwg.  in: tmp  out: o */
    KSH_SDPA_MWG_REDUCE = 7,
    /* Multi-slot decode attention in one launch (the reference runs slots
     * serially, crates/ksearch_cli/src/scheduler.rs:163-187).
     * dims: n_q, n_kv, hd, max_t, n_slots, nwg.  K/V pools are
     * [n_slots][max_t,n_kv,hd] Q4_0; meta is f32[n_slots][4].
     * in: q[n_slots,n_q*hd], Kpool, Vpool, meta   out: tmp, o[n_slots,n_q*hd]
     * dims[6] = pool slots > 0: the launch's n_slots entries are a subset, in any order, of pools that hold dims[6]
     * slots (one decode step for several sequences); a 5th input f32[n_slots] names each entry's pool slot, and
     * dims[7] is the byte distance between slots of the pools (0: max_t rows).
     * params[1] != 0: the second output is the prepared operand of a decode round's GEMM over the n_q * hd columns
     * (as KSH_ROUND_PREP writes it, row = entry) instead of f32 rows; 2 to 16 slots, 2 to 64 partitions. */
    KSH_SDPA_SLOTS = 8,
    /* QuantizeQ40: pack n f32 values (n%32==0) to Q4_0.  dims: n.  in: src  out: dst */
    KSH_QUANTIZE_Q40 = 9,
    /* RmsNorm / RmsNormAdd / RmsNormAddScale.  dims: n, has_residual, has_scale, rows.
     * params[0] = eps, params[1] = scale.  in: x, w, (residual)   out: y
     * rows > 1: rmsnorm_rows / rmsnorm_add_rows / rmsnorm_add_scale_rows (crates/ksearch_kernels/src/lib.rs:
     * 1478-1560): x, residual and y are [rows, n], the weight is shared. */
    KSH_RMSNORM = 10,
    /* RmsNormAddThenRmsNorm.  dims: n, rows.  params[0] = eps.
     * in: y, w_post, residual, w_ffn   out: x, x2   (rows > 1: rmsnorm_add_then_rmsnorm_rows, matrices [rows, n]) */
    KSH_RMSNORM_ADD_THEN_RMSNORM = 11,
    /* RmsNormPerHeadQkvQ40.  dims: n_q, n_kv, hd, max_seq, n_tok.  params[0] = eps.
     * n_tok > 1 (rmsnorm_per_head_qkv_q40_batch, crates/ksearch_kernels/src/lib.rs:1750): q, k, v and q_out hold
     * n_tok rows for consecutive positions; token i uses rope row / cache row (first position + i).
     * max_seq = 0: in: q, qw, rope_row f32[hd], k, kw, v   out: q_out f32, K row Q4_0,
     * V row Q4_0 (the caller applies the position as byte offsets, as the reference does).
     * max_seq > 0: a 7th input meta f32[4] carries the position in [3]; rope is then the
     * whole table f32[max_seq, hd] and the outputs are the cache bases.
     * dims[5] = slots > 0 (tokens of different sequences): meta is f32[n_tok][4] with token i's position in
     * [4 i + 3], an 8th input f32[n_tok] names token i's slot, the outputs are caches of dims[5] slots
     * ([slot][max_seq, n_kv, hd]; dims[6] = byte distance between slots, 0: max_seq rows). */
    KSH_RMSNORM_PER_HEAD_QKV_Q40 = 12,
    /* CopyScaleIndexed: out[i] = scale * deq(src[id*n + i]); id is read from a
     * device f32 (the reference keeps token ids as f32).  dims: n, rows in the table, n_tok (> 1:
     * copy_scale_indexed_batch_wd, idx f32[n_tok], out [n_tok, n]).
     * dtypes[0] = source dtype (Q4K | Q5K | Q6K | F16 | F32).  params[0] = scale.  in: src, idx   out: out[n] */
    KSH_COPY_SCALE_INDEXED = 13,
    /* GeluMul: out[i] = gelu_tanh(clamp(g[i])) * u[i].  dims: n.  in: g, u  out: out */
    KSH_GELU_MUL = 14,
    /* CopySlice.  dims: n.  in: src   out: dst */
    KSH_COPY_SLICE = 15,
    /* SoftcapArgmax: argmax_i cap*tanh(x_i/cap), lowest index wins ties, index
     * stored as f32.  dims: n, rows (0 or 1: one vector; more: the rows of a decode round, one index each).
     * params[0] = cap.  in: x f32[rows, n]   out: idx f32[rows] */
    KSH_SOFTCAP_ARGMAX = 16,
    /* Dequantize packed blocks to f32 (the CPU-side dequant_type_to_f32,
     * crates/ksearch_gguf/src/gguf_impl.rs:472-476, as a device kernel).
     * dims: n_elems.  dtypes[0] = Q4K | Q5K | Q6K | Q40.  in: src   out: dst f32 */
    KSH_DEQUANT = 17,
    /* quantize_f32_to_q4k (crates/ksearch_gguf/src/gguf_impl.rs:905-1016) and a
     * Q6_K packer, as device kernels.  dims: n_elems.  dtypes[0] = Q4K | Q6K.
     * in: src f32   out: packed */
    KSH_QUANTIZE_K = 18,
    /* RmsNormMatvec / RmsNormMatvecQkv / RmsNormMatvecGateUpGelu
     * (crates/ksearch_ir/src/kernel.rs:303-339): the GEMV's workgroups compute
     * the RMSNorm of the vector themselves.  Same dims as the plain kinds plus a
     * trailing has_residual flag; params[0] = eps.
     *   has_residual = 0: in: W.., x, w_norm                 out: y..
     *   has_residual = 1: in: W.., y, w_norm, w_post, res    out: y.., x_new
     *     with x_new = res + rms(y)*w_post (RmsNormAdd, the new residual stream,
     *     which must not alias res) and the GEMV input rms(x_new)*w_norm
     *     (RmsNormAddThenRmsNorm, kernel.rs:474-481, folded into its consumer).
     *     params[1] != 0: x_new = params[1] * (res + rms(y)*w_post) (RmsNormAddScale: the
     *     per-layer-embedding block's closing op, folded in the same way). */
    KSH_RMSNORM_MATVEC = 19,
    KSH_RMSNORM_MATVEC_QKV = 20,
    KSH_RMSNORM_MATVEC_GATE_UP_GELU = 21,
    /* AttendDecode: one decode step's attention in one launch.  It is the
     * composition RmsNormPerHeadQkvQ40 (n_tok = 1, position on the device)
     * -> SdpaMwgPart -> SdpaMwgReduce of the reference's forward_token
     * (crates/ksearch_gemma/src/gemma_prim.rs:984-1060); the reference has no
     * single op for it.  dims: n_q, n_kv, hd, max_seq, nwg (0 = default).
     * params[0] = eps, params[1] = softmax scale.
     * in: q f32[n_q*hd] (raw, before the per-head norm), q_norm f32[hd],
     *     rope f32[max_seq, hd], k f32[n_kv*hd], k_norm f32[hd], v f32[n_kv*hd],
     *     meta f32[4] = {tlen, start, window, pos} with start + tlen - 1 == pos
     * out: K cache, V cache (row pos is written), tmp f32[n_q, nwg, hd+2],
     *      out f32[n_q*hd].  Built for hd 128 / 256 / 512, up to 8 q heads per kv head.
     * With dims[5] = 1 the partitions are not merged: the outputs are K cache,
     * V cache and parts = { o f32[n_q, nwg, hd] (unnormalised), ml f32[n_q, nwg, 2]
     * (running max, sum) } in one buffer, for KSH_ATTN_MERGE_MATVEC.
     * With dims[6] = 1 the rope input is the row of the table for meta's pos, f32[hd], kept current by the
     * caller: the launch then has nothing to wait for between reading pos and fetching its rope values.
     * With dims[7] = 1 nothing is appended (a layer that reuses another layer's cache, whose row pos that layer
     * has written in this step; RmsNormPerHeadRope -> SdpaMwg*, gemma_prim.rs:989-1034):
     *   in: q, q_norm, rope, K cache, V cache, meta    out: tmp, out (or parts alone with dims[5] = 1) */
    KSH_ATTEND_DECODE = 22,
    /* SdpaMwgReduce (crates/ksearch_metal/src/lower.rs:5897-6087) folded into the
     * GEMV that consumes the attention output: every workgroup merges the
     * partitions' states itself while its weights are in flight, which takes
     * the cross-workgroup hand-over out of the attention launch.
     * dims: rows, n_q, hd, nwg (<= 8; n_q*hd <= 2048, hd a power of two).
     * in: W Q4_K[rows, n_q*hd], parts (as written by KSH_ATTEND_DECODE with dims[5] = 1)
     * out: y f32[rows] */
    KSH_ATTN_MERGE_MATVEC = 23,
    /* Q6_K [rows, cols] -> KSH_Q6K_ROWS, a byte permutation inside every row (done once, when weights are
     * loaded).  dims: rows, cols.  in: src Q6_K   out: dst, rows * round_up(cols/256*210, 16) bytes, 16-byte aligned */
    KSH_REPACK_ROWS = 24,
    /* Eng::rmsnorm_per_head and rmsnorm_per_head_rope_off (crates/ksearch_kernels/src/lib.rs:564-625):
     * y[h,i] = x[h,i] * rsqrt(mean_h(x^2) + eps) * w[i], then RoPE with pairs (i, i + hd/2) of the row
     * cos[0..hd/2) || sin[0..hd/2).  The query heads of layers that reuse another layer's KV cache, and the
     * per-layer-embedding prepass.  y may be x.
     * dims: n_heads, hd (64 | 128 | 256 | 512), rope (0 none; 1 the row, placed with a byte offset; 2 the whole
     *       table, row = position in meta[3]), max_seq (rope = 2), heads per token (rope = 2, > 0: the heads of
     *       several tokens, token after token; token i is at position meta[3] + i), per-token records (1: tokens of
     *       different sequences, meta is f32[n_tok][4] with token i's position in [4 i + 3])
     * params: eps.   in: x, w f32[hd] [, rope [, meta f32[4]]]   out: y */
    KSH_RMSNORM_PER_HEAD = 25,
    /* Eng::add_scale (crates/ksearch_kernels/src/lib.rs:918-937): y = scale * (a + b).
     * dims: n.  params: scale.  in: a, b   out: y */
    KSH_ADD_SCALE = 26,
    /* Eng::matvec_gelu_mul_at (crates/ksearch_kernels/src/lib.rs:791-822): y[r] = gelu(W[r].x) * ctx[r], the
     * per-layer-embedding gate; the context slice is placed with a byte offset.
     * dims: rows, cols (<= 8192), has_residual.  dtypes: Q4K, F32.  params: eps (has_residual).
     *   has_residual = 0: in: W, x, ctx f32[rows]                 out: y
     *   has_residual = 1: in: W, y_prev, ctx, w_post, res         out: y, x_new
     *     with x_new = res + rms(y_prev)*w_post (the RmsNormAdd that closes the feed-forward block, folded in;
     *     x_new must not alias res) and the GEMV input x_new */
    KSH_MATVEC_GELU_MUL = 27,
    /* Measurement aid, no counterpart in the reference: the memory-only floor of a Q4_K GEMV launch.  The grid,
     * workgroup size and LDS reservation of the default GEMV schedule (2 rows per wave, 8 waves), doing nothing
     * (mode 0), issuing exactly the GEMV's weight loads and nothing else (mode 1), or reading the same bytes with
     * flat 128-bit loads (mode 2).  dims: rows, cols (<= 4096), mode.  dtypes: Q4K.  in: W   out: sink f32[1]
     * (never written for real weights).  The empty launch takes other shapes: dims[3] workgroups, dims[4] threads per
     * workgroup (a multiple of 64 up to 512), dims[5] = 1 no LDS reservation, dims[6] = 1 an argument block of the
     * GEMV's size (0 everywhere: the GEMV's own launch shape and four scalar arguments). */
    KSH_READ_FLOOR = 28,
    /* sdpa_hybrid_kv_batch (crates/ksearch_kernels/src/lib.rs:1592-1623, lower.rs:4961-4983): causal attention of
     * n_tok consecutive prompt tokens over one Q4_0 cache that already holds their rows.  meta = f32{tlen of token
     * 0, -, window}: token i attends tlen_i = min(tlen0 + i, window) rows from start_i = tlen0 + i - tlen_i.
     * dims: n_q, n_kv, hd, max_t, n_tok, nwg (0 = default; sched.k_split sets it too).  Heads of 256 in chunks of
     * more than 16 tokens run on the matrix cores and are fastest with one partition per token (nwg = 1).
     * in: q[n_tok, n_q*hd], K, V, meta   out: tmp f32[n_tok*n_q*nwg*(hd+2)], o[n_tok, n_q*hd] */
    KSH_SDPA_BATCH = 29,
    /* The activations of a decode round (up to 16 rows, one per decoding sequence), prepared once for every GEMM
     * that reads them.  No counterpart in the reference, whose round is one decode step per request
     * (crates/ksearch_cli/src/scheduler.rs:163-231).  The operand holds x = hi + 2^-11 lo as f16 fragments of the
     * matrix instruction (a token's hi and lo part in one tile) and the per-sub-block sums of x.
     * dims: cols (a multiple of 256), batch (1..16), mode.  params: eps (modes 1, 2)
     *   mode 0: in: x f32[batch, cols]                         out: xp
     *   mode 1: the rows' RMSNorm on the way (rmsnorm_rows, crates/ksearch_kernels/src/lib.rs:1478):
     *           in: x, w f32[cols]                              out: xp of (x * inv) * w
     *   mode 2: rmsnorm_add_then_rmsnorm on rows: in: y, w_post, res, w_norm   out: xp, x_new f32[batch, cols]
     *           with x_new = res + (y * inv) * w_post (may be res) and xp of (x_new * inv2) * w_norm; params[1] != 0:
     *           x_new = params[1] * (res + ...) (rmsnorm_add_scale_rows, :1520-1560, in front of the next norm)
     *   mode 3: rmsnorm_add on rows: in: y, w, res   out: xp of x_new, x_new = res + (y * inv) * w
     * xp: 64 * cols + 2048 * (cols / 256) bytes, 16-byte aligned */
    KSH_ROUND_PREP = 30,
    /* Up to three Q4_K matrices of one width against one prepared operand, in one launch (q | k | v share their
     * input), or a gate | up pair stored as gelu(gate) * up (Eng::matvec_batch, crates/ksearch_kernels/src/lib.rs:
     * 1414-1444, is the reference's batched GEMV for up to 8 rows; fused forms: none there).  Exact integer codes on
     * the matrix cores, the GEMV's accuracy.
     * dims: rows0, cols, batch (1..16), rows1, rows2 (0: absent), pair (1: gate | up of rows0 rows each)
     * dtypes: Q4K.   in: W0, xp (KSH_ROUND_PREP) [, W1 [, W2]]
     * out: y0 f32[batch, rows0] [, y1 f32[batch, rows1] [, y2 f32[batch, rows2]]]; pair: y0 alone.
     * Rows longer than 2048 columns are split over workgroups and added by a second launch (one matrix then). */
    KSH_MATVEC_ROUND = 31,
    KSH_KIND_COUNT
};

/* OptSchedule (crates/ksearch_ir/src/kernel.rs:11-18) retargeted to gfx950.
 * All-zero means "library default, or the plan cache's entry if one exists"; tg = all ones (the other fields zero)
 * means "library default, whatever the plan cache holds". */
typedef struct {
    uint64_t tg;       /* threads per workgroup (64 * waves) */
    uint32_t vec;      /* inner-product variant.  GEMV: 1 = byte converts + f32 FMA, 3 = int8 dot over 3 digit planes,
                        * 2 (Q4_K kinds, by request only: the schedule search never offers it) = int8 dot over 2 digit
                        * planes, the activations to 2^-16 of their 32-element sub-block's largest magnitude.
                        * Attention: 1 = LDS-tile form, 3 = register (vector-ALU) form, 2 = matrix-core form of the
                        * row phase (heads of 256, up to 8 q heads per kv head.  KSH_SDPA_SLOTS with up to 16 slots:
                        * the default there; lds_tile = 32 | 16 picks four waves with tiles of 32 rows or eight with
                        * 16.  KSH_SDPA_BATCH: the default from 17 tokens on, every token's partitions workgroups of
                        * their own; vec = 2 with up to 64 tokens deals the partitions to the tokens by length) */
    uint32_t unroll;   /* superblocks in flight per lane */
    uint32_t nsg;      /* waves per workgroup */
    uint32_t nr0;      /* rows per wave */
    uint32_t k_split;  /* waves cooperating on one row along K */
    uint32_t lds_tile; /* LDS tile: KV rows per tile (SDPA), K depth (GEMM) */
} ksh_sched;

typedef struct {
    int32_t kind;          /* enum ksh_kind */
    int32_t dtypes[4];
    int64_t dims[8];
    float params[4];
    ksh_sched sched;
} ksh_kernel_desc;

/* LaunchHint / MetalKernelSource metadata (crates/ksearch_codegen/src/lib.rs:33-60) */
typedef struct {
    int32_t n_inputs, n_outputs;
    uint32_t grid[3], block[3];
    uint32_t lds_bytes;
    ksh_sched sched;       /* the schedule actually bound */
    char name[64];
} ksh_kernel_info;

const char *ksh_last_error(void);

/* MetalContext::new / Drop, crates/ksearch_metal/src/lib.rs:25-41.  Device 0,
 * one in-order stream.  Fails (never falls back) when no gfx950 GPU is usable. */
int ksh_ctx_create(ksh_ctx **out);
void ksh_ctx_destroy(ksh_ctx *ctx);
/* device_name, :43.  KSEARCH_CHIP if set, otherwise the GCN arch name. */
int ksh_device_name(ksh_ctx *ctx, char *dst, size_t n);
/* the HIP stream work is appended to (hipStream_t), for event timing by callers */
void *ksh_stream(ksh_ctx *ctx);

/* buffer_bytes / buffer_empty_*, :63-91.  init may be NULL (zero-filled). */
int ksh_buffer_alloc(ksh_ctx *ctx, size_t bytes, const void *init, ksh_buf **out);
void ksh_buffer_retain(ksh_buf *buf);
void ksh_buffer_release(ksh_buf *buf);
size_t ksh_buffer_size(const ksh_buf *buf);
void *ksh_buffer_device_ptr(const ksh_buf *buf);
/* write_buffer / write_u16s (sync=1) and their *_nosync forms (sync=0), :110-135 */
int ksh_buffer_write(ksh_ctx *ctx, ksh_buf *buf, size_t off, const void *src, size_t bytes, int sync);
/* read_f32 / read_u16 (sync=1), read_f32_nosync (sync=0), :93-108 */
int ksh_buffer_read(ksh_ctx *ctx, ksh_buf *buf, size_t off, void *dst, size_t bytes, int sync);
/* the host memset of KvPool::clear_slot (crates/ksearch_gemma/src/kv_pool.rs:148-159) */
int ksh_buffer_fill_zero(ksh_ctx *ctx, ksh_buf *buf);

/* lower_to_metal_chip + MetalContext::compile
 * (crates/ksearch_codegen/src/lib.rs:62-166, ksearch_metal/src/lib.rs:47-61):
 * binds a prebuilt kernel to the descriptor, consulting the plan cache when the
 * schedule is all-zero.  Handles are cached per context and owned by it. */
int ksh_kernel_get(ksh_ctx *ctx, const ksh_kernel_desc *desc, ksh_kernel **out);
int ksh_kernel_info_get(const ksh_kernel *k, ksh_kernel_info *info);

/* encode_offsets_multi, crates/ksearch_metal/src/lib.rs:269-374 */
int ksh_encode(ksh_ctx *ctx, ksh_kernel *k,
               ksh_buf *const *inputs, const uint64_t *in_byte_off, int n_in,
               ksh_buf *const *outputs, const uint64_t *out_byte_off, int n_out);
/* Soft-capped argmax without any allocation.  No counterpart in the reference: it is for callers that cannot
 * allocate device memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * Same result as ksh_kernel_get(KSH_SOFTCAP_ARGMAX, dims = {n}, params = {cap}) + ksh_encode, on the context's
 * stream: out f32[1] at `out_byte_off` = argmax_i cap*tanh(x_i/cap) over the n floats at `x_byte_off` (cap <= 0:
 * plain argmax), lowest index wins ties.  The per-workgroup partial results (256 value/index pairs, 2 KB) live in a
 * fixed array inside the library's device image instead of a buffer allocated per kernel handle, and the call
 * creates no kernel handle: it calls no hipMalloc / hipFree and allocates no host memory.  n must be in
 * [1, 2^24 - 1] (KSH_ARGMAX_STATIC_MAX_N: the f32 index is exact below 2^24); anything else is refused.  Every
 * call on a GPU shares that GPU's array: calls that overlap on one GPU (two contexts, two streams) race, calls
 * on one context are ordered by its stream.  Nothing needs clearing between calls: a launch writes every partial
 * it later reads. */
#define KSH_ARGMAX_STATIC_MAX_N ((1 << 24) - 1)
int ksh_softcap_argmax_static(ksh_ctx *ctx, ksh_buf *x, uint64_t x_byte_off, int64_t n, float cap,
                              ksh_buf *out, uint64_t out_byte_off);
/* run (:377-456): synchronize, then `iters` launches timed with HIP events on
 * the context's stream; *ms is the average per launch. */
int ksh_run_timed(ksh_ctx *ctx, ksh_kernel *k,
                  ksh_buf *const *inputs, const uint64_t *in_byte_off, int n_in,
                  ksh_buf *const *outputs, const uint64_t *out_byte_off, int n_out,
                  int iters, double *ms);

int ksh_flush_async(ksh_ctx *ctx);                        /* :162 */
int ksh_wait_inflight_at_most(ksh_ctx *ctx, int n);       /* :173 */
int ksh_barrier(ksh_ctx *ctx);                            /* encoder_barrier :196 */
int ksh_synchronize(ksh_ctx *ctx);                        /* :205 */
int ksh_has_gpu_work(ksh_ctx *ctx);                       /* :157 (1/0) */

/* HIP-graph capture of everything encoded between begin and end; replay with
 * ksh_graph_launch.  (The reference re-encodes every token into one Metal
 * command buffer; a graph is the gfx950 equivalent of that single commit.) */
int ksh_graph_begin(ksh_ctx *ctx);
int ksh_graph_end(ksh_ctx *ctx, ksh_graph **out);
int ksh_graph_launch(ksh_ctx *ctx, ksh_graph *g);
void ksh_graph_destroy(ksh_graph *g);

/* plan cache, crates/ksearch_codegen/src/{plan_cache.rs:9-44, beam.rs:67-139}:
 * $KSEARCH_BEAM_CACHE or ~/.cache/ksearch/beam/{key}.txt holding key=value
 * lines.  The key hash is FNV-1a 64 (the reference's DefaultHasher is not
 * stable across Rust releases and is not reproduced). */
int ksh_plan_key(const char *kind, const int64_t *dims, int n_dims, const char *chip,
                 char *dst, size_t n);
int ksh_plan_save(const char *kind, const int64_t *dims, int n_dims, const char *chip,
                  const ksh_sched *sched, double ms);
/* returns 0 and fills *sched / *ms when a plan exists, 1 when none does */
int ksh_plan_load(const char *kind, const int64_t *dims, int n_dims, const char *chip,
                  ksh_sched *sched, double *ms);
/* plan kind string for a descriptor ("matvec_q4k", "matvec_q6k", "mul_mm_q4k",
 * "sdpa_q40", ...; crates/ksearch_codegen/src/lib.rs:200-205) */
const char *ksh_plan_kind(const ksh_kernel_desc *desc);
/* BEAM: candidate schedules for a descriptor (beam.rs:26-65 retargeted) */
int ksh_beam_candidates(const ksh_kernel_desc *desc, ksh_sched *out, int cap);
/* beam_search_matvec / Eng::beam_matvec (crates/ksearch_codegen/src/lib.rs:178-246,
 * ksearch_kernels/src/lib.rs:1985-2043): time every candidate (1 warm-up +
 * `iters` timed), save the best plan, return it.  The library's own default schedule is timed first and a
 * candidate replaces it only when it is clearly faster (3 %; 10 % for cold timing, whose single launches are noisier).  force & 1 ignores a cached plan;
 * force & 2 times cold: one launch at a time, the caches evicted in between (what the model loaders use: a decode
 * step streams its weights from HBM), where the plain form launches `iters` times back to back. */
int ksh_beam_search(ksh_ctx *ctx, const ksh_kernel_desc *desc,
                    ksh_buf *const *inputs, int n_in, ksh_buf *const *outputs, int n_out,
                    int iters, int force, ksh_sched *best, double *best_ms, int *from_cache);
/* The same search with every candidate timed the way a decode loop runs it (Eng::warm_matvec_plans at model load,
 * crates/ksearch_kernels/src/lib.rs:2057-2080, gemma_prim.rs:254-290): one HIP graph of n_sets dependent launches,
 * launch i over set i (input_sets[i * n_in ..], output_sets[i * n_out ..]: another layer's weights of the same shape,
 * so that every launch streams its weights from HBM), replayed `iters` times, best replay / n_sets.  Isolated launches rank
 * schedules differently from the loop (measured: plans from them cost the decode loop 2 - 4 %). */
int ksh_beam_search_chain(ksh_ctx *ctx, const ksh_kernel_desc *desc, int n_sets,
                          ksh_buf *const *input_sets, int n_in, ksh_buf *const *output_sets, int n_out,
                          int iters, int force, ksh_sched *best, double *best_ms, int *from_cache);

/* ---- decode loop: GemmaPrimModel for the synthetic Gemma-4-E2B shape
 * (crates/ksearch_gemma/src/gemma_prim.rs:881-1275, 1658-1768), minus PLE,
 * sliding window and shared KV, which that shape does not have. ---- */
typedef struct {
    int32_t n_layers, hidden, ffn, n_q, n_kv, hd, vocab, max_seq;
    float eps, softcap, rope_theta, attn_scale;
} ksh_gemma_cfg;

typedef struct {
    ksh_buf *wq, *wk, *wv, *wo, *wgate, *wup, *wdown;             /* Q4_K */
    ksh_buf *attn_norm, *q_norm, *k_norm, *post_attn_norm, *ffn_norm, *post_ffw_norm; /* f32 */
} ksh_gemma_layer;

typedef struct ksh_gemma ksh_gemma;

int ksh_gemma_create(ksh_ctx *ctx, const ksh_gemma_cfg *cfg, const ksh_gemma_layer *layers,
                     ksh_buf *token_embd_q6k, ksh_buf *output_norm, ksh_gemma **out);
void ksh_gemma_destroy(ksh_gemma *m);
int ksh_gemma_reset(ksh_gemma *m);
/* forward_token: one token at the model's current position.  use_graph=1
 * replays a captured HIP graph.  next_id may be NULL (no host read-back). */
int ksh_gemma_forward_token(ksh_gemma *m, uint32_t token, int use_graph, uint32_t *next_id);
/* prefill_chunk (crates/ksearch_gemma/src/gemma_prim.rs:1305-1607): n tokens at the model's current position, no
 * logits; chunks of up to 1024 tokens run as one batched pass per layer (row norms, MFMA GEMMs over f32 activations,
 * batched per-head norm + RoPE + Q4_0 append, causal attention over the cache), a single token as a decode step. */
int ksh_gemma_prefill_chunk(ksh_gemma *m, const uint32_t *tokens, int n);
/* generate_timed (:1658-1768): all prompt tokens but the last through prefill_chunk (use_graph & 2: token by token
 * through the decode step instead), then n_new greedy tokens whose ids never leave the device between steps
 * (use_graph & 1: replayed from a captured HIP graph).  decode_ms covers the n_new steps only. */
int ksh_gemma_generate(ksh_gemma *m, const uint32_t *prompt, int n_prompt, int n_new,
                       int use_graph, uint32_t *out_ids, double *prefill_ms, double *decode_ms);
/* test hooks: device buffers of the last step */
ksh_buf *ksh_gemma_logits(ksh_gemma *m);
ksh_buf *ksh_gemma_hidden(ksh_gemma *m);
ksh_buf *ksh_gemma_kv(ksh_gemma *m, int layer, int which);
int ksh_gemma_pos(ksh_gemma *m);
int ksh_gemma_launches_per_token(ksh_gemma *m);

/* ---- decode loop with the layer features of the real Gemma-4 checkpoints: GemmaPrimModel::forward_token
 * (crates/ksearch_gemma/src/gemma_prim.rs:881-1275) under GemmaConfig's rules (crates/ksearch_gemma/src/lib.rs:
 * 39-167).  A layer is a sliding-window layer (head dim hd_swa, rope base rope_theta_swa, attends the last
 * sliding_window rows) or a full-attention layer (hd_full, rope_theta_full over the first hd_full*partial_rotary/2
 * pairs, attends everything); the last shared_kv_layers layers append nothing and read the cache of the nearest
 * earlier owning layer of their kind; with ple_dim > 0 every layer ends with the per-layer-embedding block.
 * Weight tensors are Q4_K or Q6_K each (what the reference keeps on the device, gemma_prim.rs:414-450; other GGUF
 * types are requantized by the loader).  The reference's attention is unscaled: attn_scale = 1. ---- */
typedef struct {
    int32_t n_layers, hidden, n_q, n_kv, vocab, max_seq;
    int32_t hd_swa, hd_full, sliding_window, shared_kv_layers, ple_dim;   /* ple_dim 0: no per-layer embeddings */
    float eps, softcap, rope_theta_swa, rope_theta_full, partial_rotary, attn_scale;
} ksh_gemma4_cfg;

typedef struct {
    int32_t is_swa, ffn;
    int32_t dt_q, dt_k, dt_v, dt_o, dt_gate, dt_up, dt_down, dt_inp_gate, dt_proj;   /* KSH_Q4K | KSH_Q6K */
    ksh_buf *wq, *wk, *wv, *wo, *wgate, *wup, *wdown;   /* wk, wv unused by layers that reuse a cache */
    ksh_buf *inp_gate, *proj;                           /* [ple_dim, hidden], [hidden, ple_dim] */
    ksh_buf *attn_norm, *q_norm, *k_norm, *post_attn_norm, *ffn_norm, *post_ffw_norm, *post_norm;   /* f32 */
    float layer_scale;                                  /* layer_output_scale (gemma_prim.rs:185) */
} ksh_gemma4_layer;

typedef struct {
    ksh_buf *token_embd;       /* [vocab, hidden], also the LM head */
    int32_t dt_embd;           /* KSH_Q4K | KSH_Q6K */
    ksh_buf *output_norm;      /* f32[hidden] */
    ksh_buf *ple_embd;         /* [vocab, n_layers*ple_dim] */
    int32_t dt_ple;            /* KSH_Q4K | KSH_Q5K | KSH_Q6K | KSH_F16 | KSH_F32 */
    ksh_buf *ple_model_proj;   /* [n_layers*ple_dim, hidden] */
    int32_t dt_ple_proj;       /* KSH_Q4K | KSH_Q6K */
    ksh_buf *ple_proj_norm;    /* f32[ple_dim] */
} ksh_gemma4_globals;

typedef struct ksh_gemma4 ksh_gemma4;

int ksh_gemma4_create(ksh_ctx *ctx, const ksh_gemma4_cfg *cfg, const ksh_gemma4_layer *layers,
                      const ksh_gemma4_globals *globals, ksh_gemma4 **out);
void ksh_gemma4_destroy(ksh_gemma4 *m);
int ksh_gemma4_reset(ksh_gemma4 *m);
/* forward_token(token, want_logits): want_logits = 0 stops after the layers (prompt tokens but the last) */
int ksh_gemma4_forward_token(ksh_gemma4 *m, uint32_t token, int want_logits, int use_graph, uint32_t *next_id);
int ksh_gemma4_generate(ksh_gemma4 *m, const uint32_t *prompt, int n_prompt, int n_new,
                        int use_graph, uint32_t *out_ids, double *prefill_ms, double *decode_ms);
/* generate_timed with its stop rule (gemma_prim.rs:1683-1710; the reference stops at ids 1 and 106): ids are
 * read one step behind the device, an id from `eos` ends the run and is the last of the *n_out ids written. */
int ksh_gemma4_generate_until(ksh_gemma4 *m, const uint32_t *prompt, int n_prompt, int n_new,
                              const uint32_t *eos, int n_eos, int use_graph, uint32_t *out_ids, int *n_out,
                              double *prefill_ms, double *decode_ms);
ksh_buf *ksh_gemma4_logits(ksh_gemma4 *m);
ksh_buf *ksh_gemma4_hidden(ksh_gemma4 *m);
/* kv_source(layer) (crates/ksearch_gemma/src/lib.rs:151-162) and that layer's cache */
int ksh_gemma4_kv_source(ksh_gemma4 *m, int layer);
ksh_buf *ksh_gemma4_kv(ksh_gemma4 *m, int layer, int which);
int ksh_gemma4_pos(ksh_gemma4 *m);
int ksh_gemma4_launches_per_token(ksh_gemma4 *m);
int ksh_gemma4_config(ksh_gemma4 *m, ksh_gemma4_cfg *cfg);

/* ---- KV slots for serving several sequences from one set of weights: KvPool, Q4_0 form
 * (crates/ksearch_gemma/src/kv_pool.rs:24-228).  max_batch slots x n_kv_layers x (K, V), each
 * max_seq * n_kv * (hd/32) * 18 bytes; the first free slot is handed out, freed slots are reused, the caller bumps
 * a slot's sequence length after the tokens it has run (kv_pool.rs:196-228), as the reference's scheduler does. ---- */
typedef struct ksh_kvpool ksh_kvpool;
int ksh_kvpool_create(ksh_ctx *ctx, int max_batch, int max_seq, int n_kv_layers, int hd, int n_kv, ksh_kvpool **out);
void ksh_kvpool_destroy(ksh_kvpool *p);
int ksh_kvpool_alloc(ksh_kvpool *p, int *slot);          /* error "KvPool full (max_batch=N)" */
int ksh_kvpool_free(ksh_kvpool *p, int slot);
int ksh_kvpool_clear_slot(ksh_kvpool *p, int slot);      /* zero the slot's caches (a fill kernel on the stream) */
int ksh_kvpool_seq_len(const ksh_kvpool *p, int slot);   /* -1: bad slot */
int ksh_kvpool_occupied(const ksh_kvpool *p, int slot);
int ksh_kvpool_bump_len_by(ksh_kvpool *p, int slot, int n, int *new_len);
int ksh_kvpool_active_batch(const ksh_kvpool *p, int *slots, int cap);   /* returns the count */
ksh_buf *ksh_kvpool_k(const ksh_kvpool *p, int slot, int layer);
ksh_buf *ksh_kvpool_v(const ksh_kvpool *p, int slot, int layer);
/* A layer's K (V) caches of all slots are one allocation, [max_batch][max_seq * n_kv * (hd/32) * 18]; the per-slot
 * buffers above are views into it.  These return the whole allocation, which a pass over several slots' tokens
 * addresses by slot index (KSH_SDPA_SLOTS with dims[6], KSH_RMSNORM_PER_HEAD_QKV_Q40 with dims[5]).  No counterpart
 * in kv_pool.rs, whose slots are separate buffers (its decode rounds are serial). */
ksh_buf *ksh_kvpool_layer_k(const ksh_kvpool *p, int layer);
ksh_buf *ksh_kvpool_layer_v(const ksh_kvpool *p, int layer);
int ksh_kvpool_dims(const ksh_kvpool *p, int *max_batch, int *max_seq, int *n_kv_layers, int *hd, int *n_kv);
/* GemmaPrimModel::bind_slot (gemma_prim.rs:1277-1292): the model's caches become the slot's (the pool needs one
 * layer per cache-owning layer and hd >= the larger head dim) and its position the slot's sequence length; the
 * device-side position follows on the stream.  Graphs are captured once per slot.  pool = NULL: back to the
 * model's own caches, at position `slot`.  The pool must outlive the binding (and the model's graphs over it:
 * bind to another pool or to NULL before destroying it). */
int ksh_gemma4_bind_slot(ksh_gemma4 *m, ksh_kvpool *pool, int slot);

/* sample_softcap_min_p (crates/ksearch_gemma/src/sample.rs:9-77), the host-side sampler of forward_token's
 * non-greedy branch, on f32 logits read back from ksh_gemma4_logits: cap*tanh(x/cap), softmax at `temperature`,
 * ids below min_p * p_max dropped, one splitmix32 draw from `seed`.  temperature < 1e-6 is the greedy argmax. */
int ksh_sample_softcap_min_p(const float *logits, size_t n, float cap, float temperature, float min_p,
                             uint32_t seed, uint32_t *out);

/* GemmaPrimModel::decode_token_sampled (gemma_prim.rs:1614-1635): one token with logits at the model's position;
 * temperature < 1e-6: the device argmax; else the logits are read back and ksh_sample_softcap_min_p draws. */
int ksh_gemma4_decode_token_sampled(ksh_gemma4 *m, uint32_t token, float temperature, float min_p, uint32_t seed,
                                    int use_graph, uint32_t *next_id);
/* GemmaPrimModel::prefill_chunk (gemma_prim.rs:1305-1607): n tokens without logits, then one synchronisation.
 * Chunks of up to 1024 tokens run as one batched pass per layer (forward_prefill_chunk), a chunk of one token as a
 * decode step.  use_graph & 1: decode steps replay the captured graph; use_graph & 2: every token goes through the
 * decode step (no batching).  ksh_gemma4_generate / _generate_until feed the prompt through this with the same flags. */
int ksh_gemma4_prefill_chunk(ksh_gemma4 *m, const uint32_t *tokens, int n, int use_graph);
/* One decode step for n (1 to 16) sequences at once: the scheduler's decode round (crates/ksearch_cli/src/scheduler.rs:
 * 163-231, there one decode_token_sampled per request) as ONE pass over the weights.  Row i feeds tokens[i] to the
 * sequence in pool slot slots[i] at that slot's sequence length: its K / V row is appended there and it attends that
 * slot's rows.  next_ids[i] is the greedy id, or, where temperature (may be NULL: all greedy) gives
 * temperature[i] >= 1e-6, the draw of ksh_sample_softcap_min_p on row i's logits with min_p[i] and seed[i].  The
 * caller bumps the slots' lengths afterwards (ksh_kvpool_bump_len_by), as after a serial step.  The model's own
 * position and binding are not touched; ksh_gemma4_bind_slot re-seeks a bound slot whose length has moved.
 * Slots must be occupied and distinct. */
int ksh_gemma4_decode_round(ksh_gemma4 *m, ksh_kvpool *pool, const int32_t *slots, const uint32_t *tokens, int n,
                            const float *temperature, const float *min_p, const uint32_t *seed, uint32_t *next_ids);
/* f32 [n][vocab]: the logits of the last round's rows */
ksh_buf *ksh_gemma4_round_logits(ksh_gemma4 *m);

/* ---- decode-before-prefill slot scheduler: spawn_scheduler and its rounds (crates/ksearch_cli/src/scheduler.rs:
 * 78-349) as a tick the host drives.  One tick = admit waiting requests into free slots (alloc + clear), one
 * decode token for every decoding request, chunked prefill for the prefilling ones (prefill_chunk tokens each
 * while anything decodes, else up to prefill_tokens_per_tick), then finished requests free their slots.  GPU
 * work is serial, as in the reference.  Requests are token ids; where the reference matches stop strings on the
 * decoded text (scheduler.rs:207-217), `stop` is asked instead (non-zero: finish with reason "stop", the token is
 * not emitted).  What the reference sends over channels is queued as events and drained with ksh_serve_poll.
 * One thread drives a scheduler (submit, cancel, tick and poll are not synchronised with one another): the
 * reference's job channel from its HTTP handlers is the embedding host's to keep. ---- */
typedef struct ksh_serve ksh_serve;
typedef int (*ksh_serve_stop_fn)(void *user, uint64_t request, uint32_t token);
typedef struct {
    int32_t slots;                     /* requests admitted at once (SchedulerConfig, scheduler.rs:60-76: 4) */
    int32_t prefill_chunk;             /* 256 */
    int32_t prefill_tokens_per_tick;   /* 2048 */
    uint32_t eos[2];                   /* EOS_IDS (scheduler.rs:14): 1, 106 */
    int32_t use_graph;                 /* replay the model's HIP graphs (1) or launch eagerly (0) */
    int32_t batched_decode;            /* from this many decoding requests on (>= 2; default 3) they take their step as one
                                        * ksh_gemma4_decode_round (the weights are read once per round); 0: always one
                                        * by one, as the reference does */
    ksh_serve_stop_fn stop;            /* may be NULL */
    void *stop_user;
} ksh_serve_cfg;
enum ksh_serve_event_kind { KSH_SERVE_TOKEN = 0, KSH_SERVE_DONE = 1, KSH_SERVE_ERROR = 2 };
/* finish_reason of StreamEvent::Done: "stop", "length", "cancelled"; "error" accompanies an error event */
enum ksh_finish_reason { KSH_FINISH_STOP = 0, KSH_FINISH_LENGTH = 1, KSH_FINISH_CANCELLED = 2, KSH_FINISH_ERROR = 3 };
typedef struct {
    uint64_t request;
    int32_t kind;                 /* ksh_serve_event_kind */
    uint32_t token;               /* KSH_SERVE_TOKEN */
    int32_t reason;               /* KSH_SERVE_DONE: ksh_finish_reason */
    uint32_t prompt_tokens, completion_tokens;   /* KSH_SERVE_DONE */
} ksh_serve_event;
int ksh_serve_default_cfg(ksh_serve_cfg *cfg);
/* the model and the pool must outlive the scheduler; the model is bound to the pool's slots from here on */
int ksh_serve_create(ksh_gemma4 *model, ksh_kvpool *pool, const ksh_serve_cfg *cfg, ksh_serve **out);
void ksh_serve_destroy(ksh_serve *s);
/* InferenceRequest (scheduler.rs:28-36).  An empty prompt is accepted here and answered with an error event at
 * admission, as the reference does.  max_tokens 0 counts as 1; the sampler's state starts at seed | 1. */
int ksh_serve_submit(ksh_serve *s, const uint32_t *prompt, size_t n_prompt, size_t max_tokens, float temperature,
                     float min_p, uint32_t seed, uint64_t *request);
/* the reference notices a dropped receiver when it sends the next token: the request then finishes "cancelled" */
int ksh_serve_cancel(ksh_serve *s, uint64_t request);
int ksh_serve_tick(ksh_serve *s);
size_t ksh_serve_poll(ksh_serve *s, ksh_serve_event *out, size_t cap);   /* returns the number written */
/* text of the oldest error event not yet asked for (one per KSH_SERVE_ERROR event, in their order); NULL: none */
const char *ksh_serve_error_text(ksh_serve *s);
int ksh_serve_pending(const ksh_serve *s, int *waiting, int *active);

/* ---- GGUF files: Gguf::open and its accessors (crates/ksearch_gguf/src/gguf_impl.rs:217-420).  The file is
 * memory-mapped; tensor data pointers stay valid until ksh_gguf_close.  A malformed file is an error here where
 * the reference panics. ---- */
enum ksh_ggml_type {   /* gguf_impl.rs:19-31 */
    KSH_GGML_F32 = 0, KSH_GGML_F16 = 1, KSH_GGML_Q4_0 = 2, KSH_GGML_Q4_1 = 3, KSH_GGML_Q5_1 = 7, KSH_GGML_Q8_0 = 8,
    KSH_GGML_Q4_K = 12, KSH_GGML_Q5_K = 13, KSH_GGML_Q6_K = 14, KSH_GGML_BF16 = 30
};
typedef struct ksh_gguf ksh_gguf;
int ksh_gguf_open(const char *path, ksh_gguf **out);
void ksh_gguf_close(ksh_gguf *g);
int ksh_gguf_version(const ksh_gguf *g);
int64_t ksh_gguf_n_tensors(const ksh_gguf *g);
int ksh_gguf_tensor_name(const ksh_gguf *g, int64_t index, char *dst, size_t n);
int ksh_gguf_has_tensor(const ksh_gguf *g, const char *name);
/* TensorInfo + tensor_raw: dims[0] is the contiguous dimension (columns), the rest multiply to the row count;
 * any out pointer may be NULL */
int ksh_gguf_tensor(const ksh_gguf *g, const char *name, int32_t *ggml_type, int64_t *dims /*[4]*/, int32_t *n_dims,
                    const void **data, size_t *bytes);
/* metadata accessors: 0 when the key exists with a fitting type, 1 otherwise (the reference's None) */
int ksh_gguf_get_u32(const ksh_gguf *g, const char *key, uint32_t *out);
int ksh_gguf_get_f32(const ksh_gguf *g, const char *key, float *out);
int ksh_gguf_get_str(const ksh_gguf *g, const char *key, char *dst, size_t n);
/* u32 / i32 / bool arrays (bools as 0/1); an integer scalar reads as a list of one (get_usize_list) */
int ksh_gguf_get_arr_u32(const ksh_gguf *g, const char *key, uint32_t *dst, int cap, int *n);
int ksh_gguf_arr_is_bool(const ksh_gguf *g, const char *key);
/* dequant_blocks for F32 / F16 / BF16 / Q4_0 / Q4_1 / Q5_1 / Q8_0 on the host (gguf_impl.rs:577-689); the
 * K-quants are dequantized by KSH_DEQUANT on the device */
int ksh_gguf_dequant_host(int32_t ggml_type, const void *src, size_t n_elems, float *out);

/* GemmaConfig::from_gguf (crates/ksearch_gemma/src/lib.rs:39-122).  ffn / is_swa (room for `cap` layers) may be
 * NULL.  ple_dim is 0 when the file has no per-layer tables. */
int ksh_gemma4_config_from_gguf(const ksh_gguf *g, int max_seq, ksh_gemma4_cfg *cfg, int32_t *ffn, int32_t *is_swa, int cap);
/* GemmaPrimModel's load path (crates/ksearch_gemma/src/gemma_prim.rs:146-450): uploads Q4_K (and Q6_K) tensors as
 * they are, converts the rest, builds the model, which then owns the buffers. */
enum { KSH_LOAD_KEEP_Q6K = 1 };   /* do not requantize Q6_K ffn_down / attn_v to Q4_K (the reference does, :418-433) */
int ksh_gemma4_load_gguf(ksh_ctx *ctx, const ksh_gguf *g, int max_seq, int flags, ksh_gemma4 **out);

#ifdef __cplusplus
}
#endif
#endif
