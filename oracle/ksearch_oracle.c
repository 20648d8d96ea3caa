/*
 * ksearch_oracle.c — CPU restatement of ksearch's quantized decode arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP path.  See the header for
 * the per-function pinning status.  Reference citations are paths inside the
 * ksearch source tree.
 *
 * Build: gcc -O2 -fno-fast-math -ffp-contract=off -fopenmp -shared -fPIC
 * (-ffp-contract=off matters: the reference rounds `d1*q` and `- mn1`
 * separately, gguf_impl.rs:710, and Rust never fuses them).
 */
#include "ksearch_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define QK_K 256

/* ------------------------------------------------------------------ f16/bf16 */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* lib.rs:10-12 */
float ko_bf16_to_f32(uint16_t v) { return u2f((uint32_t)v << 16); }
/* lib.rs:15-17 (wrapping add, then >>16) */
uint16_t ko_f32_to_bf16(float v) { return (uint16_t)((f2u(v) + 0x8000u) >> 16); }

/* lib.rs:20-35: sign * mant * 2^-24 (subnormal), inf/NaN, else
 * sign * (1 + mant/1024) * 2^(exp-15).  Every step is exact in f32. */
float ko_f16_to_f32(uint16_t v)
{
    float sign = (float)(v >> 15) * -2.0f + 1.0f;
    uint32_t e = (v >> 10) & 0x1F, mant = v & 0x3FF;
    if (e == 0) return sign * (float)mant * ldexpf(1.0f, -24);
    if (e == 31) return mant == 0 ? sign * INFINITY : NAN;
    return sign * (1.0f + (float)mant / 1024.0f) * ldexpf(1.0f, (int)e - 15);
}

/* lib.rs:39-75.  Despite its doc comment the reference rounds half UP in
 * magnitude (adds 0x1000 and truncates) and flushes [2^-25, 2^-24) to zero. */
uint16_t ko_f32_to_f16(float value)
{
    uint32_t bits = f2u(value);
    uint16_t sign = (uint16_t)((bits >> 16) & 0x8000);
    int32_t e = (int32_t)((bits >> 23) & 0xFF);
    uint32_t mant = bits & 0x7FFFFF;
    if (e == 255)
        return mant == 0 ? (uint16_t)(sign | 0x7C00) : (uint16_t)(sign | 0x7C00 | (mant >> 13));
    e -= 127;
    if (e > 15) return (uint16_t)(sign | 0x7C00);
    if (e < -14) {
        if (e < -24) return sign;
        mant |= 0x800000;
        uint32_t shift = (uint32_t)(-14 - e) + 13;
        uint32_t rounded = (mant + (1u << (shift - 1))) >> shift;
        return (uint16_t)(sign | rounded);
    }
    uint16_t half_exp = (uint16_t)(e + 15);
    uint32_t half_mant = mant + 0x1000;
    if (half_mant & 0x800000) return (uint16_t)(sign | ((half_exp + 1) << 10));
    return (uint16_t)(sign | (half_exp << 10) | (half_mant >> 13));
}

/* IEEE round-to-nearest-even f32->f16: what Metal's half() (render.rs:1033,
 * 1046) and a HIP __float2half_rn compute. */
uint16_t ko_f32_to_f16_rne(float value)
{
    uint32_t bits = f2u(value);
    uint16_t sign = (uint16_t)((bits >> 16) & 0x8000);
    uint32_t a = bits & 0x7FFFFFFF;
    if (a >= 0x7F800000) return a > 0x7F800000 ? (uint16_t)(sign | 0x7E00) : (uint16_t)(sign | 0x7C00);
    if (a >= 0x477FF000) return (uint16_t)(sign | 0x7C00);        /* >= 65520 -> inf */
    if (a < 0x33000001) return sign;                              /* <= 2^-25 -> 0 */
    int32_t e = (int32_t)(a >> 23) - 127;
    uint32_t mant = (a & 0x7FFFFF) | 0x800000;
    uint32_t shift = e < -14 ? (uint32_t)(13 + (-14 - e)) : 13;
    uint32_t q = mant >> shift, rem = mant & ((1u << shift) - 1), halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1))) q++;
    uint32_t h = e < -14 ? q : (((uint32_t)(e + 15) << 10) + (q - 0x400));
    return (uint16_t)(sign | h);
}

/* ------------------------------------------------------------------ layouts */

/* gguf_impl.rs:563-573 */
void ko_get_scale_min_k4(int j, const uint8_t *q, uint8_t *d, uint8_t *m)
{
    if (j < 4) {
        *d = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *d = (uint8_t)((q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* gguf_impl.rs:50-64 (block_spec), ksearch_ir/src/lib.rs:52-74 */
static int block_spec(int dtype, size_t *elems, size_t *bytes)
{
    switch (dtype) {
    case KO_F32:  *elems = 1;    *bytes = 4;   return 0;
    case KO_F16:  *elems = 1;    *bytes = 2;   return 0;
    case KO_BF16: *elems = 1;    *bytes = 2;   return 0;
    case KO_Q40:  *elems = 32;   *bytes = 18;  return 0;
    case KO_Q4K:  *elems = QK_K; *bytes = 144; return 0;
    case KO_Q5K:  *elems = QK_K; *bytes = 176; return 0;
    case KO_Q6K:  *elems = QK_K; *bytes = 210; return 0;
    }
    return -1;
}

size_t ko_row_bytes(int dtype, size_t cols)
{
    size_t e, b;
    if (block_spec(dtype, &e, &b) || cols % e) return 0;
    return cols / e * b;
}

static inline uint16_t rd16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }

/* gguf_impl.rs:618-633 */
static void deq_q40_block(const uint8_t *blk, float *out)
{
    float d = ko_f16_to_f32(rd16(blk));
    const uint8_t *qs = blk + 2;
    for (int i = 0; i < 16; i++) {
        int lo = (int)(qs[i] & 0x0F) - 8, hi = (int)(qs[i] >> 4) - 8;
        out[i] = (float)lo * d;
        out[i + 16] = (float)hi * d;
    }
}

/* gguf_impl.rs:690-721 */
static void deq_q4k_block(const uint8_t *blk, float *out)
{
    float d = ko_f16_to_f32(rd16(blk)), dmin = ko_f16_to_f32(rd16(blk + 2));
    const uint8_t *scales = blk + 4, *qs = blk + 16;
    int is = 0, qoff = 0;
    for (int y = 0; y < QK_K; y += 64) {
        uint8_t sc1, m1, sc2, m2;
        ko_get_scale_min_k4(is, scales, &sc1, &m1);
        ko_get_scale_min_k4(is + 1, scales, &sc2, &m2);
        float d1 = d * (float)sc1, mn1 = dmin * (float)m1;
        float d2 = d * (float)sc2, mn2 = dmin * (float)m2;
        for (int l = 0; l < 32; l++) out[y + l] = d1 * (float)(qs[qoff + l] & 0x0F) - mn1;
        for (int l = 0; l < 32; l++) out[y + 32 + l] = d2 * (float)(qs[qoff + l] >> 4) - mn2;
        qoff += 32;
        is += 2;
    }
}

/* gguf_impl.rs:722-760 */
static void deq_q5k_block(const uint8_t *blk, float *out)
{
    float d = ko_f16_to_f32(rd16(blk)), dmin = ko_f16_to_f32(rd16(blk + 2));
    const uint8_t *scales = blk + 4, *qh = blk + 16, *qs = blk + 48;
    int is = 0, qoff = 0;
    uint8_t u1 = 1, u2 = 2;
    for (int y = 0; y < QK_K; y += 64) {
        uint8_t sc1, m1, sc2, m2;
        ko_get_scale_min_k4(is, scales, &sc1, &m1);
        ko_get_scale_min_k4(is + 1, scales, &sc2, &m2);
        float d1 = d * (float)sc1, mn1 = dmin * (float)m1;
        float d2 = d * (float)sc2, mn2 = dmin * (float)m2;
        for (int l = 0; l < 32; l++) {
            float hi = (qh[l] & u1) ? 16.0f : 0.0f;
            out[y + l] = d1 * ((float)(qs[qoff + l] & 0x0F) + hi) - mn1;
        }
        for (int l = 0; l < 32; l++) {
            float hi = (qh[l] & u2) ? 16.0f : 0.0f;
            out[y + 32 + l] = d2 * ((float)(qs[qoff + l] >> 4) + hi) - mn2;
        }
        qoff += 32;
        is += 2;
        u1 = (uint8_t)(u1 << 2);
        u2 = (uint8_t)(u2 << 2);
    }
}

/* gguf_impl.rs:761-791; `d * sc * q` associates as (d*sc)*q */
static void deq_q6k_block(const uint8_t *blk, float *out)
{
    float d = ko_f16_to_f32(rd16(blk + 208));
    for (int half = 0; half < 2; half++) {
        const uint8_t *ql = blk + half * 64, *qh = blk + 128 + half * 32;
        const int8_t *sc = (const int8_t *)(blk + 192 + half * 8);
        float *y = out + half * 128;
        for (int l = 0; l < 32; l++) {
            int is = l / 16;
            int q1 = (int)((ql[l] & 0x0F) | (((qh[l] >> 0) & 3) << 4)) - 32;
            int q2 = (int)((ql[l + 32] & 0x0F) | (((qh[l] >> 2) & 3) << 4)) - 32;
            int q3 = (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
            int q4 = (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
            y[l] = d * (float)sc[is] * (float)q1;
            y[l + 32] = d * (float)sc[is + 2] * (float)q2;
            y[l + 64] = d * (float)sc[is + 4] * (float)q3;
            y[l + 96] = d * (float)sc[is + 6] * (float)q4;
        }
    }
}

static void deq_block(int dtype, const uint8_t *blk, float *out)
{
    switch (dtype) {
    case KO_Q40: deq_q40_block(blk, out); break;
    case KO_Q4K: deq_q4k_block(blk, out); break;
    case KO_Q5K: deq_q5k_block(blk, out); break;
    case KO_Q6K: deq_q6k_block(blk, out); break;
    case KO_F32: memcpy(out, blk, 4); break;
    case KO_F16: out[0] = ko_f16_to_f32(rd16(blk)); break;
    case KO_BF16: out[0] = ko_bf16_to_f32(rd16(blk)); break;
    }
}

/* gguf_impl.rs:472-476 (dequant_type_to_f32) over :577-794 */
int ko_dequant(int dtype, const uint8_t *data, size_t total_elems, float *out)
{
    size_t e, b;
    if (block_spec(dtype, &e, &b)) return -1;
    size_t nb = total_elems / e;
    for (size_t i = 0; i < nb; i++) deq_block(dtype, data + i * b, out + i * e);
    return 0;
}

/* ------------------------------------------------------------------ quantizers */

/* gguf_impl.rs:803-808 */
static inline int nearest_int(float fval)
{
    float val = fval + 12582912.0f;
    int32_t i;
    memcpy(&i, &val, 4);
    return (i & 0x007fffff) - 0x00400000;
}

static inline int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* gguf_impl.rs:811-901 */
static float make_qkx2_quants(int n, int nmax, const float *x, const float *weights,
                              uint8_t *L, float *the_min, uint8_t *Laux,
                              float rmin, float rdelta, int nstep, int use_mad)
{
    float min = x[0], max = x[0], sum_w = weights[0], sum_x = sum_w * x[0];
    for (int i = 1; i < n; i++) {
        if (x[i] < min) min = x[i];
        if (x[i] > max) max = x[i];
        float w = weights[i];
        sum_w += w;
        sum_x += w * x[i];
    }
    if (min > 0.0f) min = 0.0f;
    if (max == min) {
        for (int i = 0; i < n; i++) L[i] = 0;
        *the_min = -min;
        return 0.0f;
    }
    float iscale = (float)nmax / (max - min);
    float scale = 1.0f / iscale;
    float best_error = 0.0f;
    for (int i = 0; i < n; i++) {
        int l = clampi(nearest_int(iscale * (x[i] - min)), 0, nmax);
        L[i] = (uint8_t)l;
        float diff = scale * (float)l + min - x[i];
        diff = use_mad ? fabsf(diff) : diff * diff;
        best_error += weights[i] * diff;
    }
    if (nstep < 1) {
        *the_min = -min;
        return scale;
    }
    for (int is = 0; is <= nstep; is++) {
        iscale = (rmin + rdelta * (float)is + (float)nmax) / (max - min);
        float sum_l = 0.0f, sum_l2 = 0.0f, sum_xl = 0.0f;
        for (int i = 0; i < n; i++) {
            int l = clampi(nearest_int(iscale * (x[i] - min)), 0, nmax);
            Laux[i] = (uint8_t)l;
            float w = weights[i], lf = (float)l;
            sum_l += w * lf;
            sum_l2 += w * lf * lf;
            sum_xl += w * lf * x[i];
        }
        float D = sum_w * sum_l2 - sum_l * sum_l;
        if (D > 0.0f) {
            float this_scale = (sum_w * sum_xl - sum_x * sum_l) / D;
            float this_min = (sum_l2 * sum_x - sum_l * sum_xl) / D;
            if (this_min > 0.0f) {
                this_min = 0.0f;
                this_scale = sum_xl / sum_l2;
            }
            float cur_error = 0.0f;
            for (int i = 0; i < n; i++) {
                float diff = this_scale * (float)Laux[i] + this_min - x[i];
                diff = use_mad ? fabsf(diff) : diff * diff;
                cur_error += weights[i] * diff;
            }
            if (cur_error < best_error) {
                memcpy(L, Laux, (size_t)n);
                best_error = cur_error;
                scale = this_scale;
                min = this_min;
            }
        }
    }
    *the_min = -min;
    return scale;
}

/* gguf_impl.rs:905-1016 */
static void quantize_q4k_block(const float *x, uint8_t *blk)
{
    uint8_t L[QK_K], Laux[32];
    float weights[32], mins[QK_K / 32], scales[QK_K / 32];
    float max_scale = 0.0f, max_min = 0.0f;
    for (int j = 0; j < QK_K / 32; j++) {
        int base = 32 * j;
        float sum_x2 = 0.0f;
        for (int t = 0; t < 32; t++) sum_x2 += x[base + t] * x[base + t];
        float av_x = sqrtf(sum_x2 / 32.0f);
        for (int t = 0; t < 32; t++) weights[t] = av_x + fabsf(x[base + t]);
        scales[j] = make_qkx2_quants(32, 15, x + base, weights, L + base, &mins[j], Laux,
                                     -1.0f, 0.1f, 20, 0);
        if (scales[j] > max_scale) max_scale = scales[j];
        if (mins[j] > max_min) max_min = mins[j];
    }
    float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
    float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
    uint16_t db = ko_f32_to_f16(max_scale / 63.0f), mb = ko_f32_to_f16(max_min / 63.0f);
    blk[0] = (uint8_t)(db & 0xFF); blk[1] = (uint8_t)(db >> 8);
    blk[2] = (uint8_t)(mb & 0xFF); blk[3] = (uint8_t)(mb >> 8);
    uint8_t *sc = blk + 4;
    memset(sc, 0, 12);
    for (int j = 0; j < QK_K / 32; j++) {
        uint8_t ls = (uint8_t)nearest_int(inv_scale * scales[j]);
        uint8_t lm = (uint8_t)nearest_int(inv_min * mins[j]);
        if (ls > 63) ls = 63;
        if (lm > 63) lm = 63;
        if (j < 4) {
            sc[j] = ls;
            sc[j + 4] = lm;
        } else {
            sc[j + 4] = (uint8_t)((ls & 0x0F) | ((lm & 0x0F) << 4));
            sc[j - 4] |= (uint8_t)((ls >> 4) << 6);
            sc[j] |= (uint8_t)((lm >> 4) << 6);
        }
    }
    float d = ko_f16_to_f32(db), dmin = ko_f16_to_f32(mb);
    for (int j = 0; j < QK_K / 32; j++) {
        uint8_t s, m;
        ko_get_scale_min_k4(j, sc, &s, &m);
        float dj = d * (float)s;
        if (dj == 0.0f) continue;
        float dm = dmin * (float)m;
        for (int ii = 0; ii < 32; ii++)
            L[32 * j + ii] = (uint8_t)clampi(nearest_int((x[32 * j + ii] + dm) / dj), 0, 15);
    }
    uint8_t *qs = blk + 16;
    int qoff = 0;
    for (int j = 0; j < QK_K; j += 64) {
        for (int t = 0; t < 32; t++) qs[qoff + t] = (uint8_t)(L[j + t] | (L[j + t + 32] << 4));
        qoff += 32;
    }
}

void ko_quantize_q4k(const float *x, size_t n, uint8_t *out)
{
    size_t nb = n / QK_K;
#pragma omp parallel for schedule(static)
    for (size_t b = 0; b < nb; b++) quantize_q4k_block(x + b * QK_K, out + b * 144);
}

/* Build's own Q6_K packer (the reference has none).  Per 16-wide group the
 * scale maps the largest-magnitude value to -32; the 16 group scales are then
 * stored as int8 multiples of one f16 super-scale. */
static void quantize_q6k_block(const float *x, uint8_t *blk)
{
    float gs[16], max_abs_scale = 0.0f, max_scale = 0.0f;
    for (int g = 0; g < 16; g++) {
        float amax = 0.0f, mx = 0.0f;
        for (int i = 0; i < 16; i++) {
            float a = fabsf(x[16 * g + i]);
            if (a > amax) { amax = a; mx = x[16 * g + i]; }
        }
        gs[g] = amax > 0.0f ? mx / -32.0f : 0.0f;
        if (fabsf(gs[g]) > max_abs_scale) { max_abs_scale = fabsf(gs[g]); max_scale = gs[g]; }
    }
    memset(blk, 0, 210);
    if (max_abs_scale == 0.0f) return;
    float iscale = -128.0f / max_scale;
    uint16_t db = ko_f32_to_f16_rne(1.0f / iscale);
    blk[208] = (uint8_t)(db & 0xFF); blk[209] = (uint8_t)(db >> 8);
    float d = ko_f16_to_f32(db);
    int8_t *sc = (int8_t *)(blk + 192);
    uint8_t L[QK_K];
    for (int g = 0; g < 16; g++) {
        int s = clampi(nearest_int(iscale * gs[g]), -128, 127);
        sc[g] = (int8_t)s;
        float dg = d * (float)s;
        for (int i = 0; i < 16; i++) {
            int l = dg != 0.0f ? clampi(nearest_int(x[16 * g + i] / dg), -32, 31) : 0;
            L[16 * g + i] = (uint8_t)(l + 32);
        }
    }
    uint8_t *ql = blk, *qh = blk + 128;
    for (int half = 0; half < 2; half++) {
        const uint8_t *Lh = L + 128 * half;
        for (int l = 0; l < 32; l++) {
            uint8_t q1 = Lh[l], q2 = Lh[l + 32], q3 = Lh[l + 64], q4 = Lh[l + 96];
            ql[64 * half + l] = (uint8_t)((q1 & 0x0F) | ((q3 & 0x0F) << 4));
            ql[64 * half + l + 32] = (uint8_t)((q2 & 0x0F) | ((q4 & 0x0F) << 4));
            qh[32 * half + l] = (uint8_t)((q1 >> 4) | ((q2 >> 4) << 2) | ((q3 >> 4) << 4) | ((q4 >> 4) << 6));
        }
    }
}

void ko_quantize_q6k(const float *x, size_t n, uint8_t *out)
{
    size_t nb = n / QK_K;
#pragma omp parallel for schedule(static)
    for (size_t b = 0; b < nb; b++) quantize_q6k_block(x + b * QK_K, out + b * 210);
}

/* Metal round(): half away from zero */
static inline float round_away(float v) { return roundf(v); }

/* render.rs:1021-1059.  half_roundtrip=1 is `ksearch_pack_q40_th` (values pass
 * through half() first, RNE as on a GPU); 0 is `ksearch_pack_q40` reading
 * values that already are halves. */
void ko_pack_q40(const float *src, size_t n, uint8_t *out, int half_roundtrip)
{
    for (size_t b = 0; b < n / 32; b++) {
        float vals[32], max_abs = 0.0f;
        for (int d = 0; d < 32; d++) {
            float v = src[b * 32 + d];
            if (half_roundtrip) v = ko_f16_to_f32(ko_f32_to_f16_rne(v));
            vals[d] = v;
            max_abs = fmaxf(max_abs, fabsf(v));
        }
        float scale = max_abs > 0.0f ? max_abs / 7.0f : 1.0f;
        float inv = 1.0f / scale;
        uint8_t *blk = out + b * 18;
        uint16_t sb = ko_f32_to_f16_rne(scale);
        blk[0] = (uint8_t)(sb & 0xFF); blk[1] = (uint8_t)(sb >> 8);
        for (int i = 0; i < 16; i++) {
            int lo = clampi((int)round_away(vals[i] * inv) + 8, 0, 15);
            int hi = clampi((int)round_away(vals[i + 16] * inv) + 8, 0, 15);
            blk[2 + i] = (uint8_t)(lo | (hi << 4));
        }
    }
}

/* ------------------------------------------------------------------ GEMV / GEMM */

int ko_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

static int pick_threads(int threads)
{
    int mx = ko_max_threads();
    return (threads <= 0 || threads > mx) ? mx : threads;
}

/* check_mul_mm.rs:60-71: `s += wd[r*cols+c] * x[c]`, c ascending, f32.
 * Dequantization is fused per block, which leaves the value sequence and the
 * order of additions untouched. */
static float row_dot(int dtype, const uint8_t *row, size_t cols, const float *x,
                     size_t be, size_t bb)
{
    float buf[QK_K], s = 0.0f;
    for (size_t b = 0; b < cols / be; b++) {
        deq_block(dtype, row + b * bb, buf);
        for (size_t c = 0; c < be; c++) s += buf[c] * x[b * be + c];
    }
    return s;
}

int ko_matvec(int dtype, const uint8_t *w, size_t rows, size_t cols, const float *x,
              float *y, int threads)
{
    size_t be, bb;
    if (block_spec(dtype, &be, &bb) || cols % be) return -1;
    size_t rb = cols / be * bb;
    int nt = pick_threads(threads);
#pragma omp parallel for schedule(static) num_threads(nt)
    for (size_t r = 0; r < rows; r++) y[r] = row_dot(dtype, w + r * rb, cols, x, be, bb);
    return 0;
}

int ko_matmul(int dtype, const uint8_t *w, size_t rows, size_t cols, const float *x,
              size_t batch, float *y, int threads)
{
    size_t be, bb;
    if (block_spec(dtype, &be, &bb) || cols % be) return -1;
    size_t rb = cols / be * bb;
    int nt = pick_threads(threads);
#pragma omp parallel for schedule(static) num_threads(nt)
    for (size_t r = 0; r < rows; r++) {
        float *wd = (float *)malloc(cols * sizeof(float));
        for (size_t b = 0; b < cols / be; b++) deq_block(dtype, w + r * rb + b * bb, wd + b * be);
        for (size_t t = 0; t < batch; t++) {
            const float *xt = x + t * cols;
            float s = 0.0f;
            for (size_t c = 0; c < cols; c++) s += wd[c] * xt[c];
            y[t * rows + r] = s;
        }
        free(wd);
    }
    return 0;
}

int ko_matvec_f64(int dtype, const uint8_t *w, size_t rows, size_t cols, const float *x,
                  double *y, int threads)
{
    size_t be, bb;
    if (block_spec(dtype, &be, &bb) || cols % be) return -1;
    size_t rb = cols / be * bb;
    int nt = pick_threads(threads);
#pragma omp parallel for schedule(static) num_threads(nt)
    for (size_t r = 0; r < rows; r++) {
        float buf[QK_K];
        double s = 0.0;
        for (size_t b = 0; b < cols / be; b++) {
            deq_block(dtype, w + r * rb + b * bb, buf);
            for (size_t c = 0; c < be; c++) s += (double)buf[c] * (double)x[b * be + c];
        }
        y[r] = s;
    }
    return 0;
}

/* ------------------------------------------------------------------ attention */

static void kv_row(const uint8_t *base, int n_kv, int hd, int t, int kvh, float *out)
{
    /* element index ((start+t)*n_kv + kv_head)*hd + d, lower.rs:5086-5102 */
    const uint8_t *row = base + ((size_t)t * n_kv + kvh) * (size_t)(hd / 32) * 18;
    for (int b = 0; b < hd / 32; b++) deq_q40_block(row + b * 18, out + b * 32);
}

/* One head over rows [t0,t1): the update order of lower.rs:5140-5359. */
static void sdpa_span(const float *qh, const uint8_t *k, const uint8_t *v, int n_kv, int hd,
                      int kvh, int t0, int t1, float scale, float *m_io, float *l_io, float *O)
{
    float *kr = (float *)malloc(sizeof(float) * (size_t)hd * 2), *vr = kr + hd;
    float m = *m_io, l = *l_io;
    for (int t = t0; t < t1; t++) {
        kv_row(k, n_kv, hd, t, kvh, kr);
        kv_row(v, n_kv, hd, t, kvh, vr);
        float s = 0.0f;
        for (int d = 0; d < hd; d++) s += qh[d] * kr[d];
        s *= scale;
        float m2 = fmaxf(m, s);
        float alpha = expf(m - m2), e = expf(s - m2);
        l = l * alpha + e;
        m = m2;
        for (int d = 0; d < hd; d++) O[d] = O[d] * alpha + e * vr[d];
    }
    *m_io = m;
    *l_io = l;
    free(kr);
}

/* lower.rs:4897-5359.  `scale` multiplies q.k (1.0 reproduces the reference,
 * which has no softmax scale). */
void ko_sdpa_online(const float *q, const uint8_t *k, const uint8_t *v, int n_q, int n_kv,
                    int hd, int tlen, int start, float scale, float *out)
{
    int groups = n_q / n_kv;
    for (int h = 0; h < n_q; h++) {
        float m = -1.0e30f, l = 0.0f;
        float *O = out + (size_t)h * hd;
        for (int d = 0; d < hd; d++) O[d] = 0.0f;
        sdpa_span(q + (size_t)h * hd, k, v, n_kv, hd, h / groups, start, start + tlen, scale, &m, &l, O);
        float inv_l = 1.0f / l;
        for (int d = 0; d < hd; d++) O[d] = O[d] * inv_l;
    }
}

/* lower.rs:5367-5894 (pass 1: chunk = ceil(tlen/nwg), partials m,l,O) and
 * :5897-6087 (pass 2: log-sum-exp merge, empty partitions carry m=-1e30,l=0). */
void ko_sdpa_mwg(const float *q, const uint8_t *k, const uint8_t *v, int n_q, int n_kv, int hd,
                 int tlen, int start, float scale, int nwg, float *out)
{
    int groups = n_q / n_kv;
    int chunk = (tlen + nwg - 1) / nwg;
    float *pm = (float *)malloc(sizeof(float) * (size_t)nwg * (size_t)(hd + 2));
    for (int h = 0; h < n_q; h++) {
        for (int p = 0; p < nwg; p++) {
            float *rec = pm + (size_t)p * (hd + 2);
            int p0 = p * chunk, p1 = p0 + chunk < tlen ? p0 + chunk : tlen;
            rec[0] = -1.0e30f;
            rec[1] = 0.0f;
            for (int d = 0; d < hd; d++) rec[2 + d] = 0.0f;
            if (p0 < p1)
                sdpa_span(q + (size_t)h * hd, k, v, n_kv, hd, h / groups, start + p0, start + p1,
                          scale, &rec[0], &rec[1], rec + 2);
        }
        float m = -1.0e30f, l = 0.0f;
        float *O = out + (size_t)h * hd;
        for (int d = 0; d < hd; d++) O[d] = 0.0f;
        for (int p = 0; p < nwg; p++) {
            const float *rec = pm + (size_t)p * (hd + 2);
            float m2 = fmaxf(m, rec[0]);
            float alpha = expf(m - m2), beta = expf(rec[0] - m2);
            l = l * alpha + rec[1] * beta;
            m = m2;
            for (int d = 0; d < hd; d++) O[d] = O[d] * alpha + rec[2 + d] * beta;
        }
        float inv_l = 1.0f / l;
        for (int d = 0; d < hd; d++) O[d] = O[d] * inv_l;
    }
    free(pm);
}

/* textbook softmax(scale*q.K^T)V in f64 with a two-pass max: the brute force
 * the f32 variants are checked against. */
void ko_sdpa_f64(const float *q, const uint8_t *k, const uint8_t *v, int n_q, int n_kv, int hd,
                 int tlen, int start, float scale, double *out)
{
    int groups = n_q / n_kv;
    float *kr = (float *)malloc(sizeof(float) * (size_t)hd);
    double *s = (double *)malloc(sizeof(double) * (size_t)(tlen > 0 ? tlen : 1));
    for (int h = 0; h < n_q; h++) {
        double mx = -INFINITY;
        for (int t = 0; t < tlen; t++) {
            kv_row(k, n_kv, hd, start + t, h / groups, kr);
            double a = 0.0;
            for (int d = 0; d < hd; d++) a += (double)q[(size_t)h * hd + d] * (double)kr[d];
            s[t] = a * (double)scale;
            if (s[t] > mx) mx = s[t];
        }
        double l = 0.0;
        double *O = out + (size_t)h * hd;
        for (int d = 0; d < hd; d++) O[d] = 0.0;
        for (int t = 0; t < tlen; t++) {
            double e = exp(s[t] - mx);
            l += e;
            kv_row(v, n_kv, hd, start + t, h / groups, kr);
            for (int d = 0; d < hd; d++) O[d] += e * (double)kr[d];
        }
        for (int d = 0; d < hd; d++) O[d] /= l;
    }
    free(kr);
    free(s);
}

/* ------------------------------------------------------------------ glue ops */

/* sample.rs:18-36 (CPU twin of lower.rs:6090-6156): strict `>` scan in index
 * order, so the lowest index wins ties of the soft-capped value. */
uint32_t ko_softcap_argmax(const float *x, size_t n, float cap)
{
    uint32_t best_i = 0;
    float best_v = -INFINITY;
    for (size_t i = 0; i < n; i++) {
        float y = cap > 0.0f ? cap * tanhf(x[i] / cap) : x[i];
        if (y > best_v) {
            best_v = y;
            best_i = (uint32_t)i;
        }
    }
    return best_i;
}

/* lower.rs:4079-4162: inv = rsqrt(ss/n + eps); val = (x*inv)*w; (+res); (scale*val) */
void ko_rmsnorm(const float *x, const float *w, const float *res, float eps, float scale,
                int has_scale, size_t n, float *out)
{
    float ss = 0.0f;
    for (size_t i = 0; i < n; i++) ss += x[i] * x[i];
    float inv = 1.0f / sqrtf(ss / (float)n + eps);
    for (size_t i = 0; i < n; i++) {
        float val = x[i] * inv * w[i];
        if (res) val = val + res[i];
        if (has_scale) val = scale * val;
        out[i] = val;
    }
}

/* lower.rs:3926-4077: out_x = res + (y*inv)*w_post; out_x2 = (out_x*inv2)*w_ffn */
void ko_rmsnorm_add_then_rmsnorm(const float *y, const float *w_post, const float *res,
                                 const float *w_ffn, float eps, size_t n, float *out_x,
                                 float *out_x2)
{
    float ss = 0.0f;
    for (size_t i = 0; i < n; i++) ss += y[i] * y[i];
    float inv = 1.0f / sqrtf(ss / (float)n + eps);
    float ss2 = 0.0f;
    float *tmp = (float *)malloc(sizeof(float) * n);
    for (size_t i = 0; i < n; i++) {
        tmp[i] = res[i] + y[i] * inv * w_post[i];
        ss2 += tmp[i] * tmp[i];
    }
    float inv2 = 1.0f / sqrtf(ss2 / (float)n + eps);
    for (size_t i = 0; i < n; i++) {
        out_x[i] = tmp[i];
        out_x2[i] = tmp[i] * inv2 * w_ffn[i];
    }
    free(tmp);
}

/* gemma_prim.rs:33-56: per pos, hd floats = cos[0..half) || sin[0..half) */
void ko_rope_table(int max_seq, int hd, float theta, int rope_angles, float *out)
{
    int half = hd / 2;
    if (rope_angles > half) rope_angles = half;
    for (int pos = 0; pos < max_seq; pos++) {
        float *row = out + (size_t)pos * hd;
        for (int i = 0; i < half; i++) {
            if (i < rope_angles) {
                float freq = (float)(1.0 / pow((double)theta, (double)(2 * i) / (double)hd));
                float ang = (float)pos * freq;
                row[i] = cosf(ang);
                row[half + i] = sinf(ang);
            } else {
                row[i] = 1.0f;
                row[half + i] = 0.0f;
            }
        }
    }
}

static float head_rms_inv(const float *x, int hd, float eps)
{
    float ss = 0.0f;
    for (int i = 0; i < hd; i++) ss += x[i] * x[i];
    return 1.0f / sqrtf(ss / (float)hd + eps);
}

/* lower.rs:4356-4435: pairs (i, i+hd/2): out[i] = u*cos - v*sin, out[i+half] = u*sin + v*cos */
static void head_rms_rope(const float *x, const float *w, const float *rope, int hd, float eps,
                          float *out)
{
    int half = hd / 2;
    float inv = head_rms_inv(x, hd, eps);
    for (int i = 0; i < half; i++) {
        float u = x[i] * inv * w[i], vv = x[half + i] * inv * w[half + i];
        float c = rope[i], s = rope[half + i];
        out[i] = u * c - vv * s;
        out[half + i] = u * s + vv * c;
    }
}

/* lower.rs:4619-4702, n_tok<=1: Q rms*w + RoPE; K rms*w + RoPE -> Q4_0;
 * V rms without weight -> Q4_0.  Packs go through a half round trip
 * (Q40PackFromThread -> ksearch_pack_q40_th, render.rs:1040-1059). */
void ko_rmsnorm_per_head_qkv_q40(const float *q, const float *qw, const float *rope_row,
                                 const float *k, const float *kw, const float *v, int n_q,
                                 int n_kv, int hd, float eps, float *q_out, uint8_t *k_out,
                                 uint8_t *v_out)
{
    float *tmp = (float *)malloc(sizeof(float) * (size_t)hd);
    for (int h = 0; h < n_q; h++)
        head_rms_rope(q + (size_t)h * hd, qw, rope_row, hd, eps, q_out + (size_t)h * hd);
    for (int h = 0; h < n_kv; h++) {
        head_rms_rope(k + (size_t)h * hd, kw, rope_row, hd, eps, tmp);
        ko_pack_q40(tmp, (size_t)hd, k_out + (size_t)h * (hd / 32) * 18, 1);
        float inv = head_rms_inv(v + (size_t)h * hd, hd, eps);
        for (int i = 0; i < hd; i++) tmp[i] = v[(size_t)h * hd + i] * inv;
        ko_pack_q40(tmp, (size_t)hd, v_out + (size_t)h * (hd / 32) * 18, 1);
    }
    free(tmp);
}

/* lower.rs:2926-2955 */
float ko_gelu_mul(float g, float u)
{
    float ax = fminf(20.0f, fmaxf(-20.0f, g));
    float t = 0.79788456f * (ax + 0.044715f * ((ax * ax) * ax));
    float gelu = (0.5f * ax) * (1.0f + tanhf(t));
    return gelu * u;
}

/* lower.rs:3899-3921: out[i] = scale * deq(src[id*n + i]) */
int ko_copy_scale_indexed(int dtype, const uint8_t *src, uint32_t id, size_t n, float scale,
                          float *out)
{
    size_t rb = ko_row_bytes(dtype, n);
    if (!rb) return -1;
    ko_dequant(dtype, src + (size_t)id * rb, n, out);
    for (size_t i = 0; i < n; i++) out[i] = scale * out[i];
    return 0;
}


/* ------------------------------------------------------------------ row adoption
 * Two correct f32 implementations of a layer can round a K/V value that sits on a Q4_0 code
 * boundary to neighbouring codes.  To compare a whole decode step against another
 * implementation, the loop can take that implementation's freshly appended Q4_0 rows layer by
 * layer: it first packs its own row, measures how far the other row is from it (differing
 * bytes, and the largest difference of dequantized values in units of the own block scale),
 * then continues with the other row in its cache.  Both sides then attend over identical
 * caches, and everything downstream is comparable to f32 noise. */
static void adopt_row(uint8_t *own, const uint8_t *other, size_t nbytes, int *diff_bytes,
                      float *max_step)
{
    int nd = 0;
    float worst = 0.0f;
    for (size_t b = 0; b < nbytes / 18; b++) {
        const uint8_t *o = own + b * 18, *t = other + b * 18;
        if (!memcmp(o, t, 18)) continue;
        float vo[32], vt[32];
        ko_dequant(KO_Q40, o, 32, vo);
        ko_dequant(KO_Q40, t, 32, vt);
        float d = fabsf(ko_f16_to_f32((uint16_t)(o[0] | (o[1] << 8))));
        for (int i = 0; i < 18; i++) nd += o[i] != t[i];
        for (int i = 0; i < 32; i++) {
            float e = fabsf(vo[i] - vt[i]);
            float st = d > 0.0f ? e / d : (e > 0.0f ? INFINITY : 0.0f);
            if (st > worst) worst = st;
        }
    }
    if (diff_bytes) *diff_bytes = nd;
    if (max_step) *max_step = worst;
    memcpy(own, other, nbytes);
}

static void sync_layer(const ko_row_sync *s, int layer, uint8_t *k_own, uint8_t *v_own, size_t krow)
{
    if (!s->rows) return;
    const uint8_t *r = s->rows + (size_t)layer * 2 * s->row_stride;
    adopt_row(k_own, r, krow, s->diff_bytes ? s->diff_bytes + 2 * layer : NULL,
              s->max_step ? s->max_step + 2 * layer : NULL);
    adopt_row(v_own, r + s->row_stride, krow, s->diff_bytes ? s->diff_bytes + 2 * layer + 1 : NULL,
              s->max_step ? s->max_step + 2 * layer + 1 : NULL);
}

/* ------------------------------------------------------------------ decode loop */

struct ko_gemma {
    ko_gemma_cfg c;
    ko_gemma_layer *layers;
    const uint8_t *embd;
    const float *output_norm;
    uint8_t **kv_k, **kv_v;
    float *rope, *x, *x2, *tq, *tk, *tv, *to, *ff, *logits;
    int pos;
    ko_row_sync sync;
};

ko_gemma *ko_gemma_create(const ko_gemma_cfg *cfg, const ko_gemma_layer *layers,
                          const uint8_t *token_embd_q6k, const float *output_norm)
{
    ko_gemma *m = (ko_gemma *)calloc(1, sizeof(*m));
    m->c = *cfg;
    m->layers = (ko_gemma_layer *)malloc(sizeof(ko_gemma_layer) * (size_t)cfg->n_layers);
    memcpy(m->layers, layers, sizeof(ko_gemma_layer) * (size_t)cfg->n_layers);
    m->embd = token_embd_q6k;
    m->output_norm = output_norm;
    size_t kvb = (size_t)cfg->max_seq * cfg->n_kv * (cfg->hd / 32) * 18; /* kv_pool.rs:113-116 */
    m->kv_k = (uint8_t **)malloc(sizeof(uint8_t *) * (size_t)cfg->n_layers);
    m->kv_v = (uint8_t **)malloc(sizeof(uint8_t *) * (size_t)cfg->n_layers);
    for (int l = 0; l < cfg->n_layers; l++) {
        m->kv_k[l] = (uint8_t *)calloc(kvb, 1);
        m->kv_v[l] = (uint8_t *)calloc(kvb, 1);
    }
    m->rope = (float *)malloc(sizeof(float) * (size_t)cfg->max_seq * cfg->hd);
    ko_rope_table(cfg->max_seq, cfg->hd, cfg->rope_theta, cfg->hd / 2, m->rope);
    size_t big = (size_t)(cfg->ffn > cfg->hidden ? cfg->ffn : cfg->hidden);
    m->x = (float *)calloc((size_t)cfg->hidden, 4);
    m->x2 = (float *)calloc((size_t)cfg->hidden, 4);
    m->tq = (float *)calloc((size_t)cfg->n_q * cfg->hd, 4);
    m->tk = (float *)calloc((size_t)cfg->n_kv * cfg->hd, 4);
    m->tv = (float *)calloc((size_t)cfg->n_kv * cfg->hd, 4);
    m->to = (float *)calloc((size_t)cfg->n_q * cfg->hd, 4);
    m->ff = (float *)calloc(big, 4);
    m->logits = (float *)calloc((size_t)cfg->vocab, 4);
    return m;
}

void ko_gemma_destroy(ko_gemma *m)
{
    if (!m) return;
    for (int l = 0; l < m->c.n_layers; l++) { free(m->kv_k[l]); free(m->kv_v[l]); }
    free(m->kv_k); free(m->kv_v); free(m->layers); free(m->rope);
    free(m->x); free(m->x2); free(m->tq); free(m->tk); free(m->tv); free(m->to);
    free(m->ff); free(m->logits); free(m);
}

void ko_gemma_reset(ko_gemma *m) { m->pos = 0; }
void ko_gemma_set_row_sync(ko_gemma *m, const ko_row_sync *s)
{
    if (s) m->sync = *s; else memset(&m->sync, 0, sizeof(m->sync));
}
int ko_gemma_pos(const ko_gemma *m) { return m->pos; }
const uint8_t *ko_gemma_kv(const ko_gemma *m, int layer, int which)
{
    return which ? m->kv_v[layer] : m->kv_k[layer];
}
const float *ko_gemma_hidden(const ko_gemma *m) { return m->x; }

/* gemma_prim.rs:881-1275 with owns_kv = true for every layer, no SWA, no PLE.
 * SDPA follows sdpa_hybrid_kv (ksearch_kernels/src/lib.rs:1157-1178):
 * online below 128 rows, 16-way split-KV from 128 on. */
uint32_t ko_gemma_forward(ko_gemma *m, uint32_t token, int want_logits, float *logits_out,
                          int threads)
{
    const ko_gemma_cfg *c = &m->c;
    int h = c->hidden, hd = c->hd;
    size_t krow = (size_t)c->n_kv * (hd / 32) * 18;
    /* embed: x = sqrt(hidden) * deq(E[token]) (gemma_prim.rs:681-710) */
    ko_copy_scale_indexed(KO_Q6K, m->embd, token, (size_t)h, sqrtf((float)h), m->x);
    for (int l = 0; l < c->n_layers; l++) {
        const ko_gemma_layer *L = &m->layers[l];
        ko_rmsnorm(m->x, L->attn_norm, NULL, c->eps, 0, 0, (size_t)h, m->x2);
        ko_matvec(KO_Q4K, L->wq, (size_t)c->n_q * hd, (size_t)h, m->x2, m->tq, threads);
        ko_matvec(KO_Q4K, L->wk, (size_t)c->n_kv * hd, (size_t)h, m->x2, m->tk, threads);
        ko_matvec(KO_Q4K, L->wv, (size_t)c->n_kv * hd, (size_t)h, m->x2, m->tv, threads);
        ko_rmsnorm_per_head_qkv_q40(m->tq, L->q_norm, m->rope + (size_t)m->pos * hd, m->tk,
                                    L->k_norm, m->tv, c->n_q, c->n_kv, hd, c->eps, m->tq,
                                    m->kv_k[l] + (size_t)m->pos * krow,
                                    m->kv_v[l] + (size_t)m->pos * krow);
        sync_layer(&m->sync, l, m->kv_k[l] + (size_t)m->pos * krow,
                   m->kv_v[l] + (size_t)m->pos * krow, krow);
        int tlen = m->pos + 1;
        if (tlen >= 128)
            ko_sdpa_mwg(m->tq, m->kv_k[l], m->kv_v[l], c->n_q, c->n_kv, hd, tlen, 0,
                        c->attn_scale, 16, m->to);
        else
            ko_sdpa_online(m->tq, m->kv_k[l], m->kv_v[l], c->n_q, c->n_kv, hd, tlen, 0,
                           c->attn_scale, m->to);
        ko_matvec(KO_Q4K, L->wo, (size_t)h, (size_t)c->n_q * hd, m->to, m->x2, threads);
        ko_rmsnorm_add_then_rmsnorm(m->x2, L->post_attn_norm, m->x, L->ffn_norm, c->eps,
                                    (size_t)h, m->x, m->x2);
        /* fused gate||up + GELU on the f32 accumulators (lower.rs:2673-2968) */
        {
            float *g = m->ff, *u = (float *)malloc(sizeof(float) * (size_t)c->ffn);
            ko_matvec(KO_Q4K, L->wgate, (size_t)c->ffn, (size_t)h, m->x2, g, threads);
            ko_matvec(KO_Q4K, L->wup, (size_t)c->ffn, (size_t)h, m->x2, u, threads);
            for (int i = 0; i < c->ffn; i++) g[i] = ko_gelu_mul(g[i], u[i]);
            free(u);
        }
        ko_matvec(KO_Q4K, L->wdown, (size_t)h, (size_t)c->ffn, m->ff, m->x2, threads);
        ko_rmsnorm(m->x2, L->post_ffw_norm, m->x, c->eps, 0, 0, (size_t)h, m->x);
    }
    m->pos += 1;
    if (!want_logits) return 0;
    ko_rmsnorm(m->x, m->output_norm, NULL, c->eps, 0, 0, (size_t)h, m->x2);
    ko_matvec(KO_Q6K, m->embd, (size_t)c->vocab, (size_t)h, m->x2, m->logits, threads);
    if (logits_out) memcpy(logits_out, m->logits, sizeof(float) * (size_t)c->vocab);
    return ko_softcap_argmax(m->logits, (size_t)c->vocab, c->softcap);
}

/* ------------------------------------------------------------------ Gemma-4 extras */

void ko_rmsnorm_per_head(const float *x, const float *w, const float *rope_row, int n_heads, int hd,
                         float eps, float *out)
{
    for (int h = 0; h < n_heads; h++) {
        const float *xh = x + (size_t)h * hd;
        float *oh = out + (size_t)h * hd;
        if (rope_row) {
            float *tmp = (float *)malloc(sizeof(float) * (size_t)hd);
            head_rms_rope(xh, w, rope_row, hd, eps, tmp);
            memcpy(oh, tmp, sizeof(float) * (size_t)hd);
            free(tmp);
        } else {
            float inv = head_rms_inv(xh, hd, eps);
            for (int i = 0; i < hd; i++) oh[i] = xh[i] * inv * w[i];
        }
    }
}

void ko_add_scale(const float *a, const float *b, float scale, size_t n, float *out)
{
    for (size_t i = 0; i < n; i++) out[i] = scale * (a[i] + b[i]);
}

int ko_matvec_gelu_mul(int dtype, const uint8_t *w, size_t rows, size_t cols, const float *x,
                       const float *ctx, float *y, int threads)
{
    int rc = ko_matvec(dtype, w, rows, cols, x, y, threads);
    if (rc) return rc;
    for (size_t r = 0; r < rows; r++) y[r] = ko_gelu_mul(y[r], ctx[r]);
    return 0;
}

struct ko_gemma4 {
    ko_gemma4_cfg c;
    ko_gemma4_layer *layers;
    ko_gemma4_globals g;
    uint8_t **kv_k, **kv_v;      /* per owning layer */
    float *rope_swa, *rope_full;
    float *x, *x2, *tq, *tk, *tv, *to, *ff, *ff2, *logits;
    float *ple_tok, *ple_tmp, *ple_ctx, *ple_u;
    int pos;
    ko_row_sync sync;
};

static int g4_hd(const ko_gemma4_cfg *c, const ko_gemma4_layer *L) { return L->is_swa ? c->hd_swa : c->hd_full; }
static int g4_owns(const ko_gemma4_cfg *c, int l)
{
    int owners = c->n_layers - c->shared_kv_layers;
    return l < (owners > 0 ? owners : 0);
}

int ko_gemma4_kv_source(const ko_gemma4 *m, int layer)
{
    if (g4_owns(&m->c, layer)) return layer;
    for (int i = layer - 1; i >= 0; i--)
        if (g4_owns(&m->c, i) && m->layers[i].is_swa == m->layers[layer].is_swa) return i;
    return 0;
}

ko_gemma4 *ko_gemma4_create(const ko_gemma4_cfg *cfg, const ko_gemma4_layer *layers,
                            const ko_gemma4_globals *g)
{
    ko_gemma4 *m = (ko_gemma4 *)calloc(1, sizeof(*m));
    m->c = *cfg;
    m->g = *g;
    m->layers = (ko_gemma4_layer *)malloc(sizeof(ko_gemma4_layer) * (size_t)cfg->n_layers);
    memcpy(m->layers, layers, sizeof(ko_gemma4_layer) * (size_t)cfg->n_layers);
    m->kv_k = (uint8_t **)calloc((size_t)cfg->n_layers, sizeof(uint8_t *));
    m->kv_v = (uint8_t **)calloc((size_t)cfg->n_layers, sizeof(uint8_t *));
    int max_hd = cfg->hd_swa > cfg->hd_full ? cfg->hd_swa : cfg->hd_full, max_ff = 0;
    for (int l = 0; l < cfg->n_layers; l++) {
        if (layers[l].ffn > max_ff) max_ff = layers[l].ffn;
        if (!g4_owns(cfg, l)) continue;
        int hd = g4_hd(cfg, &layers[l]);
        size_t kvb = (size_t)cfg->max_seq * cfg->n_kv * (hd / 32) * 18; /* gemma_prim.rs:199-207 */
        m->kv_k[l] = (uint8_t *)calloc(kvb, 1);
        m->kv_v[l] = (uint8_t *)calloc(kvb, 1);
    }
    /* gemma_prim.rs:217-228: the sliding-window table rotates every pair, the full-attention table the
     * first hd*partial_rotary/2 of them */
    m->rope_swa = (float *)malloc(sizeof(float) * (size_t)cfg->max_seq * cfg->hd_swa);
    ko_rope_table(cfg->max_seq, cfg->hd_swa, cfg->rope_theta_swa, cfg->hd_swa / 2, m->rope_swa);
    m->rope_full = (float *)malloc(sizeof(float) * (size_t)cfg->max_seq * cfg->hd_full);
    ko_rope_table(cfg->max_seq, cfg->hd_full, cfg->rope_theta_full,
                  (int)((float)cfg->hd_full * cfg->partial_rotary) / 2, m->rope_full);
    size_t h = (size_t)cfg->hidden, pt = (size_t)cfg->n_layers * cfg->ple_dim;
    m->x = (float *)calloc(h, 4);
    m->x2 = (float *)calloc(h, 4);
    m->tq = (float *)calloc((size_t)cfg->n_q * max_hd, 4);
    m->tk = (float *)calloc((size_t)cfg->n_kv * max_hd, 4);
    m->tv = (float *)calloc((size_t)cfg->n_kv * max_hd, 4);
    m->to = (float *)calloc((size_t)cfg->n_q * max_hd, 4);
    m->ff = (float *)calloc((size_t)max_ff, 4);
    m->ff2 = (float *)calloc((size_t)max_ff, 4);
    m->logits = (float *)calloc((size_t)cfg->vocab, 4);
    m->ple_tok = (float *)calloc(pt + 1, 4);
    m->ple_tmp = (float *)calloc(pt + 1, 4);
    m->ple_ctx = (float *)calloc(pt + 1, 4);
    m->ple_u = (float *)calloc((size_t)cfg->ple_dim + 1, 4);
    return m;
}

void ko_gemma4_destroy(ko_gemma4 *m)
{
    if (!m) return;
    for (int l = 0; l < m->c.n_layers; l++) { free(m->kv_k[l]); free(m->kv_v[l]); }
    free(m->kv_k); free(m->kv_v); free(m->layers); free(m->rope_swa); free(m->rope_full);
    free(m->x); free(m->x2); free(m->tq); free(m->tk); free(m->tv); free(m->to); free(m->ff); free(m->ff2);
    free(m->logits); free(m->ple_tok); free(m->ple_tmp); free(m->ple_ctx); free(m->ple_u); free(m);
}

void ko_gemma4_reset(ko_gemma4 *m) { m->pos = 0; }
void ko_gemma4_set_row_sync(ko_gemma4 *m, const ko_row_sync *s)
{
    if (s) m->sync = *s; else memset(&m->sync, 0, sizeof(m->sync));
}
int ko_gemma4_pos(const ko_gemma4 *m) { return m->pos; }
const uint8_t *ko_gemma4_kv(const ko_gemma4 *m, int layer, int which)
{
    return which ? m->kv_v[layer] : m->kv_k[layer];
}
const float *ko_gemma4_hidden(const ko_gemma4 *m) { return m->x; }

uint32_t ko_gemma4_forward(ko_gemma4 *m, uint32_t token, int want_logits, float *logits_out, int threads)
{
    const ko_gemma4_cfg *c = &m->c;
    const int h = c->hidden, pd = c->ple_dim;
    const size_t pt = (size_t)c->n_layers * pd;
    /* embed (gemma_prim.rs:681-710) */
    ko_copy_scale_indexed(m->g.dt_embd, m->g.token_embd, token, (size_t)h, sqrtf((float)h), m->x);
    if (pd > 0) {
        /* ple_from_idx (:712-728): row of the per-layer table times sqrt(ple_dim);
         * ple_prepass (:845-878): model projection, per-layer norm, (ctx + tok)/sqrt(2) */
        ko_copy_scale_indexed(m->g.dt_ple, m->g.ple_embd, token, pt, sqrtf((float)pd), m->ple_tok);
        ko_matvec(m->g.dt_ple_proj, m->g.ple_model_proj, pt, (size_t)h, m->x, m->ple_tmp, threads);
        ko_rmsnorm_per_head(m->ple_tmp, m->g.ple_proj_norm, NULL, c->n_layers, pd, c->eps, m->ple_ctx);
        ko_add_scale(m->ple_ctx, m->ple_tok, 0.70710678118654752440f, pt, m->ple_ctx);
    }
    for (int l = 0; l < c->n_layers; l++) {
        const ko_gemma4_layer *L = &m->layers[l];
        const int hd = g4_hd(c, L), owns = g4_owns(c, l), src = ko_gemma4_kv_source(m, l);
        const float *rope = (L->is_swa ? m->rope_swa : m->rope_full) + (size_t)m->pos * hd;
        const size_t krow = (size_t)c->n_kv * (hd / 32) * 18;
        const size_t qd = (size_t)c->n_q * hd, kvd = (size_t)c->n_kv * hd;
        ko_rmsnorm(m->x, L->attn_norm, NULL, c->eps, 0, 0, (size_t)h, m->x2);
        ko_matvec(L->dt_q, L->wq, qd, (size_t)h, m->x2, m->tq, threads);
        if (owns) {
            ko_matvec(L->dt_k, L->wk, kvd, (size_t)h, m->x2, m->tk, threads);
            ko_matvec(L->dt_v, L->wv, kvd, (size_t)h, m->x2, m->tv, threads);
            ko_rmsnorm_per_head_qkv_q40(m->tq, L->q_norm, rope, m->tk, L->k_norm, m->tv, c->n_q, c->n_kv,
                                        hd, c->eps, m->tq, m->kv_k[src] + (size_t)m->pos * krow,
                                        m->kv_v[src] + (size_t)m->pos * krow);
            sync_layer(&m->sync, l, m->kv_k[src] + (size_t)m->pos * krow,
                       m->kv_v[src] + (size_t)m->pos * krow, krow);
        } else {
            ko_rmsnorm_per_head(m->tq, L->q_norm, rope, c->n_q, hd, c->eps, m->tq);   /* :989-1008 */
        }
        /* :1010-1017 */
        int kv_len = m->pos + 1, start = 0;
        if (L->is_swa) start = kv_len > c->sliding_window ? kv_len - c->sliding_window : 0;
        int tlen = kv_len - start;
        if (tlen >= 128)
            ko_sdpa_mwg(m->tq, m->kv_k[src], m->kv_v[src], c->n_q, c->n_kv, hd, tlen, start,
                        c->attn_scale, 16, m->to);
        else
            ko_sdpa_online(m->tq, m->kv_k[src], m->kv_v[src], c->n_q, c->n_kv, hd, tlen, start,
                           c->attn_scale, m->to);
        ko_matvec(L->dt_o, L->wo, (size_t)h, qd, m->to, m->x2, threads);
        ko_rmsnorm_add_then_rmsnorm(m->x2, L->post_attn_norm, m->x, L->ffn_norm, c->eps, (size_t)h,
                                    m->x, m->x2);
        ko_matvec(L->dt_gate, L->wgate, (size_t)L->ffn, (size_t)h, m->x2, m->ff, threads);
        ko_matvec(L->dt_up, L->wup, (size_t)L->ffn, (size_t)h, m->x2, m->ff2, threads);
        for (int i = 0; i < L->ffn; i++) m->ff[i] = ko_gelu_mul(m->ff[i], m->ff2[i]);
        ko_matvec(L->dt_down, L->wdown, (size_t)h, (size_t)L->ffn, m->ff, m->x2, threads);
        ko_rmsnorm(m->x2, L->post_ffw_norm, m->x, c->eps, 0, 0, (size_t)h, m->x);
        if (pd > 0) {
            /* :1166-1200: gate GEMV with gelu*ctx, projection, rmsnorm_add_scale */
            ko_matvec_gelu_mul(L->dt_inp_gate, L->inp_gate, (size_t)pd, (size_t)h, m->x,
                               m->ple_ctx + (size_t)l * pd, m->ple_u, threads);
            ko_matvec(L->dt_proj, L->proj, (size_t)h, (size_t)pd, m->ple_u, m->x2, threads);
            ko_rmsnorm(m->x2, L->post_norm, m->x, c->eps, L->layer_scale, 1, (size_t)h, m->x);
        }
    }
    m->pos += 1;
    if (!want_logits) return 0;
    ko_rmsnorm(m->x, m->g.output_norm, NULL, c->eps, 0, 0, (size_t)h, m->x2);
    ko_matvec(m->g.dt_embd, m->g.token_embd, (size_t)c->vocab, (size_t)h, m->x2, m->logits, threads);
    if (logits_out) memcpy(logits_out, m->logits, sizeof(float) * (size_t)c->vocab);
    return ko_softcap_argmax(m->logits, (size_t)c->vocab, c->softcap);
}

/* ------------------------------------------------------------------ sampler */

/* sample.rs:79-85 */
static uint32_t splitmix32(uint32_t *state)
{
    *state += 0x9E3779B9u;
    uint32_t z = *state;
    z = (z ^ (z >> 16)) * 0x7feb352du;
    z = (z ^ (z >> 15)) * 0x846ca68bu;
    return z ^ (z >> 16);
}

/* sample.rs:9-77 */
uint32_t ko_sample_softcap_min_p(const float *logits, size_t n, float cap, float temperature,
                                 float min_p, uint32_t seed)
{
    uint32_t best_i = 0;
    float best_v = -INFINITY;
    float *xs = (float *)malloc(sizeof(float) * n);
    for (size_t i = 0; i < n; i++) {
        float x = logits[i];
        float y = cap > 0.0f ? cap * tanhf(x / cap) : x;
        xs[i] = y;
        if (y > best_v) { best_v = y; best_i = (uint32_t)i; }
    }
    if (temperature < 1e-6f) { free(xs); return best_i; }
    float sum = 0.0f;
    for (size_t i = 0; i < n; i++) {
        xs[i] = expf((xs[i] - best_v) / temperature);
        sum += xs[i];
    }
    float inv = 1.0f / fmaxf(sum, 1e-30f);
    float p_max = 0.0f;
    for (size_t i = 0; i < n; i++) {
        xs[i] *= inv;
        if (xs[i] > p_max) p_max = xs[i];
    }
    float threshold = p_max * fmaxf(min_p, 0.0f);
    float filtered = 0.0f;
    for (size_t i = 0; i < n; i++) {
        if (xs[i] < threshold) xs[i] = 0.0f;
        else filtered += xs[i];
    }
    uint32_t pick = best_i;
    if (filtered > 1e-9f) {
        uint32_t rng = seed | 1u;
        float r = ((float)splitmix32(&rng) / 4294967296.0f) * filtered;
        float cdf = 0.0f;
        pick = (uint32_t)(n - 1);
        for (size_t i = 0; i < n; i++) {
            cdf += xs[i];
            if (r < cdf) { pick = (uint32_t)i; break; }
        }
    }
    free(xs);
    return pick;
}
