/*
 * brute.c — brute-force C restatement of the attention hot path, used ONLY to pin the
 * PyTorch oracle (oracle/xlite_oracle.py). Test infrastructure: never linked into or
 * called from the shipped library.
 *
 * Everything is written as scalar loops over raw 16-bit storage with fp64 accumulation
 * (attention, MLA) or with explicit rounding steps (rope), so that a wrong index, a
 * dropped term or a transposed operand in the vectorised oracle shows up as a mismatch.
 *
 *   brute_attention      xlite/tests/kernels/attention.py:109-117,139-184 and the paged
 *                        addressing of xlite/csrc/kernels/attention.h:147,156
 *   brute_mla            xlite/tests/kernels/mla.py:163-202
 *   brute_rope_and_cache xlite/csrc/kernels/rope_and_cache.h:93-129,486-501,563-600
 *   brute_rope_complex   xlite/csrc/kernels/rope_complex_and_cache.h:165-221
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static float bf16_to_f32(uint16_t h)
{
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static uint16_t f32_to_bf16(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        return (uint16_t)((u >> 16) | 0x40u); /* quiet NaN */
    }
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb; /* round to nearest even */
    return (uint16_t)(u >> 16);
}

static float f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t u;
    if (exp == 0) {
        if (man == 0) {
            u = sign;
        } else { /* subnormal */
            int e = -1;
            do {
                e++;
                man <<= 1;
            } while ((man & 0x400u) == 0);
            man &= 0x3ffu;
            u = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        u = sign | 0x7f800000u | (man << 13);
    } else {
        u = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static uint16_t f32_to_f16(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) {
        return (uint16_t)(sign | 0x7e00u);
    }
    if (a >= 0x47800000u) { /* >= 65536: overflow to inf (values that round up to inf too) */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (a < 0x38800000u) { /* subnormal or zero in fp16 */
        if (a < 0x33000000u) {
            return (uint16_t)sign; /* below half of the smallest subnormal */
        }
        int e = (int)(a >> 23);
        uint32_t man = (a & 0x7fffffu) | 0x800000u;
        int shift = 126 - e; /* 14..24 */
        uint32_t q = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1u))) {
            q++;
        }
        return (uint16_t)(sign | q);
    }
    uint32_t e = (a >> 23) - 112;
    uint32_t man = a & 0x7fffffu;
    uint32_t q = (e << 10) | (man >> 13);
    uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) {
        q++; /* may carry into the exponent, which is the right result (incl. inf) */
    }
    return (uint16_t)(sign | q);
}

static float ld(const uint16_t *p, int is_bf16) { return is_bf16 ? bf16_to_f32(*p) : f16_to_f32(*p); }
static uint16_t st(float f, int is_bf16) { return is_bf16 ? f32_to_bf16(f) : f32_to_f16(f); }

/* exported for direct conversion tests */
uint16_t brute_f32_to_f16(float f) { return f32_to_f16(f); }
float brute_f16_to_f32(uint16_t h) { return f16_to_f32(h); }
uint16_t brute_f32_to_bf16(float f) { return f32_to_bf16(f); }

/* out[T, nH*d] fp64. Row r of sequence i sees cache positions 0..clen+r. */
void brute_attention(const uint16_t *qkv, const uint16_t *kc, const uint16_t *vc, double *out,
                     const int32_t *qsl, const int32_t *lens, const int32_t *clens,
                     const int32_t *tables, int nH, int nKV, int d, int bs, int batch, int maxblk,
                     int is_bf16)
{
    int g = nH / nKV;
    int rowlen = (nH + 2 * nKV) * d;
    for (int i = 0; i < batch; i++) {
        for (int r = 0; r < lens[i]; r++) {
            int tok = qsl[i] + r;
            int n = clens[i] + r + 1;
            double *s = (double *)malloc(sizeof(double) * (size_t)n);
            for (int h = 0; h < nH; h++) {
                int kvh = h / g;
                const uint16_t *q = qkv + (size_t)tok * rowlen + (size_t)h * d;
                double mx = -INFINITY;
                for (int j = 0; j < n; j++) {
                    size_t blk = (size_t)tables[i * maxblk + j / bs];
                    const uint16_t *k = kc + ((blk * bs + (size_t)(j % bs)) * nKV + kvh) * d;
                    double acc = 0.0;
                    for (int e = 0; e < d; e++) {
                        acc += (double)ld(q + e, is_bf16) * (double)ld(k + e, is_bf16);
                    }
                    s[j] = acc;
                    if (acc > mx) {
                        mx = acc;
                    }
                }
                double sum = 0.0;
                for (int j = 0; j < n; j++) {
                    s[j] = exp(s[j] - mx);
                    sum += s[j];
                }
                double *o = out + (size_t)tok * nH * d + (size_t)h * d;
                for (int e = 0; e < d; e++) {
                    o[e] = 0.0;
                }
                for (int j = 0; j < n; j++) {
                    size_t blk = (size_t)tables[i * maxblk + j / bs];
                    const uint16_t *v = vc + ((blk * bs + (size_t)(j % bs)) * nKV + kvh) * d;
                    double p = s[j] / sum;
                    for (int e = 0; e < d; e++) {
                        o[e] += p * (double)ld(v + e, is_bf16);
                    }
                }
            }
            free(s);
        }
    }
}

/* Absorbed MLA attention. out[T, nH, C] fp64. topk: NULL or [T, top_k]. */
void brute_mla(const uint16_t *qa, const uint16_t *qr, const uint16_t *kc, const uint16_t *pc,
               double *out, const int32_t *qsl, const int32_t *lens, const int32_t *clens,
               const int32_t *tables, int nH, int R, int C, int bs, int batch, int maxblk,
               double scale, const int32_t *topk, int top_k)
{
    for (int i = 0; i < batch; i++) {
        for (int r = 0; r < lens[i]; r++) {
            int tok = qsl[i] + r;
            int n = clens[i] + r + 1;
            double *s = (double *)malloc(sizeof(double) * (size_t)n);
            char *keep = (char *)malloc((size_t)n);
            /* the index list only applies to rows whose causal range is longer than top_k
               (xlite/csrc/kernels/mla_v2.h:697-699) */
            if (top_k > 0 && n > top_k) {
                memset(keep, 0, (size_t)n);
                for (int t = 0; t < top_k; t++) {
                    int idx = topk[(size_t)tok * top_k + t];
                    if (idx >= 0 && idx < n) {
                        keep[idx] = 1;
                    }
                }
            } else {
                memset(keep, 1, (size_t)n);
            }
            for (int h = 0; h < nH; h++) {
                const uint16_t *q1 = qa + ((size_t)tok * nH + h) * C;
                const uint16_t *q2 = qr + ((size_t)tok * nH + h) * R;
                double mx = -INFINITY;
                for (int j = 0; j < n; j++) {
                    size_t row = (size_t)tables[i * maxblk + j / bs] * bs + (size_t)(j % bs);
                    double acc = 0.0;
                    for (int e = 0; e < C; e++) {
                        acc += (double)bf16_to_f32(q1[e]) * (double)bf16_to_f32(kc[row * C + e]);
                    }
                    for (int e = 0; e < R; e++) {
                        acc += (double)bf16_to_f32(q2[e]) * (double)bf16_to_f32(pc[row * R + e]);
                    }
                    s[j] = keep[j] ? acc * scale : -INFINITY;
                    if (s[j] > mx) {
                        mx = s[j];
                    }
                }
                double *o = out + ((size_t)tok * nH + h) * C;
                for (int e = 0; e < C; e++) {
                    o[e] = 0.0;
                }
                if (mx == -INFINITY) {
                    continue;
                }
                double sum = 0.0;
                for (int j = 0; j < n; j++) {
                    s[j] = exp(s[j] - mx);
                    sum += s[j];
                }
                for (int j = 0; j < n; j++) {
                    size_t row = (size_t)tables[i * maxblk + j / bs] * bs + (size_t)(j % bs);
                    double p = s[j] / sum;
                    for (int e = 0; e < C; e++) {
                        o[e] += p * (double)bf16_to_f32(kc[row * C + e]);
                    }
                }
            }
            free(keep);
            free(s);
        }
    }
}

/* NeoX rotation of one head, rounding each product to the storage type first. */
static void rotate_head(uint16_t *x, const uint16_t *cs, int rot, int is_bf16)
{
    int half = rot / 2;
    for (int j = 0; j < half; j++) {
        float x1 = ld(x + j, is_bf16), x2 = ld(x + j + half, is_bf16);
        float c = ld(cs + j, is_bf16), s = ld(cs + half + j, is_bf16);
        float a = ld(&(uint16_t){st(x1 * c, is_bf16)}, is_bf16);
        float b = ld(&(uint16_t){st(x2 * s, is_bf16)}, is_bf16);
        float e = ld(&(uint16_t){st(x2 * c, is_bf16)}, is_bf16);
        float f = ld(&(uint16_t){st(x1 * s, is_bf16)}, is_bf16);
        x[j] = st(a - b, is_bf16);
        x[j + half] = st(e + f, is_bf16);
    }
}

/* Single-position (no mrope) rope_and_cache on raw 16-bit storage, in place. */
void brute_rope_and_cache(uint16_t *inout, uint16_t *kcache, uint16_t *vcache,
                          const int64_t *position, const uint16_t *cosin, const int32_t *slots,
                          int T, int nH, int nKV, int d, int rot, int bs, int is_bf16)
{
    int rowlen = (nH + 2 * nKV) * d;
    float scale = 1.0f / sqrtf((float)d);
    if (!is_bf16) {
        scale = f16_to_f32(f32_to_f16(scale));
    }
    for (int t = 0; t < T; t++) {
        uint16_t *row = inout + (size_t)t * rowlen;
        const uint16_t *cs = cosin + (size_t)position[t] * rot;
        uint32_t slot = (uint32_t)slots[t];
        size_t dst = ((size_t)(slot / (uint32_t)bs) * bs + slot % (uint32_t)bs) * nKV * d;
        memcpy(vcache + dst, row + (size_t)(nH + nKV) * d, sizeof(uint16_t) * (size_t)nKV * d);
        for (int h = 0; h < nKV; h++) {
            rotate_head(row + (size_t)(nH + h) * d, cs, rot, is_bf16);
        }
        memcpy(kcache + dst, row + (size_t)nH * d, sizeof(uint16_t) * (size_t)nKV * d);
        for (int h = 0; h < nH; h++) {
            uint16_t *q = row + (size_t)h * d;
            rotate_head(q, cs, rot, is_bf16);
            for (int e = 0; e < d; e++) {
                q[e] = st(ld(q + e, is_bf16) * scale, is_bf16);
            }
        }
    }
}

/* out[T, H, rope] = de-interleaved complex product of the last `rope` elements of each head
 * of in[T, H, step] with freqs[position[t]] (interleaved fp32 cos, sin). */
void brute_rope_complex(const uint16_t *in, const float *freqs, const int64_t *position,
                        uint16_t *out, int T, int H, int step, int rope, int is_bf16)
{
    int half = rope / 2;
    for (int t = 0; t < T; t++) {
        const float *f = freqs + (size_t)position[t] * rope;
        for (int h = 0; h < H; h++) {
            const uint16_t *x = in + ((size_t)t * H + h) * step + (step - rope);
            uint16_t *o = out + ((size_t)t * H + h) * rope;
            for (int j = 0; j < half; j++) {
                float xe = ld(x + 2 * j, is_bf16), xo = ld(x + 2 * j + 1, is_bf16);
                float c = f[2 * j], s = f[2 * j + 1];
                volatile float ec = xe * c, os = xo * s, es = xe * s, oc = xo * c;
                o[j] = st(ec - os, is_bf16);
                o[j + half] = st(es + oc, is_bf16);
            }
        }
    }
}
