/* Second, independently written CPU restatement of the low-bit KV-cache path.
 * TEST INFRASTRUCTURE ONLY: it cross-checks oracle/bitdecode_oracle.py (numpy) and is
 * never linked into or called by the product library.
 *
 * Follows (paths relative to the reference tree):
 *   quantizer      csrc/bit_decode/src/include/qpack.h:224-296 (4-bit), :115-209 (2-bit)
 *   dequantize     csrc/bit_decode/src/include/dequantize.h:291,372  (code*scale+zero)
 *   attention      csrc/bit_decode/src/flash_fwd_kernel.h:406-534, softmax.h:250-310
 *   GQA mapping    csrc/bit_decode/decode_api.cpp:362-368
 * Differences from the numpy oracle that make it a useful second witness: libm roundf
 * instead of a floor-based formula, a hand-written fp32->fp16/bf16 rounding, scalar loops
 * instead of reshapes, and double-precision accumulation in the attention.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static float round_fp16(float x) {
    /* fp32 -> fp16 (round to nearest even, subnormals kept, overflow to inf) -> fp32 */
    uint32_t u; memcpy(&u, &x, 4);
    uint32_t sign = u & 0x80000000u;
    uint32_t a = u & 0x7fffffffu;
    if (a >= 0x7f800000u) return x;                       /* inf / nan */
    float ax; memcpy(&ax, &a, 4);
    if (ax >= 65520.0f) { uint32_t r = sign | 0x7f800000u; float f; memcpy(&f, &r, 4); return f; }
    float r;
    if (ax < 6.103515625e-05f) {                          /* fp16 subnormal range: ulp 2^-24 */
        r = nearbyintf(ax * 16777216.0f) / 16777216.0f;   /* default mode: ties to even */
    } else {
        int e; frexpf(ax, &e);                            /* ax = m * 2^e, m in [0.5,1) */
        float ulp = ldexpf(1.0f, e - 11);                 /* 11 significant bits */
        r = nearbyintf(ax / ulp) * ulp;
    }
    uint32_t ru; memcpy(&ru, &r, 4); ru |= sign; memcpy(&r, &ru, 4);
    return r;
}

static float round_bf16(float x) {
    uint32_t u; memcpy(&u, &x, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return x;        /* nan */
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    u &= 0xffff0000u;
    float r; memcpy(&r, &u, 4);
    return r;
}

static float round_store(float x, int bf16) { return bf16 ? round_bf16(x) : round_fp16(x); }

/* one group of n values with stride `st`; writes n codes with stride `cst` */
static void quant_group(const float* x, long st, int n, int bits, int bf16,
                        uint8_t* codes, long cst, float* scale, float* zero) {
    const float M = (float)((1 << bits) - 1);
    float mx = x[0], mn = x[0];
    for (int i = 1; i < n; ++i) { float t = x[i * st]; mx = fmaxf(mx, t); mn = fminf(mn, t); }
    /* a zero minimum is -0 if the group holds a -0 (IEEE 754-2019 minimum); libm's fminf may return either */
    if (mn == 0.0f) { for (int i = 0; i < n; ++i) if (x[i * st] == 0.0f && signbit(x[i * st])) mn = -0.0f; }
    volatile float range = mx - mn;
    volatile float scale_inv = (range > 0.0f) ? (M / range) : 0.0f;
    volatile float sc = (scale_inv == 0.0f) ? 0.0f : 1.0f / scale_inv;
    *scale = round_store(sc, bf16);
    *zero = round_store(mn, bf16);
    for (int i = 0; i < n; ++i) {
        volatile float t = x[i * st] - mn;      /* volatile: no fma contraction */
        volatile float u = t * scale_inv;
        float r = fminf(fmaxf(roundf(u), 0.0f), M);
        codes[i * cst] = (uint8_t)r;
    }
}

/* k, v: [b, S, h, d] fp32 holding storage-representable values.
 * kc, vc: uint8 [b,S,h,d]; ks,kz: [b,S/gs,h,d]; vs,vz: [b,S,h,d/gs]. */
void oracle_quantize_kv(const float* k, const float* v, int b, int S, int h, int d,
                        int bits, int gs, int bf16,
                        uint8_t* kc, float* ks, float* kz,
                        uint8_t* vc, float* vs, float* vz) {
    const long tok = (long)h * d;
    for (int bi = 0; bi < b; ++bi)
        for (int g0 = 0; g0 < S / gs; ++g0)
            for (int hi = 0; hi < h; ++hi)
                for (int c = 0; c < d; ++c) {
                    long base = ((long)bi * S + (long)g0 * gs) * tok + (long)hi * d + c;
                    long p = (((long)bi * (S / gs) + g0) * h + hi) * d + c;
                    quant_group(k + base, tok, gs, bits, bf16, kc + base, tok, ks + p, kz + p);
                }
    for (int bi = 0; bi < b; ++bi)
        for (int n = 0; n < S; ++n)
            for (int hi = 0; hi < h; ++hi)
                for (int cg = 0; cg < d / gs; ++cg) {
                    long base = ((long)bi * S + n) * tok + (long)hi * d + (long)cg * gs;
                    long p = (((long)bi * S + n) * h + hi) * (d / gs) + cg;
                    quant_group(v + base, 1, gs, bits, bf16, vc + base, 1, vs + p, vz + p);
                }
}

/* Dequantize-then-attend for one query token.
 * q [b,h,d]; codes [b,S,hk,d]; ks,kz [b,S/gs,hk,d]; vs,vz [b,S,hk,d/gs];
 * kres,vres [b,R,hk,d] (may be NULL when R == 0); seqlens/reslens [b] (may be NULL).
 * out [b,h,d] fp32, lse [b,h] fp32 (natural log; -inf for an empty row). */
void oracle_attend(const float* q, const uint8_t* kc, const float* ks, const float* kz,
                   const uint8_t* vc, const float* vs, const float* vz,
                   const float* kres, const float* vres,
                   const int* seqlens, const int* reslens,
                   int b, int h, int hk, int d, int S, int R, int gs, float softmax_scale,
                   float* out, float* lse) {
    const int g = h / hk;
    const int ncg = d / gs;
    #pragma omp parallel for collapse(2) schedule(dynamic)
    for (int bi = 0; bi < b; ++bi)
        for (int hq = 0; hq < h; ++hq) {
            const int hi = hq / g;
            const int sp = seqlens ? seqlens[bi] : S;
            const int rl = reslens ? reslens[bi] : R;
            const int n = sp + rl;
            const float* qq = q + ((long)bi * h + hq) * d;
            float* oo = out + ((long)bi * h + hq) * d;
            if (n == 0) { for (int c = 0; c < d; ++c) oo[c] = 0.f; lse[(long)bi * h + hq] = -INFINITY; continue; }
            double* s = (double*)malloc(sizeof(double) * n);
            double m = -INFINITY;
            for (int t = 0; t < n; ++t) {
                double acc = 0.0;
                if (t < sp) {
                    const long ci = (((long)bi * S + t) * hk + hi) * d;
                    const long pi = (((long)bi * (S / gs) + t / gs) * hk + hi) * d;
                    for (int c = 0; c < d; ++c) {
                        float kh = (float)kc[ci + c] * ks[pi + c] + kz[pi + c];
                        acc += (double)qq[c] * (double)kh;
                    }
                } else {
                    const long ri = (((long)bi * R + (t - sp)) * hk + hi) * d;
                    for (int c = 0; c < d; ++c) acc += (double)qq[c] * (double)kres[ri + c];
                }
                s[t] = acc * (double)softmax_scale;
                if (s[t] > m) m = s[t];
            }
            double l = 0.0;
            double* o = (double*)calloc(d, sizeof(double));
            for (int t = 0; t < n; ++t) {
                double p = exp(s[t] - m);
                l += p;
                if (t < sp) {
                    const long ci = (((long)bi * S + t) * hk + hi) * d;
                    const long pi = (((long)bi * S + t) * hk + hi) * ncg;
                    for (int c = 0; c < d; ++c) {
                        float vh = (float)vc[ci + c] * vs[pi + c / gs] + vz[pi + c / gs];
                        o[c] += p * (double)vh;
                    }
                } else {
                    const long ri = (((long)bi * R + (t - sp)) * hk + hi) * d;
                    for (int c = 0; c < d; ++c) o[c] += p * (double)vres[ri + c];
                }
            }
            for (int c = 0; c < d; ++c) oo[c] = (float)(o[c] / l);
            lse[(long)bi * h + hq] = (float)(m + log(l));
            free(s); free(o);
        }
}

float oracle_round_fp16(float x) { return round_fp16(x); }
float oracle_round_bf16(float x) { return round_bf16(x); }
