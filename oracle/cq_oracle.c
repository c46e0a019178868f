/* C restatement of the CalibQuant decode-attention step and of the prefill
 * quantise-and-pack (fp32, OpenMP over independent (batch, head) units).
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP kernels and the timed
 * "CPU port" of the benchmark.  The shipped library never links it.
 * tests/test_oracle_c.py pins it against the numpy oracle (cq_oracle.py),
 * which in turn is pinned against library routines and closed forms.
 *
 * Reference lines followed (paths relative to the reference checkout):
 *   cqo_decode_attention   patch_internvl.py:344-436 (decode branch): residual
 *                          logits :365-366, post-scaled image logits :369-373
 *                          (with calibquant.py:78-102 unpacking), calibration
 *                          :376-385, order [sys | image | text] :388, additive
 *                          mask :404-410, softmax :413, packed-V sum and value
 *                          post-scaling :418-425, residual outputs :428-434.
 *   cqo_quantize_pack      calibquant.py:24-42 (per_channel, post_scale),
 *                          patch_internvl.py:318-329 (identity LUT), and
 *                          calibquant.py:114-137 (MSB-first packing); one
 *                          rounding to the 16-bit storage dtype per torch op.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static inline int code_at(const uint8_t* row, int d, int bits) {
    const int dpe = 8 / bits;
    const int byte = row[d / dpe];
    const int shift = bits * (dpe - 1 - (d % dpe));
    return (byte >> shift) & ((1 << bits) - 1);
}

/* q (B,Hq,D) f32; codes (B,Hkv,T,D*bits/8); stats (B,Hkv,D) f32;
 * residual (B,Hkv,R,D) f32 contiguous; mask (B, T+R) f32 or NULL; out (B,Hq,D) f32. */
void cqo_decode_attention(const float* q, const uint8_t* ck, const uint8_t* cv, const float* ks, const float* kz,
                          const float* vs, const float* vz, const float* kres, const float* vres, const float* mask,
                          int B, int Hq, int Hkv, int D, int T, int R, int S, int bits, int calibrate, float off_max,
                          float off_min, float* out) {
    const int G = Hq / Hkv;
    const int nb = D * bits / 8;
    const float inv = 1.0f / sqrtf((float)D);
    const int N = T + R;
#pragma omp parallel
    {
        float* w = (float*)malloc(sizeof(float) * (size_t)(N > 0 ? N : 1));
        float* qs = (float*)malloc(sizeof(float) * (size_t)D);
#pragma omp for collapse(2) schedule(dynamic, 1)
        for (int b = 0; b < B; ++b) {
            for (int h = 0; h < Hq; ++h) {
                const int hk = h / G;
                const float* qv = q + ((size_t)b * Hq + h) * D;
                const size_t bh = (size_t)b * Hkv + hk;
                /* image logits into w[S .. S+T) */
                if (T > 0) {
                    float bias = 0.f;
                    for (int d = 0; d < D; ++d) {
                        qs[d] = qv[d] * ks[bh * D + d];
                        bias += qs[d] * kz[bh * D + d];
                    }
                    float mn = INFINITY, mx = -INFINITY;
                    for (int t = 0; t < T; ++t) {
                        const uint8_t* row = ck + (bh * T + t) * nb;
                        float acc = 0.f;
                        for (int d = 0; d < D; ++d) acc += qs[d] * (float)code_at(row, d, bits);
                        const float l = (acc - bias) * inv;
                        w[S + t] = l;
                        mn = fminf(mn, l);
                        mx = fmaxf(mx, l);
                    }
                    if (calibrate) {
                        const float tmax = mx + off_max, tmin = mn + off_min;
                        const float den = mx - mn + 1e-8f;
                        for (int t = 0; t < T; ++t) w[S + t] = (w[S + t] - mn) / den * (tmax - tmin) + tmin;
                    }
                }
                for (int r = 0; r < R; ++r) {
                    const float* kr = kres + (bh * R + r) * D;
                    float acc = 0.f;
                    for (int d = 0; d < D; ++d) acc += qv[d] * kr[d];
                    w[r < S ? r : T + r] = acc * inv;
                }
                float m = -INFINITY;
                for (int i = 0; i < N; ++i) {
                    if (mask) w[i] += mask[(size_t)b * N + i];
                    m = fmaxf(m, w[i]);
                }
                float l = 0.f;
                for (int i = 0; i < N; ++i) { w[i] = expf(w[i] - m); l += w[i]; }
                float* o = out + ((size_t)b * Hq + h) * D;
                for (int d = 0; d < D; ++d) o[d] = 0.f;
                if (T > 0) {
                    float psum = 0.f;
                    for (int t = 0; t < T; ++t) {
                        const uint8_t* row = cv + (bh * T + t) * nb;
                        const float p = w[S + t];
                        psum += p;
                        for (int d = 0; d < D; ++d) o[d] += p * (float)code_at(row, d, bits);
                    }
                    for (int d = 0; d < D; ++d) o[d] = vs[bh * D + d] * (o[d] - vz[bh * D + d] * psum);
                }
                for (int r = 0; r < R; ++r) {
                    const float* vr = vres + (bh * R + r) * D;
                    const float p = w[r < S ? r : T + r];
                    for (int d = 0; d < D; ++d) o[d] += p * vr[d];
                }
                for (int d = 0; d < D; ++d) o[d] /= l;
            }
        }
        free(w);
        free(qs);
    }
}

/* ---- storage-dtype rounding ------------------------------------------------ */
static inline float round_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return f;
    u += 0x7fffu + ((u >> 16) & 1u);
    u &= 0xffff0000u;
    memcpy(&f, &u, 4);
    return f;
}

static inline float round_fp16(float f) {
    /* fp32 -> fp16 -> fp32, round to nearest even, in integer arithmetic */
    uint32_t u;
    memcpy(&u, &f, 4);
    const uint32_t sign = u & 0x80000000u;
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return f;                 /* NaN */
    if (a >= 0x477ff000u) {                        /* >= 65520 rounds to inf */
        a = 0x7f800000u;
    } else if (a < 0x38800000u) {                  /* below 2^-14: fp16 subnormal grid, step 2^-24 */
        float af;
        memcpy(&af, &a, 4);
        const float k = 16777216.0f;               /* 2^24 */
        af = nearbyintf(af * k) / k;               /* exact: af*k < 2^10 */
        memcpy(&a, &af, 4);
    } else {
        a += 0xfffu + ((a >> 13) & 1u);
        a &= 0xffffe000u;
    }
    a |= sign;
    memcpy(&f, &a, 4);
    return f;
}

static inline float rnd(float f, int dtype) { return dtype == 0 ? round_bf16(f) : (dtype == 1 ? round_fp16(f) : f); }

/* x (B,T,H,D) f32 holding storage-dtype values; dtype 0 bf16, 1 fp16, 2 fp32.
 * codes (B,H,T,D*bits/8); scale, zero (B,H,D) f32. */
void cqo_quantize_pack(const float* x, int B, int T, int H, int D, int bits, float clip, int dtype, uint8_t* codes,
                       float* scale, float* zero) {
    const float L = (float)((1 << bits) - 1);
    const float invL = 1.0f / L;
    const int nb = D * bits / 8;
    const int dpe = 8 / bits;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; ++b) {
        for (int h = 0; h < H; ++h) {
            float* s = scale + ((size_t)b * H + h) * D;
            float* z = zero + ((size_t)b * H + h) * D;
            for (int d = 0; d < D; ++d) {
                float mn = INFINITY, mx = -INFINITY;
                for (int t = 0; t < T; ++t) {
                    const float v = x[(((size_t)b * T + t) * H + h) * D + d];
                    mn = fminf(mn, v);
                    mx = fmaxf(mx, v);
                }
                const float xmin = rnd(mn * clip, dtype), xmax = rnd(mx * clip, dtype);
                s[d] = rnd(rnd(xmax - xmin, dtype) * invL, dtype);
                z[d] = rnd(-xmin / s[d], dtype);
            }
            for (int t = 0; t < T; ++t) {
                uint8_t* row = codes + (((size_t)b * H + h) * T + t) * nb;
                memset(row, 0, (size_t)nb);
                for (int d = 0; d < D; ++d) {
                    const float v = x[(((size_t)b * T + t) * H + h) * D + d];
                    float y = rnd(rnd(v / s[d], dtype) + z[d], dtype);
                    int c = 0;
                    if (y == y) {
                        y = fminf(fmaxf(y, 0.f), L);
                        c = (int)nearbyintf(y);
                    }
                    row[d / dpe] |= (uint8_t)(c << (bits * (dpe - 1 - (d % dpe))));
                }
            }
        }
    }
}
