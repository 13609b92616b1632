/* Plain-C restatement of the Hogwild! fragmented-KV attention path.  TEST INFRASTRUCTURE ONLY:
 * the product library never links or loads this file; tests and the benchmark's CPU-baseline leg
 * use it as an independent checker next to the numpy oracle.
 *
 * Follows, in its own words:
 *   rotation ........ src/rope.cuh:18-51 (second half reads cos/sin at the first-half index) and
 *                     src/q_rope.h:18-30 (second half reads its own index) — chosen by `own_index`
 *   mask bound ...... src/kernels/kernel_v21.cuh:96-98      maxL = min(L, loc + 1)
 *   GQA ............. python/hogwild/attention.py:47-48     kv head = q head / (Hq/Hkv)
 *   softmax/output .. python/hogwild/attention.py:60-63     softmax over the union of visible keys
 *   LSE ............. natural-log logsumexp of the scaled masked logits (kernel_v21.cuh:300 is this / ln 2)
 * Pinned by tests/test_oracle_pins.py against the numpy oracle, brute force and closed forms.
 * All tensors are fp32 on entry (16-bit inputs are widened exactly by the caller); arithmetic is fp64.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static float round_bf16(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return x; /* NaN */
    u = (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u;
    memcpy(&x, &u, 4);
    return x;
}

static float round_f16(float x) {
    /* fp32 -> fp16 -> fp32, round-to-nearest-even, with subnormals and overflow to inf */
    uint32_t u;
    memcpy(&u, &x, 4);
    uint32_t sign = u & 0x80000000u;
    uint32_t a = u & 0x7fffffffu;
    if (a >= 0x7f800000u) return x;               /* inf / NaN */
    if (a >= 0x477ff000u) {                       /* >= 65520 rounds to inf */
        a = 0x7f800000u;
    } else if (a >= 0x38800000u) {                /* normal half: keep 10 mantissa bits */
        a = (a + 0xfffu + ((a >> 13) & 1u)) & 0xffffe000u;
    } else {                                      /* subnormal half: quantum 2^-24 */
        float ax;
        memcpy(&ax, &a, 4);
        float r = (ax + 0.5f) - 0.5f;             /* at magnitude 0.5 the fp32 ulp is 2^-24 (ties-to-even) */
        memcpy(&a, &r, 4);
    }
    u = sign | a;
    memcpy(&x, &u, 4);
    return x;
}

static float round_storage(double x, int storage) {
    float f = (float)x;
    if (storage == 1) return round_f16(f);
    if (storage == 2) return round_bf16(f);
    return f;
}

/* rq[F,W,Hq,S,E] = rope(q[W,Hq,S,E], cos/sin[F,W,S,R]); storage: 0 f32, 1 f16, 2 bf16 rounding of the result */
void hwo_rope(float* rq, const float* q, const float* cosv, const float* sinv,
              int F, int W, int Hq, int S, int E, int R, int storage, int own_index) {
    int h = R / 2;
    for (int f = 0; f < F; ++f)
        for (int w = 0; w < W; ++w)
            for (int hq = 0; hq < Hq; ++hq)
                for (int s = 0; s < S; ++s) {
                    const float* x = q + (((size_t)w * Hq + hq) * S + s) * E;
                    float* y = rq + ((((size_t)f * W + w) * Hq + hq) * S + s) * E;
                    const float* c = cosv + (((size_t)f * W + w) * S + s) * R;
                    const float* sn = sinv + (((size_t)f * W + w) * S + s) * R;
                    for (int e = 0; e < h; ++e) {
                        int j = own_index ? e + h : e;
                        double x1 = x[e], x2 = x[e + h];
                        y[e] = round_storage(x1 * c[e] - x2 * sn[e], storage);
                        y[e + h] = round_storage(x2 * c[j] + x1 * sn[j], storage);
                    }
                    for (int e = R; e < E; ++e) y[e] = x[e];
                }
}

/* out[W,Hq,S,Ev], lse[W,Hq,S] from pre-rotated rq[F,W,Hq,S,E]; k[f]: [Hkv,len[f],E]; v[f]: [Hkv,len[f],Ev] */
void hwo_sdpa(float* out, float* lse, const float* rq, const int* loc,
              const float* const* k, const float* const* v, const int* len, double scale,
              int F, int W, int Hq, int Hkv, int S, int E, int Ev) {
    int G = Hq / Hkv;
    size_t total = 0;
    for (int f = 0; f < F; ++f) total += (size_t)len[f];
    double* sc = (double*)malloc(sizeof(double) * (total ? total : 1));
    double* acc = (double*)malloc(sizeof(double) * Ev);
    for (int w = 0; w < W; ++w)
        for (int hq = 0; hq < Hq; ++hq)
            for (int s = 0; s < S; ++s) {
                int hkv = hq / G;
                double m = -INFINITY;
                size_t n = 0;
                for (int f = 0; f < F; ++f) {
                    int L = len[f];
                    int vis = loc[((size_t)f * W + w) * S + s] + 1;
                    if (vis > L) vis = L;
                    const float* qv = rq + ((((size_t)f * W + w) * Hq + hq) * S + s) * E;
                    for (int l = 0; l < vis; ++l) {
                        const float* kr = k[f] + ((size_t)hkv * L + l) * E;
                        double d = 0;
                        for (int e = 0; e < E; ++e) d += (double)qv[e] * (double)kr[e];
                        d *= scale;
                        sc[n++] = d;
                        if (d > m) m = d;
                    }
                }
                float* o = out + (((size_t)w * Hq + hq) * S + s) * Ev;
                size_t li = ((size_t)w * Hq + hq) * S + s;
                if (n == 0) {
                    for (int e = 0; e < Ev; ++e) o[e] = 0.f;
                    lse[li] = -INFINITY;
                    continue;
                }
                double den = 0;
                for (int e = 0; e < Ev; ++e) acc[e] = 0;
                n = 0;
                for (int f = 0; f < F; ++f) {
                    int L = len[f];
                    int vis = loc[((size_t)f * W + w) * S + s] + 1;
                    if (vis > L) vis = L;
                    for (int l = 0; l < vis; ++l) {
                        double p = exp(sc[n++] - m);
                        den += p;
                        const float* vr = v[f] + ((size_t)hkv * L + l) * Ev;
                        for (int e = 0; e < Ev; ++e) acc[e] += p * (double)vr[e];
                    }
                }
                for (int e = 0; e < Ev; ++e) o[e] = (float)(acc[e] / den);
                lse[li] = (float)(m + log(den));
            }
    free(sc);
    free(acc);
}
