/*
 * A caller of the C ABI written in plain C: no torch, no C++.  One fused decode step (hw_fused_attention) and one
 * paged step (hw_copy_to_blocks + hw_paged_sdpa) on inputs whose answer has a closed form (the fused step also with the
 * fragment lengths in device memory):
 * with q = 0 every visible key gets the same weight, so out = mean of the visible V rows and lse = ln(count).
 * V[f][h][l][e] = (l % 7) + f + 0.25 * h + e / 64, exactly representable in fp32.
 * Exit code 0 and a line "c_abi ok" on success.
 */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "hogwild_hip.h"

#define CHECK_HIP(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %d at %s:%d\n", (int)e_, __FILE__, __LINE__); return 2; } } while (0)
#define CHECK_HW(x) do { int s_ = (x); if (s_ != 0) { printf("hw status %d (%s) at %s:%d\n", s_, hw_status_string(s_), __FILE__, __LINE__); return 3; } } while (0)

enum { F = 3, W = 2, HQ = 8, HKV = 2, S = 1, D = 64 };
static const int LEN[F] = {70, 33, 5};

static float vval(int f, int h, int l, int e) { return (float)(l % 7) + (float)f + 0.25f * (float)h + (float)e / 64.0f; }

static void* to_device(const void* host, size_t bytes) {
    void* d = NULL;
    if (hipMalloc(&d, bytes ? bytes : 16) != hipSuccess) return NULL;
    if (bytes && hipMemcpy(d, host, bytes, hipMemcpyHostToDevice) != hipSuccess) return NULL;
    return d;
}

int main(void) {
    if (hw_version() != HW_ABI_VERSION) { printf("ABI version mismatch\n"); return 1; }
    /* ---------------- fragments ---------------- */
    void* kd[F]; void* vd[F];
    for (int f = 0; f < F; ++f) {
        size_t n = (size_t)HKV * LEN[f] * D;
        float* k = (float*)malloc(n * sizeof(float));
        float* v = (float*)malloc(n * sizeof(float));
        for (int h = 0; h < HKV; ++h)
            for (int l = 0; l < LEN[f]; ++l)
                for (int e = 0; e < D; ++e) {
                    k[((size_t)h * LEN[f] + l) * D + e] = (float)((l * 31 + e * 7 + h) % 13) - 6.0f;   /* irrelevant: q = 0 */
                    v[((size_t)h * LEN[f] + l) * D + e] = vval(f, h, l, e);
                }
        kd[f] = to_device(k, n * sizeof(float));
        vd[f] = to_device(v, n * sizeof(float));
        free(k); free(v);
        if (!kd[f] || !vd[f]) return 2;
    }
    /* worker w sees loc+1 keys of fragment f: full, partial, none */
    int loc[F][W][S] = {{{69}, {9}}, {{32}, {-1}}, {{2}, {4}}};
    float* q = (float*)calloc((size_t)W * HQ * S * D, sizeof(float));
    float* cs = (float*)malloc(sizeof(float) * F * W * S * D);
    for (int i = 0; i < F * W * S * D; ++i) cs[i] = 1.0f;            /* cos = 1, sin = 0: the rotation is the identity */
    float* sn = (float*)calloc((size_t)F * W * S * D, sizeof(float));
    void* dq = to_device(q, sizeof(float) * W * HQ * S * D);
    void* dloc = to_device(loc, sizeof(loc));
    void* dcos = to_device(cs, sizeof(float) * F * W * S * D);
    void* dsin = to_device(sn, sizeof(float) * F * W * S * D);
    void *dout = NULL, *dlse = NULL, *drq = NULL;
    CHECK_HIP(hipMalloc(&dout, sizeof(float) * W * HQ * S * D));
    CHECK_HIP(hipMalloc(&dlse, sizeof(float) * W * HQ * S));
    CHECK_HIP(hipMalloc(&drq, sizeof(float) * F * W * HQ * S * D));

    hw_problem p;
    memset(&p, 0, sizeof(p));
    p.dtype = HW_F32;
    p.F = F; p.W = W; p.Hq = HQ; p.Hkv = HKV; p.S = S; p.E = D; p.Ev = D; p.RotE = D;
    p.scale = 0.125f;
    p.out = dout; p.lse = (float*)dlse; p.rq = drq; p.q = dq; p.locations = (const int32_t*)dloc;
    p.cosines = (const float*)dcos; p.sines = (const float*)dsin;
    p.k = (const void* const*)kd; p.v = (const void* const*)vd; p.len = LEN;
    CHECK_HW(hw_validate(&p, 1));
    size_t ws_bytes = 0;
    CHECK_HW(hw_workspace_bytes(&p, &ws_bytes));
    CHECK_HIP(hipMalloc(&p.workspace, ws_bytes));
    p.workspace_bytes = ws_bytes;
    hipStream_t stream;
    CHECK_HIP(hipStreamCreate(&stream));
    CHECK_HW(hw_fused_attention(&p, stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    float out[W][HQ][S][D], lse[W][HQ][S];
    CHECK_HIP(hipMemcpy(out, dout, sizeof(out), hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(lse, dlse, sizeof(lse), hipMemcpyDeviceToHost));
    double worst = 0.0;
    for (int w = 0; w < W; ++w)
        for (int h = 0; h < HQ; ++h) {
            int hk = h / (HQ / HKV), count = 0;
            double mean[D];
            memset(mean, 0, sizeof(mean));
            for (int f = 0; f < F; ++f) {
                int vis = loc[f][w][0] + 1 < LEN[f] ? loc[f][w][0] + 1 : LEN[f];
                for (int l = 0; l < vis; ++l, ++count)
                    for (int e = 0; e < D; ++e) mean[e] += vval(f, hk, l, e);
            }
            for (int e = 0; e < D; ++e) {
                double err = fabs(out[w][h][0][e] - mean[e] / count);
                if (err > worst) worst = err;
            }
            double el = fabs(lse[w][h][0] - log((double)count));
            if (el > worst) worst = el;
        }
    printf("fused: worst deviation from the closed form %.3e\n", worst);
    if (!(worst < 1e-4)) return 4;

    /* the same launch with the current lengths in device memory: the fragment buffers are the planned bounds, the
       kernel sees min(bound, len_dev[f]) tokens; hw_advance_lengths moves the lengths on the device */
    {
        int cur[F] = {48, 33, 0};
        const int add[F] = {2, 0, 0};                               /* -> 50, 33, 0 */
        void* dlen = to_device(cur, sizeof(cur));
        if (!dlen) return 2;
        CHECK_HW(hw_advance_lengths((int32_t*)dlen, add, F, stream));
        p.len_dev = (const int32_t*)dlen;
        CHECK_HW(hw_fused_attention(&p, stream));
        CHECK_HIP(hipStreamSynchronize(stream));
        p.len_dev = NULL;
        CHECK_HIP(hipMemcpy(out, dout, sizeof(out), hipMemcpyDeviceToHost));
        CHECK_HIP(hipMemcpy(lse, dlse, sizeof(lse), hipMemcpyDeviceToHost));
        const int now[F] = {50, 33, 0};
        worst = 0.0;
        for (int w = 0; w < W; ++w)
            for (int h = 0; h < HQ; ++h) {
                int hk = h / (HQ / HKV), count = 0;
                double mean[D];
                memset(mean, 0, sizeof(mean));
                for (int f = 0; f < F; ++f) {
                    int vis = loc[f][w][0] + 1 < now[f] ? loc[f][w][0] + 1 : now[f];
                    for (int l = 0; l < vis; ++l, ++count)
                        for (int e = 0; e < D; ++e) mean[e] += vval(f, hk, l, e);
                }
                for (int e = 0; e < D; ++e) {
                    double err = fabs(out[w][h][0][e] - mean[e] / count);
                    if (err > worst) worst = err;
                }
                double el = fabs(lse[w][h][0] - log((double)count));
                if (el > worst) worst = el;
            }
        printf("fused, lengths in device memory: worst deviation from the closed form %.3e\n", worst);
        if (!(worst < 1e-4)) return 7;
    }

    /* an unsupported head dimension is an error, not a silent no-op */
    p.E = p.Ev = 96;
    if (hw_fused_attention(&p, stream) != HW_ERR_UNSUPPORTED) { printf("expected HW_ERR_UNSUPPORTED\n"); return 5; }

    /* ---------------- paged: append 3 tokens to a sequence of 20, attend over all 23 ---------------- */
    enum { NB = 6, BS = 8, MB = 4, OLD = 20, NEW = 3 };
    size_t cn = (size_t)NB * HKV * BS * D;
    float* vc = (float*)calloc(cn, sizeof(float));
    float* kc = (float*)calloc(cn, sizeof(float));
    int bt[1][MB] = {{4, 1, 5, 0}};
    for (int l = 0; l < OLD; ++l)
        for (int h = 0; h < HKV; ++h)
            for (int e = 0; e < D; ++e) vc[(((size_t)bt[0][l / BS] * HKV + h) * BS + l % BS) * D + e] = vval(0, h, l, e);
    float* vnew = (float*)malloc(sizeof(float) * HKV * NEW * D);
    for (int h = 0; h < HKV; ++h)
        for (int t = 0; t < NEW; ++t)
            for (int e = 0; e < D; ++e) vnew[((size_t)h * NEW + t) * D + e] = vval(0, h, OLD + t, e);
    void* dkc = to_device(kc, cn * sizeof(float));
    void* dvc = to_device(vc, cn * sizeof(float));
    void* dvn = to_device(vnew, sizeof(float) * HKV * NEW * D);
    void* dbt = to_device(bt, sizeof(bt));
    int seq[1] = {OLD};
    void* dseq = to_device(seq, sizeof(seq));
    hw_copy_blocks c;
    memset(&c, 0, sizeof(c));
    c.dtype = HW_F32; c.B = 1; c.Hkv = HKV; c.S_new = NEW; c.E = D; c.Ev = D;
    c.block_size = BS; c.max_blocks = MB; c.num_blocks = NB;
    c.key_states = dvn; c.value_states = dvn;
    c.ks_b = c.vs_b = (int64_t)HKV * NEW * D; c.ks_h = c.vs_h = (int64_t)NEW * D; c.ks_s = c.vs_s = D;
    c.key_cache = dkc; c.value_cache = dvc; c.block_table = (const int32_t*)dbt; c.seq_lengths = (const int32_t*)dseq;
    CHECK_HW(hw_copy_to_blocks(&c, stream));

    int ploc[1][1][1] = {{{OLD + NEW - 1}}};
    int pfl[1] = {BS * MB};
    void* dploc = to_device(ploc, sizeof(ploc));
    void* dpfl = to_device(pfl, sizeof(pfl));
    hw_paged_problem pp;
    memset(&pp, 0, sizeof(pp));
    pp.dtype = HW_F32; pp.F = 1; pp.W = 1; pp.Hq = HQ; pp.Hkv = HKV; pp.E = D; pp.Ev = D; pp.S = 1;
    pp.block_size = BS; pp.max_blocks = MB; pp.num_blocks = NB; pp.scale = 0.125f;
    pp.out = dout; pp.lse = (float*)dlse; pp.q = dq; pp.locations = (const int32_t*)dploc; pp.fragment_lengths = (const int32_t*)dpfl;
    pp.key_cache = dkc; pp.value_cache = dvc; pp.block_table = (const int32_t*)dbt;
    size_t pws = 0;
    CHECK_HW(hw_paged_workspace_bytes(&pp, &pws));
    CHECK_HIP(hipMalloc(&pp.workspace, pws));
    pp.workspace_bytes = pws;
    CHECK_HW(hw_paged_sdpa(&pp, stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    float pout[HQ][D], plse[HQ];
    CHECK_HIP(hipMemcpy(pout, dout, sizeof(pout), hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(plse, dlse, sizeof(plse), hipMemcpyDeviceToHost));
    worst = 0.0;
    for (int h = 0; h < HQ; ++h) {
        int hk = h / (HQ / HKV);
        for (int e = 0; e < D; ++e) {
            double m = 0.0;
            for (int l = 0; l < OLD + NEW; ++l) m += vval(0, hk, l, e);
            double err = fabs(pout[h][e] - m / (OLD + NEW));
            if (err > worst) worst = err;
        }
        double el = fabs(plse[h] - log((double)(OLD + NEW)));
        if (el > worst) worst = el;
    }
    printf("paged: worst deviation from the closed form %.3e\n", worst);
    if (!(worst < 1e-4)) return 6;
    printf("c_abi ok\n");
    return 0;
}
