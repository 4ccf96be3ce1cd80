/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the router logits.
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load
 * this library.  The product path (iris_testing_amd/) never does.
 *
 * Restates the matmul inside the reference's router
 *     routed_values = F.softmax(torch.einsum('th,he->te', tokens, router), dim=-1)
 * (reference utils.py:201) with a *specified* fp32 reduction order, so that the
 * top-k indices derived from it can be compared bit-for-bit with the HIP kernel:
 *
 *     logit[t,e] = bias[e] + chain_h( fmaf(x[t,h], w[h,e], acc) ),  h = 0 .. H-1,
 *
 * i.e. one fused-multiply-add chain per (t,e) in ascending h, starting from
 * +0.0f, every operand widened exactly to fp32 first, and the bias added last
 * with one fp32 addition.  torch's own einsum is free to use any order; this
 * one is fixed so that CPU and GPU agree on every bit.
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off; the fmaf below is
 * either the hardware FMA or libm's correctly-rounded software fmaf, both give
 * the same bits).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define CLONES __attribute__((target_clones("avx2,fma", "default")))

static inline float bf16_to_f32(uint16_t v) {
    uint32_t u = ((uint32_t)v) << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* x:[T,H] fp32, w:[H,E] fp32, bias:[E] fp32 or NULL, out:[T,E] fp32. */
CLONES
int oracle_router_logits_f32(const float* x, const float* w, const float* bias,
                             int T, int H, int E, float* out) {
    if (T < 0 || H < 0 || E <= 0) return -1;
    float* acc = (float*)malloc(sizeof(float) * (size_t)E);
    if (!acc) return -2;
    for (int t = 0; t < T; ++t) {
        for (int e = 0; e < E; ++e) acc[e] = 0.0f;
        const float* xr = x + (size_t)t * H;
        for (int h = 0; h < H; ++h) {
            const float xv = xr[h];
            const float* wr = w + (size_t)h * E;
            for (int e = 0; e < E; ++e) acc[e] = __builtin_fmaf(xv, wr[e], acc[e]);
        }
        float* o = out + (size_t)t * E;
        if (bias) {
            for (int e = 0; e < E; ++e) o[e] = acc[e] + bias[e];
        } else {
            for (int e = 0; e < E; ++e) o[e] = acc[e];
        }
    }
    free(acc);
    return 0;
}

/* Same, operands given as raw bf16 bit patterns (uint16). */
CLONES
int oracle_router_logits_bf16(const uint16_t* x, const uint16_t* w, const float* bias,
                              int T, int H, int E, float* out) {
    if (T < 0 || H < 0 || E <= 0) return -1;
    float* wf = (float*)malloc(sizeof(float) * (size_t)H * (size_t)E);
    float* acc = (float*)malloc(sizeof(float) * (size_t)E);
    if (!wf || !acc) { free(wf); free(acc); return -2; }
    for (size_t i = 0; i < (size_t)H * (size_t)E; ++i) wf[i] = bf16_to_f32(w[i]);
    for (int t = 0; t < T; ++t) {
        for (int e = 0; e < E; ++e) acc[e] = 0.0f;
        const uint16_t* xr = x + (size_t)t * H;
        for (int h = 0; h < H; ++h) {
            const float xv = bf16_to_f32(xr[h]);
            const float* wr = wf + (size_t)h * E;
            for (int e = 0; e < E; ++e) acc[e] = __builtin_fmaf(xv, wr[e], acc[e]);
        }
        float* o = out + (size_t)t * E;
        if (bias) {
            for (int e = 0; e < E; ++e) o[e] = acc[e] + bias[e];
        } else {
            for (int e = 0; e < E; ++e) o[e] = acc[e];
        }
    }
    free(wf);
    free(acc);
    return 0;
}

/*
 * Top-k selection on logits: descending logit, ties broken towards the lower
 * expert index; restates `torch.topk(routed_values, topk, dim=-1)` (reference
 * utils.py:202) with the tie rule made explicit (torch leaves it unspecified).
 * softmax is strictly monotone, so the order on logits is the order on the
 * probabilities wherever the probabilities differ.
 * idx:[T,k] int32 out.  k <= E.
 */
int oracle_topk_select(const float* logits, int T, int E, int k, int32_t* idx) {
    if (k > E || k < 0) return -1;
    unsigned char* taken = (unsigned char*)malloc((size_t)E);
    if (!taken) return -2;
    for (int t = 0; t < T; ++t) {
        const float* l = logits + (size_t)t * E;
        memset(taken, 0, (size_t)E);
        for (int j = 0; j < k; ++j) {
            int best = -1;
            for (int e = 0; e < E; ++e) {
                if (taken[e]) continue;
                if (best < 0 || l[e] > l[best]) best = e; /* strict > keeps the lower index on ties */
            }
            taken[best] = 1;
            idx[(size_t)t * k + j] = best;
        }
    }
    free(taken);
    return 0;
}
