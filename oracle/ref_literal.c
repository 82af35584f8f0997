/*
 * Literal fp32 emulation of the reference kernel on the CPU -- TEST
 * INFRASTRUCTURE (see rs_oracle.h).  One row is worked by 1024 virtual
 * threads in the reference's own element->thread mapping and with its own
 * reduction trees, so float sums round as they do there; exp2f is libm's
 * (the reference's is libdevice's -- the two agree to ~2 ulp, not bit for
 * bit).  Used to check that the canonical oracle keeps the reference's
 * semantics: same kept set away from rounding boundaries, same distribution.
 *
 * Follows sampling.cu:11-104 (primitives), :172-438 (penalty kernel),
 * :517-752 (plain kernel), :757-964 (top-p-only kernel).
 */
#include "rs_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

#define NT 1024      /* BLOCKDIM_X_SAMPLE, sampling.cu:171 */
#define NW 32        /* warps per block */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float    u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

static float sf(float x)                           /* sampling.cu:131-134 */
{
    float y = isnan(x) ? 0.0f : x;
    return isinf(y) ? copysignf(FLT_MAX, y) : y;
}

/* xor butterfly 16,8,4,2,1 inside each 32-lane warp (sampling.cu:11-17) */
static void warp_allreduce_sum_f32(float *v)       /* v: NT values */
{
    float t[NT];
    for (int off = 16; off > 0; off /= 2) {
        for (int i = 0; i < NT; i++) t[i] = v[i] + v[(i & ~31) | ((i & 31) ^ off)];
        memcpy(v, t, sizeof t);
    }
}

/* blockReduceAll<float, SumOp, 1024, false> (sampling.cu:19-33,44-46) */
static float block_sum_f32(float *v)
{
    warp_allreduce_sum_f32(v);
    float w[NT];
    for (int i = 0; i < NT; i++) w[i] = (i < NW) ? v[i * 32 + 31] : 0.0f;
    /* only the first warp butterflies (:31) */
    float t[32];
    for (int off = 16; off > 0; off /= 2) {
        for (int i = 0; i < 32; i++) t[i] = w[i] + w[i ^ off];
        memcpy(w, t, sizeof t);
    }
    return w[0];
}

/* blockReduceAll<float, SumOp, 1024, true>: thread 0 adds the 32 warp
 * results in order (sampling.cu:34-43) */
static float block_sum_monotone_f32(float *v)
{
    warp_allreduce_sum_f32(v);
    float s = v[31];
    for (int w = 1; w < NW; w++) s += v[w * 32 + 31];
    return s;
}

/* warpInclusiveScan + blockInclusiveScan (sampling.cu:48-104) */
void ref_literal_block_scan_f32(const float *in, float *out, float *total, int descending_ladder)
{
    float v[NT], t[NT];
    memcpy(v, in, sizeof v);
    int offs_desc[5] = {16, 8, 4, 2, 1}, offs_asc[5] = {1, 2, 4, 8, 16};
    const int *offs = descending_ladder ? offs_desc : offs_asc;
    for (int s = 0; s < 5; s++) {
        int off = offs[s];
        for (int i = 0; i < NT; i++) t[i] = ((i & 31) >= off) ? v[i] + v[i - off] : v[i];
        memcpy(v, t, sizeof t);
    }
    float ws[NW];
    for (int w = 0; w < NW; w++) ws[w] = v[w * 32 + 31];
    float s = ws[0];
    for (int w = 1; w < NW; w++) { s += ws[w]; ws[w] = s; }     /* :85-92 */
    for (int i = 32; i < NT; i++) v[i] += ws[i / 32 - 1];        /* :96-98 */
    memcpy(out, v, sizeof v);
    if (total) *total = v[NT - 1];
}

static void block_scan_u32(const uint32_t *in, uint32_t *out, uint32_t *total)
{
    uint32_t s = 0;                 /* integer: any order gives the same */
    for (int i = 0; i < NT; i++) { s += in[i]; out[i] = s; }
    if (total) *total = s;
}

void ref_literal_wave64_scan_f32(const float *in, float *out, int descending)
{
    float v[64], t[64];
    memcpy(v, in, sizeof v);
    for (int s = 0; s < 6; s++) {
        int off = descending ? (32 >> s) : (1 << s);
        for (int i = 0; i < 64; i++) t[i] = (i >= off) ? v[i] + v[i - off] : v[i];
        memcpy(v, t, sizeof t);
    }
    memcpy(out, v, sizeof v);
}

void ref_literal_row(const float *logits, float *penalties, int32_t V,
                     float c, int32_t top_k, float top_p, int variant,
                     float u1, float u2,
                     float presence, float repetition, float decay,
                     float *probs_out, ref_literal_diag *diag)
{
    const int V4 = V / 4;
    float *probs = (float *)malloc(sizeof(float) * (size_t)V);
    float acc[NT];
    ref_literal_diag dg;
    memset(&dg, 0, sizeof dg);

    /* stage A (:208-227 / :547-559 / :784-796) */
    float maxu = -INFINITY;
    for (int i = 0; i < V; i++) {
        float fl = penalties ? sf((sf(logits[i]) - penalties[i]) * c) : sf(logits[i] * c);
        probs[i] = fl;
        maxu = fmaxf(maxu, fl);
    }
    dg.xmax = maxu;

    /* stage B (:228-240): per thread, per float4 partial `em` */
    for (int t = 0; t < NT; t++) {
        float d = 0.0f;
        for (int i = t; i < V4; i += NT) {
            float em = 0.0f;
            for (int j = 0; j < 4; j++) em += exp2f(probs[4 * i + j] - maxu);
            d += em;
        }
        acc[t] = d;
    }
    float denom = block_sum_f32(acc);
    dg.denom = denom;

    /* stage C (:241-258) */
    float pmax = -INFINITY, pmin = INFINITY;
    for (int i = 0; i < V; i++) {
        float fr = exp2f(probs[i] - maxu) / denom;
        probs[i] = fr;
        pmax = fmaxf(pmax, fr);
        pmin = fminf(pmin, fr);
    }
    dg.pmax = pmax; dg.pmin = pmin;

    /* stage D (:261-329 / :829-876) */
    uint32_t left = f2u(pmin), right = f2u(pmax) + 1;
    uint32_t cntx = (uint32_t)V;
    float lx = 1.0f;
    uint32_t rounds = 0;
    float my_[NT], mz_[NT], mw_[NT];
    while (((variant == 0 && cntx > (uint32_t)top_k) || lx > top_p) && left < right - 1) {
        uint32_t pz = (left + right) / 2;
        uint32_t py = (left + pz) / 2;
        uint32_t pw = (pz + right) / 2;
        float fy = u2f(py), fz = u2f(pz), fw = u2f(pw);
        uint32_t cy = 0, cz = 0, cw = 0;
        for (int t = 0; t < NT; t++) {
            float ay = 0, az = 0, aw = 0;
            for (int i = t; i < V4; i += NT)
                for (int j = 0; j < 4; j++) {
                    float p = probs[4 * i + j];
                    if (p >= fy) { cy++; ay += p; }
                    if (p >= fz) { cz++; az += p; }
                    if (p >= fw) { cw++; aw += p; }
                }
            my_[t] = ay; mz_[t] = az; mw_[t] = aw;
        }
        rounds++;
        float ly = block_sum_monotone_f32(my_);
        int ky = (variant == 0) ? (cy < (uint32_t)top_k) : 1;
        if (ky && ly < top_p) { right = py; continue; }
        float lz = block_sum_monotone_f32(mz_);
        int kz = (variant == 0) ? (cz < (uint32_t)top_k) : 1;
        if (kz && lz < top_p) { left = py; right = pz; cntx = cy; lx = ly; continue; }
        float lw = block_sum_monotone_f32(mw_);
        int kw = (variant == 0) ? (cw < (uint32_t)top_k) : 1;
        if (kw && lw < top_p) { left = pz; right = pw; cntx = cz; lx = lz; continue; }
        left = pw; cntx = cw; lx = lw;
    }
    float threshold = u2f(left);
    dg.threshold = threshold; dg.rounds = rounds;

    /* stage E (:332-355) */
    float gtp[NT], scan_f[NT];
    uint32_t eqk[NT], gtk[NT], scan_u[NT];
    uint32_t kept = 0;
    for (int t = 0; t < NT; t++) {
        float g = 0; uint32_t e = 0, k = 0;
        for (int i = t; i < V4; i += NT)
            for (int j = 0; j < 4; j++) {
                float p = probs[4 * i + j];
                if (p == threshold) e++;
                if (p > threshold) { k++; g += p; }
            }
        gtp[t] = g; eqk[t] = e; gtk[t] = k;
        kept += e + k;
    }
    float sgtp; uint32_t seqk, sgtk;
    ref_literal_block_scan_f32(gtp, scan_f, &sgtp, 1);
    block_scan_u32(eqk, scan_u, &seqk);
    block_scan_u32(gtk, scan_u, &sgtk);
    dg.kept = kept; dg.n_eq = seqk; dg.n_gt = sgtk;

    /* stage F (:365-371 / :903-908) */
    uint32_t neqk = seqk;
    float comp = 1.0f;
    if (neqk > 0) {
        comp = fminf(sf((top_p - sgtp) / (threshold * (float)neqk)), comp);
        if (variant == 0)
            comp = fminf(sf((float)((uint32_t)top_k - sgtk) / (float)neqk), comp);
        comp = fmaxf(comp, 0.0f);
    }
    dg.comp = comp;

    /* stage G1 (:374-398): bucket = thread */
    float actual[NT], cumu[NT], sum_p;
    for (int t = 0; t < NT; t++) actual[t] = gtp[t] + (threshold * (float)eqk[t]) * comp;
    ref_literal_block_scan_f32(actual, cumu, &sum_p, 1);
    float randp = sum_p * u1;
    int idxt = 0;
    for (int t = 0; t < NT; t++) {
        int u = randp <= cumu[t];
        int u_ = (t == 0) ? 0 : (randp <= cumu[t - 1]);
        if (u != u_) idxt = t;
    }
    dg.idxt = idxt;

    /* stage G2 (:400-426): the <=1024 elements owned by thread idxt */
    float o[NT], cumo[NT], sum_o;
    int idn[NT];
    for (int t = 0; t < NT; t++) {
        idn[t] = idxt * 4 + (t / 4) * 4 * NT + (t % 4);
        float o0 = (idn[t] < V) ? probs[idn[t]] : 0.0f;
        o[t] = (o0 < threshold) ? 0.0f : (o0 == threshold) ? (o0 * comp) : o0;
    }
    ref_literal_block_scan_f32(o, cumo, &sum_o, 1);
    float rand_2 = sum_o * u2;
    int out_id = 0;
    for (int t = 0; t < NT; t++) {
        int u = rand_2 <= cumo[t];
        int u_ = (t == 0) ? 0 : (rand_2 <= cumo[t - 1]);
        if (u != u_) out_id = (idn[t] < V) ? idn[t] : 0;
    }
    dg.index = out_id;

    /* stage H (:427-437) */
    if (penalties) {
        for (int i = 0; i < V; i++) {
            float p = penalties[i];
            penalties[i] = fmaf(p, decay, (out_id != i) ? 0.0f : (p == 0.0f ? presence : repetition));
        }
    }
    if (probs_out) memcpy(probs_out, probs, sizeof(float) * (size_t)V);
    if (diag) *diag = dg;
    free(probs);
}
