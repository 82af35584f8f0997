/*
 * Canonical CPU restatement of the sampling path -- TEST INFRASTRUCTURE.
 * See rs_oracle.h for who may use it.  Build with -ffp-contract=off: every
 * fused multiply-add below is an explicit fmaf().
 *
 * What is kept from the reference, step by step (sampling.cu:N):
 *   x   = sf((sf(l) - pen) * c)              :208-225  (plain: sf(l*c) :553)
 *   e   = exp2(x - max)                      :228-240
 *   threshold search on bit patterns, 4-way  :261-329
 *   recount above / at the threshold         :332-355
 *   tie compensation                         :365-371
 *   inverse-CDF pick, first index reached    :374-426
 *   penalty decay with one-hot add           :427-437
 * What is restated so that the result is independent of summation order AND
 * of where the row maximum sits (so that a slice of a row can be worked
 * before the maximum of the whole row is known):
 *   - exp2 splits x itself, not x - max:  n = floor(x), f = x - n (exact),
 *     e = poly5(f) * 2^(n - M) with M = floor(max x), a fixed degree-5 Horner
 *     polynomial with positive coefficients (monotone, poly(1) < 2).  The
 *     significand of e depends on x alone; the maximum only shifts the
 *     exponent.  Below 2^-40 e is flushed to zero, as the reference's
 *     exp2f(x - max) underflows to zero 149 octaves down (:235): such a token
 *     has probability exactly 0, takes no part in the selection and can never
 *     be returned (a logit masked with -inf must not come back, however large
 *     top_k and top_p are).  So e = 0 or 2^-40 <= e < 2, and e_max in [1,2);
 *   - the probability of token i is carried as the exact integer
 *         W_i = e_i * 2^63  =  significand24(e_i) << (exponent(e_i) - 87),
 *     the row total D = sum W_i (up to 2^84: 128-bit) replaces the float
 *     denominator, and "mass >= top_p" becomes  sum W >= P = ceil(top_p * D)
 *     in exact arithmetic (the reference divides by the float denominator
 *     and sums floats, :248,:285-292);
 *   - tie compensation and the CDF are integer: each token equal to the
 *     threshold weighs  min(W_thr, (P-G)/n_eq, W_thr*(k-n_gt)/n_eq)
 *     (the reference's  thr * min(1,(top_p-sgtp)/(thr*neqk),(top_k-sgtk)/neqk)
 *     :368-371,:404), and one uniform picks the first index whose inclusive
 *     CDF reaches r = ceil(u*S) (the reference spends two uniforms on a
 *     bucket and then an element of it, :384-423 -- same distribution).
 */
#include "rs_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

typedef unsigned __int128 u128;

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float    u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline void     put128(uint64_t out[2], u128 v) { out[0] = (uint64_t)v; out[1] = (uint64_t)(v >> 64); }

/* sampling.cu:131-134 : NaN -> 0, +-Inf -> +-FLT_MAX */
float rs_oracle_sf(float x)
{
    float y = isnan(x) ? 0.0f : x;
    return isinf(y) ? copysignf(FLT_MAX, y) : y;
}

/* sampling.cu:220 (penalty kernel) and :553 (plain kernel) */
float rs_oracle_scale(float logit, float penalty, int has_penalty, float c)
{
    if (has_penalty)
        return rs_oracle_sf((rs_oracle_sf(logit) - penalty) * c);
    return rs_oracle_sf(logit * c);
}

/*
 * Bit pattern of e = 2^(x - M) for a row whose maximum has floor M
 * (sampling.cu:235 computes exp2f(x - max); the common factor 2^(max - M)
 * cancels in every probability).  n = floor(x) and f = x - n are exact, f in
 * [0,1]; 2^f is a degree-5 minimax polynomial (relative error 8.3e-8)
 * evaluated by Horner with fmaf, all coefficients positive, so it is monotone
 * in f and poly(1) < 2 = 2*poly(0): e is monotone in x.  The exponent n - M
 * is added to the exponent field; below 2^-40 the result is flushed to zero
 * (bit pattern 0): a dead token.
 */
static const float RS_C1 = 0x1.62e4bap-1f;
static const float RS_C2 = 0x1.ebdb56p-3f;
static const float RS_C3 = 0x1.c91ce6p-5f;
static const float RS_C4 = 0x1.277856p-7f;
static const float RS_C5 = 0x1.e974fap-10f;

uint32_t rs_oracle_e_bits(float x, float M)
{
    float n = floorf(x);
    float f = x - n;
    float p = RS_C5;
    p = fmaf(p, f, RS_C4);
    p = fmaf(p, f, RS_C3);
    p = fmaf(p, f, RS_C2);
    p = fmaf(p, f, RS_C1);
    p = fmaf(p, f, 1.0f);
    float k = fmaxf(n - M, -41.0f);             /* <= 0; anything below -40 is clamped anyway */
    uint32_t b = f2u(p) + ((uint32_t)(int32_t)k << 23);
    return b < RS_E_MIN_BITS ? 0u : b;
}

/* exact weight of a token: e * 2^63 = significand24 << (exponent - 87), in [2^23, 2^64);
 * 0 for a dead token (e flushed to zero) */
uint64_t rs_oracle_w(uint32_t e_bits)
{
    if (e_bits < RS_E_MIN_BITS) return 0;
    uint64_t m = (e_bits & 0x7FFFFFu) | 0x800000u;
    int ex = (int)(e_bits >> 23);
    return m << (ex - 87);
}

/* ceil(f * s) for a float 0 < f <= 1 and s < 2^100, exact; clamped to [1, s] */
static u128 ceil_mul128(float f, u128 s)
{
    if (!(f > 0.0f)) return 1;
    if (f >= 1.0f) return s;
    uint32_t b = f2u(f);
    int ex = (int)(b >> 23);
    uint64_t m = b & 0x7FFFFFu;
    if (ex == 0) ex = 1; else m |= 0x800000u;     /* subnormal / normal   */
    int sh = 150 - ex;                            /* f = m * 2^-sh, sh>=24 */
    u128 prod = (u128)m * s;                      /* < 2^24 * 2^100        */
    u128 r;
    if (sh >= 126) r = 1;                         /* 0 < prod < 2^124 < 2^sh */
    else r = (prod + (((u128)1 << sh) - 1)) >> sh;
    if (r < 1) r = 1;
    if (r > s) r = s;
    return r;
}

void rs_oracle_ceil_mul(float f, uint64_t s_lo, uint64_t s_hi, uint64_t out[2])
{
    put128(out, ceil_mul128(f, ((u128)s_hi << 64) | s_lo));
}

/* 64 random bits -> r in [1,S]: floor(u64 * S / 2^64) + 1 */
static u128 r_from_bits128(uint64_t u64, u128 S)
{
    uint64_t s_lo = (uint64_t)S, s_hi = (uint64_t)(S >> 64);
    return (u128)u64 * s_hi + (uint64_t)(((u128)u64 * s_lo) >> 64) + 1;
}

void rs_oracle_r_from_bits(uint64_t u64, uint64_t s_lo, uint64_t s_hi, uint64_t out[2])
{
    put128(out, r_from_bits128(u64, ((u128)s_hi << 64) | s_lo));
}

/* sampling.cu:474-486 / :986-1011 */
int rs_oracle_normalize(double temperature, int64_t top_k, double top_p,
                        int64_t B, int64_t T, int64_t V,
                        float *c_out, int32_t *k_out, float *p_out)
{
    if (!(V > 0 && V <= 1048576 && V % 4 == 0)) return -1;
    if (!(B > 0 && T > 0)) return -2;
    if (!(temperature >= 0.001 && temperature <= 1000)) return -3;
    if (top_k <= 0 || top_k > V) top_k = V;
    if (top_p < 0 || top_p > 1) top_p = 1;
    if (top_p == 0) { top_k = 1; top_p = 1; }
    *c_out = (float)(M_LOG2E / temperature);
    *k_out = (int32_t)top_k;
    *p_out = (float)top_p;
    return 0;
}

/* ---- Philox4x32-10 (Salmon et al., SC'11); the generator behind
 * curandStatePhilox4_32_10_t (sampling.cu:9).  curand_init(seed, b, 0)
 * (sampling.cu:137) sets key = seed and counter = (0, 0, b_lo, b_hi); each
 * curand_uniform4 (sampling.cu:383) consumes one counter value. ---------- */
void rs_oracle_philox(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4])
{
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
    uint32_t k0 = key[0], k1 = key[1];
    for (int i = 0; i < 10; i++) {
        uint64_t p0 = (uint64_t)0xD2511F53u * c0;
        uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
        uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
        uint32_t n1 = (uint32_t)p1;
        uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        uint32_t n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

void rs_oracle_philox_draw(uint64_t seed, uint64_t row, uint64_t n, uint32_t out[4])
{
    uint32_t ctr[4] = { (uint32_t)n, (uint32_t)(n >> 32), (uint32_t)row, (uint32_t)(row >> 32) };
    uint32_t key[2] = { (uint32_t)seed, (uint32_t)(seed >> 32) };
    rs_oracle_philox(ctr, key, out);
}

void rs_oracle_rng_init(uint32_t *rng, uint64_t seed, int32_t B)
{
    for (int32_t b = 0; b < B; b++) {
        uint32_t *s = rng + 16 * (size_t)b;
        memset(s, 0, 64);
        s[0] = (uint32_t)seed; s[1] = (uint32_t)(seed >> 32);
        s[2] = 0; s[3] = 0;                 /* draw counter */
        s[4] = (uint32_t)b; s[5] = 0;       /* subsequence = row */
    }
}

/* ---- definitional threshold: the largest t with
 *      count{e >= t} >= top_k  or  sum{W : e >= t} >= P   ------------------ */
static int cmp_desc_u32(const void *a, const void *b)
{
    uint32_t x = *(const uint32_t *)a, y = *(const uint32_t *)b;
    return (x < y) - (x > y);
}

uint32_t rs_oracle_thr_by_sort(const uint32_t *e_bits, int32_t V, int32_t top_k, uint64_t P_lo, uint64_t P_hi)
{
    const u128 P = ((u128)P_hi << 64) | P_lo;
    uint32_t *s = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)V);
    memcpy(s, e_bits, sizeof(uint32_t) * (size_t)V);
    qsort(s, (size_t)V, sizeof(uint32_t), cmp_desc_u32);
    u128 mass = 0;
    uint32_t thr = s[V - 1];
    for (int32_t i = 0; i < V;) {
        int32_t j = i;
        while (j < V && s[j] == s[i]) { mass += rs_oracle_w(s[j]); j++; }
        if ((int64_t)j >= top_k || mass >= P) { thr = s[i]; break; }
        i = j;
    }
    free(s);
    return thr;
}

void rs_oracle_row(const float *logits, float *penalties, int32_t V,
                   float c, int32_t top_k, float top_p,
                   int use_u, float u, uint64_t u64,
                   float presence, float repetition, float decay,
                   uint32_t *e_bits_out, rs_oracle_diag *diag)
{
    float    *x  = (float *)malloc(sizeof(float) * (size_t)V);
    uint32_t *eb = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)V);
    rs_oracle_diag dg;
    memset(&dg, 0, sizeof dg);

    /* 1. scaled logits and their maximum (sampling.cu:208-227) */
    float xmax = -INFINITY;
    for (int32_t i = 0; i < V; i++) {
        x[i] = rs_oracle_scale(logits[i], penalties ? penalties[i] : 0.0f, penalties != NULL, c);
        if (x[i] > xmax) xmax = x[i];
    }
    dg.xmax = xmax;
    const float M = floorf(xmax);

    /* 2. e = 2^(x - M), total D (sampling.cu:228-258 without the division).
     *    Dead tokens (e = 0) weigh nothing and are left out of everything that
     *    follows; the token at the maximum has e >= 1, so a row is never all dead. */
    u128 D = 0;
    uint32_t emin = 0xFFFFFFFFu, emax = 0;
    uint64_t n_live = 0;
    for (int32_t i = 0; i < V; i++) {
        eb[i] = rs_oracle_e_bits(x[i], M);
        if (eb[i] == 0) continue;
        n_live++;
        D += rs_oracle_w(eb[i]);
        if (eb[i] < emin) emin = eb[i];
        if (eb[i] > emax) emax = eb[i];
    }
    const u128 P = ceil_mul128(top_p, D);
    put128(dg.D, D); put128(dg.P, P); dg.emin_bits = emin;

    /* 3. the reference's quaternary search, literally (sampling.cu:261-329),
     *    with exact counts and integer masses */
    uint32_t left = emin, right = emax + 1;
    uint64_t cnt_x = n_live;
    u128 mass_x = D;
    uint32_t rounds = 0;
    while ((cnt_x > (uint64_t)top_k || mass_x > P) && left < right - 1) {
        uint32_t pz = (left + right) / 2;
        uint32_t py = (left + pz) / 2;
        uint32_t pw = (pz + right) / 2;
        uint64_t cy = 0, cz = 0, cw = 0;
        u128 my = 0, mz = 0, mw = 0;
        for (int32_t i = 0; i < V; i++) {
            uint32_t b = eb[i];
            if (b == 0) continue;
            uint64_t w = rs_oracle_w(b);
            if (b >= py) { cy++; my += w; }
            if (b >= pz) { cz++; mz += w; }
            if (b >= pw) { cw++; mw += w; }
        }
        rounds++;
        if (cy < (uint64_t)top_k && my < P) { right = py; continue; }
        if (cz < (uint64_t)top_k && mz < P) { left = py; right = pz; cnt_x = cy; mass_x = my; continue; }
        if (cw < (uint64_t)top_k && mw < P) { left = pz; right = pw; cnt_x = cz; mass_x = mz; continue; }
        left = pw; cnt_x = cw; mass_x = mw;
    }
    dg.left_bits = left; dg.rounds = rounds;

    /* 4. canonical threshold = smallest kept e; recount (sampling.cu:332-355) */
    uint32_t thr = 0xFFFFFFFFu;
    for (int32_t i = 0; i < V; i++) if (eb[i] >= left && eb[i] < thr) thr = eb[i];
    uint32_t n_gt = 0, n_eq = 0;
    u128 G = 0;
    for (int32_t i = 0; i < V; i++) {
        if (eb[i] == thr) n_eq++;
        else if (eb[i] > thr) { n_gt++; G += rs_oracle_w(eb[i]); }
    }
    dg.thr_bits = thr; dg.n_gt = n_gt; dg.n_eq = n_eq; put128(dg.G, G);

    /* 5. tie compensation (sampling.cu:365-371), integer form */
    const uint64_t w_thr = rs_oracle_w(thr);
    u128 w_tie = w_thr;
    u128 a = (P > G) ? (P - G) / n_eq : 0;
    u128 bk = ((uint32_t)top_k > n_gt) ? ((u128)w_thr * ((uint32_t)top_k - n_gt)) / n_eq : 0;
    if (a < w_tie) w_tie = a;
    if (bk < w_tie) w_tie = bk;
    if (w_tie == 0 && G == 0) w_tie = 1;
    const u128 S = G + (u128)n_eq * w_tie;
    dg.w_tie = (uint64_t)w_tie; put128(dg.S, S);

    /* 6. inverse CDF in index order; first index whose inclusive CDF >= r
     *    (the single false->true transition of sampling.cu:388-397,410-423) */
    const u128 r = use_u ? ceil_mul128(u, S) : r_from_bits128(u64, S);
    put128(dg.r, r);
    u128 cdf = 0;
    int32_t idx = -1;
    for (int32_t i = 0; i < V; i++) {
        u128 w = (eb[i] > thr) ? (u128)rs_oracle_w(eb[i]) : (eb[i] == thr ? w_tie : 0);
        cdf += w;
        if (cdf >= r) { idx = i; break; }
    }
    dg.index = idx;

    /* 7. penalty decay + one-hot add, evaluated on the pre-decay value
     *    (sampling.cu:427-437) */
    if (penalties) {
        for (int32_t i = 0; i < V; i++) {
            float p = penalties[i];
            float add = (i != idx) ? 0.0f : (p == 0.0f ? presence : repetition);
            penalties[i] = fmaf(p, decay, add);
        }
    }

    if (e_bits_out) memcpy(e_bits_out, eb, sizeof(uint32_t) * (size_t)V);
    if (diag) *diag = dg;
    free(x); free(eb);
}

void rs_oracle_batch(const float *logits, int64_t row_stride, float *penalties,
                     int32_t *out, uint32_t *rng, const float *injected_u,
                     int32_t B, int32_t V, float c, int32_t top_k, float top_p,
                     float presence, float repetition, float decay,
                     rs_oracle_diag *diag)
{
    rs_oracle_batch_e(logits, row_stride, penalties, out, rng, injected_u, B, V, c, top_k, top_p,
                      presence, repetition, decay, diag, NULL);
}

void rs_oracle_batch_e(const float *logits, int64_t row_stride, float *penalties,
                       int32_t *out, uint32_t *rng, const float *injected_u,
                       int32_t B, int32_t V, float c, int32_t top_k, float top_p,
                       float presence, float repetition, float decay,
                       rs_oracle_diag *diag, uint32_t *e_bits_out)
{
    for (int32_t b = 0; b < B; b++) {
        rs_oracle_diag dg;
        uint64_t u64 = 0;
        if (!injected_u) {
            uint32_t *s = rng + 16 * (size_t)b;
            uint32_t ctr[4] = { s[2], s[3], s[4], s[5] };
            uint32_t key[2] = { s[0], s[1] };
            uint32_t o[4];
            rs_oracle_philox(ctr, key, o);
            u64 = ((uint64_t)o[0] << 32) | o[1];
            if (++s[2] == 0) ++s[3];
        }
        rs_oracle_row(logits + (int64_t)b * row_stride,
                      penalties ? penalties + (int64_t)b * V : NULL, V, c, top_k, top_p,
                      injected_u != NULL, injected_u ? injected_u[b] : 0.0f, u64,
                      presence, repetition, decay, e_bits_out ? e_bits_out + (size_t)b * V : NULL, &dg);
        out[b] = dg.index;
        if (diag) diag[b] = dg;
    }
}
