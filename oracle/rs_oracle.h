/*
 * CPU oracle for the batched token sampler -- TEST INFRASTRUCTURE, NOT PRODUCT.
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
 * build, load or call anything in this directory.  The shipped library never
 * links it and has no CPU fallback.
 *
 * Two restatements of the reference algorithm live here:
 *
 *   rs_oracle.c    the CANONICAL arithmetic the GPU library must reproduce
 *                  bit for bit: the reference's steps (fused logit/penalty
 *                  scale, base-2 softmax, quaternary threshold search on bit
 *                  patterns, tie compensation, inverse-CDF pick, penalty
 *                  decay) with every cross-element sum done in exact integer
 *                  fixed point, so the result does not depend on the order of
 *                  summation and any parallel decomposition agrees with a
 *                  plain loop.
 *   ref_literal.c  a LITERAL fp32 emulation of the reference kernel's thread
 *                  layout (1024 virtual threads, 32-lane butterflies, serial
 *                  32-way combine, two-uniform strided pick).  It is the
 *                  cross-check that the canonical restatement keeps the
 *                  reference's semantics; it is never compared bit for bit
 *                  with the GPU.
 *
 * Every function cites the reference lines it follows (sampling.cu:N is
 * /root/reference/sampling.cu line N).
 */
#ifndef RS_ORACLE_H
#define RS_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* The smallest live e is 2^-40 (bit pattern 0x2B800000); below it e is flushed to zero. */
#define RS_E_MIN_BITS 0x2B800000u

/* Per-row diagnostics; mirrors rs_row_diag of include/rapid_sampling.h.
 * 128-bit quantities are (low word, high word). */
typedef struct {
    float    xmax;        /* row maximum of the scaled logits                 */
    uint32_t emin_bits;   /* bit pattern of the smallest live (non-zero) e     */
    uint64_t D[2];        /* sum of the weights W over the row                */
    uint64_t P[2];        /* ceil(top_p * D)                                  */
    uint32_t left_bits;   /* `left` when the reference's search loop ends     */
    uint32_t thr_bits;    /* smallest kept e  (the canonical threshold)       */
    uint32_t rounds;      /* passes of the search loop                        */
    uint32_t n_gt;        /* count of e >  thr                                */
    uint32_t n_eq;        /* count of e == thr                                */
    int32_t  index;       /* sampled token                                    */
    uint64_t G[2];        /* sum of W over e > thr                            */
    uint64_t w_tie;       /* weight of each token with e == thr               */
    uint64_t S[2];        /* G + n_eq * w_tie                                 */
    uint64_t r[2];        /* target of the inverse CDF, 1 <= r <= S           */
} rs_oracle_diag;

/* ---- element-wise canonical arithmetic -------------------------------- */
float    rs_oracle_sf(float x);
float    rs_oracle_scale(float logit, float penalty, int has_penalty, float c);
uint32_t rs_oracle_e_bits(float x, float M);
uint64_t rs_oracle_w(uint32_t e_bits);
void     rs_oracle_ceil_mul(float f, uint64_t s_lo, uint64_t s_hi, uint64_t out[2]);

/* ---- host argument normalisation -------------------------------------- */
/* returns 0, or -1 (V), -2 (B,T), -3 (temperature) like the reference's throws */
int rs_oracle_normalize(double temperature, int64_t top_k, double top_p,
                        int64_t B, int64_t T, int64_t V,
                        float *c_out, int32_t *k_out, float *p_out);

/* ---- Philox4x32-10 ---------------------------------------------------- */
void     rs_oracle_philox(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]);
/* draw #n of row `row` for `seed`: counter (n_lo, n_hi, row_lo, row_hi) */
void     rs_oracle_philox_draw(uint64_t seed, uint64_t row, uint64_t n, uint32_t out[4]);
void     rs_oracle_r_from_bits(uint64_t u64, uint64_t s_lo, uint64_t s_hi, uint64_t out[2]);

/* ---- one row, canonical ------------------------------------------------ */
/*
 * logits: V floats.  penalties: V floats updated in place, or NULL.
 * use_u != 0: the uniform is the float `u` in (0,1];  else the 64 random bits
 * `u64`.  e_bits_out: V uint32 (bit patterns of e), or NULL.
 */
void rs_oracle_row(const float *logits, float *penalties, int32_t V,
                   float c, int32_t top_k, float top_p,
                   int use_u, float u, uint64_t u64,
                   float presence, float repetition, float decay,
                   uint32_t *e_bits_out, rs_oracle_diag *diag);

/* definitional threshold by sorting (independent of the search loop) */
uint32_t rs_oracle_thr_by_sort(const uint32_t *e_bits, int32_t V, int32_t top_k, uint64_t P_lo, uint64_t P_hi);

/* ---- a batch, canonical ------------------------------------------------ */
/*
 * Row b reads logits + b*row_stride.  rng: B records of 16 uint32 laid out as
 * the library's state tensor (key0,key1,ctr_lo,ctr_hi,row_lo,row_hi,...);
 * advanced by one draw per row when injected_u is NULL.
 */
void rs_oracle_batch(const float *logits, int64_t row_stride, float *penalties,
                     int32_t *out, uint32_t *rng, const float *injected_u,
                     int32_t B, int32_t V, float c, int32_t top_k, float top_p,
                     float presence, float repetition, float decay,
                     rs_oracle_diag *diag /* B entries or NULL */);

/* the same, also returning the bit patterns of e of every token: e_bits_out (B,V) or NULL */
void rs_oracle_batch_e(const float *logits, int64_t row_stride, float *penalties,
                       int32_t *out, uint32_t *rng, const float *injected_u,
                       int32_t B, int32_t V, float c, int32_t top_k, float top_p,
                       float presence, float repetition, float decay,
                       rs_oracle_diag *diag, uint32_t *e_bits_out);

void rs_oracle_rng_init(uint32_t *rng, uint64_t seed, int32_t B);

/* ---- literal fp32 emulation of the reference kernel -------------------- */
typedef struct {
    float    threshold;   /* float(left) after the loop (sampling.cu:329)     */
    float    comp;        /* tie compensation (sampling.cu:366-371)           */
    float    pmax, pmin, denom, xmax;
    uint32_t kept;        /* count of p >= threshold                          */
    uint32_t n_eq, n_gt;
    uint32_t rounds;
    int32_t  idxt;        /* bucket picked by the first uniform               */
    int32_t  index;       /* sampled token                                    */
} ref_literal_diag;

/*
 * variant 0: general kernel (sampling.cu:517-752 / 172-438 with penalties)
 * variant 1: top-p-only kernel (sampling.cu:757-964)
 * probs_out: V floats (the scratch `probs` row) or NULL.
 */
void ref_literal_row(const float *logits, float *penalties, int32_t V,
                     float c, int32_t top_k, float top_p, int variant,
                     float u1, float u2,
                     float presence, float repetition, float decay,
                     float *probs_out, ref_literal_diag *diag);

/* the reference's two block scans on n<=1024 values (sampling.cu:48-104) */
void ref_literal_block_scan_f32(const float *in, float *out, float *total, int descending_ladder);
/* a 64-lane ladder scan; descending!=0: offsets 32,16,...,1  else 1,2,...,32 */
void ref_literal_wave64_scan_f32(const float *in, float *out, int descending);

#ifdef __cplusplus
}
#endif
#endif
