/*
 * C ABI of the MI355X token sampler (librapid_sampling_hip.so).
 *
 * The reference exposes this path only as three ATen functions bound with
 * pybind11 (/root/reference/sampling.cpp:2-8); it has no C interface.  The
 * entry points below are what those three functions need from the device
 * side, with plain pointers and sizes, so that any host (the pybind module in
 * rapid_sampling_amd/csrc/sampling.cpp, ctypes, cgo, JNI ...) can bind them.
 *
 * Conventions: every pointer named *device* is device memory owned by the
 * caller; `stream` is a hipStream_t passed as void* (NULL = the null stream);
 * calls enqueue work on `stream` and return without synchronising; the return
 * value is RS_OK or a negative RS_ERR_* code; nothing throws, and only the
 * calls that say so allocate.  The library keeps no state of its own between
 * calls: what a call needs beyond its arguments lives in the workspace and,
 * optionally, in an rs_policy object, both owned by the caller.
 */
#ifndef RAPID_SAMPLING_H
#define RAPID_SAMPLING_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RS_OK               0
#define RS_ERR_VOCAB       -1   /* V <= 0, V > 1048576 or V % 4 != 0   (sampling.cu:461,986)  */
#define RS_ERR_BATCH       -2   /* B <= 0 or T <= 0                    (sampling.cu:467,992)  */
#define RS_ERR_TEMPERATURE -3   /* outside [0.001, 1000]               (sampling.cu:474,999)  */
#define RS_ERR_NULL        -4   /* a required pointer is NULL                                 */
#define RS_ERR_WORKSPACE   -5   /* workspace too small or misaligned                          */
#define RS_ERR_ALIGN       -6   /* a row of logits/penalties is not 16-byte aligned           */
#define RS_ERR_ARG         -7   /* top_k / top_p not normalised (use rs_normalize_args)       */
#define RS_ERR_LAUNCH      -8   /* the HIP runtime refused the launch                         */
#define RS_ERR_DEVICE      -9   /* a kernel gave up waiting for its peer workgroups           */
#define RS_ERR_SCRATCH     -10  /* rs_sample_static: the call needs more than RS_STATIC_SCRATCH_BYTES */
#define RS_ERR_UNSUPPORTED -11  /* the current device is not a whole MI355X (256 compute units)     */

/* Bytes of RNG state per row.  Same size as the reference's
 * curandStatePhilox4_32_10_t record (sampling.cu:9,141) so that the opaque
 * tensor returned by setup_rand keeps its shape. */
#define RS_STATE_BYTES_PER_ROW 64

/* Optional per-row diagnostics (device memory, B records).  128-bit
 * quantities are (low word, high word). */
typedef struct rs_row_diag {
    float    xmax;        /* row maximum of the scaled logits                 */
    uint32_t emin_bits;   /* unused by the library (0)                        */
    uint64_t D[2];        /* sum of the exact weights W = e * 2^63 over the row */
    uint64_t P[2];        /* ceil(top_p * D)                                  */
    uint32_t left_bits;   /* same as thr_bits                                 */
    uint32_t thr_bits;    /* bit pattern of the smallest kept e               */
    uint32_t rounds;      /* histogram levels summed over the cluster; 0 = row
                             finished by the streaming path, 8 = by its
                             finishing workgroup alone from the logits, 9 = a
                             call that keeps every token (top_k = V, top_p = 1)
                             on the streaming path                            */
    uint32_t n_gt;        /* tokens with e >  threshold                       */
    uint32_t n_eq;        /* tokens with e == threshold                       */
    int32_t  index;       /* sampled token                                    */
    uint64_t G[2];        /* sum of W over e > threshold                      */
    uint64_t w_tie;       /* weight of each token with e == threshold         */
    uint64_t S[2];        /* G + n_eq * w_tie                                 */
    uint64_t r[2];        /* target of the inverse CDF, 1 <= r <= S           */
} rs_row_diag;

/* Library version, major*10000 + minor*100 + patch. */
int rs_version(void);

/* Static text for an RS_ERR_* code. */
const char *rs_error_string(int code);

/*
 * Host-side argument normalisation of both reference wrappers
 * (sampling.cu:461-486 and :986-1011): range checks, top_k<=0||top_k>V -> V,
 * top_p<0||top_p>1 -> 1, top_p==0 -> greedy (top_k=1, top_p=1), and
 * log2e_inv_temp = (float)(log2(e) / temperature).  No device work.
 */
int rs_normalize_args(double temperature, int64_t top_k, double top_p,
                      int64_t B, int64_t T, int64_t V,
                      float *log2e_inv_temp, int32_t *top_k_out, float *top_p_out);

/*
 * Size of the workspace rs_sample needs for a batch of B rows of V tokens.
 * Replaces the reference's per-call `probs` scratch tensor of B*V floats
 * (sampling.cu:488,1014): a fixed record per row (about 38 KB) plus, for the
 * streaming paths, about 1.05 bytes per token (per slice of 16384 tokens the
 * stash of its largest tokens, its counts and bins, and 4 KB for its note of
 * the non-zero penalties; up to 3.2 bytes per token for the first 6M tokens,
 * where slices are shorter; 1.5 bytes per token in rows of up to 262144
 * tokens, for the slices of 8192 tokens the one-pass wide path and the
 * counting-only pass cut there); a quarter to two fifths of the reference's
 * scratch.  It does not grow with T.  (A call is also accepted with a
 * workspace that lacks the room for those slices of 8192 tokens -- the size
 * versions before 414 asked for -- and then works on the long slices.)
 *
 * One workspace may serve calls of different shapes if it is at least
 * rs_workspace_bytes(largest B, largest V) of those calls and the same
 * (pointer, size) pair is passed every time: per-row records are addressed from
 * its end, per-slice data from its front.
 */
int rs_workspace_bytes(int32_t B, int32_t V, size_t *bytes);

/*
 * Zero a freshly allocated workspace (device memory, 256-byte aligned) with a
 * fill kernel on `stream`.  Call once after allocation, and again after a call
 * reported RS_ERR_DEVICE; rs_sample leaves the workspace ready for the next
 * call on the same stream.  Allocates nothing.
 */
int rs_workspace_init(void *workspace_device, size_t bytes, void *stream);

/*
 * How long a workgroup waits for its peers before it gives up with
 * RS_ERR_DEVICE, in milliseconds (0 = the default, 2000).  Stored in the
 * workspace header by a one-thread kernel on `stream`; rs_workspace_init
 * resets it to the default.  For tests of the error path.
 */
int rs_workspace_set_wait_limit(void *workspace_device, uint32_t milliseconds, void *stream);

/*
 * Read back the sticky device error word of a workspace (synchronises
 * `stream`).  *status is RS_OK or RS_ERR_DEVICE.
 */
int rs_workspace_status(const void *workspace_device, int32_t *status, void *stream);

/*
 * Where the first wait that gave up was (synchronises `stream`; no counterpart
 * in the reference).  where[0] = the wait (0 none; 1 a histogram level,
 * 2 the first level's totals, 3 the candidates of a level, 4 the masses,
 * 5 the index, 6 the verdict of the one-launch kernel, 7 the slots and bins
 * the workgroups of a row post ahead of the first exchange), where[1] =
 * row << 16 | slice of the workgroup that gave up, where[2] and where[3] = what
 * it had seen and what it waited for.  Cleared by rs_workspace_init.
 */
int rs_workspace_where(const void *workspace_device, uint32_t where[4], void *stream);

/*
 * Routing state of the streaming paths and an asynchronous error report, owned
 * by the caller (optional; one per workspace).  No counterpart in the
 * reference.
 *
 * A row the wait-free streaming path cannot finish from what its pass over
 * the logits set aside is done by one workgroup alone, from the logits again,
 * which takes several times as long as the general kernel needs for a whole
 * call of moderate size: with a bounding top_k (<= 1024) that takes unusual
 * rows (ties of thousands of tokens), without one (top_p < 1 alone) a flat
 * distribution (a call without a bounding top_k also counts a row as slow
 * when it is finished from a list of more than V/20, at least 2048, tokens:
 * the general kernel is faster for such calls; a call with a bounding top_k
 * does the same, and also counts a row as slow when its stashes hold more
 * tokens than the finishing workgroup's list and have to be gone through
 * twice more -- flat rows cut into many slices -- if it is of fewer than 2^24
 * tokens or of a shape the row kernel takes, see rs_sample, which does such
 * rows faster whatever the size of the call).  The
 * two-pass wide path (kept sets of any size, two passes over the logits) does a
 * row the slow way when its slices are no fair samples of the row; the one-pass
 * wide path (a sample of the row, then one pass over all of it; calls of at
 * least 2^26 tokens, 12 million in rows of up to 262144) when the sample is
 * no fair picture of the row (a few
 * tokens that carry most of the mass under top_p).  Calls that are
 * given a policy report "a row went the slow way: yes/no" to a word of pinned
 * host memory inside it (yes at once, no by the next call on the workspace),
 * and rs_sample_ex reads that word, without waiting, before it routes the
 * next call: while it is set, calls of that kind go to the general kernel (a
 * call without a bounding top_k to a wide path when it is large enough, a call
 * that would take the one-pass wide path to the two-pass one, calls of a
 * shape the row kernel takes to the row kernel);
 * after 64 of them the path is tried again, each try that fails doubles that
 * number (up to 1024), and a run of good calls as long as the last stay away
 * puts it back to 64.  There is a word per KIND of call -- streaming with a
 * bounding top_k, streaming without, one-pass wide, two-pass wide -- and per
 * SIZE CLASS (tokens per
 * call below 2^20, below 2^24, from 2^24 on), so that workloads that share a
 * policy do not flip each other's route.  The first call without a bounding
 * top_k of a size class, and every such call that tries again after a stay
 * away, runs as a PROBE: on the wide path, whose time does not depend on the
 * kept set, with the finishing workgroups reporting whether the rows' kept sets
 * (more than 512 tokens?) would have fitted the streaming path's stashes --
 * so a workload of flat rows never pays for a row done the slow way.  A probe
 * reports on itself when it has run; until then its word is pending and calls
 * of its kind and size class are probes too (at most 64 of them, then they stay
 * away as after a slow row), so a caller
 * that issues many calls without synchronising does not run attempts on rows
 * nobody has looked at yet.  Without
 * a policy, calls with a bounding top_k always stream and calls without never
 * do.  Results do not depend on the routing.
 *
 * A kernel that gives up waiting (RS_ERR_DEVICE) also writes the code into a
 * pinned word, which rs_policy_error reads without synchronising.
 *
 * rs_policy_create allocates (a small host object and 64 bytes of pinned host
 * memory); rs_policy_destroy frees them -- only after the last call that was
 * given the policy has completed on the device.
 * rs_policy_state (over all size classes): bit 0 set: calls without a bounding
 * top_k currently leave the streaming path, bit 1 set: so do calls with one,
 * bit 2 set: calls that would take the one-pass wide path take the two-pass
 * one, bit 3 set: calls that would take the two-pass wide path take the
 * general kernel.
 * rs_policy_error: *error = RS_OK or RS_ERR_DEVICE as last reported; with
 * clear != 0 the word is reset.
 */
typedef struct rs_policy rs_policy;
int  rs_policy_create(rs_policy **policy_out);
void rs_policy_destroy(rs_policy *policy);
int  rs_policy_state(const rs_policy *policy, int32_t *state);
int  rs_policy_error(rs_policy *policy, int32_t *error, int32_t clear);

/*
 * setup_rand (sampling.cu:136-144): initialise B records of RNG state for
 * Philox4x32-10 with key = seed and subsequence = row, draw counter 0.
 * state_device: B * RS_STATE_BYTES_PER_ROW bytes.  Runs on `stream` (the
 * reference uses the null stream).
 */
int rs_philox_init(void *state_device, uint64_t seed, int32_t B, void *stream);

/*
 * One sampling call; replaces the kernel launches at sampling.cu:500,
 * :1025 and :1033.
 *
 *   logits_device     first sampled row; row b starts b*row_stride floats on.
 *                     For a (B,T,V) tensor pass base + (T-1)*V and
 *                     row_stride = T*V (sampling.cu:176,202).
 *   penalties_device  (B,V) contiguous, updated in place, or NULL for the
 *                     plain path (sampling.cu:427-437).
 *   out_device        (B,) int32 sampled token ids.
 *   rng_state_device  from rs_philox_init; each row's draw counter advances
 *                     by one.  Ignored (may be NULL) when injected_u is given.
 *   injected_u_device (B,) floats in (0,1] used instead of the RNG, or NULL.
 *   top_k, top_p, log2e_inv_temp   as produced by rs_normalize_args:
 *                     1 <= top_k <= V, 0 < top_p <= 1.
 *   workspace_device  rs_workspace_bytes(B,V) bytes, initialised once.
 *   diag_device       B rs_row_diag records, or NULL.
 *   e_bits_device     (B,V) uint32: bit patterns of e = 2^(x - floor(max x))
 *                     per token (2^-40 <= e < 2, or 0 for a dead token: e
 *                     below 2^-40 has probability 0 and is never returned),
 *                     or NULL.  Together with diag.thr_bits this is the kept
 *                     set {e >= thr}.
 *
 * Calls that share a workspace must be ordered on one stream.
 *
 * The call is one kernel launch (the general kernel: rows of fewer than 8192
 * tokens in calls of fewer than 2^17, and whatever the other paths do not
 * take; with penalties and top_k <= 1024 the one-launch streaming kernel while
 * the call fits the GPU at once), two for calls without penalties whose kept
 * set is expected to be small (a wait-free pass over the logits and a per-row
 * finish; see rs_policy; plain temperature sampling -- top_k = V, top_p = 1,
 * every token kept -- takes these two launches as well: the pass only counts,
 * and the finish reads one slice of the row again), four for kept sets of
 * thousands of tokens in calls of at least 3 * 2^23 tokens in rows of more
 * than 262144 tokens (the two-pass wide
 * path: the counting pass, a one-workgroup-per-row plan, a second pass over
 * the logits that counts the boundary bin's next digit and sets the tokens
 * around the expected threshold aside, a per-row finish), three for the same
 * from 2^26 tokens on, and from 12 million tokens on in rows of 49152 to
 * 262144 tokens (the one-pass wide path: a one-workgroup-per-row look at
 * a sample of the row, an eighth of it at most, one pass over the logits that
 * counts the row's bins and, finely, the range in which the sample expects the
 * threshold, and sets the tokens around it aside, a per-row finish that checks
 * the guess against the exact counts), one again for such kept sets in rows of
 * 8192 to 65536 tokens when the call has 64 rows (128 from 32768 tokens on)
 * or more (the row kernel: one workgroup of 1024 threads per row, the row in
 * its registers; calls of more than 256 rows only from 32768 tokens per row
 * on), or three for calls of at least
 * 2^23 tokens with penalties and top_k <= 1024 (a pass over logits and
 * penalties that also writes the decayed penalties, the finish, which patches
 * the sampled tokens' penalties, and a fix-up kernel for slices the pass left
 * alone); results are identical either way.  No environment variable is read.
 * A device that is not a whole MI355X (256 compute units) is refused with
 * RS_ERR_UNSUPPORTED: the kernels' waits are only known to end on one.
 */
int rs_sample(const float *logits_device, int64_t row_stride,
              float *penalties_device, int32_t *out_device,
              void *rng_state_device, const float *injected_u_device,
              int32_t B, int32_t V,
              float presence_penalty, float repetition_penalty, float penalty_decay,
              float log2e_inv_temp, int32_t top_k, float top_p,
              void *workspace_device, size_t workspace_bytes,
              rs_row_diag *diag_device, uint32_t *e_bits_device,
              void *stream);

/*
 * The same call for logits stored as bfloat16 or IEEE half (RS_DTYPE_BF16,
 * RS_DTYPE_F16; RS_DTYPE_F32 makes it rs_sample).  An extension: the reference
 * rejects anything but float32 (sampling.cu:452-457, :976-981), and so do the
 * drop-in Python functions unless the caller opts in.  Both formats widen to
 * float32 exactly, so the result is that of rs_sample on the widened logits,
 * bit for bit; rows of V elements, row_stride in elements, rows 8-byte aligned.
 * Half the algorithmic bytes per row (2 V).
 */
#define RS_DTYPE_F32  0
#define RS_DTYPE_BF16 1
#define RS_DTYPE_F16  2
int rs_sample_dtype(const void *logits_device, int32_t logits_dtype, int64_t row_stride,
                    float *penalties_device, int32_t *out_device,
                    void *rng_state_device, const float *injected_u_device,
                    int32_t B, int32_t V,
                    float presence_penalty, float repetition_penalty, float penalty_decay,
                    float log2e_inv_temp, int32_t top_k, float top_p,
                    void *workspace_device, size_t workspace_bytes,
                    rs_row_diag *diag_device, uint32_t *e_bits_device,
                    void *stream);

/*
 * rs_sample_dtype with explicit options (NULL = all defaults, which makes it
 * rs_sample_dtype).  `path` forces the way through the library (tests,
 * benchmarks): RS_PATH_CLUSTER the general one-launch kernel, RS_PATH_STREAM
 * the streaming path when top_k <= 1024 or the call keeps every token (else
 * the general kernel),
 * RS_PATH_ATTEMPT the streaming path whatever top_k is (penalties take the
 * general kernel on these three), RS_PATH_FUSED the streaming pass and the
 * finish in one launch (any call whose rows span at least two slices, with or
 * without penalties; else the general kernel), RS_PATH_WIDE the two-pass wide
 * path and RS_PATH_WIDE1 the one-pass wide path (any call without penalties; a
 * call that keeps every token takes the counting-only streaming variant),
 * RS_PATH_ROW the row kernel (any call without penalties in rows of up to
 * 65536 tokens; else the general kernel).  `slice_r` forces the float4 groups per thread of the
 * general kernel (1, 2, 4, 8, 16 or 32; 0 = chosen by the library).
 * `policy` see rs_policy.  No counterpart in the reference.
 */
#define RS_PATH_AUTO    0
#define RS_PATH_CLUSTER 1
#define RS_PATH_STREAM  2
#define RS_PATH_ATTEMPT 3
#define RS_PATH_FUSED   4
#define RS_PATH_WIDE    5
#define RS_PATH_WIDE1   6
#define RS_PATH_ROW     7
typedef struct rs_options {
    int32_t    path;
    int32_t    slice_r;
    rs_policy *policy;
} rs_options;
int rs_sample_ex(const void *logits_device, int32_t logits_dtype, int64_t row_stride,
                 float *penalties_device, int32_t *out_device,
                 void *rng_state_device, const float *injected_u_device,
                 int32_t B, int32_t V,
                 float presence_penalty, float repetition_penalty, float penalty_decay,
                 float log2e_inv_temp, int32_t top_k, float top_p,
                 void *workspace_device, size_t workspace_bytes,
                 rs_row_diag *diag_device, uint32_t *e_bits_device,
                 const rs_options *options, void *stream);

/*
 * rs_sample_ex without a workspace argument, for callers that cannot allocate
 * device memory or carry a workspace along: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  No counterpart in the
 * reference.
 *
 * The workspace is a static array in device memory inside the library,
 * RS_STATIC_SCRATCH_BYTES (32 MiB) on every GPU the library is used on, held
 * until the process ends.  A call that cannot do with that much (what
 * rs_workspace_bytes(B, V) asks for, less the room for slices of 8192 tokens
 * in large calls, which such a call then does without)
 * is refused with RS_ERR_SCRATCH (64 rows of 152064 tokens need 16 MiB,
 * 32 rows of 131072 tokens 14 MiB; 128 rows of 1048576 tokens, 105 MB, do not
 * fit).  Every check that can refuse a call -- arguments, alignment, size, the
 * device -- is made before anything is launched.  The call allocates nothing
 * and synchronises nothing: it enqueues one small kernel that clears the
 * launch counters of the array's header and the B row records the call is
 * about to use, then exactly what rs_sample_ex enqueues; so a call starts from
 * clean records whatever the one before it left, also after RS_ERR_DEVICE.
 * The sticky error word of the array, the place of the first wait that gave
 * up, the wait limit and the words of the routing report survive that clearing:
 * with `options->policy` the reports work as they do with a workspace of the
 * caller's own, and without one a caller learns of a kernel that gave up a
 * wait from rs_static_status (the call that gave up returned RS_OK and left
 * garbage in out_device, as rs_sample_ex does).
 *
 * The address of the array is looked up once per device, with
 * hipGetSymbolAddress, on the first call made while that device is current --
 * which must therefore happen outside stream capture: call rs_static_prepare()
 * (or make one ordinary call) on each device before capturing.  The array of
 * the CURRENT device is used; a `stream` of another device is refused
 * (RS_ERR_ARG).
 *
 * Every call on a GPU uses that GPU's one array: calls must be ordered on one
 * stream (or otherwise serialised); calls that overlap on one GPU race.
 */
#define RS_STATIC_SCRATCH_BYTES (32u << 20)
int rs_sample_static(const void *logits_device, int32_t logits_dtype, int64_t row_stride,
                     float *penalties_device, int32_t *out_device,
                     void *rng_state_device, const float *injected_u_device,
                     int32_t B, int32_t V,
                     float presence_penalty, float repetition_penalty, float penalty_decay,
                     float log2e_inv_temp, int32_t top_k, float top_p,
                     rs_row_diag *diag_device, uint32_t *e_bits_device,
                     const rs_options *options, void *stream);

/* Looks up the static array's address on the current device (no GPU work, no
 * allocation); to be called once per device before rs_sample_static is used
 * under stream capture.  No counterpart in the reference. */
int rs_static_prepare(void);

/* Device address of the current device's static array (RS_STATIC_SCRATCH_BYTES
 * long), or NULL; for rs_workspace_where / rs_workspace_set_wait_limit and for
 * tests.  No counterpart in the reference. */
void *rs_static_workspace(void);

/*
 * The sticky error word of the current device's static array (synchronises
 * `stream`): *status = RS_OK or RS_ERR_DEVICE; where[4], if not NULL, as
 * rs_workspace_where.  With clear != 0 a reported error is put back to RS_OK
 * by a one-thread kernel on `stream`.  No counterpart in the reference.
 */
int rs_static_status(int32_t *status, uint32_t where[4], int32_t clear, void *stream);

/*
 * Launch-plus-one-read floor: a kernel that reads every logit of the B rows once
 * and max-combines one int per row into out_device (which it does not clear),
 * every thread issuing all its loads before it uses the first.  variant 0: the
 * general kernel's grid for (B,V), plain loads; 1: the same with loads marked
 * non-temporal (as the sampling kernels read the logits); 2, 3: the same two
 * on the streaming pass's grid; 4 to 8: other shapes of a read-only kernel,
 * all non-temporal, which max-combine into out_device[0] only -- 4 a
 * persistent grid of 2048 workgroups that sweeps the rows front to back with
 * four loads per thread in flight, 5 the same with an eighth of the data per
 * XCD, 6 contiguous 256 KiB per workgroup, 7 a persistent grid of 1024
 * workgroups per XCD with eight loads in flight, 8 one of 4096 workgroups with
 * two.  Measurement aid for the B=1 latency bound and for the read bandwidth
 * the hardware delivers; no counterpart in the reference.
 */
int rs_floor_read(const float *logits_device, int64_t row_stride, int32_t *out_device,
                  int32_t B, int32_t V, int32_t variant, void *stream);

#ifdef __cplusplus
}
#endif
#endif
